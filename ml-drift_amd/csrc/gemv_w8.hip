// Streaming int8 GEMV for gfx950 (decode: 1..4 tokens, fp32 or fp16 tensors, per-channel or
// group-wise scales, optional zero points).
//
// Packed buffer (the reference's I4O4 layout with one byte per weight): row ks (4 input
// channels) holds Ns blocks of 16 bytes; in a block, word i is input channel i and its bytes
// are the output channels 0..3 of the slice, stored as u = w + 128.
//
// All arithmetic is fp32: a byte becomes a float with one conversion (v_cvt_f32_ubyte0..3) and
// enters one fused multiply-add.  The constant centre is not subtracted per weight:
// sum_k a_k (u_k - c) = sum_k a_k u_k - c sum_k a_k with c = 128 + zero point, removed once per
// chunk of 32 input channels (one scale group when group-wise), where the scale is applied too.
//
// Thread layout as in the int4 kernel: LPR lanes cover one contiguous row segment (LPR x 16 B =
// LPR slices), 64/LPR rows per wave, WAVES waves per work-group; a thread owns whole chunks of
// 8 consecutive K-slices, issues its 8 weight loads back to back and prefetches the next
// chunk while it computes.  K is reduced through LDS in a fixed order.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mldhip {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct W8Params {
  const u32x4* weights;
  const void* act;
  const void* scale;
  const void* zero_point;  // same shape as scale, or null
  const void* bias;
  void* dst;
  int m, ks, ns;
  int chunks;        // ceil(ks / 8)
  int group_chunks;  // chunks per scale group (grouped only)
  int groups;
  int grouped;
  // Batched weights selected by runtime ids (fully_connected.cc:654-665, 804-822;
  // fully_connected_util.cc:279-290): blockIdx.z = dst row, m tokens per row; the matrices lie one
  // after the other, scales are [group][weights_batch][Ns][4].
  const int32_t* batch_ids;
  int rows, src_rows, weights_batch;
  // Runtime channel bounds (the streaming kernel only): int32 values in device memory, read at the top
  // of the kernel; an index < 0 = not set; null = no bounds.
  const int32_t* rt_params;
  int src_end_idx, dst_end_idx, k_channels;
};

__device__ __forceinline__ void Load4(const float* p, size_t i, float v[4]) {
  const float4 r = *reinterpret_cast<const float4*>(p + i);
  v[0] = r.x;
  v[1] = r.y;
  v[2] = r.z;
  v[3] = r.w;
}
__device__ __forceinline__ void Load4(const __half* p, size_t i, float v[4]) {
  const uint2 r = *reinterpret_cast<const uint2*>(p + i);
  const __half2 lo = *reinterpret_cast<const __half2*>(&r.x);
  const __half2 hi = *reinterpret_cast<const __half2*>(&r.y);
  v[0] = __low2float(lo);
  v[1] = __high2float(lo);
  v[2] = __low2float(hi);
  v[3] = __high2float(hi);
}
// Four values as they lie in memory, and their conversion: a load and its conversion are kept apart
// where several loads must be in flight at once.
__device__ __forceinline__ float4 LoadRaw4(const float* p, size_t i) { return *reinterpret_cast<const float4*>(p + i); }
__device__ __forceinline__ uint2 LoadRaw4(const __half* p, size_t i) { return *reinterpret_cast<const uint2*>(p + i); }
__device__ __forceinline__ void Cvt4(const float4& r, float v[4]) {
  v[0] = r.x;
  v[1] = r.y;
  v[2] = r.z;
  v[3] = r.w;
}
__device__ __forceinline__ void Cvt4(const uint2& r, float v[4]) {
  const __half2 lo = *reinterpret_cast<const __half2*>(&r.x);
  const __half2 hi = *reinterpret_cast<const __half2*>(&r.y);
  v[0] = __low2float(lo);
  v[1] = __high2float(lo);
  v[2] = __low2float(hi);
  v[3] = __high2float(hi);
}
__device__ __forceinline__ void Store1(float* dst, size_t i, float r, const float* bias, size_t bi) {
  dst[i] = bias ? r + bias[bi] : r;
}
__device__ __forceinline__ void Store1(__half* dst, size_t i, float r, const __half* bias, size_t bi) {
  __half h = __float2half_rn(r);
  if (bias) h = __hadd(h, bias[bi]);
  dst[i] = h;
}

template <typename T, int LPR, int WAVES, int M, bool BATCHED>
__global__ __launch_bounds__(WAVES * 64) void fc_w8_stream_kernel(W8Params p) {
  constexpr int THREADS = WAVES * 64;
  constexpr int ROWS = THREADS / LPR;  // chunks the work-group covers per step
  constexpr int RPW = 64 / LPR;        // rows per wave
  constexpr int STRIP = LPR * 4;       // output channels per work-group
  constexpr int PARTS = THREADS / STRIP > ROWS ? ROWS : THREADS / STRIP;
  constexpr int RPP = ROWS / PARTS;    // rows per part
  __shared__ float red[ROWS][M][STRIP];
  __shared__ float red2[PARTS][M][STRIP];

  // BATCHED: this row's matrix (an id outside the batch is clamped into it), its source row (one
  // shared row is broadcast) and the token strides of the two tensors
  const int brow = BATCHED ? (int)blockIdx.z : 0;
  int wb = BATCHED ? p.batch_ids[brow] : 0;
  if (BATCHED) wb = min(max(wb, 0), p.weights_batch - 1);
  const u32x4* weights = p.weights + (BATCHED ? (size_t)wb * p.ks * p.ns : 0);
  const T* act = static_cast<const T*>(p.act);
  const T* scale = static_cast<const T*>(p.scale) + (BATCHED ? (size_t)wb * p.ns * 4 : 0);
  const T* zero_point = p.zero_point ? static_cast<const T*>(p.zero_point) + (BATCHED ? (size_t)wb * p.ns * 4 : 0) : nullptr;
  const size_t group_stride = (size_t)p.ns * 4 * (BATCHED ? p.weights_batch : 1);
  const int act_stride = BATCHED ? p.src_rows * M : M, act_tok0 = BATCHED ? min(brow, p.src_rows - 1) * M : 0;
  const int dst_stride = BATCHED ? p.rows * M : M, dst_tok0 = BATCHED ? brow * M : 0;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int col = lane % LPR;
  const int row = wave * RPW + lane / LPR;
  const int slice_raw = blockIdx.x * LPR + col;
  const int slice = slice_raw < p.ns ? slice_raw : p.ns - 1;  // clamp: loads stay in range, result unused
  // runtime channel bounds: K-slices that count (the loop over scale groups runs over all of them in
  // the reference), dst slices that are written
  int ks_live = p.ks, ns_live = p.ns, chunks_live = p.chunks;
  if (p.rt_params != nullptr) {
    if (!p.grouped && p.src_end_idx >= 0) ks_live = SrcEndSlices(p.rt_params[p.src_end_idx], p.k_channels, p.ks);
    if (p.dst_end_idx >= 0) ns_live = DstEndSlice(p.rt_params[p.dst_end_idx], p.ns);
    if ((int)blockIdx.x * LPR >= ns_live) return;  // (the whole work-group: no barrier is left waiting)
    chunks_live = (ks_live + 7) / 8;
  }

  float acc[M][4];
#pragma unroll
  for (int m = 0; m < M; ++m)
#pragma unroll
    for (int o = 0; o < 4; ++o) acc[m][o] = 0.0f;

  // per-channel constants
  float s_lin[4] = {1.0f, 1.0f, 1.0f, 1.0f}, z_lin[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (!p.grouped) {
    Load4(scale, (size_t)slice * 4, s_lin);
    if (zero_point) Load4(zero_point, (size_t)slice * 4, z_lin);
  }

  auto load_weights = [&](int c, u32x4 (&w)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int ks = min(c * 8 + j, p.ks - 1);  // rows past K re-read the last one; their activations are zero
      w[j] = __builtin_nontemporal_load(weights + (size_t)ks * p.ns + slice);
    }
  };
  auto load_acts = [&](int c, float (&a)[8][M][4]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int ks = c * 8 + j;
#pragma unroll
      for (int m = 0; m < M; ++m) {
        // unconditional load at a clamped row, zeroed by selects: a branch here would make every
        // wait of the chunk a wait for all loads
        float v[4];
        Load4(act, ((size_t)min(ks, p.ks - 1) * act_stride + act_tok0 + m) * 4, v);
#pragma unroll
        for (int i = 0; i < 4; ++i) a[j][m][i] = ks < ks_live ? v[i] : 0.0f;
      }
    }
  };

  for (int c = row; c < chunks_live; c += ROWS) {
    u32x4 w[8];
    float a[8][M][4];
    load_weights(c, w);
    load_acts(c, a);
    float s[4], z[4];
#pragma unroll
    for (int o = 0; o < 4; ++o) {
      s[o] = s_lin[o];
      z[o] = z_lin[o];
    }
    if (p.grouped) {
      int g = c / p.group_chunks;
      if (g >= p.groups) g = p.groups - 1;
      Load4(scale, (size_t)g * group_stride + (size_t)slice * 4, s);
      if (zero_point) Load4(zero_point, (size_t)g * group_stride + (size_t)slice * 4, z);
    }
    float t[M][4], asum[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
      asum[m] = 0.0f;
#pragma unroll
      for (int o = 0; o < 4; ++o) t[m][o] = 0.0f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t word = w[j][i];
        const float u0 = (float)(word & 0xFFu), u1 = (float)((word >> 8) & 0xFFu);
        const float u2 = (float)((word >> 16) & 0xFFu), u3 = (float)(word >> 24);
#pragma unroll
        for (int m = 0; m < M; ++m) {
          const float av = a[j][m][i];
          asum[m] += av;
          t[m][0] = fmaf(av, u0, t[m][0]);
          t[m][1] = fmaf(av, u1, t[m][1]);
          t[m][2] = fmaf(av, u2, t[m][2]);
          t[m][3] = fmaf(av, u3, t[m][3]);
        }
      }
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int o = 0; o < 4; ++o) acc[m][o] = fmaf(s[o], fmaf(-(128.0f + z[o]), asum[m], t[m][o]), acc[m][o]);
  }

  // K reduction through LDS: every thread stores its 4*M sums, PARTS threads per output add
  // ROWS/PARTS rows each, then one thread per output adds the PARTS results.
#pragma unroll
  for (int m = 0; m < M; ++m)
    *reinterpret_cast<float4*>(&red[row][m][col * 4]) = make_float4(acc[m][0], acc[m][1], acc[m][2], acc[m][3]);
  __syncthreads();
  const int nl = tid % STRIP;
  const int part = tid / STRIP;
  if (part < PARTS) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float v = 0.0f;
#pragma unroll
      for (int r = 0; r < RPP; ++r) v += red[part * RPP + r][m][nl];
      red2[part][m][nl] = v;
    }
  }
  __syncthreads();
  T* dst = static_cast<T*>(p.dst);
  const T* bias = static_cast<const T*>(p.bias);
  const int n0 = blockIdx.x * STRIP;
  for (int idx = tid; idx < M * STRIP; idx += THREADS) {
    const int m = idx / STRIP, ol = idx % STRIP;
    const int n = n0 + ol;
    if (n >= ns_live * 4) continue;
    float v = 0.0f;
#pragma unroll
    for (int q = 0; q < PARTS; ++q) v += red2[q][m][ol];
    Store1(dst, ((size_t)(n >> 2) * dst_stride + dst_tok0 + m) * 4 + (n & 3), v, bias, (size_t)n);
  }
}

// ------------------------------------------------------------------------------------------
// One token over weights packed in output groups of one slice (the layout FullyConnectedOI reads,
// fully_connected_oi.cc:122-133): the K rows of a slice are one contiguous run of 16-byte blocks,
// so a work-group streams the whole K of 4 output channels and layers of a few thousand channels
// give every CU several work-groups without a split of K.  Lane l reads rows l, l + T, l + 2T, ...
// (T threads): every load instruction of a wave covers 1 KB of contiguous memory, eight of them in
// flight per lane.  Same arithmetic as the kernel above (fp32, one conversion and one fused
// multiply-add per weight, the centre removed per row with group-wise scales, once otherwise);
// K is reduced inside the wave by butterflies, across waves through LDS in wave order.
// group_chunks carries log2 of the K-slices per scale group here.
// ------------------------------------------------------------------------------------------
template <typename T, int WAVES, bool GROUPED>
__global__ __launch_bounds__(WAVES * 64) void fc_w8_rows_kernel(W8Params p) {
  constexpr int TH = WAVES * 64;
  __shared__ float red[WAVES][4];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  // Work-groups go round-robin to the 8 XCDs.  The scales of 8 neighbouring slices share a line, so
  // of every 64 work-groups XCD x takes slices 8x .. 8x + 7 (its L2 then fetches the line once).
  int slice = blockIdx.x;
  if (slice < (int)(gridDim.x & ~63u)) slice = (slice & ~63) + ((slice & 7) << 3) + ((slice >> 3) & 7);
  const int ks = p.ks;
  const u32x4* wrow = p.weights + (size_t)slice * ks;
  const T* act = static_cast<const T*>(p.act);
  const T* scale = static_cast<const T*>(p.scale);
  const T* zero_point = static_cast<const T*>(p.zero_point);
  const size_t group_stride = (size_t)p.ns * 4;
  const int group_shift = p.group_chunks;

  float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f}, asum_all = 0.0f;
  float s_lin[4] = {1.0f, 1.0f, 1.0f, 1.0f}, z_lin[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (!GROUPED) {
    Load4(scale, (size_t)slice * 4, s_lin);
    if (zero_point) Load4(zero_point, (size_t)slice * 4, z_lin);
  }
  // zero points come from the scales' address when there are none, and are dropped behind the fence
  const bool has_zp = zero_point != nullptr;
  const T* zsrc = has_zp ? zero_point : scale;
  for (int r0 = tid; r0 < ks; r0 += 8 * TH) {
    u32x4 w[8];
    decltype(LoadRaw4(act, 0)) araw[8], sraw[8], zraw[8];
    // small loads that come from cache first, then the eight weight loads back to back; rows past
    // K re-read the last one.  Conversions, and the zeroing of activations past K, come behind the
    // fence: next to their loads they would make the kernel wait for every load in turn.
#pragma unroll
    for (int j = 0; j < 8; ++j) araw[j] = LoadRaw4(act, (size_t)min(r0 + TH * j, ks - 1) * 4);
    if (GROUPED) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const size_t so = (size_t)(min(r0 + TH * j, ks - 1) >> group_shift) * group_stride + (size_t)slice * 4;
        sraw[j] = LoadRaw4(scale, so);
        zraw[j] = LoadRaw4(zsrc, so);
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) w[j] = __builtin_nontemporal_load(wrow + min(r0 + TH * j, ks - 1));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float a[4], t[4] = {0.0f, 0.0f, 0.0f, 0.0f}, asum = 0.0f;
      Cvt4(araw[j], a);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t word = w[j][i];
        const float u0 = (float)(word & 0xFFu), u1 = (float)((word >> 8) & 0xFFu);
        const float u2 = (float)((word >> 16) & 0xFFu), u3 = (float)(word >> 24);
        const float av = r0 + TH * j < ks ? a[i] : 0.0f;
        asum += av;
        t[0] = fmaf(av, u0, t[0]);
        t[1] = fmaf(av, u1, t[1]);
        t[2] = fmaf(av, u2, t[2]);
        t[3] = fmaf(av, u3, t[3]);
      }
      if (GROUPED) {
        float sc[4], zp[4];
        Cvt4(sraw[j], sc);
        Cvt4(zraw[j], zp);
#pragma unroll
        for (int o = 0; o < 4; ++o) acc[o] = fmaf(sc[o], fmaf(-(128.0f + (has_zp ? zp[o] : 0.0f)), asum, t[o]), acc[o]);
      } else {
        asum_all += asum;
#pragma unroll
        for (int o = 0; o < 4; ++o) acc[o] += t[o];
      }
    }
  }
  if (!GROUPED) {
#pragma unroll
    for (int o = 0; o < 4; ++o) acc[o] = s_lin[o] * fmaf(-(128.0f + z_lin[o]), asum_all, acc[o]);
  }
  // Every lane holds sums of the same 4 channels.  Two exchange steps halve what a lane carries
  // (lanes 32.. keep channels 2 and 3, then lanes 16.. of each half the odd one), four more add
  // the 16 lanes that are left with the same channel: lane l ends with channel 2 * (l / 32) + (l / 16) % 2.
  // (register exchanges and data-parallel moves: nothing goes through the LDS crossbar)
  typedef unsigned u32x2s __attribute__((ext_vector_type(2)));
  const u32x2s e0 = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[0]), __float_as_uint(acc[2]), false, false);
  const u32x2s e1 = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[1]), __float_as_uint(acc[3]), false, false);
  const float x0 = __uint_as_float(e0[0]) + __uint_as_float(e0[1]);
  const float x1 = __uint_as_float(e1[0]) + __uint_as_float(e1[1]);
  const u32x2s e2 = __builtin_amdgcn_permlane16_swap(__float_as_uint(x0), __float_as_uint(x1), false, false);
  float v = __uint_as_float(e2[0]) + __uint_as_float(e2[1]);
  v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
  {
    const uint32_t up = __builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x104 /* row_shl:4 */, 0xf, 0x5, false);
    const uint32_t both = __builtin_amdgcn_update_dpp(up, __float_as_uint(v), 0x114 /* row_shr:4 */, 0xf, 0xA, false);
    v += __uint_as_float(both);
  }
  v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x4E /* quad_perm:[2,3,0,1] */, 0xf, 0xf, false));
  v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0xB1 /* quad_perm:[1,0,3,2] */, 0xf, 0xf, false));
  const int ch = 2 * (lane >> 5) + ((lane >> 4) & 1);
  if (WAVES > 1) {
    if ((lane & 15) == 0) red[wave][ch] = v;
    __syncthreads();
    if (tid >= 64) return;
    v = 0.0f;
#pragma unroll
    for (int q = 0; q < WAVES; ++q) v += red[q][ch];
  }
  if ((lane & 15) != 0) return;
  const size_t n = (size_t)slice * 4 + ch;
  Store1(static_cast<T*>(p.dst), n, v, static_cast<const T*>(p.bias), n);
}

// ------------------------------------------------------------------------------------------
// The same walk for 2..4 tokens: every weight row is converted once and used for MT token slots
// (tensors are [slice][token][4], so the MT activation vectors of a K-slice are neighbours in
// memory).  3 tokens run in 4 slots: the last slot re-reads token 2 and is not stored.  Fewer rows
// are in flight per lane as the slots grow (8 at 2 slots, 4 at 4), which keeps the kernel clear of
// register spills.
// ------------------------------------------------------------------------------------------
template <typename T, int WAVES, int MT, bool GROUPED>
__global__ __launch_bounds__(WAVES * 64) void fc_w8_rows_tokens_kernel(W8Params p) {
  constexpr int TH = WAVES * 64;
  constexpr int U = MT == 2 ? 8 : 4;
  __shared__ float red[WAVES][MT][4];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  int slice = blockIdx.x;
  if (slice < (int)(gridDim.x & ~63u)) slice = (slice & ~63) + ((slice & 7) << 3) + ((slice >> 3) & 7);
  const int ks = p.ks;
  const int m = p.m;
  const u32x4* wrow = p.weights + (size_t)slice * ks;
  const T* act = static_cast<const T*>(p.act);
  const T* scale = static_cast<const T*>(p.scale);
  const T* zero_point = static_cast<const T*>(p.zero_point);
  const size_t group_stride = (size_t)p.ns * 4;
  const int group_shift = p.group_chunks;

  float acc[MT][4], asum_all[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    asum_all[t] = 0.0f;
#pragma unroll
    for (int o = 0; o < 4; ++o) acc[t][o] = 0.0f;
  }
  float s_lin[4] = {1.0f, 1.0f, 1.0f, 1.0f}, z_lin[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (!GROUPED) {
    Load4(scale, (size_t)slice * 4, s_lin);
    if (zero_point) Load4(zero_point, (size_t)slice * 4, z_lin);
  }
  const bool has_zp = zero_point != nullptr;
  const T* zsrc = has_zp ? zero_point : scale;
  for (int r0 = tid; r0 < ks; r0 += U * TH) {
    u32x4 w[U];
    decltype(LoadRaw4(act, 0)) araw[U][MT], sraw[U], zraw[U];
#pragma unroll
    for (int j = 0; j < U; ++j)
#pragma unroll
      for (int t = 0; t < MT; ++t)
        araw[j][t] = LoadRaw4(act, ((size_t)min(r0 + TH * j, ks - 1) * m + min(t, m - 1)) * 4);
    if (GROUPED) {
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const size_t so = (size_t)(min(r0 + TH * j, ks - 1) >> group_shift) * group_stride + (size_t)slice * 4;
        sraw[j] = LoadRaw4(scale, so);
        zraw[j] = LoadRaw4(zsrc, so);
      }
    }
#pragma unroll
    for (int j = 0; j < U; ++j) w[j] = __builtin_nontemporal_load(wrow + min(r0 + TH * j, ks - 1));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const bool live = r0 + TH * j < ks;
      float u[4][4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t word = w[j][i];
        u[i][0] = (float)(word & 0xFFu);
        u[i][1] = (float)((word >> 8) & 0xFFu);
        u[i][2] = (float)((word >> 16) & 0xFFu);
        u[i][3] = (float)(word >> 24);
      }
      float sc[4], zp[4];
      if (GROUPED) {
        Cvt4(sraw[j], sc);
        Cvt4(zraw[j], zp);
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        float a[4], tt[4] = {0.0f, 0.0f, 0.0f, 0.0f}, asum = 0.0f;
        Cvt4(araw[j][t], a);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float av = live ? a[i] : 0.0f;
          asum += av;
#pragma unroll
          for (int o = 0; o < 4; ++o) tt[o] = fmaf(av, u[i][o], tt[o]);
        }
        if (GROUPED) {
#pragma unroll
          for (int o = 0; o < 4; ++o)
            acc[t][o] = fmaf(sc[o], fmaf(-(128.0f + (has_zp ? zp[o] : 0.0f)), asum, tt[o]), acc[t][o]);
        } else {
          asum_all[t] += asum;
#pragma unroll
          for (int o = 0; o < 4; ++o) acc[t][o] += tt[o];
        }
      }
    }
  }
  // per token the reduction of the one-token kernel: lane l ends with channel 2 * (l / 32) + (l / 16) % 2
  typedef unsigned u32x2s __attribute__((ext_vector_type(2)));
  float v[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    if (!GROUPED) {
#pragma unroll
      for (int o = 0; o < 4; ++o) acc[t][o] = s_lin[o] * fmaf(-(128.0f + z_lin[o]), asum_all[t], acc[t][o]);
    }
    const u32x2s e0 = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[t][0]), __float_as_uint(acc[t][2]), false, false);
    const u32x2s e1 = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[t][1]), __float_as_uint(acc[t][3]), false, false);
    const float x0 = __uint_as_float(e0[0]) + __uint_as_float(e0[1]);
    const float x1 = __uint_as_float(e1[0]) + __uint_as_float(e1[1]);
    const u32x2s e2 = __builtin_amdgcn_permlane16_swap(__float_as_uint(x0), __float_as_uint(x1), false, false);
    float x = __uint_as_float(e2[0]) + __uint_as_float(e2[1]);
    x += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
    {
      const uint32_t up = __builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0x104 /* row_shl:4 */, 0xf, 0x5, false);
      const uint32_t both = __builtin_amdgcn_update_dpp(up, __float_as_uint(x), 0x114 /* row_shr:4 */, 0xf, 0xA, false);
      x += __uint_as_float(both);
    }
    x += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0x4E /* quad_perm:[2,3,0,1] */, 0xf, 0xf, false));
    x += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0xB1 /* quad_perm:[1,0,3,2] */, 0xf, 0xf, false));
    v[t] = x;
  }
  const int ch = 2 * (lane >> 5) + ((lane >> 4) & 1);
  if (WAVES > 1) {
    if ((lane & 15) == 0) {
#pragma unroll
      for (int t = 0; t < MT; ++t) red[wave][t][ch] = v[t];
    }
    __syncthreads();
    if (tid >= 64) return;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      v[t] = 0.0f;
#pragma unroll
      for (int q = 0; q < WAVES; ++q) v[t] += red[q][t][ch];
    }
  }
  if ((lane & 15) != 0) return;
  const size_t n = (size_t)slice * 4 + ch;
#pragma unroll
  for (int t = 0; t < MT; ++t)
    if (t < m) Store1(static_cast<T*>(p.dst), ((size_t)slice * m + t) * 4 + ch, v[t], static_cast<const T*>(p.bias), n);
}

template <typename T, int WAVES, int MT>
hipError_t LaunchRowsTokensG(const W8Params& p, dim3 grid, hipStream_t stream) {
  if (p.grouped)
    hipLaunchKernelGGL((fc_w8_rows_tokens_kernel<T, WAVES, MT, true>), grid, dim3(WAVES * 64), 0, stream, p);
  else
    hipLaunchKernelGGL((fc_w8_rows_tokens_kernel<T, WAVES, MT, false>), grid, dim3(WAVES * 64), 0, stream, p);
  return hipGetLastError();
}
template <typename T, int MT>
hipError_t LaunchRowsTokensT(const W8Params& p, int waves, hipStream_t stream) {
  const dim3 grid(p.ns);
  switch (waves) {
    case 1: return LaunchRowsTokensG<T, 1, MT>(p, grid, stream);
    case 2: return LaunchRowsTokensG<T, 2, MT>(p, grid, stream);
    case 4: return LaunchRowsTokensG<T, 4, MT>(p, grid, stream);
    default: return LaunchRowsTokensG<T, 8, MT>(p, grid, stream);
  }
}

template <typename T, int WAVES>
hipError_t LaunchRowsG(const W8Params& p, dim3 grid, hipStream_t stream) {
  if (p.grouped)
    hipLaunchKernelGGL((fc_w8_rows_kernel<T, WAVES, true>), grid, dim3(WAVES * 64), 0, stream, p);
  else
    hipLaunchKernelGGL((fc_w8_rows_kernel<T, WAVES, false>), grid, dim3(WAVES * 64), 0, stream, p);
  return hipGetLastError();
}
template <typename T>
hipError_t LaunchRowsT(const W8Params& p, int waves, hipStream_t stream) {
  const dim3 grid(p.ns);
  switch (waves) {
    case 1: return LaunchRowsG<T, 1>(p, grid, stream);
    case 2: return LaunchRowsG<T, 2>(p, grid, stream);
    case 4: return LaunchRowsG<T, 4>(p, grid, stream);
    default: return LaunchRowsG<T, 8>(p, grid, stream);
  }
}

template <typename T, int LPR, int WAVES, bool BATCHED>
hipError_t LaunchMB(const W8Params& p, dim3 grid, hipStream_t stream) {
  const dim3 block(WAVES * 64);
  // 16 waves leave a lane 128 registers, which only the one-token form fits without spills; more
  // tokens run with 8 waves at most (256 registers)
  if constexpr (WAVES == 16) {
    if (p.m != 1) return hipErrorInvalidValue;
    hipLaunchKernelGGL((fc_w8_stream_kernel<T, LPR, WAVES, 1, BATCHED>), grid, block, 0, stream, p);
  } else {
    switch (p.m) {
      case 1: hipLaunchKernelGGL((fc_w8_stream_kernel<T, LPR, WAVES, 1, BATCHED>), grid, block, 0, stream, p); break;
      case 2: hipLaunchKernelGGL((fc_w8_stream_kernel<T, LPR, WAVES, 2, BATCHED>), grid, block, 0, stream, p); break;
      case 3: hipLaunchKernelGGL((fc_w8_stream_kernel<T, LPR, WAVES, 3, BATCHED>), grid, block, 0, stream, p); break;
      case 4: hipLaunchKernelGGL((fc_w8_stream_kernel<T, LPR, WAVES, 4, BATCHED>), grid, block, 0, stream, p); break;
      default: return hipErrorInvalidValue;
    }
  }
  return hipGetLastError();
}
template <typename T, int LPR, int WAVES>
hipError_t LaunchM(const W8Params& p, dim3 grid, hipStream_t stream) {
  return p.batch_ids ? LaunchMB<T, LPR, WAVES, true>(p, grid, stream) : LaunchMB<T, LPR, WAVES, false>(p, grid, stream);
}

template <typename T>
hipError_t LaunchT(const W8Params& p, int lpr, int waves, hipStream_t stream) {
  const dim3 grid(DivUp(p.ns, lpr), 1, p.batch_ids ? p.rows : 1);
  if (lpr == 4)
    return waves == 4 ? LaunchM<T, 4, 4>(p, grid, stream)
         : waves == 8 ? LaunchM<T, 4, 8>(p, grid, stream) : LaunchM<T, 4, 16>(p, grid, stream);
  return waves == 4 ? LaunchM<T, 8, 4>(p, grid, stream)
       : waves == 8 ? LaunchM<T, 8, 8>(p, grid, stream) : LaunchM<T, 8, 16>(p, grid, stream);
}

}  // namespace

bool FcW8StreamSupported(const FcArgs& a) {
  if (a.weight_bits != 8 || a.act_f16 != a.dst_f16) return false;
  if (a.params != nullptr && (a.packed_params_offset >= 0 || a.ring_i_index >= 0 || a.ring_o_index >= 0)) return false;
  if (EffectiveGroup(a.group, DivUp(a.n, 4)) != DivUp(a.n, 4)) return false;  // one output group only
  if (a.m < 1 || a.m > kGemvMaxTokens) return false;
  if (a.has_zero_point && a.zero_point == nullptr) return false;  // a scalar zero point: generic kernel
  if (a.scale_kind == kScaleScalar) return false;
  if (a.scale_kind == kScaleBlock) {
    const int ks = DivUp(a.k, 4);
    if (a.groups <= 0 || ks % a.groups != 0) return false;
    if ((ks / a.groups) % 8 != 0) return false;  // a chunk of 8 K-slices must not straddle groups
  }
  return true;
}

// The row-interleaved kernels serve: 1..4 tokens, output groups of one slice, scale groups of a
// power-of-two number of K-slices.
bool FcW8RowsSupported(const FcArgs& a) {
  if (a.weight_bits != 8 || a.act_f16 != a.dst_f16 || a.m < 1 || a.m > 4 || a.batch_ids != nullptr) return false;
  if (a.params != nullptr) return false;  // runtime channel bounds: the streaming kernel
  const int ns = DivUp(a.n, 4), ks = DivUp(a.k, 4);
  if (ns < 2 || EffectiveGroup(a.group, ns) != 1) return false;
  if (a.has_zero_point && a.zero_point == nullptr) return false;  // a scalar zero point: generic kernel
  if (a.scale_kind == kScaleScalar) return false;
  if (a.scale_kind == kScaleBlock) {
    if (a.groups <= 0 || ks % a.groups != 0) return false;
    const int group_slices = ks / a.groups;
    if (group_slices & (group_slices - 1)) return false;
  }
  return true;
}

hipError_t LaunchFcW8Rows(const FcArgs& a, hipStream_t stream, const char** kernel_name) {
  W8Params p;
  p.weights = reinterpret_cast<const u32x4*>(a.weights);
  p.act = a.act;
  p.scale = a.scale;
  p.zero_point = a.has_zero_point ? a.zero_point : nullptr;
  p.bias = a.bias;
  p.dst = a.dst;
  p.m = a.m;
  p.ks = DivUp(a.k, 4);
  p.ns = DivUp(a.n, 4);
  p.chunks = DivUp(p.ks, 8);
  p.grouped = a.scale_kind == kScaleBlock;
  p.groups = p.grouped ? a.groups : 1;
  p.group_chunks = 0;  // here: log2 of the K-slices per scale group
  if (p.grouped)
    for (int gs = p.ks / a.groups; gs > 1; gs >>= 1) ++p.group_chunks;
  p.batch_ids = nullptr;
  p.rows = p.src_rows = p.weights_batch = 1;
  p.rt_params = nullptr;
  p.src_end_idx = p.dst_end_idx = -1;
  p.k_channels = a.k;
  // eight rows per thread where K allows: all of a thread's loads are in flight at once
  int waves = 1;
  while (waves < 8 && waves * 64 * 8 < p.ks) waves *= 2;
  if (GetTuning().gemv_waves > 0) waves = GetTuning().gemv_waves;
  if (a.m > 1) {
    // rows in flight per lane: 8 at 2 token slots, 4 at 4
    const int per_lane = a.m == 2 ? 8 : 4;
    waves = 1;
    while (waves < 8 && waves * 64 * per_lane < p.ks) waves *= 2;
    if (GetTuning().gemv_waves > 0) waves = GetTuning().gemv_waves;
    if (kernel_name) *kernel_name = "fc_w8_rows_tokens_kernel";
    if (a.m == 2)
      return a.act_f16 ? LaunchRowsTokensT<__half, 2>(p, waves, stream) : LaunchRowsTokensT<float, 2>(p, waves, stream);
    return a.act_f16 ? LaunchRowsTokensT<__half, 4>(p, waves, stream) : LaunchRowsTokensT<float, 4>(p, waves, stream);
  }
  if (kernel_name) *kernel_name = "fc_w8_rows_kernel";
  return a.act_f16 ? LaunchRowsT<__half>(p, waves, stream) : LaunchRowsT<float>(p, waves, stream);
}

hipError_t LaunchFcW8Stream(const FcArgs& a, hipStream_t stream, const char** kernel_name) {
  W8Params p;
  p.weights = reinterpret_cast<const u32x4*>(a.weights);
  p.act = a.act;
  p.scale = a.scale;
  p.zero_point = a.has_zero_point ? a.zero_point : nullptr;
  p.bias = a.bias;
  p.dst = a.dst;
  p.m = a.m;
  p.ks = DivUp(a.k, 4);
  p.ns = DivUp(a.n, 4);
  p.chunks = DivUp(p.ks, 8);
  p.grouped = a.scale_kind == kScaleBlock;
  p.groups = p.grouped ? a.groups : 1;
  p.group_chunks = p.grouped ? (p.ks / a.groups) / 8 : p.chunks;
  p.batch_ids = a.batch_ids;
  p.rows = a.rows;
  p.src_rows = a.src_rows;
  p.weights_batch = a.weights_batch;
  p.rt_params = a.params;
  p.src_end_idx = a.src_end_ch_index;
  p.dst_end_idx = a.dst_end_ch_index;
  p.k_channels = a.k;
  // 128-byte row segments (8 slices) when that still gives a work-group to half the CUs, else
  // 64-byte ones; small work-groups when K is covered by 64 / 128 rows of chunks
  const int lpr = (long)DivUp(p.ns, 8) * (a.batch_ids ? a.rows : 1) >= 128 ? 8 : 4;
  const int waves = p.chunks <= 4 * 64 / lpr ? 4 : p.m > 1 ? 8 : 16;
  if (kernel_name) *kernel_name = "fc_w8_stream_kernel";
  return a.act_f16 ? LaunchT<__half>(p, lpr, waves, stream) : LaunchT<float>(p, lpr, waves, stream);
}

}  // namespace mldhip
