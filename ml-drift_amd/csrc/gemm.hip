// Prefill-side kernels for gfx950: LDS-tiled MFMA GEMMs.
//
//  fc_w4_mfma_gemm_kernel   multi-token FullyConnected over the packed int4 I4O4 buffer: the
//                           work-group dequantizes its weight tile into LDS as fp16 (one
//                           rounding per weight: round((u-8)*s), like the reference's
//                           fma(u, s, -8s)), then v_mfma_f32_32x32x16_f16 with fp32 accumulation.
//  conv_int8_mfma_kernel    int8 codes x int8 weights with v_mfma_i32_32x32x32_i8 (int32
//                           accumulators, exact), then the reference's rescale epilogue.
//
// Both share one skeleton.  Operand roles: the MFMA "A" operand is the weight tile (rows =
// output channels), "B" is the activation tile (columns = tokens).  In the 32x32 result a lane
// then holds, for one token, groups of 4 consecutive output channels: exactly one 4-channel
// slice of the slice-major output tensor, so a lane stores 8 (fp16) or 16 bytes and 32 lanes
// store consecutive tokens.
//
// LDS holds both tiles as [k-group][row][16 bytes]; a k-group is 8 halfs (fp16 path) or 16
// bytes (int8 path), i.e. what one lane feeds to one MFMA.  A K-step is 4 k-groups (32 or 64
// input channels): two MFMA steps.  Tiles are double-buffered: the global loads of step t+1
// are issued before the MFMAs of step t and written to the other buffer afterwards.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "../../include/mldhip.h"
#include "kernels.h"

namespace mldhip {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef int int16v_t __attribute__((ext_vector_type(16)));
typedef int int4v_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int KG = 4;  // k-groups per K-step

struct GemmParams {
  int m, n, k;
  int ns;        // output slices, ceil(n/4)
  int k_steps;   // K-steps
  void* dst;
  const void* bias;
  int dst_type;
  // fp16 / int4 path
  const uint8_t* w4;    // [Ks][Ns] blocks of 8 bytes
  const __half* act;    // [Ks][m][4]
  const __half* scale;  // [groups][Ns][4]
  int ks;               // input slices, ceil(k/4)
  int steps_per_group;  // K-steps per scale group
  int groups;
  uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
  // int8 path
  const u32x4* wi8;    // [k16][n]
  const u32x4* codes;  // [k16][m]
  int k16;
  const float* params;  // [m][4]
  const int32_t* wsum;
  const float* wscale;
  const float* wzp;
  // byte sizes of the A (weights), B (activations / codes) and scale buffers
  uint32_t a_bytes, b_bytes, s_bytes;
  int group_size;   // input channels per scale group (fp16 path)
  int group_shift;  // log2(group_size / 16) when that is a power of two, else -1 (not supported by the direct kernel)
};

__device__ __forceinline__ half2_t AsHalf2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }
__device__ __forceinline__ uint32_t AsU32(half2_t v) { return __builtin_bit_cast(uint32_t, v); }

__device__ __forceinline__ uint32_t AndOr(uint32_t x, uint32_t mask, uint32_t magic) {
  uint32_t d;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(x), "s"(mask), "v"(magic));
  return d;
}

// The reference's rescale of an int32 accumulator: every product and sum is a separate
// rounding, in this order.
#pragma clang fp contract(off)
__device__ __forceinline__ float Rescale(int acc, float ws, int wsum, float src_scale, float src_zp,
                                         bool has_zp, float wzp, float src_sum, float in_channels) {
  float res = (float)acc;
  const float f0 = ws * src_scale;
  res = res * f0;
  const float f1 = ws * src_zp;
  const float f2 = f1 * (float)wsum;
  res = res + f2;
  if (has_zp) {
    const float g0 = src_scale * wzp;
    const float g1 = g0 * src_sum;
    res = res + g1;
    const float g2 = src_zp * wzp;
    const float g3 = g2 * in_channels;
    res = res + g3;
  }
  return res;
}
#pragma clang fp contract(fast)

template <bool W4, int FN, int FM, int D>  // D: register stages, even
__global__ __launch_bounds__(kThreads) void mfma_gemm_kernel(GemmParams p) {
  constexpr int BN = 2 * FN * 32;
  constexpr int BM = 2 * FM * 32;
  __shared__ u32x4 sA[2][KG][BN];
  __shared__ u32x4 sB[2][KG][BM];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wn = wave & 1, wm = wave >> 1;
  const int n0 = blockIdx.x * BN;
  const int m0 = blockIdx.y * BM;
  const int r32 = lane & 31, g2 = lane >> 5;

  // ---- staging registers -----------------------------------------------------------------
  // fp16 path: A items (k-group g, slice nsl) -> two 8-byte blocks; B items (K-slice, token) 8 B.
  // int8 path: A / B items (k-group, row) -> 16 bytes.
  constexpr int A_ITEMS = W4 ? KG * (BN / 4) : KG * BN;
  constexpr int B_ITEMS = W4 ? (KG * 2) * BM : KG * BM;
  constexpr int NA = (A_ITEMS + kThreads - 1) / kThreads;
  constexpr int NB = (B_ITEMS + kThreads - 1) / kThreads;
  // D register stages: tile t is fetched D K-steps before it is multiplied, so D-1 tiles of
  // global loads are in flight while the MFMAs of the current tile run.
  u32x4 ra_[D][NA];  // fp16 path: {blk0.x, blk0.y, blk1.x, blk1.y}
  u32x2 rs_[D][NA];  // fp16 path: the 4 scales of the item's slice
  u32x4 rb_[D][W4 ? 1 : NB];
  u32x2 rb2_[D][W4 ? NB : 1];  // fp16 path: 8-byte activation items

  // All tile loads are raw buffer loads: out-of-range items get an offset beyond the buffer and
  // read as zero, so the loop body stays free of branches and the loads of several stages stay
  // in flight (a zero activation or a zero scale makes the padded product vanish).
  constexpr uint32_t kOob = 0x7FFFFFF0u;
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<void*>(W4 ? static_cast<const void*>(p.w4) : static_cast<const void*>(p.wi8)), 0, p.a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<void*>(W4 ? static_cast<const void*>(p.act) : static_cast<const void*>(p.codes)), 0, p.b_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_s =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half*>(p.scale), 0, p.s_bytes, 0x00020000);

  auto load_tiles = [&](int kt, u32x4 (&ra)[NA], u32x2 (&rs)[NA], u32x4 (&rb)[W4 ? 1 : NB],
                        u32x2 (&rb2)[W4 ? NB : 1]) {
    if (W4) {
#pragma unroll
      for (int q = 0; q < NA; ++q) {
        const int it = tid + q * kThreads;
        const int g = it / (BN / 4), nsl = it % (BN / 4);
        const int nsi = n0 / 4 + nsl;
        const int ksa = (kt * KG + g) * 2;
        const bool ok = it < A_ITEMS && nsi < p.ns;
        const uint32_t off0 = ok ? (uint32_t)(ksa * p.ns + nsi) * 8u : kOob;
        const uint32_t off1 = ok ? off0 + (uint32_t)p.ns * 8u : kOob;
        const u32x2 b0 = __builtin_amdgcn_raw_buffer_load_b64(rsrc_a, off0, 0, 0);
        const u32x2 b1 = __builtin_amdgcn_raw_buffer_load_b64(rsrc_a, off1, 0, 0);
        ra[q] = u32x4{b0[0], b0[1], b1[0], b1[1]};
        int grp = kt / p.steps_per_group;
        grp = grp < p.groups ? grp : p.groups - 1;
        rs[q] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_s, ok ? (uint32_t)(grp * p.ns + nsi) * 8u : kOob, 0, 0);
      }
#pragma unroll
      for (int q = 0; q < NB; ++q) {
        const int it = tid + q * kThreads;
        const int ksl = it / BM, ml = it % BM;
        const int ksi = kt * KG * 2 + ksl;
        const int mi = m0 + ml;
        const bool ok = it < B_ITEMS && mi < p.m;
        rb2[q] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_b, ok ? (uint32_t)(ksi * p.m + mi) * 8u : kOob, 0, 0);
      }
    } else {
#pragma unroll
      for (int q = 0; q < NA; ++q) {
        const int it = tid + q * kThreads;
        const int g = it / BN, r = it % BN;
        const int kg = kt * KG + g;
        const bool ok = it < A_ITEMS && n0 + r < p.n;
        ra[q] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, ok ? (uint32_t)(kg * p.n + n0 + r) * 16u : kOob, 0, 0);
      }
#pragma unroll
      for (int q = 0; q < NB; ++q) {
        const int it = tid + q * kThreads;
        const int g = it / BM, r = it % BM;
        const int kg = kt * KG + g;
        const bool ok = it < B_ITEMS && m0 + r < p.m;
        rb[q] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, ok ? (uint32_t)(kg * p.m + m0 + r) * 16u : kOob, 0, 0);
      }
    }
  };

  auto store_tiles = [&](int buf, u32x4 (&ra)[NA], u32x2 (&rs)[NA], u32x4 (&rb)[W4 ? 1 : NB],
                         u32x2 (&rb2)[W4 ? NB : 1]) {
    if (W4) {
      const half2_t off_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f};
      const half2_t off_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
#pragma unroll
      for (int q = 0; q < NA; ++q) {
        const int it = tid + q * kThreads;
        if (it >= A_ITEMS) continue;
        const int g = it / (BN / 4), nsl = it % (BN / 4);
#pragma unroll
        for (int o = 0; o < 4; ++o) {
          // scale of output o in both halves
          const uint32_t sw = rs[q][o >> 1];
          const uint32_t s16 = (o & 1) ? (sw >> 16) : (sw & 0xFFFFu);
          const half2_t s2 = AsHalf2(s16 | (s16 << 16));
          u32x4 row;
#pragma unroll
          for (int wd = 0; wd < 4; ++wd) {
            const uint32_t x = (o & 2) ? (ra[q][wd] >> 8) : ra[q][wd];
            const uint32_t bits = (o & 1) ? AndOr(x, p.mask_hi, p.magic_hi) : AndOr(x, p.mask_lo, p.magic_lo);
            const half2_t centered = AsHalf2(bits) + ((o & 1) ? off_hi : off_lo);
            row[wd] = AsU32(centered * s2);
          }
          sA[buf][g][nsl * 4 + o] = row;
        }
      }
#pragma unroll
      for (int q = 0; q < NB; ++q) {
        const int it = tid + q * kThreads;
        if (it >= B_ITEMS) continue;
        const int ksl = it / BM, ml = it % BM;
        u32x2* dst2 = reinterpret_cast<u32x2*>(&sB[buf][ksl >> 1][ml]) + (ksl & 1);
        *dst2 = rb2[q];
      }
    } else {
#pragma unroll
      for (int q = 0; q < NA; ++q) {
        const int it = tid + q * kThreads;
        if (it < A_ITEMS) sA[buf][it / BN][it % BN] = ra[q];
      }
#pragma unroll
      for (int q = 0; q < NB; ++q) {
        const int it = tid + q * kThreads;
        if (it < B_ITEMS) sB[buf][it / BM][it % BM] = rb[q];
      }
    }
  };

  // ---- accumulators -----------------------------------------------------------------------
  float16_t accf[FN][FM];
  int16v_t acci[FN][FM];
#pragma unroll
  for (int fn = 0; fn < FN; ++fn)
#pragma unroll
    for (int fm = 0; fm < FM; ++fm)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        if (W4)
          accf[fn][fm][v] = 0.0f;
        else
          acci[fn][fm][v] = 0;
      }

  // prologue: tiles 0 .. D-1 into the register stages, tile 0 on into LDS.  The loop below
  // has no conditions: it runs a multiple of D steps, tiles beyond K read as zeros (buffer
  // range check) and add nothing.
#pragma unroll
  for (int d = 0; d < D; ++d) load_tiles(d, ra_[d], rs_[d], rb_[d], rb2_[d]);
  store_tiles(0, ra_[0], rs_[0], rb_[0], rb2_[0]);
  __syncthreads();
  const int k_steps_padded = (p.k_steps + D - 1) / D * D;
  for (int kt0 = 0; kt0 < k_steps_padded; kt0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int kt = kt0 + d;
      const int buf = d & 1;  // D is even, so the LDS buffer of a stage is fixed
      // stage d held tile kt (already in LDS): refill it with tile kt + D
      load_tiles(kt + D, ra_[d], rs_[d], rb_[d], rb2_[d]);
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        u32x4 a[FN], b[FM];
#pragma unroll
        for (int fn = 0; fn < FN; ++fn) a[fn] = sA[buf][2 * s + g2][(wn * FN + fn) * 32 + r32];
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) b[fm] = sB[buf][2 * s + g2][(wm * FM + fm) * 32 + r32];
#pragma unroll
        for (int fn = 0; fn < FN; ++fn)
#pragma unroll
          for (int fm = 0; fm < FM; ++fm) {
            if (W4)
              accf[fn][fm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(half8_t, a[fn]), __builtin_bit_cast(half8_t, b[fm]), accf[fn][fm], 0, 0, 0);
            else
              acci[fn][fm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                  __builtin_bit_cast(int4v_t, a[fn]), __builtin_bit_cast(int4v_t, b[fm]), acci[fn][fm], 0, 0, 0);
          }
      }
      {
        const int dn = (d + 1) % D;
        store_tiles(buf ^ 1, ra_[dn], rs_[dn], rb_[dn], rb2_[dn]);
      }
      __syncthreads();
    }
  }

  // ---- epilogue ---------------------------------------------------------------------------
#pragma unroll
  for (int fm = 0; fm < FM; ++fm) {
    const int mi = m0 + (wm * FM + fm) * 32 + r32;
    if (mi >= p.m) continue;
    float src_scale = 0.0f, src_zp = 0.0f, src_sum = 0.0f;
    if (!W4 && p.dst_type != MLDHIP_INT32) {
      const float4 pr = *reinterpret_cast<const float4*>(p.params + (size_t)mi * 4);
      src_scale = pr.x;
      src_zp = pr.y;
      src_sum = pr.z;
    }
#pragma unroll
    for (int fn = 0; fn < FN; ++fn) {
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        const int nb = n0 + (wn * FN + fn) * 32 + 8 * v4 + 4 * g2;  // first of 4 consecutive channels
        const int slice = nb >> 2;
        if (slice >= p.ns) continue;
        const size_t o_idx = ((size_t)slice * p.m + mi) * 4;
        float r[4];
        if (W4) {
#pragma unroll
          for (int c = 0; c < 4; ++c) r[c] = accf[fn][fm][v4 * 4 + c];
        } else if (p.dst_type == MLDHIP_INT32) {
          int4v_t o = {acci[fn][fm][v4 * 4], acci[fn][fm][v4 * 4 + 1], acci[fn][fm][v4 * 4 + 2],
                       acci[fn][fm][v4 * 4 + 3]};
          *reinterpret_cast<int4v_t*>(static_cast<int*>(p.dst) + o_idx) = o;
          continue;
        } else {
#pragma unroll
          for (int c = 0; c < 4; ++c)
            r[c] = Rescale(acci[fn][fm][v4 * 4 + c], p.wscale[nb + c], p.wsum[nb + c], src_scale, src_zp,
                           p.wzp != nullptr, p.wzp ? p.wzp[nb + c] : 0.0f, src_sum, (float)p.k);
        }
        if (p.dst_type == MLDHIP_FLOAT32) {
          const float* bias = static_cast<const float*>(p.bias);
          float4 o = make_float4(r[0], r[1], r[2], r[3]);
          if (bias) {
            o.x += bias[nb];
            o.y += bias[nb + 1];
            o.z += bias[nb + 2];
            o.w += bias[nb + 3];
          }
          *reinterpret_cast<float4*>(static_cast<float*>(p.dst) + o_idx) = o;
        } else {
          const __half* bias = static_cast<const __half*>(p.bias);
          __half h[4];
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            h[c] = __float2half_rn(r[c]);
            if (bias) h[c] = __hadd(h[c], bias[nb + c]);
          }
          u32x2 o;
          o[0] = (uint32_t)__half_as_ushort(h[0]) | ((uint32_t)__half_as_ushort(h[1]) << 16);
          o[1] = (uint32_t)__half_as_ushort(h[2]) | ((uint32_t)__half_as_ushort(h[3]) << 16);
          *reinterpret_cast<u32x2*>(static_cast<__half*>(p.dst) + o_idx) = o;
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// int4 prefill GEMM without LDS in the main loop.
//
// Work-group = 4 waves on one output tile of 128 channels x (FM*32) tokens; the waves split K
// four ways and add their fp32 tiles through LDS at the end (fixed order).  Inside a wave every
// MFMA operand comes straight from global memory in the layout the instruction wants:
//  - A (weights): the 32 "rows" of MFMA number t are the output channels 4*i + t, i = lane % 32,
//    so a lane's two 8-byte blocks (K-slices 2q, 2q+1 of slice i; 8 input channels x 4 output
//    channels) dequantize to exactly its A operands for t = 0..3.  No transposition, and each
//    weight is dequantized once per wave: fp16 round((u-8)*s) with two packed ops per pair.
//  - B (activations): column j = token; a lane's 8 halfs are the two 8-byte slices
//    [2q][token][4], [2q+1][token][4] of the slice-major tensor.
// In the 32x32 result, register v of lane j holds row 8*(v/4) + 4*(lane/32) + v%4 = slice i, so
// the 4 MFMAs t = 0..3 together hold one whole 4-channel output slice per (v, token): one
// 8-byte store.  Loads are raw buffer loads (out-of-range reads as zero), U steps ahead.
// ------------------------------------------------------------------------------------------
// Work-group barrier that waits for this wave's LDS traffic only: global stores issued before
// it stay in flight.
__device__ __forceinline__ void LdsBarrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int FM, int U, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void fc_w4_mfma_direct_kernel(GemmParams p) {
  constexpr int BN = 128;
  constexpr int BM = FM * 32;
  static_assert(WAVES == 4 || WAVES == 8 || WAVES == 16, "the reduction handles WAVES registers per phase");
  __shared__ float4 red[WAVES][WAVES][64];  // [copy][register within the phase][lane]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int i32 = lane & 31, g2 = lane >> 5;
  // XCD-aware tile order.  Work-groups go round-robin to the 8 XCDs (id % 8), each with its own
  // L2.  Tiles are numbered token-tile-major and XCD x takes the contiguous range
  // [x*per_xcd, (x+1)*per_xcd): the work-groups that share an L2 then share a few activation
  // tiles (the big fp16 operand), and every weight tile streams through that L2 once.
  const int tiles_n = (p.n + BN - 1) / BN;
  const int tiles_m = (p.m + BM - 1) / BM;
  const int per_xcd = (tiles_n * tiles_m + 7) / 8;
  const int tile = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (tile >= tiles_n * tiles_m) return;
  const int n0 = (tile % tiles_n) * BN;
  const int m0 = (tile / tiles_n) * BM;
  const int nsi = n0 / 4 + i32;
  const bool n_ok = nsi < p.ns;

  // This wave's range of 16-channel steps.  The buffer descriptors of the weights and the
  // activations end where the wave's share of K ends, so the prefetches that run past it (and
  // past K itself) read zeros without a test in the loop; a lane without an output slice or
  // a token gets an offset beyond every buffer.
  const int steps_total = (p.k + 15) / 16;
  const int per_wave = ((steps_total + WAVES - 1) / WAVES + U - 1) / U * U;  // multiple of U
  const int t_begin = __builtin_amdgcn_readfirstlane(wave * per_wave);
  const uint32_t row_w = (uint32_t)p.ns * 8u;  // bytes per K-slice row of the weights
  const uint32_t row_x = (uint32_t)p.m * 8u;   // bytes per K-slice row of the activations
  const uint32_t k_slices_end = (uint32_t)(t_begin + per_wave) * 4u;
  const uint32_t w_end = min((uint64_t)p.a_bytes, (uint64_t)k_slices_end * row_w);
  const uint32_t x_end = min((uint64_t)p.b_bytes, (uint64_t)k_slices_end * row_x);

  constexpr uint32_t kOob = 0x7FFFFFF0u;
  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.w4), 0, w_end, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_x =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half*>(p.act), 0, x_end, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_s =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half*>(p.scale), 0, p.s_bytes, 0x00020000);

  // Per-lane byte offsets of the next step to fetch; each fetch advances them by one step.
  // Only the per-lane offset takes part in the range check of a buffer load, so the whole
  // address lives there.
  const uint32_t step_w = 4u * row_w, step_x = 4u * row_x;
  uint32_t vw0 = n_ok ? ((uint32_t)t_begin * 4u + (uint32_t)g2 * 2u) * row_w + (uint32_t)nsi * 8u : kOob;
  uint32_t vw1 = n_ok ? vw0 + row_w : kOob;
  const uint32_t vs = n_ok ? (uint32_t)nsi * 8u : kOob;
  uint32_t vx[FM][2];
#pragma unroll
  for (int fm = 0; fm < FM; ++fm) {
    const int mi = m0 + fm * 32 + i32;
    vx[fm][0] = mi < p.m ? ((uint32_t)t_begin * 4u + (uint32_t)g2 * 2u) * row_x + (uint32_t)mi * 8u : kOob;
    vx[fm][1] = mi < p.m ? vx[fm][0] + row_x : kOob;
  }
  const uint32_t group_bytes = row_w;  // one scale group: [Ns][4] halfs

  u32x2 rw[U][2], rsc[U], rx[U][FM][2];
  auto load_step = [&](int t, u32x2 (&w)[2], u32x2& sc, u32x2 (&x)[FM][2]) {
    w[0] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, vw0, 0, 0);
    w[1] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, vw1, 0, 0);
    vw0 += step_w;
    vw1 += step_w;
    // scale group of this step (groups hold a power-of-two number of steps); a group past the
    // last one reads zeros
    sc = __builtin_amdgcn_raw_buffer_load_b64(rsrc_s, vs + (uint32_t)(t >> p.group_shift) * group_bytes, 0, 0);
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) {
      x[fm][0] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_x, vx[fm][0], 0, 0);
      x[fm][1] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_x, vx[fm][1], 0, 0);
      vx[fm][0] += step_x;
      vx[fm][1] += step_x;
    }
  };

  float16_t acc[4][FM];
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4)
#pragma unroll
    for (int fm = 0; fm < FM; ++fm)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t4][fm][v] = 0.0f;

  const half2_t off_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f};
  const half2_t off_hi = {(_Float16)-72.0f, (_Float16)-72.0f};

  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    load_step(t_begin + u, rw[u], rsc[u], rx[u]);
    __builtin_amdgcn_sched_barrier(0);
  }
  for (int tt = 0; tt < per_wave; tt += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int t = t_begin + tt + u;
      // consume stage u
      const u32x4 blk = {rw[u][0][0], rw[u][0][1], rw[u][1][0], rw[u][1][1]};
      const u32x4 blk8 = {blk[0] >> 8, blk[1] >> 8, blk[2] >> 8, blk[3] >> 8};
      const half2_t sc01 = AsHalf2(rsc[u][0]), sc23 = AsHalf2(rsc[u][1]);
#pragma unroll
      for (int t4 = 0; t4 < 4; ++t4) {
        const half2_t sp = (t4 & 2) ? sc23 : sc01;
        const half2_t s2 = (t4 & 1) ? __builtin_shufflevector(sp, sp, 1, 1) : __builtin_shufflevector(sp, sp, 0, 0);
        u32x4 aop;
#pragma unroll
        for (int wd = 0; wd < 4; ++wd) {
          const uint32_t x = (t4 & 2) ? blk8[wd] : blk[wd];
          const uint32_t bits = (t4 & 1) ? AndOr(x, p.mask_hi, p.magic_hi) : AndOr(x, p.mask_lo, p.magic_lo);
          aop[wd] = AsU32((AsHalf2(bits) + ((t4 & 1) ? off_hi : off_lo)) * s2);
        }
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) {
          const u32x4 bop = {rx[u][fm][0][0], rx[u][fm][0][1], rx[u][fm][1][0], rx[u][fm][1][1]};
          acc[t4][fm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, aop),
                                                               __builtin_bit_cast(half8_t, bop), acc[t4][fm], 0, 0, 0);
        }
      }
      // refill stage u with step t + U; the fences keep the loads of a stage together and in
      // program order, so that waiting for one stage leaves the younger ones in flight
      __builtin_amdgcn_sched_barrier(0);
      load_step(t + U, rw[u], rsc[u], rx[u]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // K-split reduction, spread over all waves.  The tile goes through LDS in phases of WAVES
  // accumulator registers per lane (x 4 MFMAs): every wave writes its copy, then wave w adds the
  // WAVES copies of register w in a fixed order and stores that part of the output.  In the
  // 32x32 result, register v of lane (g2, i32) belongs to output slice 8*(v/4) + 4*g2 + v%4 and
  // token i32, and the four MFMAs hold the slice's four channels: one 8-byte store.
  const __half* bias = static_cast<const __half*>(p.bias);
  __half* dst = static_cast<__half*>(p.dst);
#pragma unroll
  for (int fm = 0; fm < FM; ++fm) {
    const int mi = m0 + fm * 32 + i32;
#pragma unroll
    for (int ph = 0; ph < 16 / WAVES; ++ph) {
#pragma unroll
      for (int j = 0; j < WAVES; ++j) {
        const int v = ph * WAVES + j;
        red[wave][j][lane] = make_float4(acc[0][fm][v], acc[1][fm][v], acc[2][fm][v], acc[3][fm][v]);
      }
      LdsBarrier();
      float4 sum = red[0][wave][lane];
#pragma unroll
      for (int c = 1; c < WAVES; ++c) {
        const float4 o = red[c][wave][lane];
        sum.x += o.x;
        sum.y += o.y;
        sum.z += o.z;
        sum.w += o.w;
      }
      const int v = ph * WAVES + wave;
      const int slice = n0 / 4 + 8 * (v >> 2) + 4 * g2 + (v & 3);
      if (mi < p.m && slice < p.ns) {
        __half h[4] = {__float2half_rn(sum.x), __float2half_rn(sum.y), __float2half_rn(sum.z), __float2half_rn(sum.w)};
        if (bias) {
#pragma unroll
          for (int t4 = 0; t4 < 4; ++t4) h[t4] = __hadd(h[t4], bias[slice * 4 + t4]);
        }
        u32x2 o;
        o[0] = (uint32_t)__half_as_ushort(h[0]) | ((uint32_t)__half_as_ushort(h[1]) << 16);
        o[1] = (uint32_t)__half_as_ushort(h[2]) | ((uint32_t)__half_as_ushort(h[3]) << 16);
        *reinterpret_cast<u32x2*>(dst + ((size_t)slice * p.m + mi) * 4) = o;
      }
      if (fm + 1 < FM || ph + 1 < 16 / WAVES) LdsBarrier();
    }
  }
}

template <bool W4>
hipError_t LaunchGemm(const GemmParams& p, hipStream_t stream) {
  // Tile choice: the largest work-group tile that still gives every CU a work-group;
  // small problems fall back to 64x64-per-wave tiles... the candidates are (FN, FM) in
  // {(4,4), (4,2), (2,2), (2,1)} -> work-group tiles 256x256, 256x128, 128x128, 128x64 (N x M).
  auto groups = [&](int bn, int bm) { return (long)DivUp(p.n, bn) * DivUp(p.m, bm); };
  const long want = 200;
  if (groups(256, 256) >= want) {
    hipLaunchKernelGGL((mfma_gemm_kernel<W4, 4, 4, 2>), dim3(DivUp(p.n, 256), DivUp(p.m, 256)), dim3(kThreads), 0,
                       stream, p);
  } else if (groups(256, 128) >= want) {
    hipLaunchKernelGGL((mfma_gemm_kernel<W4, 4, 2, (W4 ? 6 : 4)>), dim3(DivUp(p.n, 256), DivUp(p.m, 128)), dim3(kThreads), 0,
                       stream, p);
  } else if (groups(128, 128) >= want || p.m > 64) {
    hipLaunchKernelGGL((mfma_gemm_kernel<W4, 2, 2, (W4 ? 8 : 6)>), dim3(DivUp(p.n, 128), DivUp(p.m, 128)), dim3(kThreads), 0,
                       stream, p);
  } else {
    hipLaunchKernelGGL((mfma_gemm_kernel<W4, 2, 1, (W4 ? 8 : 6)>), dim3(DivUp(p.n, 128), DivUp(p.m, 64)), dim3(kThreads), 0,
                       stream, p);
  }
  return hipGetLastError();
}

}  // namespace

bool FcW4MfmaSupported(const FcArgs& a) {
  if (a.weight_bits != 4 || !a.act_f16 || !a.dst_f16) return false;
  if (a.has_zero_point || a.scale_kind == kScaleScalar) return false;
  if (a.m <= kGemvMaxTokens) return false;
  // 32-bit buffer offsets
  if ((size_t)DivUp(a.k, 4) * DivUp(a.n, 4) * 8 >= 0x7FFFFFF0u || (size_t)DivUp(a.k, 4) * a.m * 8 >= 0x7FFFFFF0u)
    return false;
  if (a.scale_kind == kScaleBlock) {
    // an MFMA step of 16 input channels must not straddle scale groups
    if (a.groups <= 0 || a.k % a.groups != 0 || (a.k / a.groups) % 16 != 0) return false;
    const int steps_per_group = (a.k / a.groups) / 16;
    if (steps_per_group & (steps_per_group - 1)) return false;  // the kernel finds the group by a shift
  }
  return true;
}

hipError_t LaunchFcW4Mfma(const FcArgs& a, hipStream_t stream, const char** kernel_name) {
  GemmParams p = {};
  p.m = a.m;
  p.n = a.n;
  p.k = a.k;
  p.ns = DivUp(a.n, 4);
  p.ks = DivUp(a.k, 4);
  p.k_steps = DivUp(a.k, 32);
  p.dst = a.dst;
  p.bias = a.bias;
  p.dst_type = MLDHIP_FLOAT16;
  p.w4 = a.weights;
  p.act = static_cast<const __half*>(a.act);
  p.scale = static_cast<const __half*>(a.scale);
  p.groups = a.scale_kind == kScaleBlock ? a.groups : 1;
  p.steps_per_group = a.scale_kind == kScaleBlock ? (a.k / a.groups) / 32 : p.k_steps;
  p.mask_lo = 0x000F000Fu;
  p.mask_hi = 0x00F000F0u;
  p.magic_lo = 0x64006400u;
  p.magic_hi = 0x54005400u;
  p.a_bytes = (uint32_t)((size_t)p.ks * p.ns * 8);
  p.b_bytes = (uint32_t)((size_t)p.ks * p.m * 8);
  p.s_bytes = (uint32_t)((size_t)p.groups * p.ns * 8);
  p.group_size = a.scale_kind == kScaleBlock ? a.k / a.groups : a.k;
  p.group_shift = -1;
  if (a.scale_kind != kScaleBlock) {
    p.group_shift = 30;  // one group
  } else {
    const int spg = p.group_size / 16;
    for (int sh = 0; sh < 30; ++sh)
      if ((1 << sh) == spg) p.group_shift = sh;
  }
  if (kernel_name) *kernel_name = "fc_w4_mfma_gemm_kernel";
  // token tile: 64 when that still yields a work-group per CU or M is large, else 32
  const long tiles64 = (long)DivUp(a.n, 128) * DivUp(a.m, 64);
  int fm = (a.m > 32 && (tiles64 >= 128 || a.m > 64)) ? 2 : 1;
  int u = 4;
  if (const char* e = std::getenv("MLDHIP_GEMM_FM")) fm = std::atoi(e);
  if (const char* e = std::getenv("MLDHIP_GEMM_U")) u = std::atoi(e);
  const int tiles = DivUp(a.n, 128) * DivUp(a.m, fm * 32);
  const dim3 grid(DivUp(tiles, 8) * 8);
  int waves = 8;
  if (const char* e = std::getenv("MLDHIP_GEMM_WAVES")) waves = std::atoi(e);
  if (fm == 2) {
    if (waves == 8)
      hipLaunchKernelGGL((fc_w4_mfma_direct_kernel<2, 4, 8>), grid, dim3(512), 0, stream, p);
    else if (u == 8)
      hipLaunchKernelGGL((fc_w4_mfma_direct_kernel<2, 8, 4>), grid, dim3(256), 0, stream, p);
    else
      hipLaunchKernelGGL((fc_w4_mfma_direct_kernel<2, 4, 4>), grid, dim3(256), 0, stream, p);
  } else {
    if (waves == 8)
      hipLaunchKernelGGL((fc_w4_mfma_direct_kernel<1, 4, 8>), grid, dim3(512), 0, stream, p);
    else
      hipLaunchKernelGGL((fc_w4_mfma_direct_kernel<1, 4, 4>), grid, dim3(256), 0, stream, p);
  }
  return hipGetLastError();
}

hipError_t LaunchConvInt8(const ConvInt8Args& a, hipStream_t stream, const char** kernel_name) {
  GemmParams p = {};
  p.m = a.m;
  p.n = a.n;
  p.k = a.k;
  p.ns = DivUp(a.n, 4);
  p.k16 = DivUp(a.k, 16);
  p.k_steps = DivUp(p.k16, KG);
  p.dst = a.dst;
  p.bias = a.bias;
  p.dst_type = a.dst_type;
  p.wi8 = reinterpret_cast<const u32x4*>(a.weights);
  p.codes = reinterpret_cast<const u32x4*>(a.codes);
  p.params = a.params;
  p.wsum = a.weights_sum;
  p.wscale = a.weights_scale;
  p.wzp = a.weights_zero_point;
  if ((size_t)p.k16 * p.n * 16 >= 0x7FFFFFF0u || (size_t)p.k16 * p.m * 16 >= 0x7FFFFFF0u) return hipErrorInvalidValue;
  p.a_bytes = (uint32_t)((size_t)p.k16 * p.n * 16);
  p.b_bytes = (uint32_t)((size_t)p.k16 * p.m * 16);
  p.s_bytes = 0;
  if (kernel_name) *kernel_name = "conv_int8_mfma_kernel";
  return LaunchGemm<false>(p, stream);
}

}  // namespace mldhip
