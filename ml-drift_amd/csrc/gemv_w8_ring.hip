// FullyConnected over ringed uint8 weights whose ring runs over the input channels
// (ConvRuntimeCheckDesc::ring_i_offset_index over a kOSpatialIOGroupI4O4 buffer,
// common/kernels/fully_connected.cc:424-441, 676-706), 1..4 tokens per row: the matmul of a decode
// step with a cache as its weights (attention probabilities x value cache), where the cache is
// long and the output narrow.
//
// The reference's kernel walks the source slices and gathers, for source channel c, the word of
// ring channel (c + offset) % ring_size: four 4-byte reads per slice and output slice.  Here the
// walk is over the ring's own K-slice rows instead: a row (4 ring channels x all output channels)
// is contiguous and aligned, so a thread reads its 16-byte block (4 ring channels x 4 output
// channels) with one load, and what shifts with the offset is the index of the activations:
// row w of the window (w = 0 .. rows touched) is buffer row (offset / 4 + w) % rows and holds
// source channels 4 w - offset % 4 + {0, 1, 2, 3}; those outside [0, channels multiplied) count as
// zero.  That needs ring_size % 4 == 0.
//
// Work-group = 256 threads = LS lanes along the output slices x 256 / LS rows in flight, four
// rows per thread and pass; the window is split across blockIdx.x, the slices (in chunks of LS)
// across blockIdx.y, the dst rows of a launch with batched weights across blockIdx.z.  Every
// thread keeps sum(a * (u - 128)) per token and output channel and sum(a) per token; a work-group
// adds its rows through LDS and writes fp32 partial sums to the op's workspace, a second kernel
// adds the parts in their order (fixed), applies scale * (sum - zp * sum(a)), converts and adds
// the bias in the destination type.  MT = token slots per row (1, 2 or 4).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "kernels.h"

namespace mldhip {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kRingThreads = 256;
// window rows per thread and pass, all of their loads in flight at once: 8 at one token, 4 at more
// (the activations of a row are 8 values per token)
__host__ __device__ constexpr int RingUnroll(int token_slots) { return token_slots == 1 ? 8 : 4; }
constexpr int kRingMaxParts = 256;

struct RingParams {
  const void* act;
  const u32x4* weights;
  const void* scale;
  const void* zero_point;
  const void* bias;
  void* dst;
  float* partial;  // [part][row][token][ns * 4 + 4]: the sums, then sum(a)
  const int32_t* params;
  const int32_t* batch_ids;
  int m, ks, ns;
  int ring_rows;  // ring_size / 4
  int ring_size, ring_index, src_end_ch_index, dst_end_ch_index, k_channels;
  int rows, src_rows, weights_batch;
  int scale_kind, has_zero_point;
  float scalar_scale, scalar_zero_point;
  int parts;
};

__device__ __forceinline__ float LoadF(const float* p, size_t i) { return p[i]; }
__device__ __forceinline__ float LoadF(const __half* p, size_t i) { return __half2float(p[i]); }
__device__ __forceinline__ void Load4(const float* p, size_t i, float v[4]) {
  const float4 r = *reinterpret_cast<const float4*>(p + i);
  v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
}
__device__ __forceinline__ void Load4(const __half* p, size_t i, float v[4]) {
  const uint2 r = *reinterpret_cast<const uint2*>(p + i);
  const __half2 lo = *reinterpret_cast<const __half2*>(&r.x), hi = *reinterpret_cast<const __half2*>(&r.y);
  v[0] = __low2float(lo); v[1] = __high2float(lo); v[2] = __low2float(hi); v[3] = __high2float(hi);
}

// source slices the launch multiplies and dst slices it writes (the runtime channel bounds of the
// unspecialised kernel: fully_connected.cc:750-755, 795)
__device__ __forceinline__ int RingSrcEndSlices(const RingParams& p) {
  if (p.src_end_ch_index < 0) return p.ks;
  return min(max(SrcEndSlices(p.params[p.src_end_ch_index], p.k_channels, p.ks), 0), p.ks);
}
__device__ __forceinline__ int RingDstEndSlice(const RingParams& p) {
  if (p.dst_end_ch_index < 0) return p.ns;
  return min(max(DstEndSlice(p.params[p.dst_end_ch_index], p.ns), 0), p.ns);
}

template <typename T, int LS, int MT>
__global__ __launch_bounds__(kRingThreads) void fc_w8_ring_i_kernel(RingParams p) {
  constexpr int RW = kRingThreads / LS;  // window rows in flight per pass
  constexpr int U = RingUnroll(MT);
  __shared__ float red[RW][LS][5 * MT];
  const int tid = threadIdx.x;
  const int s_lane = tid % LS, rsub = tid / LS;
  const int ds = blockIdx.y * LS + s_lane;
  const int row = blockIdx.z;
  int wb = p.batch_ids ? p.batch_ids[row] : 0;
  wb = min(max(wb, 0), p.weights_batch - 1);
  const size_t act_stride = (size_t)p.src_rows * p.m;
  const size_t act_tok0 = (size_t)min(row, p.src_rows - 1) * p.m;
  const T* act = static_cast<const T*>(p.act);
  const int off = ((p.params[p.ring_index] % p.ring_size) + p.ring_size) % p.ring_size;
  const int sh = off & 3, row0 = off >> 2;
  const int ks_end = RingSrcEndSlices(p);
  const int k_eff = ks_end * 4;                      // source channels multiplied (whole slices)
  const int nrows = k_eff > 0 ? (sh + k_eff + 3) >> 2 : 0;  // window rows touched (at most ring_rows + 1)
  const int per = (nrows + p.parts - 1) / p.parts;
  const int w_begin = blockIdx.x * per, w_end = min(nrows, w_begin + per);
  const bool slice_ok = ds < RingDstEndSlice(p);
  const u32x4* wcol = p.weights + (size_t)wb * p.ring_rows * p.ns + min(ds, p.ns - 1);

  float acc[MT][4], asum[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    asum[t] = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[t][c] = 0.0f;
  }
  for (int w0 = w_begin + rsub; w0 < w_end; w0 += RW * U) {
    u32x4 blk[U];
    float a[U][MT][8];  // [row][token]: source slices w - 1 and w of the window row
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int w = w0 + u * RW;
      const bool live = w < w_end;
      int kb = row0 + min(w, w_end - 1);
      if (kb >= p.ring_rows) kb -= p.ring_rows;
      blk[u] = __builtin_nontemporal_load(wcol + (size_t)kb * p.ns);
      if (!live) blk[u] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const bool tok = live && t < p.m;
        // slice w holds source channels 4 w .. 4 w + 3; the row needs 4 w - sh .. 4 w - sh + 3
        const bool lo_ok = tok && sh > 0 && w >= 1 && w - 1 < ks_end, hi_ok = tok && w < ks_end;
        const size_t tk = act_tok0 + min(t, p.m - 1);
        Load4(act, ((size_t)max(min(w - 1, ks_end - 1), 0) * act_stride + tk) * 4, &a[u][t][0]);
        Load4(act, ((size_t)max(min(w, ks_end - 1), 0) * act_stride + tk) * 4, &a[u][t][4]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          a[u][t][i] = lo_ok ? a[u][t][i] : 0.0f;
          a[u][t][4 + i] = hi_ok ? a[u][t][4 + i] : 0.0f;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t word = blk[u][i];
        const float u0 = (float)(word & 0xFFu) - 128.0f, u1 = (float)((word >> 8) & 0xFFu) - 128.0f;
        const float u2 = (float)((word >> 16) & 0xFFu) - 128.0f, u3 = (float)(word >> 24) - 128.0f;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          // ring channel i of the row = source channel 4 w - sh + i = value 4 - sh + i of the two slices
          const float* v = a[u][t];
          const float av = sh == 0 ? v[4 + i] : (sh == 1 ? v[3 + i] : (sh == 2 ? v[2 + i] : v[1 + i]));
          asum[t] += av;
          acc[t][0] = fmaf(av, u0, acc[t][0]);
          acc[t][1] = fmaf(av, u1, acc[t][1]);
          acc[t][2] = fmaf(av, u2, acc[t][2]);
          acc[t][3] = fmaf(av, u3, acc[t][3]);
        }
      }
    }
  }
  // rows of the work-group through LDS, in their order
#pragma unroll
  for (int t = 0; t < MT; ++t) {
#pragma unroll
    for (int c = 0; c < 4; ++c) red[rsub][s_lane][t * 5 + c] = acc[t][c];
    red[rsub][s_lane][t * 5 + 4] = asum[t];
  }
  __syncthreads();
  if (rsub != 0) return;
  const size_t width = (size_t)p.ns * 4 + 4;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    if (t >= p.m) break;
    float* out = p.partial + (((size_t)blockIdx.x * p.rows + row) * 4 + t) * width;
    float v[5] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int q = 0; q < RW; ++q) {
#pragma unroll
      for (int c = 0; c < 5; ++c) v[c] += red[q][s_lane][t * 5 + c];
    }
    if (slice_ok) *reinterpret_cast<float4*>(out + (size_t)ds * 4) = make_float4(v[0], v[1], v[2], v[3]);
    if (blockIdx.y == 0 && s_lane == 0) out[(size_t)p.ns * 4] = v[4];
  }
}

// Work-group = 16 output channels x 16 part lanes of one (dst row, token): lane q adds the parts
// q, q + 16, ... in their order, eight loads in flight at a time; the 16 lanes' sums are added in
// lane order, then the write-out.
template <typename T, typename DstT>
__global__ __launch_bounds__(256) void fc_w8_ring_finish_kernel(RingParams p) {
  __shared__ float red[16][16][2];
  const int n_all = p.ns * 4;
  const int cl = threadIdx.x & 15, q = threadIdx.x >> 4;
  const int n = blockIdx.x * 16 + cl;  // (n_all is a multiple of 4; the grid covers it in chunks of 16)
  const int t = blockIdx.y, row = blockIdx.z;
  const size_t width = (size_t)n_all + 4;
  const int nc = min(n, n_all - 1);
  float sum = 0.0f, asum = 0.0f;
  for (int part0 = q; part0 < p.parts; part0 += 16 * 8) {
    float v[8], av[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int part = min(part0 + 16 * j, p.parts - 1);
      const float* in = p.partial + (((size_t)part * p.rows + row) * 4 + t) * width;
      v[j] = in[nc];
      av[j] = in[n_all];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (part0 + 16 * j < p.parts) {
        sum += v[j];
        asum += av[j];
      }
    }
  }
  red[q][cl][0] = sum;
  red[q][cl][1] = asum;
  __syncthreads();
  if (q != 0 || n >= n_all || (n >> 2) >= RingDstEndSlice(p)) return;
  sum = asum = 0.0f;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    sum += red[j][cl][0];
    asum += red[j][cl][1];
  }
  int wb = p.batch_ids ? p.batch_ids[row] : 0;
  wb = min(max(wb, 0), p.weights_batch - 1);
  float s = p.scalar_scale, z = p.has_zero_point ? p.scalar_zero_point : 0.0f;
  if (p.scale_kind == kScaleLinear) {
    s = LoadF(static_cast<const T*>(p.scale), (size_t)wb * n_all + n);
    if (p.zero_point) z = LoadF(static_cast<const T*>(p.zero_point), (size_t)wb * n_all + n);
  }
  const float r = s * fmaf(-z, asum, sum);
  const size_t o = ((size_t)(n >> 2) * p.rows * p.m + (size_t)row * p.m + t) * 4 + (n & 3);
  DstT* dst = static_cast<DstT*>(p.dst);
  const DstT* bias = static_cast<const DstT*>(p.bias);
  if constexpr (std::is_same<DstT, float>::value) {
    dst[o] = bias ? r + bias[n] : r;
  } else {
    __half h = __float2half_rn(r);
    if (bias) h = __hadd(h, bias[n]);
    dst[o] = h;
  }
}

template <typename T, int LS>
hipError_t LaunchRingT(const RingParams& p, bool dst_f16, hipStream_t stream) {
  const dim3 grid(p.parts, DivUp(p.ns, LS), p.rows);
  if (p.m == 1)
    hipLaunchKernelGGL((fc_w8_ring_i_kernel<T, LS, 1>), grid, dim3(kRingThreads), 0, stream, p);
  else if (p.m == 2)
    hipLaunchKernelGGL((fc_w8_ring_i_kernel<T, LS, 2>), grid, dim3(kRingThreads), 0, stream, p);
  else
    hipLaunchKernelGGL((fc_w8_ring_i_kernel<T, LS, 4>), grid, dim3(kRingThreads), 0, stream, p);
  const dim3 fgrid(DivUp(p.ns * 4, 16), p.m, p.rows);
  if (dst_f16)
    hipLaunchKernelGGL((fc_w8_ring_finish_kernel<T, __half>), fgrid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((fc_w8_ring_finish_kernel<T, float>), fgrid, dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace

size_t FcW8RingWorkspaceFloats(int max_tokens, int o) {
  const int n_pad = DivUp(o, 4) * 4;
  // (a launch's dst rows x tokens per row are at most max_tokens; every row keeps 4 token slots)
  const size_t rows_tokens = (size_t)std::min(std::max(max_tokens, 1), 16) * 4;
  return std::min((size_t)kRingMaxParts * rows_tokens * (n_pad + 4), (size_t)8 << 20);
}

bool FcW8RingSupported(const FcArgs& a) {
  if (a.params == nullptr || a.ring_i_index < 0 || a.ring_o_index >= 0) return false;
  if (a.weight_bits != 8 || a.ring_size < 4 || a.ring_size % 4 != 0) return false;
  if (a.packed_params_offset >= 0 || a.scale_kind == kScaleBlock) return false;
  if (a.act_f16 != a.dst_f16) return false;
  if (a.m < 1 || a.m > 4 || a.rows < 1 || (long)a.rows * a.m > 16) return false;
  if (a.k > a.ring_size) return false;  // (the window stays within one turn of the ring)
  const int ns = DivUp(a.n, 4);
  if (EffectiveGroup(a.group, ns) != ns) return false;
  const int w_ks = DivUp(a.weights_k > 0 ? a.weights_k : a.k, 4);
  if (a.ring_size > 4 * w_ks || (a.weights_batch > 1 && a.ring_size != 4 * w_ks)) return false;
  if (a.partial == nullptr) return false;
  // at least one part must fit the workspace
  return (size_t)a.rows * 4 * ((size_t)ns * 4 + 4) <= a.partial_floats;
}

hipError_t LaunchFcW8Ring(const FcArgs& a, hipStream_t stream, const char** kernel_name) {
  if (!FcW8RingSupported(a)) return hipErrorInvalidValue;
  RingParams p;
  p.act = a.act;
  p.weights = reinterpret_cast<const u32x4*>(a.weights);
  p.scale = a.scale;
  p.zero_point = a.has_zero_point ? a.zero_point : nullptr;
  p.bias = a.bias;
  p.dst = a.dst;
  p.partial = a.partial;
  p.params = a.params;
  p.batch_ids = a.batch_ids;
  p.m = a.m;
  p.ks = DivUp(a.k, 4);
  p.ns = DivUp(a.n, 4);
  p.ring_size = a.ring_size;
  p.ring_rows = a.ring_size / 4;
  p.ring_index = a.ring_i_index;
  p.src_end_ch_index = a.src_end_ch_index;
  p.dst_end_ch_index = a.dst_end_ch_index;
  p.k_channels = a.k;
  p.rows = a.rows;
  p.src_rows = a.src_rows;
  p.weights_batch = a.weights_batch;
  p.scale_kind = a.scale_kind;
  p.has_zero_point = a.has_zero_point ? 1 : 0;
  p.scalar_scale = a.scalar_scale;
  p.scalar_zero_point = a.scalar_zero_point;
  // lanes along the output slices: a power of two up to 64; parts: about 32 KB of weights each, at
  // most what the workspace holds
  int ls = 16;
  while (ls < 64 && ls < p.ns) ls *= 2;
  const int rows_in_flight = kRingThreads / ls * RingUnroll(p.m == 1 ? 1 : (p.m == 2 ? 2 : 4));
  const int window = std::min(p.ks + 1, p.ring_rows + 1);
  const size_t bytes = (size_t)window * p.ns * 16;
  int parts = (int)std::min<size_t>(kRingMaxParts, std::max<size_t>(1, bytes / 32768));
  parts = std::min(parts, std::max(1, DivUp(window, rows_in_flight)));
  const size_t per_part = (size_t)a.rows * 4 * ((size_t)p.ns * 4 + 4);
  parts = (int)std::min<size_t>(parts, a.partial_floats / per_part);
  p.parts = std::max(parts, 1);
  if (kernel_name) *kernel_name = "fc_w8_ring_i_kernel";
  if (a.act_f16) {
    if (ls == 16) return LaunchRingT<__half, 16>(p, a.dst_f16, stream);
    if (ls == 32) return LaunchRingT<__half, 32>(p, a.dst_f16, stream);
    return LaunchRingT<__half, 64>(p, a.dst_f16, stream);
  }
  if (ls == 16) return LaunchRingT<float, 16>(p, a.dst_f16, stream);
  if (ls == 32) return LaunchRingT<float, 32>(p, a.dst_f16, stream);
  return LaunchRingT<float, 64>(p, a.dst_f16, stream);
}

}  // namespace mldhip
