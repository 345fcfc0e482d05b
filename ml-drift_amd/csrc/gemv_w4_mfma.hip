// Streaming int4 GEMV on the matrix cores, for gfx950: 1..16 tokens, fp16 tensors, per-channel
// scales, optional per-channel zero points.  HBM-bound like the vector-ALU GEMV (gemv_w4.hip),
// but the multiply-accumulate work does not grow with the token count and the vector ALU only
// unpacks nibbles: one v_and_or_b32 per two weights.
//
// Work-group = 16 waves on a strip of 16 output slices (64 channels) and all of K; the waves
// split K sixteen ways and add their fp32 tiles through LDS in a fixed order.  A wave step covers
// 8 K-slices (32 input channels) with v_mfma_f32_16x16x32_f16:
//  - A (weights): row r of MFMA number t (t = 0..3) is output channel 4*(slice r) + t.  Lane
//    (r = lane % 16, g = lane / 16) loads the two 8-byte blocks (K-slices 2g, 2g+1 of the step,
//    slice r): in a block, word h holds inputs (2h, 2h+1) of the four outputs, 16 bits apart, so
//    (word >> 4t) & 0x000F000F | 0x64006400 is the half pair (1024+u, 1024+u) of output t (a
//    nibble in bits 4..7 is read in place with 0x5400: 64+u).  Four such words are the lane's A
//    operand for t: its 8 consecutive input channels.
//  - B (activations): column j = token; lane (j, g) loads the token's two 8-byte slices.
//  - The constant offsets are not subtracted per weight: a fifth MFMA with an all-ones A operand
//    accumulates sum_k a_k per token in the accumulator layout, and every accumulator is
//    corrected once at the end: acc - (c + 8 + zero point) * sum(a), c = 1024 or 64.
// All loads of a wave's share of K (up to 8 steps) are issued back to back, unconditionally:
// rows past K or past the wave's share re-read a valid row against zeroed activations.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mldhip {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4v_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kMsWaves = 16;
constexpr int kMsSteps = 8;  // steps whose loads are in flight together

struct MsParams {
  const uint8_t* weights;  // [Ks][Ns] blocks of 8 bytes
  const __half* act;       // [Ks][m][4]
  const __half* scale;     // [Ns * 4]
  const __half* zero_point;
  const __half* bias;
  __half* dst;  // [Ns][m][4]
  int m, ks, ns;
  int group;  // slices per output group of the packed weights (ns: one group)
  int steps_per_wave;
  uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};

// (x & mask) | magic.  Plain C on purpose: the result feeds an MFMA directly, and the compiler
// only inserts the wait states between a vector write and the MFMA that reads it when it can
// see the writing instruction (an inline-asm v_and_or_b32 here gave wrong sums).  The exponent
// patterns are parked in vector registers so that the expression still selects to one
// v_and_or_b32 (the instruction reads at most one scalar register).
__device__ __forceinline__ uint32_t AndOrMs(uint32_t x, uint32_t mask, uint32_t magic) {
  return (x & mask) | magic;
}

__device__ __forceinline__ float4v_t Mfma16(u32x4 a, u32x4 b, float4v_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
}

// FT: token blocks of 16.
template <int FT, bool ZP>
__global__ __launch_bounds__(kMsWaves * 64) void fc_w4_mfma_stream_kernel(MsParams p) {
  constexpr int TOK = FT * 16;
  __shared__ float red[kMsWaves][64][TOK + 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int slice0 = blockIdx.x * 16;
  const int slice = min(slice0 + r, p.ns - 1);  // clamp: loads stay in range, result unused
  const uint32_t row_w = (uint32_t)p.group * 8u;  // bytes per K-slice row of the weights (of one output group)
  const size_t col_w = ((size_t)(slice / p.group) * p.ks * p.group + slice % p.group) * 8;
  const uint32_t row_x = (uint32_t)p.m * 8u;

  int tok[FT];
#pragma unroll
  for (int ft = 0; ft < FT; ++ft) tok[ft] = min(ft * 16 + r, p.m - 1);

  float4v_t acc[4][FT], ones[FT];
#pragma unroll
  for (int ft = 0; ft < FT; ++ft) {
    ones[ft] = float4v_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[t][ft] = float4v_t{0.0f, 0.0f, 0.0f, 0.0f};
  }
  const u32x4 all_ones = {0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
  uint32_t magic_lo = p.magic_lo, magic_hi = p.magic_hi;
  asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));

  const int step_begin = wave * p.steps_per_wave;
  const int step_end = step_begin + p.steps_per_wave;
  for (int s0 = step_begin; s0 < step_end; s0 += kMsSteps) {
    u32x2 w[kMsSteps][2], x[kMsSteps][FT][2];
    // activations first (they come from cache), then the weights: waiting for the former leaves
    // the latter in flight
#pragma unroll
    for (int u = 0; u < kMsSteps; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int ksc = min((s0 + u) * 8 + 2 * g + h, p.ks - 1);
#pragma unroll
        for (int ft = 0; ft < FT; ++ft)
          x[u][ft][h] = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint8_t*>(p.act) + (size_t)ksc * row_x +
                                                         (size_t)tok[ft] * 8);
      }
#pragma unroll
    for (int u = 0; u < kMsSteps; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int ksc = min((s0 + u) * 8 + 2 * g + h, p.ks - 1);
        w[u][h] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p.weights + (size_t)ksc * row_w + col_w));
      }
    // keep the loads together and ahead of the arithmetic (the scheduler would otherwise sink
    // them next to their uses to save registers, a few at a time)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < kMsSteps; ++u) {
      const u32x4 blk = {w[u][0][0], w[u][0][1], w[u][1][0], w[u][1][1]};
      const u32x4 blk8 = {blk[0] >> 8, blk[1] >> 8, blk[2] >> 8, blk[3] >> 8};
      u32x4 bop[FT];
      // a K-slice past K or past this wave's share contributes nothing: zero activations
      const int ks_u = (s0 + u) * 8 + 2 * g;
      const bool live = s0 + u < step_end;
      const bool ok0 = live && ks_u < p.ks, ok1 = live && ks_u + 1 < p.ks;
#pragma unroll
      for (int ft = 0; ft < FT; ++ft) {
        bop[ft] = u32x4{ok0 ? x[u][ft][0][0] : 0u, ok0 ? x[u][ft][0][1] : 0u, ok1 ? x[u][ft][1][0] : 0u,
                        ok1 ? x[u][ft][1][1] : 0u};
        ones[ft] = Mfma16(all_ones, bop[ft], ones[ft]);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        u32x4 aop;
#pragma unroll
        for (int wd = 0; wd < 4; ++wd) {
          const uint32_t v = (t & 2) ? blk8[wd] : blk[wd];
          aop[wd] = (t & 1) ? AndOrMs(v, p.mask_hi, magic_hi) : AndOrMs(v, p.mask_lo, magic_lo);
        }
#pragma unroll
        for (int ft = 0; ft < FT; ++ft) acc[t][ft] = Mfma16(aop, bop[ft], acc[t][ft]);
      }
    }
  }

  // In the 16x16 result, register v of lane (j = lane % 16, g) is row 4*g + v (slice of the
  // strip) and column j (token); the four MFMAs hold the slice's four channels.
  // Remove the constant part, then stage this wave's tile for the K reduction.
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int sl = 4 * g + v;
    float zp[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (ZP) {
      const int s_c = min(slice0 + sl, p.ns - 1);
#pragma unroll
      for (int t = 0; t < 4; ++t) zp[t] = __half2float(p.zero_point[s_c * 4 + t]);
    }
#pragma unroll
    for (int ft = 0; ft < FT; ++ft) {
      const int token = ft * 16 + r;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const float centre = ((t & 1) ? 72.0f : 1032.0f) + zp[t];
        red[wave][sl * 4 + t][token] = fmaf(-centre, ones[ft][v], acc[t][ft][v]);
      }
    }
  }
  __syncthreads();
  // one thread per (slice, token, channel), in the order of the output tensor
  const int items = 64 * p.m;
  for (int idx = tid; idx < items; idx += kMsWaves * 64) {
    const int c = idx & 3;
    const int token = (idx >> 2) % p.m;
    const int sl = (idx >> 2) / p.m;
    const int s_out = slice0 + sl;
    if (s_out >= p.ns) continue;
    float sum = red[0][sl * 4 + c][token];
#pragma unroll
    for (int w2 = 1; w2 < kMsWaves; ++w2) sum += red[w2][sl * 4 + c][token];
    sum *= __half2float(p.scale[s_out * 4 + c]);
    __half h = __float2half_rn(sum);
    if (p.bias) h = __hadd(h, p.bias[s_out * 4 + c]);
    p.dst[((size_t)s_out * p.m + token) * 4 + c] = h;
  }
}

}  // namespace

bool FcW4MfmaStreamSupported(const FcArgs& a) {
  if (a.weight_bits != 4 || !a.act_f16 || !a.dst_f16) return false;
  if (a.params != nullptr || a.batch_ids != nullptr) return false;  // runtime channel bounds, batched weights: the other kernels
  if (a.scale_kind != kScaleLinear) return false;
  if (a.has_zero_point && a.zero_point == nullptr) return false;  // a scalar zero point: generic kernel
  if (a.m < 1 || a.m > 16) return false;
  // strips of 64 channels must give most CUs a work-group (K is not split across work-groups)
  return DivUp(DivUp(a.n, 4), 16) >= 128;
}

hipError_t LaunchFcW4MfmaStream(const FcArgs& a, hipStream_t stream, const char** kernel_name) {
  MsParams p;
  p.weights = a.weights;
  p.act = static_cast<const __half*>(a.act);
  p.scale = static_cast<const __half*>(a.scale);
  p.zero_point = a.has_zero_point ? static_cast<const __half*>(a.zero_point) : nullptr;
  p.bias = static_cast<const __half*>(a.bias);
  p.dst = static_cast<__half*>(a.dst);
  p.m = a.m;
  p.ks = DivUp(a.k, 4);
  p.ns = DivUp(a.n, 4);
  p.group = EffectiveGroup(a.group, p.ns);
  if (p.ns % p.group != 0) return hipErrorInvalidValue;
  p.steps_per_wave = DivUp(DivUp(p.ks, 8), kMsWaves);
  p.mask_lo = 0x000F000Fu;
  p.mask_hi = 0x00F000F0u;
  p.magic_lo = 0x64006400u;
  p.magic_hi = 0x54005400u;
  if (kernel_name) *kernel_name = "fc_w4_mfma_stream_kernel";
  const dim3 grid(DivUp(p.ns, 16)), block(kMsWaves * 64);
  const bool zp = p.zero_point != nullptr;
  if (zp)
    hipLaunchKernelGGL((fc_w4_mfma_stream_kernel<1, true>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((fc_w4_mfma_stream_kernel<1, false>), grid, block, 0, stream, p);
  return hipGetLastError();
}

}  // namespace mldhip
