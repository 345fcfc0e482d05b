// Dynamic per-token activation quantization for gfx950 (fp16/fp32 -> int8/uint8 codes plus
// fp32 (inv_scale, offset, sum) per token), following the arithmetic of the reference's
// generated kernel operation by operation: separate multiply and add (no fused
// multiply-add), round half up through floor(x*scale + zp + 0.5) or truncation of
// (x-min)*scale + 0.5.
//
// Work-group = 32 tokens x 8 reduction lanes.  Tokens are the contiguous axis of the
// slice-major tensor, so the 32 token lanes of a wave read 32 x 8 B (fp16) contiguous bytes
// per slice.  Each thread owns groups of 4 consecutive slices (16 channels), which is one
// 16-byte store of codes in the C16 layout.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "kernels.h"

// Every multiply and add below is a separate rounding, as in the reference's kernel text:
// no fused multiply-add may be formed.
#pragma clang fp contract(off)

namespace mldhip {
namespace {

// Single IEEE operations.  They are written with plain operators inside this file so that
// they carry no permission to contract (library intrinsics inline with that permission).
__device__ __forceinline__ float Mul(float a, float b) { return a * b; }
__device__ __forceinline__ float Add(float a, float b) { return a + b; }
__device__ __forceinline__ float Sub(float a, float b) { return a - b; }
__device__ __forceinline__ float Div(float a, float b) { return a / b; }

constexpr int kTok = 32;
constexpr int kRed = 8;

struct QuantParams {
  const void* src;
  uint8_t* codes;
  float* params;
  int tokens, channels, slices, batch;
  int is_signed, c16, symmetric, calculate_sum;
};

__device__ __forceinline__ void Load4(const __half* src, size_t idx, float v[4]) {
  const uint2 raw = *reinterpret_cast<const uint2*>(src + idx);
  const __half2 lo = *reinterpret_cast<const __half2*>(&raw.x);
  const __half2 hi = *reinterpret_cast<const __half2*>(&raw.y);
  v[0] = __low2float(lo);
  v[1] = __high2float(lo);
  v[2] = __low2float(hi);
  v[3] = __high2float(hi);
}
__device__ __forceinline__ void Load4(const float* src, size_t idx, float v[4]) {
  const float4 raw = *reinterpret_cast<const float4*>(src + idx);
  v[0] = raw.x;
  v[1] = raw.y;
  v[2] = raw.z;
  v[3] = raw.w;
}

// max - min in the source type.
__device__ __forceinline__ float RangeInSrcType(const __half*, float mx, float mn) {
  return __half2float(__hsub(__float2half_rn(mx), __float2half_rn(mn)));
}
__device__ __forceinline__ float RangeInSrcType(const float*, float mx, float mn) {
  return Sub(mx, mn);
}

template <typename SrcT>
__global__ __launch_bounds__(kTok* kRed) void quantize_kernel(QuantParams p) {
  __shared__ float s_a[kRed][kTok];
  __shared__ float s_b[kRed][kTok];
  __shared__ int s_sum[kRed][kTok];
  const SrcT* src = static_cast<const SrcT*>(p.src);
  const int lt = threadIdx.x % kTok;
  const int lr = threadIdx.x / kTok;
  const int tok_raw = blockIdx.x * kTok + lt;
  const bool tok_ok = tok_raw < p.tokens;
  const int tok = tok_ok ? tok_raw : p.tokens - 1;
  const int s16_count = (p.slices + 3) / 4;
  constexpr bool kHalf = sizeof(SrcT) == 2;

  // pass 1: abs-max, or min/max seeded with element (batch b, y 0, x 0, channel 0)
  float r0, r1;
  if (p.symmetric) {
    r0 = 0.0f;
    r1 = 0.0f;
  } else {
    const int b = p.batch > 0 ? tok % p.batch : 0;
    float seed[4];
    Load4(src, (size_t)b * 4, seed);
    r0 = seed[0];
    r1 = seed[0];
  }
  for (int g = lr; g < s16_count; g += kRed) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = g * 4 + j;
      if (s >= p.slices) break;
      float v[4];
      Load4(src, ((size_t)s * p.tokens + tok) * 4, v);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if (s * 4 + c < p.channels) {
          if (p.symmetric) {
            r0 = fmaxf(r0, fabsf(v[c]));
          } else {
            r0 = fminf(r0, v[c]);
            r1 = fmaxf(r1, v[c]);
          }
        }
      }
    }
  }
  s_a[lr][lt] = r0;
  s_b[lr][lt] = r1;
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kRed; ++r) {
    if (p.symmetric) {
      r0 = fmaxf(r0, s_a[r][lt]);
    } else {
      r0 = fminf(r0, s_a[r][lt]);
      r1 = fmaxf(r1, s_b[r][lt]);
    }
  }

  float inv_scale = 0.0f, scale = 0.0f, offset = 0.0f, min_value = 0.0f;
  if (p.symmetric) {
    const float abs_max = r0;
    if (abs_max > 0.0f) {
      const float min_scale = kHalf ? 6.103515625e-05f : 1.0e-30f;
      inv_scale = fmaxf(min_scale, Div(abs_max, 127.0f));
      if (!p.is_signed && kHalf) inv_scale = fminf(inv_scale, Div(65504.0f, 128.0f));
      scale = Div(1.0f, inv_scale);
      if (!p.is_signed) offset = Mul(-inv_scale, 128.0f);
    }
  } else {
    min_value = r0;
    const float src_range = RangeInSrcType(src, r1, r0);
    offset = min_value;
    scale = Div(255.0f, src_range);
    inv_scale = Div(src_range, 255.0f);
    if (p.is_signed) offset = Add(offset, Mul(src_range, Div(128.0f, 255.0f)));
  }

  // pass 2: codes
  int sum = 0;
  const int code_shift = p.is_signed ? 128 : 0;
  for (int g = lr; g < s16_count; g += kRed) {
    uint32_t packed[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = g * 4 + j;
      if (s >= p.slices) break;
      float v[4];
      Load4(src, ((size_t)s * p.tokens + tok) * 4, v);
      uint32_t word = 0;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        int q;
        if (p.symmetric) {
          float f = Mul(v[c], scale);
          f = Add(f, 128.5f);
          f = floorf(f);
          f = fminf(255.0f, fmaxf(0.0f, f));
          q = (int)f;
        } else {
          float f = Mul(Sub(v[c], min_value), scale);
          f = Add(f, 0.5f);
          q = (f != f) ? 0 : (int)f;  // NaN (constant row: 0 * inf) converts to 0
          q = max(0, min(255, q));
        }
        q -= code_shift;
        if (s * 4 + c < p.channels) sum += q;
        word |= (uint32_t)(q & 0xFF) << (8 * c);
      }
      packed[j] = word;
      if (!p.c16 && tok_ok)
        *reinterpret_cast<uint32_t*>(p.codes + ((size_t)s * p.tokens + tok) * 4) = word;
    }
    if (p.c16 && tok_ok)
      *reinterpret_cast<uint4*>(p.codes + ((size_t)g * p.tokens + tok) * 16) =
          make_uint4(packed[0], packed[1], packed[2], packed[3]);
  }
  if (p.calculate_sum) {
    s_sum[lr][lt] = sum;
    __syncthreads();
    sum = 0;
#pragma unroll
    for (int r = 0; r < kRed; ++r) sum += s_sum[r][lt];
  }
  if (lr == 0 && tok_ok)
    *reinterpret_cast<float4*>(p.params + (size_t)tok * 4) =
        make_float4(inv_scale, offset, p.calculate_sum ? (float)sum : 0.0f, 0.0f);
}

}  // namespace

hipError_t LaunchQuantize(const QuantArgs& a, hipStream_t stream, const char** kernel_name) {
  QuantParams p;
  p.src = a.src;
  p.codes = static_cast<uint8_t*>(a.codes);
  p.params = a.params;
  p.tokens = a.tokens;
  p.channels = a.channels;
  p.slices = DivUp(a.channels, 4);
  p.batch = a.batch;
  p.is_signed = a.packed_type == 2 || a.packed_type == 5;
  p.c16 = a.packed_type == 5 || a.packed_type == 6;
  p.symmetric = a.symmetric;
  p.calculate_sum = a.calculate_sum;
  if (kernel_name) *kernel_name = "quantize_kernel";
  dim3 grid(DivUp(a.tokens, kTok));
  dim3 block(kTok * kRed);
  if (a.src_f16)
    hipLaunchKernelGGL(quantize_kernel<__half>, grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL(quantize_kernel<float>, grid, block, 0, stream, p);
  return hipGetLastError();
}

}  // namespace mldhip
