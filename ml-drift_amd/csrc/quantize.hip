// Dynamic per-token activation quantization for gfx950 (fp16/fp32 -> 8-bit or 4-bit codes in the
// C4, W4C4, C16 or C32 packing plus fp32 (inv_scale, offset, sum) per token), following the arithmetic of the reference's
// generated kernel operation by operation: separate multiply and add (no fused
// multiply-add), round half up through floor(x*scale + zp + 0.5) or truncation of
// (x-min)*scale + 0.5.
//
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

// Groups of 16 channels per thread that stay in registers between the two passes.
constexpr int kMaxWaves = 16;

struct QuantParams {
  const void* src;
  uint8_t* codes;
  float* params;
  int tokens, channels, slices, batch;
  int is_signed, layout, symmetric, calculate_sum;
  int bits;           // 8, or 4 for the C32 types
  int width, height;  // tokens = height * width * batch, token = (y * width + x) * batch + b
  int nearest_even;   // codes by round-to-nearest-even of the scaled value instead of the reference's floor(v + 0.5)
};
// where the codes of a token go
enum : int { kCodesC4 = 0, kCodesC16 = 1, kCodesC32 = 2, kCodesW4C4 = 3 };

template <typename SrcT>
struct Raw;
template <>
struct Raw<__half> {
  using type = uint2;
};
template <>
struct Raw<float> {
  using type = float4;
};

__device__ __forceinline__ void Unpack(const uint2& raw, float v[4]) {
  const __half2 lo = *reinterpret_cast<const __half2*>(&raw.x);
  const __half2 hi = *reinterpret_cast<const __half2*>(&raw.y);
  v[0] = __low2float(lo);
  v[1] = __high2float(lo);
  v[2] = __low2float(hi);
  v[3] = __high2float(hi);
}
__device__ __forceinline__ void Unpack(const float4& raw, float v[4]) {
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

template <bool SYM, bool RNE>
struct Quantizer {
  float scale, min_value;
  float round_offset;  // symmetric: range / 2 + 0.5
  float top;           // the largest code, range - 1
  // The unsigned code of x as an integral float, at most `top`; the caller's conversion to a byte
  // saturates it at 0.  Asymmetric: truncation of a value >= 0.5, i.e. floor; a NaN (constant
  // row: 0 * inf) becomes code 0.
  __device__ __forceinline__ float Value(float x) const {
    // RNE (not the reference's rule): rint(x * scale) + range / 2 and rint((x - min) * scale), ties to even
    if (SYM) {
      if (RNE) return fminf(Add(rintf(Mul(x, scale)), round_offset - 0.5f), top);
      return fminf(floorf(Add(Mul(x, scale), round_offset)), top);
    }
    const float scaled = Mul(Sub(x, min_value), scale);
    if (scaled != scaled) return 0.0f;
    return fminf(RNE ? rintf(scaled) : floorf(Add(scaled, 0.5f)), top);
  }
};

// Work-group = TT tokens x (blockDim.x / TT) reduction lanes.  Tokens are the contiguous axis
// of the slice-major tensor, so the TT token lanes read TT x 8 B (fp16) contiguous bytes per
// slice.  Each thread owns groups of 4 consecutive slices (16 channels, one 16-byte store of
// codes in the C16 layout); the first CACHE groups of a thread stay in registers between the
// min/max pass and the encoding pass, so a row of up to 16 * CACHE * lanes channels is read
// from memory once.
// The value of the lane whose number differs in bit OFF (8, 16 or 32), paired with the lane's own:
// {own or partner, partner or own} in some order, which is all a symmetric reduction (max, min, sum)
// needs.  Register exchanges and a data-parallel move instead of a trip through the LDS crossbar.
typedef uint32_t u32x2q __attribute__((ext_vector_type(2)));
template <int OFF>
__device__ __forceinline__ u32x2q PairAcross(uint32_t v) {
  if constexpr (OFF == 32) {
    return __builtin_amdgcn_permlane32_swap(v, v, false, false);
  } else if constexpr (OFF == 16) {
    return __builtin_amdgcn_permlane16_swap(v, v, false, false);
  } else if constexpr (OFF == 8) {
    return u32x2q{v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x128 /* row_ror:8 */, 0xf, 0xf, false)};
  } else {
    return u32x2q{v, (uint32_t)__shfl_xor((int)v, OFF)};
  }
}
template <int FROM, typename Op>
__device__ __forceinline__ float ReduceAcross(float v, Op op) {
  if constexpr (FROM < 64) {
    const u32x2q r = PairAcross<FROM>(__float_as_uint(v));
    return ReduceAcross<FROM * 2>(op(__uint_as_float(r[0]), __uint_as_float(r[1])), op);
  } else {
    return v;
  }
}
template <int FROM>
__device__ __forceinline__ int SumAcross(int v) {
  if constexpr (FROM < 64) {
    const u32x2q r = PairAcross<FROM>((uint32_t)v);
    return SumAcross<FROM * 2>((int)r[0] + (int)r[1]);
  } else {
    return v;
  }
}

template <typename SrcT, int TT, bool SYM, int CACHE, bool RNE = false>
__global__ __launch_bounds__(1024) void quantize_kernel(QuantParams p) {
  using RawT = typename Raw<SrcT>::type;
  __shared__ float s_a[kMaxWaves][TT];
  __shared__ float s_b[kMaxWaves][TT];
  __shared__ int s_sum[kMaxWaves][TT];
  const SrcT* src = static_cast<const SrcT*>(p.src);
  const RawT* src4 = static_cast<const RawT*>(p.src);
  const int red = blockDim.x / TT;
  const int lt = threadIdx.x % TT;
  const int lr = threadIdx.x / TT;
  const int wave = threadIdx.x / 64;
  const int waves = blockDim.x / 64;
  const int tok_raw = blockIdx.x * TT + lt;
  const bool tok_ok = tok_raw < p.tokens;
  const int tok = tok_ok ? tok_raw : p.tokens - 1;
  const int s16_count = (p.slices + 3) / 4;
  constexpr bool kHalf = sizeof(SrcT) == 2;

  // Loads of the cached groups; slices past the end re-read the last one and are masked below.
  RawT cache[CACHE][4];
#pragma unroll
  for (int i = 0; i < CACHE; ++i) {
    const int g = lr + i * red;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = min(g * 4 + j, p.slices - 1);
      cache[i][j] = src4[(size_t)s * p.tokens + tok];
    }
  }

  // pass 1: abs-max, or min/max seeded with element (batch b, y 0, x 0, channel 0)
  float r0, r1;
  if (SYM) {
    r0 = 0.0f;
    r1 = 0.0f;
  } else {
    const int b = p.batch > 0 ? tok % p.batch : 0;
    float seed[4];
    Unpack(src4[b], seed);
    r0 = seed[0];
    r1 = seed[0];
  }
  // Channels past the end are replaced by the running value, which leaves it unchanged.
  auto reduce4 = [&](const RawT& raw, int s) {
    float v[4];
    Unpack(raw, v);
    const int nvalid = p.channels - s * 4;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (SYM) {
        r0 = fmaxf(r0, c < nvalid ? fabsf(v[c]) : 0.0f);
      } else {
        r0 = fminf(r0, c < nvalid ? v[c] : r0);
        r1 = fmaxf(r1, c < nvalid ? v[c] : r1);
      }
    }
  };
#pragma unroll
  for (int i = 0; i < CACHE; ++i) {
    const int g = lr + i * red;
#pragma unroll
    for (int j = 0; j < 4; ++j) reduce4(cache[i][j], g * 4 + j);
  }
  for (int g = lr + CACHE * red; g < s16_count; g += red) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = g * 4 + j;
      if (s < p.slices) reduce4(src4[(size_t)s * p.tokens + tok], s);
    }
  }
  // lanes of a wave that share a token, then the waves of the work-group
  if (SYM) {
    r0 = ReduceAcross<TT>(r0, [](float a, float b) { return fmaxf(a, b); });
  } else {
    r0 = ReduceAcross<TT>(r0, [](float a, float b) { return fminf(a, b); });
    r1 = ReduceAcross<TT>(r1, [](float a, float b) { return fmaxf(a, b); });
  }
  if (threadIdx.x % 64 < TT) {
    s_a[wave][lt] = r0;
    if (!SYM) s_b[wave][lt] = r1;
  }
  __syncthreads();
  for (int w = 0; w < waves; ++w) {
    if (SYM) {
      r0 = fmaxf(r0, s_a[w][lt]);
    } else {
      r0 = fminf(r0, s_a[w][lt]);
      r1 = fmaxf(r1, s_b[w][lt]);
    }
  }

  float inv_scale = 0.0f, offset = 0.0f;
  Quantizer<SYM, RNE> qz;
  qz.scale = 0.0f;
  qz.min_value = 0.0f;
  // code range: 256 values, or 16 for the 4-bit types
  const int half_codes = p.bits == 4 ? 8 : 128;
  const float zero_point = (float)half_codes, top = (float)(2 * half_codes - 1);
  qz.round_offset = zero_point + 0.5f;
  qz.top = top;
  // unsigned code - range / 2 as a two's complement byte / nibble
  const uint32_t sign_flip = !p.is_signed ? 0u : (p.bits == 4 ? 0x08080808u : 0x80808080u);
  const uint32_t code_mask = p.bits == 4 ? 0x0F0F0F0Fu : 0xFFFFFFFFu;
  const int code_shift = p.is_signed ? half_codes : 0;
  if (SYM) {
    const float abs_max = r0;
    if (abs_max > 0.0f) {
      const float min_scale = kHalf ? 6.103515625e-05f : 1.0e-30f;
      inv_scale = fmaxf(min_scale, Div(abs_max, zero_point - 1.0f));
      if (!p.is_signed && kHalf) inv_scale = fminf(inv_scale, Div(65504.0f, zero_point));
      qz.scale = Div(1.0f, inv_scale);
      if (!p.is_signed) offset = Mul(-inv_scale, zero_point);
    }
  } else {
    qz.min_value = r0;
    const float src_range = RangeInSrcType(src, r1, r0);
    offset = qz.min_value;
    qz.scale = Div(top, src_range);
    inv_scale = Div(src_range, top);
    if (p.is_signed) offset = Add(offset, Mul(src_range, Div(zero_point, top)));
  }

  // pass 2: codes
  uint32_t sum = 0;
  auto encode4 = [&](const RawT& raw, int s) -> uint32_t {
    float v[4];
    Unpack(raw, v);
    const int nvalid = max(0, min(4, p.channels - s * 4));
    uint32_t word = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) word = __builtin_amdgcn_cvt_pk_u8_f32(qz.Value(v[c]), c, word);
    const uint32_t valid = nvalid >= 4 ? 0xFFFFFFFFu : (1u << (8 * nvalid)) - 1u;
    sum = __builtin_amdgcn_udot4(word & valid, 0x01010101u, sum, false) - code_shift * nvalid;
    return (word ^ sign_flip) & code_mask;
  };
  // four bytes of 4-bit codes -> 16 bits, channel c in nibble c
  auto nibbles = [](uint32_t w) -> uint32_t {
    return (w & 0xFu) | ((w >> 4) & 0xF0u) | ((w >> 8) & 0xF00u) | ((w >> 12) & 0xF000u);
  };
  // W4C4: the token's column, row and batch element
  int tb = 0, tx = 0, ty = 0;
  if (p.layout == kCodesW4C4) {
    tb = tok % p.batch;
    tx = (tok / p.batch) % p.width;
    ty = tok / (p.batch * p.width);
  }
  // packed[j]: the codes of slice 4 g + j; slices at or beyond the end hold the last slice's
  auto store_group = [&](int g, const uint32_t packed[4]) {
    if (!tok_ok) return;
    if (p.layout == kCodesC16) {
      *reinterpret_cast<uint4*>(p.codes + ((size_t)g * p.tokens + tok) * 16) =
          make_uint4(packed[0], packed[1], packed[2], packed[3]);
    } else if (p.layout == kCodesC32) {
      const uint2 half = make_uint2(nibbles(packed[0]) | (nibbles(packed[1]) << 16),
                                    nibbles(packed[2]) | (nibbles(packed[3]) << 16));
      uint8_t* d = p.codes + ((size_t)(g >> 1) * p.tokens + tok) * 16;
      *reinterpret_cast<uint2*>(d + (g & 1) * 8) = half;
      if ((g & 1) == 0 && g == s16_count - 1) {  // no thread owns the upper half: the last slice again
        const uint32_t last = nibbles(packed[3]) * 0x00010001u;
        *reinterpret_cast<uint2*>(d + 8) = make_uint2(last, last);
      }
    } else if (p.layout == kCodesW4C4) {
      const int w4 = (p.width + 3) / 4;
      // this column, and the columns that pad the width to a multiple of 4 when it is the last one
      const int x_end = tx == p.width - 1 ? w4 * 4 : tx + 1;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int s = g * 4 + j;
        if (s >= p.slices) continue;
        for (int x = tx; x < x_end; ++x)
          *reinterpret_cast<uint32_t*>(p.codes + ((((size_t)s * p.height + ty) * w4 + x / 4) * p.batch + tb) * 16 +
                                       (x % 4) * 4) = packed[j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int s = g * 4 + j;
        if (s < p.slices)
          *reinterpret_cast<uint32_t*>(p.codes + ((size_t)s * p.tokens + tok) * 4) = packed[j];
      }
    }
  };
#pragma unroll
  for (int i = 0; i < CACHE; ++i) {
    const int g = lr + i * red;
    if (g < s16_count) {
      uint32_t packed[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) packed[j] = encode4(cache[i][j], g * 4 + j);  // (the load clamped the slice)
      store_group(g, packed);
    }
  }
  for (int g = lr + CACHE * red; g < s16_count; g += red) {
    uint32_t packed[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = g * 4 + j;
      packed[j] = encode4(src4[(size_t)min(s, p.slices - 1) * p.tokens + tok], s);
    }
    store_group(g, packed);
  }
  if (p.calculate_sum) {
    int total = (int)sum;
    total = SumAcross<TT>(total);
    if (threadIdx.x % 64 < TT) s_sum[wave][lt] = total;
    __syncthreads();
    total = 0;
    for (int w = 0; w < waves; ++w) total += s_sum[w][lt];
    sum = (uint32_t)total;
  }
  if (lr == 0 && tok_ok)
    *reinterpret_cast<float4*>(p.params + (size_t)tok * 4) =
        make_float4(inv_scale, offset, p.calculate_sum ? (float)(int)sum : 0.0f, 0.0f);
}

template <int TT, int CACHE, bool RNE>
void Launch3(bool f16, bool sym, dim3 grid, dim3 block, hipStream_t stream, const QuantParams& p) {
  if (f16 && sym)
    hipLaunchKernelGGL((quantize_kernel<__half, TT, true, CACHE, RNE>), grid, block, 0, stream, p);
  else if (f16)
    hipLaunchKernelGGL((quantize_kernel<__half, TT, false, CACHE, RNE>), grid, block, 0, stream, p);
  else if (sym)
    hipLaunchKernelGGL((quantize_kernel<float, TT, true, CACHE, RNE>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((quantize_kernel<float, TT, false, CACHE, RNE>), grid, block, 0, stream, p);
}
template <int TT, int CACHE>
void Launch2(bool f16, bool sym, dim3 grid, dim3 block, hipStream_t stream, const QuantParams& p) {
  if (p.nearest_even)
    Launch3<TT, CACHE, true>(f16, sym, grid, block, stream, p);
  else
    Launch3<TT, CACHE, false>(f16, sym, grid, block, stream, p);
}
// One register-cached group per thread when that covers the row, four otherwise.
template <int TT>
void Launch(bool f16, bool sym, dim3 grid, dim3 block, hipStream_t stream, const QuantParams& p) {
  const int red = (int)block.x / TT;
  if (DivUp(p.slices, 4) <= red)
    Launch2<TT, 1>(f16, sym, grid, block, stream, p);
  else
    Launch2<TT, 4>(f16, sym, grid, block, stream, p);
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
  // PackedType: 1 uint8c4, 2 int8c4, 3 uint8w4c4, 4 int8w4c4, 5 int8c16, 6 uint8c16, 7 int4c32, 8 uint4c32
  p.is_signed = a.packed_type == 2 || a.packed_type == 4 || a.packed_type == 5 || a.packed_type == 7;
  p.layout = (a.packed_type == 5 || a.packed_type == 6)   ? kCodesC16
             : (a.packed_type == 7 || a.packed_type == 8) ? kCodesC32
             : (a.packed_type == 3 || a.packed_type == 4) ? kCodesW4C4
                                                          : kCodesC4;
  p.bits = p.layout == kCodesC32 ? 4 : 8;
  p.width = a.width;
  p.height = a.height;
  if (p.layout == kCodesW4C4 && (long long)a.width * a.height * a.batch != a.tokens) return hipErrorInvalidValue;
  p.symmetric = a.symmetric;
  p.calculate_sum = a.calculate_sum;
  p.nearest_even = a.nearest_even ? 1 : 0;
  if (kernel_name) *kernel_name = "quantize_kernel";
  // Few channel groups: wide token tiles (32 tokens x >= 2 lanes); otherwise 8 tokens per
  // work-group and as many reduction lanes as there are groups, up to 128.
  const int groups16 = DivUp(p.slices, 4);
  int red = 1;
  while (red < groups16 && red < 128) red *= 2;
  if (red <= 8) {
    red = red < 2 ? 2 : red;
    dim3 grid(DivUp(a.tokens, 32)), block(32 * red);
    Launch<32>(a.src_f16, a.symmetric, grid, block, stream, p);
  } else {
    dim3 grid(DivUp(a.tokens, 8)), block(8 * red);
    Launch<8>(a.src_f16, a.symmetric, grid, block, stream, p);
  }
  return hipGetLastError();
}

}  // namespace mldhip
