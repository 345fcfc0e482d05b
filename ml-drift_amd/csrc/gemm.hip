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

template <bool W4, int FN, int FM>
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
  u32x4 ra[NA];  // fp16 path: {blk0.x, blk0.y, blk1.x, blk1.y}
  u32x2 rs[NA];  // fp16 path: the 4 scales of the item's slice
  u32x4 rb[NB];  // fp16 path uses .xy only

  auto load_tiles = [&](int kt) {
    if (W4) {
#pragma unroll
      for (int q = 0; q < NA; ++q) {
        const int it = tid + q * kThreads;
        const int g = it / (BN / 4), nsl = it % (BN / 4);
        const int nsi = n0 / 4 + nsl;
        const int ksa = (kt * KG + g) * 2;
        u32x4 v = {0x88888888u, 0x88888888u, 0x88888888u, 0x88888888u};
        u32x2 sc = {0u, 0u};
        if (it < A_ITEMS && nsi < p.ns) {
          if (ksa < p.ks) {
            const u32x2 b0 = *reinterpret_cast<const u32x2*>(p.w4 + ((size_t)ksa * p.ns + nsi) * 8);
            v[0] = b0[0];
            v[1] = b0[1];
          }
          if (ksa + 1 < p.ks) {
            const u32x2 b1 = *reinterpret_cast<const u32x2*>(p.w4 + ((size_t)(ksa + 1) * p.ns + nsi) * 8);
            v[2] = b1[0];
            v[3] = b1[1];
          }
          int grp = kt / p.steps_per_group;
          if (grp >= p.groups) grp = p.groups - 1;
          sc = *reinterpret_cast<const u32x2*>(p.scale + ((size_t)grp * p.ns + nsi) * 4);
        }
        ra[q] = v;
        rs[q] = sc;
      }
#pragma unroll
      for (int q = 0; q < NB; ++q) {
        const int it = tid + q * kThreads;
        const int ksl = it / BM, ml = it % BM;
        const int ksi = kt * KG * 2 + ksl;
        const int mi = m0 + ml;
        u32x2 v = {0u, 0u};
        if (it < B_ITEMS && ksi < p.ks && mi < p.m)
          v = *reinterpret_cast<const u32x2*>(p.act + ((size_t)ksi * p.m + mi) * 4);
        rb[q] = u32x4{v[0], v[1], 0u, 0u};
      }
    } else {
#pragma unroll
      for (int q = 0; q < NA; ++q) {
        const int it = tid + q * kThreads;
        const int g = it / BN, r = it % BN;
        const int kg = kt * KG + g;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (it < A_ITEMS && kg < p.k16 && n0 + r < p.n) v = p.wi8[(size_t)kg * p.n + n0 + r];
        ra[q] = v;
      }
#pragma unroll
      for (int q = 0; q < NB; ++q) {
        const int it = tid + q * kThreads;
        const int g = it / BM, r = it % BM;
        const int kg = kt * KG + g;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (it < B_ITEMS && kg < p.k16 && m0 + r < p.m) v = p.codes[(size_t)kg * p.m + m0 + r];
        rb[q] = v;
      }
    }
  };

  auto store_tiles = [&](int buf) {
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
        *dst2 = u32x2{rb[q][0], rb[q][1]};
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

  load_tiles(0);
  store_tiles(0);
  __syncthreads();
  for (int kt = 0; kt < p.k_steps; ++kt) {
    const int buf = kt & 1;
    const bool more = kt + 1 < p.k_steps;
    if (more) load_tiles(kt + 1);
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
    if (more) store_tiles(buf ^ 1);
    __syncthreads();
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

template <bool W4>
hipError_t LaunchGemm(const GemmParams& p, hipStream_t stream) {
  // Tile choice: the largest work-group tile that still gives every CU a work-group;
  // small problems fall back to 64x64-per-wave tiles... the candidates are (FN, FM) in
  // {(4,4), (4,2), (2,2), (2,1)} -> work-group tiles 256x256, 256x128, 128x128, 128x64 (N x M).
  auto groups = [&](int bn, int bm) { return (long)DivUp(p.n, bn) * DivUp(p.m, bm); };
  const long want = 200;
  if (groups(256, 256) >= want) {
    hipLaunchKernelGGL((mfma_gemm_kernel<W4, 4, 4>), dim3(DivUp(p.n, 256), DivUp(p.m, 256)), dim3(kThreads), 0,
                       stream, p);
  } else if (groups(256, 128) >= want) {
    hipLaunchKernelGGL((mfma_gemm_kernel<W4, 4, 2>), dim3(DivUp(p.n, 256), DivUp(p.m, 128)), dim3(kThreads), 0,
                       stream, p);
  } else if (groups(128, 128) >= want || p.m > 64) {
    hipLaunchKernelGGL((mfma_gemm_kernel<W4, 2, 2>), dim3(DivUp(p.n, 128), DivUp(p.m, 128)), dim3(kThreads), 0,
                       stream, p);
  } else {
    hipLaunchKernelGGL((mfma_gemm_kernel<W4, 2, 1>), dim3(DivUp(p.n, 128), DivUp(p.m, 64)), dim3(kThreads), 0,
                       stream, p);
  }
  return hipGetLastError();
}

}  // namespace

bool FcW4MfmaSupported(const FcArgs& a) {
  if (a.weight_bits != 4 || !a.act_f16 || !a.dst_f16) return false;
  if (a.has_zero_point || a.scale_kind == kScaleScalar) return false;
  if (a.m <= kGemvMaxTokens) return false;
  if (a.scale_kind == kScaleBlock) {
    // a K-step of 32 input channels must not straddle scale groups
    if (a.groups <= 0 || a.k % a.groups != 0 || (a.k / a.groups) % 32 != 0) return false;
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
  if (kernel_name) *kernel_name = "fc_w4_mfma_gemm_kernel";
  return LaunchGemm<true>(p, stream);
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
  if (kernel_name) *kernel_name = "conv_int8_mfma_kernel";
  return LaunchGemm<false>(p, stream);
}

}  // namespace mldhip
