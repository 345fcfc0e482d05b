// Decode-side FullyConnected kernels for gfx950: HBM-streaming GEMV over the reference's
// packed I4O4 weight buffers.
//
//  fc_generic_kernel   any weight width / scale kind / zero point / tensor type, fp32 math.
//  fc_w4_stream_kernel int4 weights, fp16 tensors, <= 4 tokens: 128-bit loads of packed
//                      nibbles, magic-number nibble->half conversion, v_dot2_f32_f16
//                      accumulation, deterministic split-K across work-groups.
//  fc_int8_math_kernel int8 activations x uint8/uint4 weights -> int32 (bit-exact).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "kernels.h"

namespace mldhip {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float LoadF(const float* p, size_t i) { return p[i]; }
__device__ __forceinline__ float LoadF(const __half* p, size_t i) { return __half2float(p[i]); }

// Converts the accumulator to the destination type, then adds the bias in that type
// (the order the reference's write-out uses).
__device__ __forceinline__ void StoreOut(float* dst, size_t i, float r, const float* bias, size_t bi) {
  dst[i] = bias ? r + bias[bi] : r;
}
__device__ __forceinline__ void StoreOut(__half* dst, size_t i, float r, const __half* bias, size_t bi) {
  __half h = __float2half_rn(r);
  if (bias) h = __hadd(h, bias[bi]);
  dst[i] = h;
}

// ------------------------------------------------------------------------------------------
// Generic kernel.  Block (64, 4): x = output slice inside a strip of 64, y = K lane.
// ------------------------------------------------------------------------------------------
struct GenericParams {
  const void* act;
  const uint8_t* weights;
  const void* scale;
  const void* zero_point;
  const void* bias;
  void* dst;
  int m, ks, ns;
  int scale_kind, groups, group_slices;
  float scalar_scale, scalar_zero_point;
  int has_zero_point;
};

template <typename ActT, typename DstT, int WBITS, int TB>
__global__ __launch_bounds__(256) void fc_generic_kernel(GenericParams p) {
  __shared__ float red[4][64][TB * 4];
  const int tx = threadIdx.x, ty = threadIdx.y;
  const int ds = blockIdx.x * 64 + tx;
  const int tok0 = blockIdx.y * TB;
  const ActT* act = static_cast<const ActT*>(p.act);
  const ActT* scale = static_cast<const ActT*>(p.scale);
  const ActT* zp = static_cast<const ActT*>(p.zero_point);
  const float shift = WBITS == 8 ? 128.0f : 8.0f;

  float acc[TB][4];
#pragma unroll
  for (int t = 0; t < TB; ++t)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[t][c] = 0.0f;

  if (ds < p.ns) {
    float s[4], z[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      s[c] = p.scalar_scale;
      z[c] = p.has_zero_point ? p.scalar_zero_point : 0.0f;
    }
    if (p.scale_kind == kScaleLinear) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        s[c] = LoadF(scale, (size_t)ds * 4 + c);
        if (zp) z[c] = LoadF(zp, (size_t)ds * 4 + c);
      }
    }
    for (int ks = ty; ks < p.ks; ks += 4) {
      if (p.scale_kind == kScaleBlock) {
        int g = ks / p.group_slices;
        if (g >= p.groups) g = p.groups - 1;
        const size_t sidx = ((size_t)g * p.ns + ds) * 4;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          s[c] = LoadF(scale, sidx + c);
          if (zp) z[c] = LoadF(zp, sidx + c);
        }
      }
      const size_t blk = (size_t)ks * p.ns + ds;
      float wf[4][4];
      if (WBITS == 8) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(p.weights + blk * 16);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int c = 0; c < 4; ++c)
            wf[i][c] = ((float)((w[i] >> (8 * c)) & 0xFFu) - (shift + z[c])) * s[c];
      } else {
        const u32x2 w = *reinterpret_cast<const u32x2*>(p.weights + blk * 8);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int c = 0; c < 4; ++c)
            wf[i][c] = ((float)((w[i >> 1] >> (16 * (i & 1) + 4 * c)) & 0xFu) - (shift + z[c])) * s[c];
      }
#pragma unroll
      for (int t = 0; t < TB; ++t) {
        const int tok = tok0 + t;
        if (tok < p.m) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float a = LoadF(act, ((size_t)ks * p.m + tok) * 4 + i);
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[t][c] = fmaf(a, wf[i][c], acc[t][c]);
          }
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < TB; ++t)
#pragma unroll
    for (int c = 0; c < 4; ++c) red[ty][tx][t * 4 + c] = acc[t][c];
  __syncthreads();
  if (ty == 0 && ds < p.ns) {
    DstT* dst = static_cast<DstT*>(p.dst);
    const DstT* bias = static_cast<const DstT*>(p.bias);
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      const int tok = tok0 + t;
      if (tok >= p.m) continue;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float r = (red[0][tx][t * 4 + c] + red[1][tx][t * 4 + c]) +
                        (red[2][tx][t * 4 + c] + red[3][tx][t * 4 + c]);
        StoreOut(dst, ((size_t)ds * p.m + tok) * 4 + c, r, bias, (size_t)ds * 4 + c);
      }
    }
  }
}

template <typename ActT, typename DstT, int WBITS>
hipError_t LaunchGenericT(const GenericParams& p, hipStream_t stream) {
  constexpr int TB = 4;
  dim3 grid(DivUp(p.ns, 64), DivUp(p.m, TB));
  dim3 block(64, 4);
  hipLaunchKernelGGL((fc_generic_kernel<ActT, DstT, WBITS, TB>), grid, block, 0, stream, p);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// Streaming int4 GEMV.
//
// Packed buffer: row ks (4 input channels) holds Ns blocks of 8 bytes; one 16-byte load
// covers two neighbouring blocks = 8 output channels x 4 input channels.  In a 32-bit word
// of a block, nibble j (j = 0..3) is (input 2h, output j) and nibble 4+j is (input 2h+1,
// output j) for word h of the block, so (word >> 4j) & 0x000F000F yields the pair
// (input 2h, input 2h+1) of output j in the two 16-bit halves: exactly the operand shape of
// v_dot2_f32_f16 against the activation pair.  OR-ing 0x6400 makes each half the fp16 number
// 1024+u; subtracting 1032 (exact) leaves the signed weight u-8.
//
// Thread layout: LPR lanes cover one row segment (LPR x 16 B contiguous), 256/LPR rows per
// work-group step.  A thread walks chunks of 8 consecutive K-slices (32 input channels = one
// scale group when group-wise), so a group's scale is fetched once per chunk.
// Work-groups of the same output strip split K (blockIdx.y); partial sums go to a private
// workspace and the last-arriving work-group adds them in a fixed order.
// ------------------------------------------------------------------------------------------
struct StreamParams {
  const u32x4* weights;
  const __half* act;
  const __half* scale;
  const __half* bias;
  __half* dst;
  float* partial;
  int* counters;
  int m, ks, ns, n_pad;  // n_pad = ns * 4
  int row_u4;            // uint4 per packed row = ns / 2
  int chunks;            // ceil(ks / 8)
  int chunks_per_split;
  int ksplit;
  int group_chunks;  // chunks per scale group (grouped only)
  int groups;
};

// Reinterprets a 32-bit word as two halfs.  Taking the word by value matters: applying
// __builtin_bit_cast directly to a vector element reads element 0 whatever the index.
__device__ __forceinline__ half2_t AsHalf2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }

__device__ __forceinline__ half2_t NibblePair(uint32_t word, int j) {
  const uint32_t bits = ((word >> (4 * j)) & 0x000F000Fu) | 0x64006400u;
  half2_t h = AsHalf2(bits);
  const half2_t off = {(_Float16)1032.0f, (_Float16)1032.0f};
  return h - off;
}

template <int LPR, int M, bool GROUPED>
__global__ __launch_bounds__(256) void fc_w4_stream_kernel(StreamParams p) {
  constexpr int ROWS = 256 / LPR;
  constexpr int STRIP = LPR * 8;  // output channels per work-group
  __shared__ float red[ROWS][M][STRIP];
  __shared__ int s_last;

  const int tid = threadIdx.x;
  const int col = tid % LPR;
  const int row = tid / LPR;
  const int pcol = blockIdx.x * LPR + col;  // uint4 column = output channels 8*pcol .. +7
  const bool col_ok = pcol < p.row_u4;
  const int ky = blockIdx.y;
  const int c_begin = ky * p.chunks_per_split;
  const int c_end = min(c_begin + p.chunks_per_split, p.chunks);

  float acc[M][8];
#pragma unroll
  for (int m = 0; m < M; ++m)
#pragma unroll
    for (int o = 0; o < 8; ++o) acc[m][o] = 0.0f;

  if (col_ok) {
    for (int c = c_begin + row; c < c_end; c += ROWS) {
      const int ks0 = c * 8;
      u32x4 w[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int ks = ks0 + j;
        if (ks < p.ks) {
          w[j] = __builtin_nontemporal_load(p.weights + (size_t)ks * p.row_u4 + pcol);
        } else {
          w[j] = u32x4{0x88888888u, 0x88888888u, 0x88888888u, 0x88888888u};
        }
      }
      float t[M][8];
#pragma unroll
      for (int m = 0; m < M; ++m)
#pragma unroll
        for (int o = 0; o < 8; ++o) t[m][o] = GROUPED ? 0.0f : acc[m][o];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int ks = ks0 + j;
        half2_t a01[M], a23[M];
#pragma unroll
        for (int m = 0; m < M; ++m) {
          u32x2 av = {0u, 0u};
          if (ks < p.ks) av = *reinterpret_cast<const u32x2*>(p.act + ((size_t)ks * M + m) * 4);
          a01[m] = AsHalf2(av[0]);
          a23[m] = AsHalf2(av[1]);
        }
#pragma unroll
        for (int o = 0; o < 4; ++o) {
          const half2_t w0 = NibblePair(w[j][0], o);  // inputs 0,1 -> output o
          const half2_t w1 = NibblePair(w[j][1], o);  // inputs 2,3 -> output o
          const half2_t w2 = NibblePair(w[j][2], o);  // inputs 0,1 -> output 4+o
          const half2_t w3 = NibblePair(w[j][3], o);  // inputs 2,3 -> output 4+o
#pragma unroll
          for (int m = 0; m < M; ++m) {
            t[m][o] = __builtin_amdgcn_fdot2(w0, a01[m], t[m][o], false);
            t[m][o] = __builtin_amdgcn_fdot2(w1, a23[m], t[m][o], false);
            t[m][4 + o] = __builtin_amdgcn_fdot2(w2, a01[m], t[m][4 + o], false);
            t[m][4 + o] = __builtin_amdgcn_fdot2(w3, a23[m], t[m][4 + o], false);
          }
        }
      }
      if (GROUPED) {
        int g = c / p.group_chunks;
        if (g >= p.groups) g = p.groups - 1;
        const u32x4 sv = *reinterpret_cast<const u32x4*>(p.scale + ((size_t)g * p.ns + 2 * pcol) * 4);
#pragma unroll
        for (int o = 0; o < 8; ++o) {
          const half2_t sp = AsHalf2(sv[o >> 1]);
          const float s = (float)sp[o & 1];
#pragma unroll
          for (int m = 0; m < M; ++m) acc[m][o] = fmaf(s, t[m][o], acc[m][o]);
        }
      } else {
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
          for (int o = 0; o < 8; ++o) acc[m][o] = t[m][o];
      }
    }
  }

  // Work-group reduction over the rows.
#pragma unroll
  for (int m = 0; m < M; ++m)
#pragma unroll
    for (int o = 0; o < 8; ++o) red[row][m][col * 8 + o] = acc[m][o];
  __syncthreads();

  const int n0 = blockIdx.x * STRIP;
  const bool single = p.ksplit == 1;
  for (int idx = tid; idx < M * STRIP; idx += 256) {
    const int m = idx / STRIP, nl = idx % STRIP;
    const int n = n0 + nl;
    if (n >= p.n_pad) continue;
    float v = 0.0f;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) v += red[r][m][nl];
    if (single) {
      if (!GROUPED) v *= __half2float(p.scale[n]);
      StoreOut(p.dst, ((size_t)(n >> 2) * M + m) * 4 + (n & 3), v, p.bias, (size_t)n);
    } else {
      p.partial[((size_t)ky * M + m) * p.n_pad + n] = v;
    }
  }
  if (single) return;

  // Split-K: publish the partial sums, count arrivals, the last work-group of this strip
  // adds all partials in split order (so the result does not depend on arrival order).
  __threadfence();
  __syncthreads();
  if (tid == 0) {
    const int prev = atomicAdd(&p.counters[blockIdx.x], 1);
    s_last = prev == p.ksplit - 1;
  }
  __syncthreads();
  if (!s_last) return;
  __threadfence();
  for (int idx = tid; idx < M * STRIP; idx += 256) {
    const int m = idx / STRIP, nl = idx % STRIP;
    const int n = n0 + nl;
    if (n >= p.n_pad) continue;
    float v = 0.0f;
    for (int s = 0; s < p.ksplit; ++s)
      v += __builtin_nontemporal_load(&p.partial[((size_t)s * M + m) * p.n_pad + n]);
    if (!GROUPED) v *= __half2float(p.scale[n]);
    StoreOut(p.dst, ((size_t)(n >> 2) * M + m) * 4 + (n & 3), v, p.bias, (size_t)n);
  }
  if (tid == 0) p.counters[blockIdx.x] = 0;  // ready for the next launch on this stream
}

template <int LPR, int M>
hipError_t LaunchStreamLM(const StreamParams& p, bool grouped, dim3 grid, hipStream_t stream) {
  if (grouped)
    hipLaunchKernelGGL((fc_w4_stream_kernel<LPR, M, true>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((fc_w4_stream_kernel<LPR, M, false>), grid, dim3(256), 0, stream, p);
  return hipGetLastError();
}

template <int LPR>
hipError_t LaunchStreamL(const StreamParams& p, bool grouped, dim3 grid, hipStream_t stream) {
  switch (p.m) {
    case 1: return LaunchStreamLM<LPR, 1>(p, grouped, grid, stream);
    case 2: return LaunchStreamLM<LPR, 2>(p, grouped, grid, stream);
    case 3: return LaunchStreamLM<LPR, 3>(p, grouped, grid, stream);
    case 4: return LaunchStreamLM<LPR, 4>(p, grouped, grid, stream);
    default: return hipErrorInvalidValue;
  }
}

int EnvInt(const char* name, int fallback) {
  const char* v = std::getenv(name);
  return v ? std::atoi(v) : fallback;
}

// ------------------------------------------------------------------------------------------
// int8-math kernel: same thread layout as the generic kernel, int32 accumulators.
// ------------------------------------------------------------------------------------------
template <int WBITS, int TB>
__global__ __launch_bounds__(256) void fc_int8_math_kernel(const int8_t* __restrict__ act,
                                                           const uint8_t* __restrict__ weights,
                                                           int32_t* __restrict__ dst, int m, int ks_n,
                                                           int ns) {
  __shared__ int red[4][64][TB * 4];
  const int tx = threadIdx.x, ty = threadIdx.y;
  const int ds = blockIdx.x * 64 + tx;
  const int tok0 = blockIdx.y * TB;
  int acc[TB][4];
#pragma unroll
  for (int t = 0; t < TB; ++t)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[t][c] = 0;
  if (ds < ns) {
    for (int ks = ty; ks < ks_n; ks += 4) {
      const size_t blk = (size_t)ks * ns + ds;
      uint32_t w0, w1, w2, w3;  // per output channel: the 4 input-channel values, one per byte
      if (WBITS == 4) {
        const u32x2 w = *reinterpret_cast<const u32x2*>(weights + blk * 8);
        // 4x4 nibble-matrix transpose by two swap stages.
        uint32_t t = (w[1] ^ (w[0] >> 16)) & 0x0000FFFFu;
        uint32_t t0 = w[0] ^ (t << 16);
        uint32_t t1 = w[1] ^ t;
        t = (t1 ^ (t0 >> 8)) & 0x00FF00FFu;
        t1 ^= t;
        t0 ^= (t << 8);
        w0 = t0 & 0x0F0F0F0Fu;
        w1 = (t0 >> 4) & 0x0F0F0F0Fu;
        w2 = t1 & 0x0F0F0F0Fu;
        w3 = (t1 >> 4) & 0x0F0F0F0Fu;
      } else {
        const u32x4 w = *reinterpret_cast<const u32x4*>(weights + blk * 16);
        // 4x4 byte-matrix transpose, then u-128 per byte (flip the top bit) = the int8 weight.
        uint32_t t = (w[2] ^ (w[0] >> 16)) & 0x0000FFFFu;
        w2 = w[2] ^ t;
        w0 = w[0] ^ (t << 16);
        t = (w[3] ^ (w[1] >> 16)) & 0x0000FFFFu;
        w3 = w[3] ^ t;
        w1 = w[1] ^ (t << 16);
        t = (w1 ^ (w0 >> 8)) & 0x00FF00FFu;
        w1 ^= t;
        w0 ^= (t << 8);
        t = (w3 ^ (w2 >> 8)) & 0x00FF00FFu;
        w3 ^= t;
        w2 ^= (t << 8);
        w0 ^= 0x80808080u;
        w1 ^= 0x80808080u;
        w2 ^= 0x80808080u;
        w3 ^= 0x80808080u;
      }
#pragma unroll
      for (int t = 0; t < TB; ++t) {
        const int tok = tok0 + t;
        if (tok >= m) continue;
        const int v = *reinterpret_cast<const int*>(act + ((size_t)ks * m + tok) * 4);
        acc[t][0] = __builtin_amdgcn_sdot4(v, (int)w0, acc[t][0], false);
        acc[t][1] = __builtin_amdgcn_sdot4(v, (int)w1, acc[t][1], false);
        acc[t][2] = __builtin_amdgcn_sdot4(v, (int)w2, acc[t][2], false);
        acc[t][3] = __builtin_amdgcn_sdot4(v, (int)w3, acc[t][3], false);
        if (WBITS == 4) {
          // nibble values are u = w + 8: remove 8 * sum(act) (the reference's r_sum term)
          const int s8 = 8 * __builtin_amdgcn_sdot4(v, 0x01010101, 0, false);
          acc[t][0] -= s8;
          acc[t][1] -= s8;
          acc[t][2] -= s8;
          acc[t][3] -= s8;
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < TB; ++t)
#pragma unroll
    for (int c = 0; c < 4; ++c) red[ty][tx][t * 4 + c] = acc[t][c];
  __syncthreads();
  if (ty == 0 && ds < ns) {
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      const int tok = tok0 + t;
      if (tok >= m) continue;
#pragma unroll
      for (int c = 0; c < 4; ++c)
        dst[((size_t)ds * m + tok) * 4 + c] = red[0][tx][t * 4 + c] + red[1][tx][t * 4 + c] +
                                              red[2][tx][t * 4 + c] + red[3][tx][t * 4 + c];
    }
  }
}

}  // namespace

hipError_t LaunchFcGeneric(const FcArgs& a, hipStream_t stream, const char** kernel_name) {
  GenericParams p;
  p.act = a.act;
  p.weights = a.weights;
  p.scale = a.scale;
  p.zero_point = a.zero_point;
  p.bias = a.bias;
  p.dst = a.dst;
  p.m = a.m;
  p.ks = DivUp(a.k, 4);
  p.ns = DivUp(a.n, 4);
  p.scale_kind = a.scale_kind;
  p.groups = a.groups;
  p.group_slices = a.scale_kind == kScaleBlock ? (p.ks / a.groups > 0 ? p.ks / a.groups : 1) : p.ks;
  p.scalar_scale = a.scalar_scale;
  p.scalar_zero_point = a.scalar_zero_point;
  p.has_zero_point = a.has_zero_point;
  if (kernel_name) *kernel_name = "fc_generic_kernel";
  const bool w8 = a.weight_bits == 8;
  if (a.act_f16 && a.dst_f16)
    return w8 ? LaunchGenericT<__half, __half, 8>(p, stream) : LaunchGenericT<__half, __half, 4>(p, stream);
  if (!a.act_f16 && !a.dst_f16)
    return w8 ? LaunchGenericT<float, float, 8>(p, stream) : LaunchGenericT<float, float, 4>(p, stream);
  if (a.act_f16 && !a.dst_f16)
    return w8 ? LaunchGenericT<__half, float, 8>(p, stream) : LaunchGenericT<__half, float, 4>(p, stream);
  return w8 ? LaunchGenericT<float, __half, 8>(p, stream) : LaunchGenericT<float, __half, 4>(p, stream);
}

bool FcW4StreamSupported(const FcArgs& a) {
  if (a.weight_bits != 4 || !a.act_f16 || !a.dst_f16) return false;
  if (a.m < 1 || a.m > kGemvMaxTokens) return false;
  if (a.has_zero_point) return false;
  const int ks = DivUp(a.k, 4), ns = DivUp(a.n, 4);
  if (ns % 2 != 0) return false;  // 16-byte loads need an even number of 8-byte blocks per row
  if (a.scale_kind == kScaleScalar) return false;
  if (a.scale_kind == kScaleBlock) {
    if (a.groups <= 0 || ks % a.groups != 0) return false;
    if ((ks / a.groups) % 8 != 0) return false;  // a chunk of 8 K-slices must not straddle groups
  }
  return a.partial != nullptr && a.counters != nullptr;
}

hipError_t LaunchFcW4Stream(const FcArgs& a, hipStream_t stream, const char** kernel_name) {
  StreamParams p;
  p.weights = reinterpret_cast<const u32x4*>(a.weights);
  p.act = static_cast<const __half*>(a.act);
  p.scale = static_cast<const __half*>(a.scale);
  p.bias = static_cast<const __half*>(a.bias);
  p.dst = static_cast<__half*>(a.dst);
  p.partial = a.partial;
  p.counters = a.counters;
  p.m = a.m;
  p.ks = DivUp(a.k, 4);
  p.ns = DivUp(a.n, 4);
  p.n_pad = p.ns * 4;
  p.row_u4 = p.ns / 2;
  p.chunks = DivUp(p.ks, 8);
  const bool grouped = a.scale_kind == kScaleBlock;
  p.groups = grouped ? a.groups : 1;
  p.group_chunks = grouped ? (p.ks / a.groups) / 8 : p.chunks;

  // Shape heuristic: fill the 256 CUs with >= 2 work-groups each while keeping row segments
  // of at least 256 contiguous bytes; narrower strips for small N, deeper K-splits for small N
  // with large K.
  int lpr = 64;
  if (p.row_u4 <= 1024) lpr = 32;
  if (p.row_u4 <= 256) lpr = 16;
  lpr = EnvInt("MLDHIP_GEMV_LPR", lpr);
  if (lpr != 16 && lpr != 32 && lpr != 64) lpr = 64;
  const int strips = DivUp(p.row_u4, lpr);
  const int rows = 256 / lpr;
  int ksplit = DivUp(512, strips);
  const int max_split = DivUp(p.chunks, rows);  // at least one chunk per thread row
  if (ksplit > max_split) ksplit = max_split;
  ksplit = EnvInt("MLDHIP_GEMV_KSPLIT", ksplit);
  if (ksplit > kGemvMaxKSplit) ksplit = kGemvMaxKSplit;
  if (ksplit < 1) ksplit = 1;
  if (strips > a.n_counters) ksplit = 1;
  while (ksplit > 1 && (size_t)ksplit * p.m * p.n_pad > a.partial_floats) --ksplit;
  // every thread row gets the same number of chunks
  p.chunks_per_split = DivUp(DivUp(p.chunks, ksplit), rows) * rows;
  p.ksplit = DivUp(p.chunks, p.chunks_per_split);
  dim3 grid(strips, p.ksplit);
  if (kernel_name) *kernel_name = "fc_w4_stream_kernel";
  switch (lpr) {
    case 16: return LaunchStreamL<16>(p, grouped, grid, stream);
    case 32: return LaunchStreamL<32>(p, grouped, grid, stream);
    default: return LaunchStreamL<64>(p, grouped, grid, stream);
  }
}

hipError_t LaunchFcInt8Math(const int8_t* act, const uint8_t* weights, int32_t* dst, int m, int k,
                            int n, int weight_bits, hipStream_t stream, const char** kernel_name) {
  constexpr int TB = 4;
  const int ks = DivUp(k, 4), ns = DivUp(n, 4);
  dim3 grid(DivUp(ns, 64), DivUp(m, TB));
  dim3 block(64, 4);
  if (kernel_name) *kernel_name = "fc_int8_math_kernel";
  if (weight_bits == 8)
    hipLaunchKernelGGL((fc_int8_math_kernel<8, TB>), grid, block, 0, stream, act, weights, dst, m, ks, ns);
  else
    hipLaunchKernelGGL((fc_int8_math_kernel<4, TB>), grid, block, 0, stream, act, weights, dst, m, ks, ns);
  return hipGetLastError();
}

}  // namespace mldhip
