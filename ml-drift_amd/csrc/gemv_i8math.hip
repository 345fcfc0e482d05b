// Streaming int8-math GEMV for gfx950: int8 activations x uint8 / uint4 weights -> int32, the
// FullyConnected variant the reference compiles when the source tensor is int8
// (common/kernels/fully_connected.cc:543-621 ReadWeightsAs4Uint8x4, :630, :714-716;
// fully_connected_util.cc:205-229 AccumulateUint / AdjustUintSum).  1..4 tokens.
//
// Packed buffers (I4O4): row ks (4 input channels) holds Ns blocks.  uint8: a block is 16 bytes,
// word i = input channel i, its bytes = output channels 0..3 of the slice, u = w + 128.  uint4: a
// block is 8 bytes, nibble 4*i + o of the 16 = (input i, output o), u = w + 8.
//
// The integer dot product wants the 4 input channels of ONE output in one register: the block
// is transposed in registers with byte permutes (v_perm_b32).  uint8: 8 permutes, then the top
// bit of every byte is flipped (u - 128 as a signed byte) and v_dot4_i32_i8 does the rest.
// uint4: 2 permutes gather the bytes that hold outputs (0,1) and (2,3) of the four inputs, low
// and high nibbles are split off with a mask; the codes stay unsigned (0..15) and the reference's
// correction "r -= shift * sum(act)" is applied once per thread at the end.  Integer sums are
// exact, so the order of the K reduction (rows of a work-group through LDS) does not matter.
//
// Thread layout as in the float GEMV kernels: LPR lanes cover one contiguous row segment
// (LPR x 16 B), 64/LPR rows per wave, WAVES waves per work-group; a thread owns whole chunks of
// 8 consecutive K-slices and issues its 8 weight loads back to back, unconditionally (rows past
// K re-read the last row, their activations are zeroed by a select).
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mldhip {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct I8MathParams {
  const u32x4* weights;
  const int* act;  // [Ks][m] words of 4 int8
  int* dst;        // [Ns][m][4]
  int m, ks, ns;
  int row_u4;  // 16-byte items per K-slice row
  int gu4;     // 16-byte items per row of one output group of the packed weights (row_u4: one group)
  int chunks;  // ceil(ks / 8)
  FcBatchRows batch;  // batched weights selected by runtime ids: blockIdx.z = dst row
};

__device__ __forceinline__ uint32_t Perm(uint32_t hi, uint32_t lo, uint32_t sel) {
  return __builtin_amdgcn_perm(hi, lo, sel);
}

// WBITS 8: a lane's 16 bytes are one slice (4 outputs); WBITS 4: two slices (8 outputs).
template <int WBITS, int LPR, int WAVES, int M, bool BATCHED>
__global__ __launch_bounds__(WAVES * 64) void fc_i8math_stream_kernel(I8MathParams p) {
  constexpr int THREADS = WAVES * 64;
  constexpr int ROWS = THREADS / LPR;
  constexpr int RPW = 64 / LPR;
  constexpr int OUTS = WBITS == 4 ? 8 : 4;  // outputs per lane
  constexpr int STRIP = LPR * OUTS;         // outputs per work-group
  constexpr int PARTS = THREADS / STRIP > ROWS ? ROWS : THREADS / STRIP;
  constexpr int RPP = ROWS / PARTS;
  __shared__ int red[ROWS][M][STRIP];
  __shared__ int red2[PARTS][M][STRIP];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int col = lane % LPR;
  const int row = wave * RPW + lane / LPR;
  const int item_raw = blockIdx.x * LPR + col;
  const int item = item_raw < p.row_u4 ? item_raw : p.row_u4 - 1;  // clamp: loads stay in range, result unused
  // BATCHED: this row's matrix (an id outside the batch is clamped into it), its source row (one
  // shared row is broadcast) and the token strides of the two tensors
  const int brow = BATCHED ? (int)blockIdx.z : 0;
  int wb = BATCHED ? p.batch.ids[brow] : 0;
  if (BATCHED) wb = min(max(wb, 0), p.batch.weights_batch - 1);
  // column of this lane: with output groups, the rows of a group lie one after the other
  // (batched: the matrices of an output group lie one after the other)
  const u32x4* weights = p.weights + ((size_t)(item / p.gu4) * (BATCHED ? p.batch.weights_batch : 1) + wb) * p.ks * p.gu4 +
                         item % p.gu4;
  const int act_stride = BATCHED ? p.batch.src_rows * M : M, act_tok0 = BATCHED ? min(brow, p.batch.src_rows - 1) * M : 0;
  const int dst_stride = BATCHED ? p.batch.rows * M : M, dst_tok0 = BATCHED ? brow * M : 0;

  int acc[M][OUTS], asum[M];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    asum[m] = 0;
#pragma unroll
    for (int o = 0; o < OUTS; ++o) acc[m][o] = 0;
  }

  for (int c = row; c < p.chunks; c += ROWS) {
    u32x4 w[8];
    int a[8][M];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int ks = c * 8 + j;
      const int ksc = min(ks, p.ks - 1);
      w[j] = __builtin_nontemporal_load(weights + (size_t)ksc * p.gu4);
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const int v = p.act[(size_t)ksc * act_stride + act_tok0 + m];
        a[j][m] = ks < p.ks ? v : 0;
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint32_t t[OUTS];  // per output: its 4 input-channel values, one per byte
      if (WBITS == 8) {
        const uint32_t x01 = Perm(w[j][1], w[j][0], 0x05010400u);  // i0o0 i1o0 i0o1 i1o1
        const uint32_t y01 = Perm(w[j][1], w[j][0], 0x07030602u);  // i0o2 i1o2 i0o3 i1o3
        const uint32_t x23 = Perm(w[j][3], w[j][2], 0x05010400u);
        const uint32_t y23 = Perm(w[j][3], w[j][2], 0x07030602u);
        t[0] = Perm(x23, x01, 0x05040100u) ^ 0x80808080u;
        t[1] = Perm(x23, x01, 0x07060302u) ^ 0x80808080u;
        t[2] = Perm(y23, y01, 0x05040100u) ^ 0x80808080u;
        t[3] = Perm(y23, y01, 0x07060302u) ^ 0x80808080u;
      } else {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          // bytes of a block: word 0 = (i0: o0|o1, o2|o3), (i1: ...); word 1 = i2, i3
          const uint32_t p01 = Perm(w[j][2 * b + 1], w[j][2 * b], 0x06040200u);  // (o0|o1) of i0..i3
          const uint32_t p23 = Perm(w[j][2 * b + 1], w[j][2 * b], 0x07050301u);  // (o2|o3) of i0..i3
          t[4 * b + 0] = p01 & 0x0F0F0F0Fu;
          t[4 * b + 1] = (p01 >> 4) & 0x0F0F0F0Fu;
          t[4 * b + 2] = p23 & 0x0F0F0F0Fu;
          t[4 * b + 3] = (p23 >> 4) & 0x0F0F0F0Fu;
        }
      }
#pragma unroll
      for (int m = 0; m < M; ++m) {
#pragma unroll
        for (int o = 0; o < OUTS; ++o) acc[m][o] = __builtin_amdgcn_sdot4(a[j][m], (int)t[o], acc[m][o], false);
        if (WBITS == 4) asum[m] = __builtin_amdgcn_sdot4(a[j][m], 0x01010101, asum[m], false);
      }
    }
  }
  if (WBITS == 4) {
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int o = 0; o < OUTS; ++o) acc[m][o] -= 8 * asum[m];
  }

  // K reduction through LDS: every thread stores its sums, PARTS threads per output add
  // ROWS/PARTS rows each, then one thread per output adds the PARTS results.
#pragma unroll
  for (int m = 0; m < M; ++m)
#pragma unroll
    for (int o4 = 0; o4 < OUTS / 4; ++o4)
      *reinterpret_cast<int4*>(&red[row][m][col * OUTS + o4 * 4]) =
          make_int4(acc[m][o4 * 4], acc[m][o4 * 4 + 1], acc[m][o4 * 4 + 2], acc[m][o4 * 4 + 3]);
  __syncthreads();
  const int nl = tid % STRIP;
  const int part = tid / STRIP;
  if (part < PARTS) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      int v = 0;
#pragma unroll
      for (int r = 0; r < RPP; ++r) v += red[part * RPP + r][m][nl];
      red2[part][m][nl] = v;
    }
  }
  __syncthreads();
  const int n0 = blockIdx.x * STRIP;
  for (int idx = tid; idx < M * STRIP; idx += THREADS) {
    const int m = idx / STRIP, ol = idx % STRIP;
    const int n = n0 + ol;
    if (n >= p.ns * 4) continue;
    int v = 0;
#pragma unroll
    for (int q = 0; q < PARTS; ++q) v += red2[q][m][ol];
    p.dst[((size_t)(n >> 2) * dst_stride + dst_tok0 + m) * 4 + (n & 3)] = v;
  }
}

// uint4 weights, one token, strips of 64 channels that lie inside one output group of the packed
// weights (grid x = strip of the group, y = group): 8 lanes cover a 128-byte row segment, a thread
// owns chunks of 8 consecutive K-slices (ONE: exactly one, no loop), the 8 channel sums of a lane
// are added across the 8 rows of a wave by register exchanges that halve the live values per
// step and across waves through 4 KB of LDS.  CONTIG: output groups of 16 slices, a strip's rows
// lie one after the other (128 bytes apart: immediate offsets).  Integer sums: any order is exact.
typedef unsigned u32x2s __attribute__((ext_vector_type(2)));
template <int WAVES, bool ONE, bool CONTIG>
__global__ __launch_bounds__(WAVES * 64) void fc_i8math_strip_kernel(I8MathParams p) {
  constexpr int ROWS = WAVES * 8;
  __shared__ int red[WAVES][64];
  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63, wave = tid >> 6;
  const uint32_t col = tid & 7, row = tid >> 3;
  const uint32_t row_bytes = CONTIG ? 128u : (uint32_t)p.gu4 * 16u;
  const char* gbase = reinterpret_cast<const char*>(p.weights + (size_t)blockIdx.y * p.ks * p.gu4 + (size_t)blockIdx.x * 8);
  const int4* act4 = reinterpret_cast<const int4*>(p.act);
  int acc[8], asum = 0;
#pragma unroll
  for (int o = 0; o < 8; ++o) acc[o] = 0;
  for (uint32_t c = row; ONE ? c == row : c < (uint32_t)p.chunks; c += ROWS) {
    u32x4 w[8];
    const uint32_t voff = __umul24(c * 8u, row_bytes) + col * 16u;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      w[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(gbase + voff + (CONTIG ? (uint32_t)j * 128u : __umul24((uint32_t)j, row_bytes))));
    const int4 a0 = act4[c * 2], a1 = act4[c * 2 + 1];
    const int a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    if (!ONE) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const uint32_t p01 = Perm(w[j][2 * b + 1], w[j][2 * b], 0x06040200u);  // (o0|o1) of i0..i3
        const uint32_t p23 = Perm(w[j][2 * b + 1], w[j][2 * b], 0x07050301u);  // (o2|o3) of i0..i3
        acc[4 * b + 0] = __builtin_amdgcn_sdot4(a[j], (int)(p01 & 0x0F0F0F0Fu), acc[4 * b + 0], false);
        acc[4 * b + 1] = __builtin_amdgcn_sdot4(a[j], (int)((p01 >> 4) & 0x0F0F0F0Fu), acc[4 * b + 1], false);
        acc[4 * b + 2] = __builtin_amdgcn_sdot4(a[j], (int)(p23 & 0x0F0F0F0Fu), acc[4 * b + 2], false);
        acc[4 * b + 3] = __builtin_amdgcn_sdot4(a[j], (int)((p23 >> 4) & 0x0F0F0F0Fu), acc[4 * b + 3], false);
      }
      asum = __builtin_amdgcn_sdot4(a[j], 0x01010101, asum, false);
    }
  }
#pragma unroll
  for (int o = 0; o < 8; ++o) acc[o] -= 8 * asum;
  int s4[4], s2[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const u32x2s r = __builtin_amdgcn_permlane32_swap((uint32_t)acc[i], (uint32_t)acc[i + 4], false, false);
    s4[i] = (int)(r[0] + r[1]);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const u32x2s r = __builtin_amdgcn_permlane16_swap((uint32_t)s4[i], (uint32_t)s4[i + 2], false, false);
    s2[i] = (int)(r[0] + r[1]);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
    s2[i] += (int)__builtin_amdgcn_update_dpp(0u, (uint32_t)s2[i], 0x128 /* row_ror:8 */, 0xf, 0xf, false);
  const int mine = (lane & 8) ? s2[1] : s2[0];
  red[wave][col * 8 + ((lane >> 3) & 7)] = mine;  // (lanes that hold the same channel write the same value)
  __syncthreads();
  if (tid < 64) {
    int v = 0;
#pragma unroll
    for (int q = 0; q < WAVES; ++q) v += red[q][tid];
    const uint32_t strip = blockIdx.y * ((uint32_t)p.gu4 >> 3) + blockIdx.x;
    p.dst[strip * 64u + tid] = v;
  }
}

template <int WAVES>
hipError_t LaunchStripI8(const I8MathParams& p, dim3 grid, hipStream_t stream) {
  const dim3 block(WAVES * 64);
  const bool one = p.chunks == WAVES * 8, contig = p.gu4 == 8;
#define MLD_I8STRIP(O, C) hipLaunchKernelGGL((fc_i8math_strip_kernel<WAVES, O, C>), grid, block, 0, stream, p)
  if (one) { if (contig) MLD_I8STRIP(true, true); else MLD_I8STRIP(true, false); }
  else     { if (contig) MLD_I8STRIP(false, true); else MLD_I8STRIP(false, false); }
#undef MLD_I8STRIP
  return hipGetLastError();
}

template <int WBITS, int LPR, int WAVES, bool BATCHED>
hipError_t LaunchMB(const I8MathParams& p, dim3 grid, hipStream_t stream) {
  const dim3 block(WAVES * 64);
  switch (p.m) {
    case 1: hipLaunchKernelGGL((fc_i8math_stream_kernel<WBITS, LPR, WAVES, 1, BATCHED>), grid, block, 0, stream, p); break;
    case 2: hipLaunchKernelGGL((fc_i8math_stream_kernel<WBITS, LPR, WAVES, 2, BATCHED>), grid, block, 0, stream, p); break;
    case 3: hipLaunchKernelGGL((fc_i8math_stream_kernel<WBITS, LPR, WAVES, 3, BATCHED>), grid, block, 0, stream, p); break;
    case 4: hipLaunchKernelGGL((fc_i8math_stream_kernel<WBITS, LPR, WAVES, 4, BATCHED>), grid, block, 0, stream, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}
template <int WBITS, int LPR, int WAVES>
hipError_t LaunchM(const I8MathParams& p, dim3 grid, hipStream_t stream) {
  return p.batch.ids ? LaunchMB<WBITS, LPR, WAVES, true>(p, grid, stream) : LaunchMB<WBITS, LPR, WAVES, false>(p, grid, stream);
}

template <int WBITS>
hipError_t LaunchW(const I8MathParams& p, int lpr, int waves, hipStream_t stream) {
  const dim3 grid(DivUp(p.row_u4, lpr), 1, p.batch.ids ? p.batch.rows : 1);
  if (lpr == 4) return waves == 4 ? LaunchM<WBITS, 4, 4>(p, grid, stream) : LaunchM<WBITS, 4, 16>(p, grid, stream);
  return waves == 4 ? LaunchM<WBITS, 8, 4>(p, grid, stream) : LaunchM<WBITS, 8, 16>(p, grid, stream);
}

}  // namespace

bool FcInt8MathStreamSupported(int m, int k, int n, int weight_bits) {
  if (m < 1 || m > kGemvMaxTokens) return false;
  if (weight_bits == 8) return true;
  // uint4: a lane's 16 bytes are two slices, so the rows must hold an even number of them
  return weight_bits == 4 && DivUp(n, 4) % 2 == 0;
}

hipError_t LaunchFcInt8MathStream(const int8_t* act, const uint8_t* weights, int32_t* dst, int m, int k, int n,
                                  int weight_bits, hipStream_t stream, const char** kernel_name,
                                  const FcBatchRows& batch) {
  I8MathParams p;
  p.batch = batch;
  p.weights = reinterpret_cast<const u32x4*>(weights);
  p.act = reinterpret_cast<const int*>(act);
  p.dst = dst;
  p.m = m;
  p.ks = DivUp(k, 4);
  p.ns = DivUp(n, 4);
  p.row_u4 = weight_bits == 4 ? p.ns / 2 : p.ns;
  const int group = EffectiveGroup(batch.group, p.ns);
  if (p.ns % group != 0 || (weight_bits == 4 && group % 2 != 0)) return hipErrorInvalidValue;
  p.gu4 = weight_bits == 4 ? group / 2 : group;
  p.chunks = DivUp(p.ks, 8);
  // 128-byte row segments when that still gives a work-group to half the CUs, else 64-byte ones;
  // small work-groups for several tokens (LDS) and when K is covered by few rows of chunks
  const int lpr = (long)DivUp(p.row_u4, 8) * (batch.ids ? batch.rows : 1) >= 128 ? 8 : 4;
  const int waves = (m > 1 || p.chunks <= 4 * 64 / lpr) ? 4 : 16;
  if (kernel_name) *kernel_name = "fc_i8math_stream_kernel";
  // one token over uint4 strips of 64 channels inside one output group, whole chunks of K, enough
  // strips for the chip, offsets within 24-bit factors: the strip form
  if (weight_bits == 4 && m == 1 && batch.ids == nullptr && p.gu4 % 8 == 0 && p.row_u4 % 8 == 0 && p.ks % 8 == 0 &&
      p.row_u4 / 8 >= 128 && p.ks < (1 << 20) && p.gu4 < (1 << 20) && (size_t)p.ks * p.gu4 * 16 < ((size_t)1 << 32) &&
      GetTuning().gemv_one_chunk != 0) {
    const dim3 grid(p.gu4 / 8, p.row_u4 / p.gu4);
    if (kernel_name) *kernel_name = "fc_i8math_strip_kernel";
    if (p.chunks <= 32) return LaunchStripI8<4>(p, grid, stream);
    if (p.chunks <= 64) return LaunchStripI8<8>(p, grid, stream);
    return LaunchStripI8<16>(p, grid, stream);
  }
  return weight_bits == 4 ? LaunchW<4>(p, lpr, waves, stream) : LaunchW<8>(p, lpr, waves, stream);
}

}  // namespace mldhip
