// Streaming int4 GEMV for gfx950 (decode: 1..4 tokens, fp16 tensors, symmetric weights,
// per-channel scales or group-wise scales whose groups are multiples of 32 input channels).
//
// Packed buffer (the reference's I4O4 layout): row ks (4 input channels) holds Ns blocks of
// 8 bytes; one 16-byte load covers two neighbouring blocks = 8 output channels x 4 input
// channels.  In word h (0/1) of a block, nibble j (j = 0..3) is (input 2h, output j) and
// nibble 4+j is (input 2h+1, output j).  Masking a word with 0x000F000F after a shift by 4j
// therefore leaves the pair (input 2h, input 2h+1) of output j in the two 16-bit halves:
// the operand shape of v_dot2_f32_f16 against the activation pair.  OR-ing 0x6400 turns a
// half into the fp16 number 1024+u; a nibble sitting in bits 4..7 of a half is read in place
// by OR-ing 0x5400, which gives 64+u (the mantissa's unit there is 1/16).  The constant
// offsets (1024+8 and 64+8) are not subtracted per weight: sum_k a_k (c + u_k - 8 - c) =
// sum_k a_k (c + u_k) - (c + 8) sum_k a_k, so the kernel accumulates the biased products and
// removes (c+8) * sum(a) once per chunk.
//
// Thread layout: LPR lanes cover one contiguous row segment (LPR x 16 B), 64/LPR rows per
// wave, WAVES waves per work-group.  A thread owns whole chunks of 8 consecutive K-slices
// (32 input channels, one scale group when group-wise), issues its 8 weight loads back to
// back and prefetches the next chunk while it computes.  Launch shapes are chosen so that a
// thread usually owns exactly one chunk: then every load of the problem is in flight at
// once, which is what a ~4 us kernel needs to approach HBM speed.
// K is reduced across the rows of a wave with lane shuffles, across waves through LDS, and
// (only when the strip count is too small to fill the chip) across work-groups through a
// partial-sum workspace that a second small kernel adds up in a fixed order.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <mutex>

#include "../../include/mldhip.h"
#include "gated.h"
#include "kernels.h"

namespace mldhip {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Reinterprets a 32-bit word as two halfs.  Taking the word by value matters: applying
// __builtin_bit_cast directly to a vector element reads element 0 whatever the index.
__device__ __forceinline__ half2_t AsHalf2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }

// (x & mask) | magic in one instruction.  The three-operand form reads at most one scalar
// register, so the mask stays scalar and the exponent pattern lives in a vector register.
__device__ __forceinline__ uint32_t AndOr(uint32_t x, uint32_t mask, uint32_t magic) {
  uint32_t d;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(x), "s"(mask), "v"(magic));
  return d;
}

// One weight matrix of a launch.  A launch covers up to kMaxSegments matrices that read the
// same activations (same K): work-groups [strip_end of the previous, strip_end) belong to it.
constexpr int kMaxSegments = 3;
struct StreamSegment {
  const u32x4* weights;
  const __half* scale;
  const __half* zero_point;  // same shape as scale, or null
  const __half* bias;
  __half* dst;
  int ns, n_pad;  // n_pad = ns * 4
  int row_u4;     // uint4 per packed row = ns / 2
  int gu4;        // uint4 per row of one output group of the packed weights (row_u4: one group)
  int strip_end;
  int n_off;      // channels of the launch's matrices before this one (split-K sums of fused launches)
};

struct StreamParams {
  StreamSegment seg[kMaxSegments];
  int segments;
  const __half* act;
  float* partial;  // split-K sums: [split][token][n_total]
  int n_total;     // padded channels of all matrices of the launch
  int m, ks;
  int chunks;            // ceil(ks / 8)
  int chunks_per_split;
  int ksplit;
  int group_chunks;  // chunks per scale group (grouped only)
  int groups;
  // nibble masks and fp16 exponent patterns, passed as run-time values so that the compiler
  // keeps them in registers and forms single v_and_or_b32 instructions
  uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
  // Batched weights selected by runtime ids (fully_connected.cc:654-665, 804-822;
  // fully_connected_util.cc:279-290): blockIdx.z = dst row, m tokens per row.  seg[0].weights
  // holds weights_batch matrices one after the other, scales are [group][weights_batch][Ns][4].
  const int32_t* batch_ids;
  int rows, src_rows, weights_batch;
  // Runtime channel bounds (the streaming kernel only): int32 values in device memory, read at the top
  // of the kernel; an index < 0 = not set; null = no bounds.  The K loop stops after the bounded
  // K-slices (not with group-wise scales, whose loop runs over all groups in the reference too), dst
  // slices beyond the bound are not written.
  const int32_t* rt_params;
  int src_end_idx, dst_end_idx, k_channels;
};

__device__ __forceinline__ void StoreHalf(__half* dst, size_t i, float r, const __half* bias, size_t bi) {
  __half h = __float2half_rn(r);
  if (bias) h = __hadd(h, bias[bi]);
  dst[i] = h;
}

// Branch-free: a K-slice past the end re-reads the last row of weights against zeroed
// activations, so the eight loads of a chunk are issued back to back and the waits for them can
// be counted down one by one while the arithmetic of the earlier slices runs.
// act_stride / act_tok0: tokens per K-slice row of the activation tensor and the first token of
// this launch row in it (M and 0 unless the launch has batched weights).
// wcol: the lane's column of the packed weights (K-slice row 0), rstride: uint4 per K-slice row.
// ks_live: K-slices that count (p.ks, or fewer under a runtime bound): activations from there on read as zero.
template <int M>
__device__ __forceinline__ void LoadChunk(const StreamParams& p, const u32x4* wcol, int rstride, int c,
                                          u32x4 w[8], u32x2 a[8][M], int ks_live, int act_stride = M, int act_tok0 = 0) {
  const int ks0 = c * 8;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int ks = ks0 + j;
    const int ksc = min(ks, p.ks - 1);
    w[j] = __builtin_nontemporal_load(wcol + (size_t)ksc * rstride);
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const u32x2 v = *reinterpret_cast<const u32x2*>(p.act + ((size_t)ksc * act_stride + act_tok0 + m) * 4);
      a[j][m] = u32x2{ks < ks_live ? v[0] : 0u, ks < ks_live ? v[1] : 0u};
    }
  }
}

// t[m][o] += sum over the chunk of a * (c_o + u), c_o = 1024 for even o, 64 for odd o;
// asum[m] += sum over the chunk of a.
template <int M, typename Params>
__device__ __forceinline__ void ComputeChunk(const Params& p, const u32x4 w[8], const u32x2 a[8][M],
                                             float t[M][8], float asum[M]) {
  const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    half2_t a01[M], a23[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
      a01[m] = AsHalf2(a[j][m][0]);
      a23[m] = AsHalf2(a[j][m][1]);
      asum[m] = __builtin_amdgcn_fdot2(a01[m], ones, asum[m], false);
      asum[m] = __builtin_amdgcn_fdot2(a23[m], ones, asum[m], false);
    }
#pragma unroll
    for (int h = 0; h < 4; ++h) {  // word h: inputs (2(h&1), 2(h&1)+1), outputs 4*(h>>1) .. +3
      const uint32_t lo = w[j][h];
      const uint32_t hi = lo >> 8;
      const half2_t q0 = AsHalf2(AndOr(lo, p.mask_lo, p.magic_lo));
      const half2_t q1 = AsHalf2(AndOr(lo, p.mask_hi, p.magic_hi));
      const half2_t q2 = AsHalf2(AndOr(hi, p.mask_lo, p.magic_lo));
      const half2_t q3 = AsHalf2(AndOr(hi, p.mask_hi, p.magic_hi));
      const int ob = 4 * (h >> 1);
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const half2_t av = (h & 1) ? a23[m] : a01[m];
        t[m][ob + 0] = __builtin_amdgcn_fdot2(q0, av, t[m][ob + 0], false);
        t[m][ob + 1] = __builtin_amdgcn_fdot2(q1, av, t[m][ob + 1], false);
        t[m][ob + 2] = __builtin_amdgcn_fdot2(q2, av, t[m][ob + 2], false);
        t[m][ob + 3] = __builtin_amdgcn_fdot2(q3, av, t[m][ob + 3], false);
      }
    }
  }
}

// ZP: the weights have a zero-point tensor (same shape as the scales): the centre of the codes
// moves from 8 to 8 + zp, per channel or per (group, channel).
// MULTI: the launch covers more than one matrix (the single-matrix instantiation reads its
// arguments at fixed offsets, which saves a dependent scalar load in front of the first weight
// load: 0.2 us on a 29 MB matrix).
// BATCHED: batched weights selected by runtime ids, one dst row per blockIdx.z (no K split, one
// matrix list entry).
template <int LPR, int WAVES, int M, bool GROUPED, bool ZP, bool MULTI, bool BATCHED = false>
__global__ __launch_bounds__(WAVES * 64) void fc_w4_stream_kernel(StreamParams p) {
  static_assert(!BATCHED || !MULTI, "a batched launch has one matrix list entry");
  constexpr int THREADS = WAVES * 64;
  constexpr int ROWS = THREADS / LPR;  // chunks the work-group covers per step
  constexpr int RPW = 64 / LPR;        // rows per wave
  constexpr int STRIP = LPR * 8;       // output channels per work-group
  __shared__ float red[ROWS][M][STRIP];
  __shared__ float red2[(THREADS / STRIP > 0 ? THREADS / STRIP : 1)][M][STRIP];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int col = lane % LPR;
  const int row = wave * RPW + lane / LPR;
  // which matrix of the launch this work-group belongs to, and which strip of it
  int si = 0, strip = blockIdx.x;
  if (MULTI && p.segments > 1 && strip >= p.seg[0].strip_end) {
    si = (p.segments > 2 && strip >= p.seg[1].strip_end) ? 2 : 1;
    strip -= p.seg[si - 1].strip_end;
  }
  const StreamSegment& sg = p.seg[MULTI ? si : 0];
  const int row_u4 = sg.row_u4;
  // BATCHED: this row's matrix (an id outside the batch is clamped into it), its source row
  // (one shared row is broadcast) and the token strides of the two tensors
  const int brow = BATCHED ? (int)blockIdx.z : 0;
  int wb = BATCHED ? p.batch_ids[brow] : 0;
  if (BATCHED) wb = __builtin_amdgcn_readfirstlane(min(max(wb, 0), p.weights_batch - 1));
  const u32x4* weights = sg.weights;
  const __half* scale_base = sg.scale + (BATCHED ? (size_t)wb * sg.n_pad : 0);
  const __half* zp_base = ZP ? sg.zero_point + (BATCHED ? (size_t)wb * sg.n_pad : 0) : nullptr;
  const size_t group_stride = (size_t)sg.n_pad * (BATCHED ? p.weights_batch : 1);  // elements per scale group
  const int act_stride = BATCHED ? p.src_rows * M : M, act_tok0 = BATCHED ? min(brow, p.src_rows - 1) * M : 0;
  const int dst_stride = BATCHED ? p.rows * M : M, dst_tok0 = BATCHED ? brow * M : 0;
  const int pcol_raw = strip * LPR + col;  // uint4 column = output channels 8*pcol .. +7
  const bool col_ok = pcol_raw < row_u4;
  const int pcol = col_ok ? pcol_raw : row_u4 - 1;  // clamp: loads stay in range, result unused
  // with output groups, the rows of a group lie one after the other (batched: of its matrices, one
  // after the other)
  const u32x4* wcol = weights + ((size_t)(pcol / sg.gu4) * (BATCHED ? p.weights_batch : 1) + wb) * p.ks * sg.gu4 + pcol % sg.gu4;
  const int rstride = sg.gu4;
  const int ky = blockIdx.y;
  const int c_begin = ky * p.chunks_per_split;
  // runtime channel bounds: K-slices that count, dst slices that are written
  int ks_live = p.ks, ns_live = sg.ns;
  if (p.rt_params != nullptr) {
    if (!GROUPED && p.src_end_idx >= 0) ks_live = SrcEndSlices(p.rt_params[p.src_end_idx], p.k_channels, p.ks);
    if (p.dst_end_idx >= 0) ns_live = DstEndSlice(p.rt_params[p.dst_end_idx], sg.ns);
    if (strip * (STRIP / 4) >= ns_live) return;  // (the whole work-group: no barrier is left waiting)
  }
  const int c_end = min(c_begin + p.chunks_per_split, p.rt_params != nullptr ? (ks_live + 7) / 8 : p.chunks);

  float acc[M][8];
#pragma unroll
  for (int m = 0; m < M; ++m)
#pragma unroll
    for (int o = 0; o < 8; ++o) acc[m][o] = 0.0f;

  // The per-channel scale and the bias of the output this thread writes at the end (output
  // tid % STRIP of the strip, for every token it handles): fetched now, so that their latency
  // does not follow the reduction.
  // (Unconditional loads of the raw halfs at a clamped index: a branch, or a conversion, here
  // would make the kernel wait for them before it issues the weight loads.)
  const int n_out = min(strip * STRIP + tid % STRIP, sg.n_pad - 1);
  const unsigned short* bias_src = reinterpret_cast<const unsigned short*>(sg.bias ? sg.bias : sg.scale);
  const unsigned short out_scale_raw = reinterpret_cast<const unsigned short*>(scale_base)[n_out];
  const unsigned short out_bias_raw = bias_src[n_out];

  int c = c_begin + row;
  u32x4 zv = {0u, 0u, 0u, 0u};  // zero points of this thread's 8 channels (halfs)
  if (ZP && !GROUPED) zv = *reinterpret_cast<const u32x4*>(zp_base + (size_t)2 * pcol * 4);
  if (c < c_end) {
    u32x4 w[8];
    u32x2 a[8][M];
    LoadChunk<M>(p, wcol, rstride, c, w, a, ks_live, act_stride, act_tok0);
    while (true) {
      const int cn = c + ROWS;
      const bool more = cn < c_end;
      u32x4 wn[8];
      u32x2 an[8][M];
      if (more) LoadChunk<M>(p, wcol, rstride, cn, wn, an, ks_live, act_stride, act_tok0);
      u32x4 sv;
      if (GROUPED) {
        int g = c / p.group_chunks;
        if (g >= p.groups) g = p.groups - 1;
        sv = *reinterpret_cast<const u32x4*>(scale_base + (size_t)g * group_stride + (size_t)2 * pcol * 4);
        if (ZP) zv = *reinterpret_cast<const u32x4*>(zp_base + (size_t)g * group_stride + (size_t)2 * pcol * 4);
      }
      float t[M][8], asum[M];
#pragma unroll
      for (int m = 0; m < M; ++m) {
        asum[m] = 0.0f;
#pragma unroll
        for (int o = 0; o < 8; ++o) t[m][o] = 0.0f;
      }
      ComputeChunk<M>(p, w, a, t, asum);
#pragma unroll
      for (int m = 0; m < M; ++m)
#pragma unroll
        for (int o = 0; o < 8; ++o) {
          float centre = (o & 1) ? -72.0f : -1032.0f;
          if (ZP) centre -= (float)AsHalf2(zv[o >> 1])[o & 1];
          const float centered = fmaf(centre, asum[m], t[m][o]);
          if (GROUPED) {
            const half2_t sp = AsHalf2(sv[o >> 1]);
            acc[m][o] = fmaf((float)sp[o & 1], centered, acc[m][o]);
          } else {
            acc[m][o] += centered;
          }
        }
      if (!more) break;
      c = cn;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        w[j] = wn[j];
#pragma unroll
        for (int m = 0; m < M; ++m) a[j][m] = an[j][m];
      }
    }
  }

  // K reduction inside the work-group, through LDS only: every thread stores its 8*M sums,
  // PARTS threads per output add ROWS/PARTS rows each, then one thread per output adds the
  // PARTS results.
  constexpr int PARTS = THREADS / STRIP >= 1 ? (THREADS / STRIP > ROWS ? ROWS : THREADS / STRIP) : 1;
  constexpr int RPP = ROWS / PARTS;  // rows per part
#pragma unroll
  for (int m = 0; m < M; ++m) {
    float4* dst4 = reinterpret_cast<float4*>(&red[row][m][col * 8]);
    dst4[0] = make_float4(acc[m][0], acc[m][1], acc[m][2], acc[m][3]);
    dst4[1] = make_float4(acc[m][4], acc[m][5], acc[m][6], acc[m][7]);
  }
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
  const int n0 = strip * STRIP;
  for (int idx = tid; idx < M * STRIP; idx += THREADS) {
    const int m = idx / STRIP, ol = idx % STRIP;
    const int n = n0 + ol;
    if (n >= ns_live * 4) continue;
    float v = 0.0f;
#pragma unroll
    for (int q = 0; q < PARTS; ++q) v += red2[q][m][ol];
    if (p.ksplit == 1) {
      if (!GROUPED) v *= __half2float(__ushort_as_half(out_scale_raw));
      __half h = __float2half_rn(v);
      if (sg.bias) h = __hadd(h, __ushort_as_half(out_bias_raw));
      sg.dst[((size_t)(n >> 2) * dst_stride + dst_tok0 + m) * 4 + (n & 3)] = h;
    } else {
      p.partial[((size_t)ky * M + m) * sg.n_pad + n] = v;
    }
  }
}

// Adds the split-K partial sums in split order and writes the output.  The sums of a launch are
// [split][token][channels of all its matrices]; n_total = those channels.
template <bool GROUPED>
__global__ __launch_bounds__(256) void fc_w4_reduce_kernel(StreamParams p, int n_total) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.m * n_total) return;
  const int m = idx / n_total, nt = idx % n_total;
  int si = 0;
  if (p.segments > 1 && nt >= p.seg[1].n_off) si = (p.segments > 2 && nt >= p.seg[2].n_off) ? 2 : 1;
  const StreamSegment& sg = p.seg[si];
  const int n = nt - sg.n_off;
  if (p.rt_params != nullptr && p.dst_end_idx >= 0 && (n >> 2) >= DstEndSlice(p.rt_params[p.dst_end_idx], sg.ns)) return;
  // The parts are fetched eight at a time before any is added (a part past the last re-reads the
  // last one and is dropped by a select), so that their latencies overlap; added in split order.
  const float scale = GROUPED ? 1.0f : __half2float(sg.scale[n]);
  float v = 0.0f;
  for (int s0 = 0; s0 < p.ksplit; s0 += 8) {
    float part[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      part[j] = p.partial[((size_t)min(s0 + j, p.ksplit - 1) * p.m + m) * n_total + nt];
#pragma unroll
    for (int j = 0; j < 8; ++j) v += s0 + j < p.ksplit ? part[j] : 0.0f;
  }
  v *= scale;
  StoreHalf(sg.dst, ((size_t)(n >> 2) * p.m + m) * 4 + (n & 3), v, sg.bias, (size_t)n);
}

// ------------------------------------------------------------------------------------------
// Gated pair: dst = activation(gate(x)) * up(x), the MLP step that follows the gate and up
// projections in the decoder layers of the LLM sample (samples/llm/gemma3_model_builder.cc:
// 1054-1090 CreateGeluTanhMulOp, samples/llm/qwen3_model_builder.cc:850-883 CreateSiluMulOp).
// The two projections run as in the kernel above, in one work-group per strip (seg[0] = gate,
// seg[1] = up, same shape); their sums are rounded to fp16 (+ bias) exactly as the two separate
// FullyConnected nodes would store them, then combined in fp32 in the operation order of the
// sample's elementwise kernel.  Only seg[0].dst is written.
// ------------------------------------------------------------------------------------------
template <int LPR, int WAVES, int M, bool GROUPED>
__global__ __launch_bounds__(WAVES * 64) void fc_w4_gated_stream_kernel(StreamParams p, int activation) {
  constexpr int THREADS = WAVES * 64;
  constexpr int ROWS = THREADS / LPR;
  constexpr int RPW = 64 / LPR;
  constexpr int STRIP = LPR * 8;
  constexpr int PARTS = THREADS / STRIP > ROWS ? ROWS : THREADS / STRIP;
  constexpr int RPP = ROWS / PARTS;
  __shared__ float red[ROWS][2 * M][STRIP];
  __shared__ float red2[PARTS][2 * M][STRIP];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int col = lane % LPR;
  const int row = wave * RPW + lane / LPR;
  const int strip = blockIdx.x;
  const int row_u4 = p.seg[0].row_u4;
  const int pcol_raw = strip * LPR + col;
  const int pcol = pcol_raw < row_u4 ? pcol_raw : row_u4 - 1;  // clamp: loads stay in range, result unused
  const int rstride = p.seg[0].gu4;
  const size_t wcol_off = (size_t)(pcol / rstride) * p.ks * rstride + pcol % rstride;

  // scales / biases of the output this thread finishes, fetched ahead (raw halfs, clamped index)
  const int n_out = min(strip * STRIP + tid % STRIP, p.seg[0].n_pad - 1);
  unsigned short scale_raw[2], bias_raw[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const unsigned short* bias_src = reinterpret_cast<const unsigned short*>(p.seg[q].bias ? p.seg[q].bias : p.seg[q].scale);
    scale_raw[q] = reinterpret_cast<const unsigned short*>(p.seg[q].scale)[n_out];
    bias_raw[q] = bias_src[n_out];
  }

  float acc[2][M][8];
#pragma unroll
  for (int q = 0; q < 2; ++q)
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int o = 0; o < 8; ++o) acc[q][m][o] = 0.0f;

  for (int c = row; c < p.chunks; c += ROWS) {
    u32x4 w[2][8];
    u32x2 a[8][M];
    LoadChunk<M>(p, p.seg[0].weights + wcol_off, rstride, c, w[0], a, p.ks);
    {
      const int ks0 = c * 8;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        w[1][j] = __builtin_nontemporal_load(p.seg[1].weights + wcol_off + (size_t)min(ks0 + j, p.ks - 1) * rstride);
    }
    u32x4 sv[2];
    if (GROUPED) {
      int g = c / p.group_chunks;
      if (g >= p.groups) g = p.groups - 1;
#pragma unroll
      for (int q = 0; q < 2; ++q)
        sv[q] = *reinterpret_cast<const u32x4*>(p.seg[q].scale + ((size_t)g * p.seg[q].ns + 2 * pcol) * 4);
    }
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      float t[M][8], asum[M];
#pragma unroll
      for (int m = 0; m < M; ++m) {
        asum[m] = 0.0f;
#pragma unroll
        for (int o = 0; o < 8; ++o) t[m][o] = 0.0f;
      }
      ComputeChunk<M>(p, w[q], a, t, asum);
#pragma unroll
      for (int m = 0; m < M; ++m)
#pragma unroll
        for (int o = 0; o < 8; ++o) {
          const float centered = fmaf((o & 1) ? -72.0f : -1032.0f, asum[m], t[m][o]);
          if (GROUPED) {
            const half2_t sp = AsHalf2(sv[q][o >> 1]);
            acc[q][m][o] = fmaf((float)sp[o & 1], centered, acc[q][m][o]);
          } else {
            acc[q][m][o] += centered;
          }
        }
    }
  }

#pragma unroll
  for (int q = 0; q < 2; ++q)
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float4* dst4 = reinterpret_cast<float4*>(&red[row][q * M + m][col * 8]);
      dst4[0] = make_float4(acc[q][m][0], acc[q][m][1], acc[q][m][2], acc[q][m][3]);
      dst4[1] = make_float4(acc[q][m][4], acc[q][m][5], acc[q][m][6], acc[q][m][7]);
    }
  __syncthreads();
  const int nl = tid % STRIP;
  const int part = tid / STRIP;
  if (part < PARTS) {
#pragma unroll
    for (int qm = 0; qm < 2 * M; ++qm) {
      float v = 0.0f;
#pragma unroll
      for (int r = 0; r < RPP; ++r) v += red[part * RPP + r][qm][nl];
      red2[part][qm][nl] = v;
    }
  }
  __syncthreads();
  const int n0 = strip * STRIP;
  for (int idx = tid; idx < M * STRIP; idx += THREADS) {
    const int m = idx / STRIP, ol = idx % STRIP;
    const int n = n0 + ol;
    if (n >= p.seg[0].n_pad) continue;
    float gu[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      float v = 0.0f;
#pragma unroll
      for (int k = 0; k < PARTS; ++k) v += red2[k][q * M + m][ol];
      if (!GROUPED) v *= __half2float(__ushort_as_half(scale_raw[q]));
      __half h = __float2half_rn(v);
      if (p.seg[q].bias) h = __hadd(h, __ushort_as_half(bias_raw[q]));
      gu[q] = __half2float(h);
    }
    p.seg[0].dst[((size_t)(n >> 2) * M + m) * 4 + (n & 3)] = __float2half_rn(GatedActivation(activation, gu[0], gu[1]));
  }
}

template <int LPR, int WAVES>
hipError_t LaunchGatedM(const StreamParams& p, bool grouped, int activation, dim3 grid, hipStream_t stream) {
  const dim3 block(WAVES * 64);
#define MLD_GATED(MM)                                                                                             \
  if (grouped)                                                                                                    \
    hipLaunchKernelGGL((fc_w4_gated_stream_kernel<LPR, WAVES, MM, true>), grid, block, 0, stream, p, activation); \
  else                                                                                                            \
    hipLaunchKernelGGL((fc_w4_gated_stream_kernel<LPR, WAVES, MM, false>), grid, block, 0, stream, p, activation);
  switch (p.m) {
    case 1: MLD_GATED(1) break;
    case 2: MLD_GATED(2) break;
    default: return hipErrorInvalidValue;
  }
#undef MLD_GATED
  return hipGetLastError();
}

template <int LPR, int WAVES, int M, bool GROUPED, bool ZP>
hipError_t LaunchCfgS(const StreamParams& p, dim3 grid, hipStream_t stream) {
  if (p.segments > 1)
    hipLaunchKernelGGL((fc_w4_stream_kernel<LPR, WAVES, M, GROUPED, ZP, true>), grid, dim3(WAVES * 64), 0, stream, p);
  else
    hipLaunchKernelGGL((fc_w4_stream_kernel<LPR, WAVES, M, GROUPED, ZP, false>), grid, dim3(WAVES * 64), 0, stream, p);
  return hipGetLastError();
}

template <int LPR, int WAVES, int M>
hipError_t LaunchCfg(const StreamParams& p, bool grouped, dim3 grid, hipStream_t stream) {
  const bool zp = p.seg[0].zero_point != nullptr;
  if (grouped && zp) return LaunchCfgS<LPR, WAVES, M, true, true>(p, grid, stream);
  if (grouped) return LaunchCfgS<LPR, WAVES, M, true, false>(p, grid, stream);
  if (zp) return LaunchCfgS<LPR, WAVES, M, false, true>(p, grid, stream);
  return LaunchCfgS<LPR, WAVES, M, false, false>(p, grid, stream);
}

template <int LPR, int WAVES>
hipError_t LaunchCfgM(const StreamParams& p, bool grouped, dim3 grid, hipStream_t stream) {
  switch (p.m) {
    case 1: return LaunchCfg<LPR, WAVES, 1>(p, grouped, grid, stream);
    case 2: return LaunchCfg<LPR, WAVES, 2>(p, grouped, grid, stream);
    case 3: return LaunchCfg<LPR, WAVES, 3>(p, grouped, grid, stream);
    case 4: return LaunchCfg<LPR, WAVES, 4>(p, grouped, grid, stream);
    default: return hipErrorInvalidValue;
  }
}

// The compiled launch shapes (lanes per row segment, waves): narrow strips come with small
// work-groups, 256-byte segments with the largest.
hipError_t LaunchShape(const StreamParams& p, int lpr, int waves, bool grouped, dim3 grid, hipStream_t stream) {
  if (lpr == 2) return LaunchCfgM<2, 4>(p, grouped, grid, stream);
  if (lpr == 4) return LaunchCfgM<4, 4>(p, grouped, grid, stream);
  if (lpr == 16) return LaunchCfgM<16, 16>(p, grouped, grid, stream);
  if (waves == 4) return LaunchCfgM<8, 4>(p, grouped, grid, stream);
  if (waves == 8) return LaunchCfgM<8, 8>(p, grouped, grid, stream);
  return LaunchCfgM<8, 16>(p, grouped, grid, stream);
}

// Batched weights: two launch shapes (128-byte row segments with 8 waves, 64-byte ones with 4).
template <int LPR, int WAVES, int M>
hipError_t LaunchBatchedCfg(const StreamParams& p, bool grouped, dim3 grid, hipStream_t stream) {
  const bool zp = p.seg[0].zero_point != nullptr;
  const dim3 block(WAVES * 64);
  if (grouped && zp)
    hipLaunchKernelGGL((fc_w4_stream_kernel<LPR, WAVES, M, true, true, false, true>), grid, block, 0, stream, p);
  else if (grouped)
    hipLaunchKernelGGL((fc_w4_stream_kernel<LPR, WAVES, M, true, false, false, true>), grid, block, 0, stream, p);
  else if (zp)
    hipLaunchKernelGGL((fc_w4_stream_kernel<LPR, WAVES, M, false, true, false, true>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((fc_w4_stream_kernel<LPR, WAVES, M, false, false, false, true>), grid, block, 0, stream, p);
  return hipGetLastError();
}
template <int LPR, int WAVES>
hipError_t LaunchBatchedM(const StreamParams& p, bool grouped, dim3 grid, hipStream_t stream) {
  switch (p.m) {
    case 1: return LaunchBatchedCfg<LPR, WAVES, 1>(p, grouped, grid, stream);
    case 2: return LaunchBatchedCfg<LPR, WAVES, 2>(p, grouped, grid, stream);
    case 3: return LaunchBatchedCfg<LPR, WAVES, 3>(p, grouped, grid, stream);
    case 4: return LaunchBatchedCfg<LPR, WAVES, 4>(p, grouped, grid, stream);
    default: return hipErrorInvalidValue;
  }
}

// ------------------------------------------------------------------------------------------
// One token over weights packed in output groups of 16 slices (64 channels): the share of a
// work-group, 64 channels x its range of K, is one contiguous run of 128-byte rows, which HBM
// delivers at the rate of a plain copy.  Lane = (column of 16 bytes, row): a thread owns 8
// consecutive K-slices (one 32-channel scale group), its 8 loads are one base address plus
// immediate offsets, the 8 slices of its activations are 64 contiguous bytes.  Nothing in front of
// the loads but the address: the kernel's time is the stream's, and every instruction ahead of
// the first load delays all of it.
// K reduction: inside a wave by register exchanges that halve the live values per step (the two
// row halves with v_permlane32_swap, the 16-lane rows with v_permlane16_swap, the 8-lane halves
// of a row with a DPP rotate), after which lane l holds channel (l % 8) * 8 + l / 8 of the
// strip; across waves through 4 KB of LDS, fixed order.
// ------------------------------------------------------------------------------------------
typedef uint32_t u32x2s __attribute__((ext_vector_type(2)));

// LPR lanes (16 bytes each) cover a row; a wave holds 64 / LPR rows.  Sum over the rows of a wave
// of the 8 channel sums of every lane; the result of channel (lane % LPR) * 8 + (lane / 8) % 8 is
// returned in this lane (lanes that differ only in the bits between LPR and 8 hold the same
// sums).  All 64 lanes must be active.
// v + the value of the lane that differs in one bit of the lane number, as data-parallel moves
// inside the rows of 16 lanes (no trip through the LDS crossbar): bits 0 and 1 are quad
// permutations, bit 2 a shift by 4 lanes in either direction, each for the banks it is valid in.
__device__ __forceinline__ float AddLaneXor1(float v) {
  return v + __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0xB1 /* quad_perm:[1,0,3,2] */, 0xf, 0xf, false));
}
__device__ __forceinline__ float AddLaneXor2(float v) {
  return v + __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x4E /* quad_perm:[2,3,0,1] */, 0xf, 0xf, false));
}
__device__ __forceinline__ float AddLaneXor4(float v) {
  const uint32_t up = __builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x104 /* row_shl:4 */, 0xf, 0x5, false);
  const uint32_t both = __builtin_amdgcn_update_dpp(up, __float_as_uint(v), 0x114 /* row_shr:4 */, 0xf, 0xA, false);
  return v + __uint_as_float(both);
}

template <int LPR>
__device__ __forceinline__ float WaveStripSum(const float acc[8], int lane) {
  float s4[4], s2[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const u32x2s r = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[i]), __float_as_uint(acc[i + 4]), false, false);
    s4[i] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const u32x2s r = __builtin_amdgcn_permlane16_swap(__float_as_uint(s4[i]), __float_as_uint(s4[i + 2]), false, false);
    s2[i] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
    s2[i] += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(s2[i]), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
  float v = (lane & 8) ? s2[1] : s2[0];
  // narrower rows: the lanes 4 (and 2) apart hold further rows of the same channels
  if (LPR <= 4) v = AddLaneXor4(v);
  if (LPR <= 2) v = AddLaneXor2(v);
  if (LPR <= 1) v = AddLaneXor1(v);
  return v;
}

// Launch parameters of the strip kernel: what a single-matrix launch reads sits in the first
// 128 bytes, so that two scalar loads issued at the top of the kernel bring all of it.
struct StripSegment {
  const u32x4* weights;
  const __half* scale;
  const __half* zero_point;  // same shape as scale, or null
  const __half* bias;
  __half* dst;
  int n_pad;      // channels of the matrix (a multiple of 64)
  int strip_end;  // work-groups [strip_end of the previous, strip_end) belong to this matrix
  int n_off;      // channels of the launch's matrices before this one (split-K sums)
  int row_u4;     // STRIDED only: 16-byte items between two K-slice rows of a strip (one output group over all slices)
};
struct StripParams {
  const __half* act;
  float* partial;  // split-K sums: [split][n_total]
  int ks, chunks, chunks_per_split, ksplit;
  int group_chunks, n_total, segments, reserved;
  uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
  StripSegment seg[kMaxSegments];
  // batched weights selected by runtime ids (BATCHED instantiations only): dst row blockIdx.z
  const int32_t* batch_ids;
  int rows, src_rows, weights_batch;
};

// The matrix a work-group belongs to and its strip number inside it.  Every field of every list
// entry sits at a fixed offset of the kernel arguments, so all of them are fetched by the scalar
// loads at the top of the kernel and chosen with scalar selects; indexing the list with a run-time
// number would make the entry's loads wait for a first round trip (the strip ends).
template <bool MULTI>
__device__ __forceinline__ StripSegment SelectSegment(const StripParams& p, int& strip) {
  StripSegment sg = p.seg[0];
  if (MULTI) {
    const int e0 = p.seg[0].strip_end, e1 = p.seg[1].strip_end;
    const bool second = p.segments > 1 && strip >= e0;
    const bool third = p.segments > 2 && strip >= e1;
    const StripSegment s1 = p.seg[1], s2 = p.seg[2];
    // (an input-only operand keeps the pointers' address space; it makes the compiler fetch the
    // entries with the first batch of scalar loads instead of behind the first wait)
    asm volatile("" : : "s"(s1.weights), "s"(s2.weights), "s"(s1.scale), "s"(s2.scale), "s"(sg.weights), "s"(sg.scale));
#define MLD_PICK(f) sg.f = third ? s2.f : (second ? s1.f : sg.f)
    MLD_PICK(weights); MLD_PICK(scale); MLD_PICK(zero_point); MLD_PICK(bias); MLD_PICK(dst);
    MLD_PICK(n_pad); MLD_PICK(n_off); MLD_PICK(row_u4);
#undef MLD_PICK
    strip -= third ? e1 : (second ? e0 : 0);
  }
  return sg;
}

// BATCHED: batched weights selected by runtime ids, one dst row of one token per blockIdx.z (no K
// split, one matrix list entry): the strip of matrix b is the b-th of its output group's runs,
// scales are [group][matrix][channel], the token of source row r is every src_rows-th 8 bytes.
// ONE: every thread owns exactly one chunk and K is not split across work-groups (the launch shape
// of the wide layers: c.f. the launcher).  The kernel then has no chunk loop, no test for a first
// chunk and no split-K branch, the lane's byte offsets are 32-bit values over scalar bases, and
// the compiler is left to order loads and arithmetic (it defers the last weight loads behind the
// first rows' arithmetic).  At a launch of a few microseconds every instruction in front of the
// first load and behind the last one counts: 4 waves per SIMD issue them one after the other.
// STRIDED (with ONE): the weights are packed in one output group over all slices (the reference's
// own layout): the 128-byte rows of a strip lie a whole K-slice row of the matrix apart.
template <int LPR, int WAVES, bool GROUPED, bool ZP, bool MULTI, bool BATCHED = false, bool ONE = false, bool STRIDED = false>
__global__ __launch_bounds__(WAVES * 64) void fc_w4_strip_kernel(StripParams p) {
  static_assert(!BATCHED || !MULTI, "a batched launch has one matrix list entry");
  static_assert(!ONE || (!BATCHED && !ZP), "the one-chunk form serves plain launches");
  static_assert(!STRIDED || ONE, "strided strips are served by the one-chunk form");
  constexpr int ROWS = WAVES * 64 / LPR;  // chunks of 8 K-slices the work-group covers per pass
  constexpr int STRIP = LPR * 8;          // channels of a strip (one output group of the layout)
  __shared__ float red[WAVES][STRIP];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int col = lane % LPR;
  const int row = tid / LPR;
  int strip = blockIdx.x;
  const StripSegment sg = SelectSegment<MULTI>(p, strip);
  // Everything the loop reads from the arguments, fetched here in one go: a scalar load first
  // issued inside the loop would be a second round trip in front of the weight loads.
  struct { uint32_t mask_lo, mask_hi, magic_lo, magic_hi; } up = {p.mask_lo, p.mask_hi, p.magic_lo, p.magic_hi};
  const u32x4* weights = sg.weights;
  const u32x4* astrip = reinterpret_cast<const u32x4*>(p.act);  // chunk c: 4 uint4 (8 slices x 4 halfs)
  // (input-only operands: the pointers keep their address space, and their scalar loads join the
  // first batch instead of being issued where the pointer is first used)
  asm volatile("" : : "s"(p.act), "s"(sg.dst), "s"(sg.bias), "s"(sg.scale));
  int ks = p.ks, group_chunks = p.group_chunks, n_pad = sg.n_pad;
  asm volatile("" : "+s"(up.mask_lo), "+s"(up.mask_hi), "+s"(ks), "+s"(group_chunks), "+s"(n_pad));
  // BATCHED: this row's matrix (an id outside the batch is clamped into it) and its source row (one
  // shared row is broadcast)
  const int brow = BATCHED ? (int)blockIdx.z : 0;
  int wb = 0, nb = 1, src_rows = 1, arow = 0;
  if (BATCHED) {
    nb = p.weights_batch;
    src_rows = p.src_rows;
    wb = __builtin_amdgcn_readfirstlane(min(max(p.batch_ids[brow], 0), nb - 1));
    arow = min(brow, src_rows - 1);
  }
  const u32x2* arows = reinterpret_cast<const u32x2*>(p.act) + arow;  // BATCHED: K-slice s of the row at s * src_rows
  const __half* scale = sg.scale + (size_t)wb * n_pad;
  const __half* zero_point = ZP ? sg.zero_point + (size_t)wb * n_pad : nullptr;
  const size_t group_stride = (size_t)n_pad * nb;  // elements per scale group
  // (the pointers are left to the compiler: through an asm operand they would lose their address
  // space and turn every load into a flat one)
  const int ky = ONE ? 0 : (int)blockIdx.y;
  const int c_begin = ONE ? 0 : ky * p.chunks_per_split;
  const int c_end = ONE ? ROWS : min(c_begin + p.chunks_per_split, p.chunks);
  // the output this thread finishes: channel `ch` of the strip (the channel the wave sum leaves in
  // this lane when the work-group is one wave, else thread order)
  const int ch_wave = col * 8 + ((lane >> 3) & 7);  // the channel whose wave sum this lane holds
  const int ch = WAVES == 1 ? ch_wave : (tid % STRIP);
  const int n_out = strip * STRIP + ch;
  const unsigned short* bias_src = reinterpret_cast<const unsigned short*>(sg.bias ? sg.bias : sg.scale);

  float acc[8];
#pragma unroll
  for (int o = 0; o < 8; ++o) acc[o] = 0.0f;
  u32x4 zv = {0u, 0u, 0u, 0u};
  // row r of the strip: LPR uint4; chunk c: 8 rows
  const u32x4* wstrip = STRIDED ? weights + (size_t)strip * LPR : weights + ((size_t)strip * nb + wb) * ks * LPR + (ONE ? 0 : col);
  const uint32_t row_items = STRIDED ? (uint32_t)sg.row_u4 : (uint32_t)LPR;  // 16-byte items from one K-slice row to the next
  // Loads of one chunk, in the order the memory pipeline returns them (loads return in order): the
  // small ones that come from cache first (activations, group scales), then the eight weight loads
  // back to back.
  u32x4 w[8], a4[4], sv;
  u32x2 ab[8];
  auto issue = [&](int c) {
    const u32x4* wp = wstrip + (size_t)c * (8 * LPR);
    if (ONE) {  // c = row: byte offsets of the lane in 32 bits, the strip's base is scalar
      const uint32_t voff = (__umul24((uint32_t)row * 8u, row_items) + (uint32_t)col) * 16u;
      wp = reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(wstrip) + voff);
      const u32x4* ap = reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(p.act) + (uint32_t)row * 64u);
#pragma unroll
      for (int j = 0; j < 4; ++j) a4[j] = ap[j];
    } else if (BATCHED) {
#pragma unroll
      for (int j = 0; j < 8; ++j) ab[j] = arows[(size_t)(c * 8 + j) * src_rows];
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) a4[j] = astrip[c * 4 + j];
    }
    if (GROUPED) {
      const int g = c / group_chunks;
      const size_t so = (size_t)g * group_stride + (size_t)strip * STRIP + col * 8;
      sv = *reinterpret_cast<const u32x4*>(scale + so);
      if (ZP) zv = *reinterpret_cast<const u32x4*>(zero_point + so);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) w[j] = __builtin_nontemporal_load(wp + (STRIDED ? (size_t)j * row_items : (size_t)j * LPR));
  };
  auto consume = [&]() {
    u32x2 a[8][1];
#pragma unroll
    for (int j = 0; j < 8; ++j) a[j][0] = BATCHED ? ab[j] : u32x2{a4[j >> 1][2 * (j & 1)], a4[j >> 1][2 * (j & 1) + 1]};
    float t[1][8], asum[1] = {0.0f};
#pragma unroll
    for (int o = 0; o < 8; ++o) t[0][o] = 0.0f;
    ComputeChunk<1>(up, w, a, t, asum);
#pragma unroll
    for (int o = 0; o < 8; ++o) {
      float centre = (o & 1) ? -72.0f : -1032.0f;
      if (ZP) centre -= (float)AsHalf2(zv[o >> 1])[o & 1];
      const float centered = fmaf(centre, asum[0], t[0][o]);
      if (GROUPED) {
        const half2_t sp = AsHalf2(sv[o >> 1]);
        acc[o] = ONE ? (float)sp[o & 1] * centered : fmaf((float)sp[o & 1], centered, acc[o]);
      } else {
        acc[o] = ONE ? centered : acc[o] + centered;
      }
    }
  };
  // First chunk (the only one in the launch shapes that give every thread one chunk).  The scale
  // and bias of the output this thread finishes are fetched behind its weight loads: in front of
  // them, their trip to memory would hold back the use of every weight that arrives before they do.
  int c = c_begin + row;
  const bool first = ONE ? true : c < c_end;
  if (ZP && !GROUPED) zv = *reinterpret_cast<const u32x4*>(zero_point + (size_t)strip * STRIP + col * 8);
  if (first) issue(c);
  const unsigned short out_scale_raw = reinterpret_cast<const unsigned short*>(scale)[n_out];
  const unsigned short out_bias_raw = bias_src[n_out];
  // the fence keeps the arithmetic behind all the loads, so that the waits count the weight loads
  // down one by one instead of some of them being issued after the first wait
  if (!ONE) __builtin_amdgcn_sched_barrier(0);
  if (first) {
    consume();
    if (!ONE) {
      for (c += ROWS; c < c_end; c += ROWS) {
        issue(c);
        __builtin_amdgcn_sched_barrier(0);
        consume();
      }
    }
  }
  float v = WaveStripSum<LPR>(acc, lane);
  if (WAVES > 1) {
    red[wave][ch_wave] = v;  // (lanes that hold the same channel write the same value)
    __syncthreads();
    if (tid >= STRIP) return;
    v = 0.0f;
#pragma unroll
    for (int q = 0; q < WAVES; ++q) v += red[q][tid];
  }
  if (ONE || p.ksplit == 1) {
    if (!GROUPED) v *= __half2float(__ushort_as_half(out_scale_raw));
    __half h = __float2half_rn(v);
    if (sg.bias) h = __hadd(h, __ushort_as_half(out_bias_raw));
    if (BATCHED)
      sg.dst[((size_t)(n_out >> 2) * p.rows + brow) * 4 + (n_out & 3)] = h;
    else
      sg.dst[n_out] = h;
  } else {
    p.partial[(size_t)ky * p.n_total + sg.n_off + n_out] = v;
  }
}

// Second pass of a K-split strip launch: one 64-thread work-group per 64 channels, numbered like
// the strips of the first pass.  Work-groups go round-robin to the 8 XCDs, so with a strip count
// that is a multiple of 8 the sums of a strip are added on the XCD whose L2 they were written
// through.  Added in split order (fixed), up to 8 sums in flight at a time.
template <bool GROUPED>
__global__ __launch_bounds__(64) void fc_w4_strip_reduce_kernel(StripParams p) {
  const int nt = blockIdx.x * 64 + threadIdx.x;
  if (nt >= p.n_total) return;
  int si = 0;
  if (p.segments > 1 && nt >= p.seg[1].n_off) si = (p.segments > 2 && nt >= p.seg[2].n_off) ? 2 : 1;
  const StripSegment& sg = p.seg[si];
  const int n = nt - sg.n_off;
  const unsigned short* bias_src = reinterpret_cast<const unsigned short*>(sg.bias ? sg.bias : sg.scale);
  const unsigned short scale_raw = reinterpret_cast<const unsigned short*>(sg.scale)[n];
  const unsigned short bias_raw = bias_src[n];
  float v = 0.0f;
  for (int s0 = 0; s0 < p.ksplit; s0 += 8) {
    float part[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) part[j] = p.partial[(size_t)min(s0 + j, p.ksplit - 1) * p.n_total + nt];
#pragma unroll
    for (int j = 0; j < 8; ++j) v += s0 + j < p.ksplit ? part[j] : 0.0f;
  }
  if (!GROUPED) v *= __half2float(__ushort_as_half(scale_raw));
  __half h = __float2half_rn(v);
  if (sg.bias) h = __hadd(h, __ushort_as_half(bias_raw));
  sg.dst[n] = h;
}

template <int LPR, int WAVES>
hipError_t LaunchStripW(const StripParams& p, bool grouped, bool strided, dim3 grid, hipStream_t stream) {
  const bool zp = p.seg[0].zero_point != nullptr, multi = p.segments > 1;
  const dim3 block(WAVES * 64);
  if (p.batch_ids != nullptr) {  // batched weights: strips of 64 channels only
    if constexpr (LPR == 8) {
#define MLD_STRIP_B(G, Z) hipLaunchKernelGGL((fc_w4_strip_kernel<LPR, WAVES, G, Z, false, true>), grid, block, 0, stream, p)
      if (grouped) { if (zp) MLD_STRIP_B(true, true); else MLD_STRIP_B(true, false); }
      else         { if (zp) MLD_STRIP_B(false, true); else MLD_STRIP_B(false, false); }
#undef MLD_STRIP_B
      return hipGetLastError();
    }
    return hipErrorInvalidValue;
  }
  // every thread exactly one chunk, K inside the work-group: the one-chunk form (strips of 64 channels)
  if constexpr (LPR == 8) {
    if (!zp && p.ksplit == 1 && p.chunks == WAVES * 64 / LPR && GetTuning().gemv_one_chunk != 0) {
#define MLD_STRIP_1(G, MU, ST) hipLaunchKernelGGL((fc_w4_strip_kernel<LPR, WAVES, G, false, MU, false, true, ST>), grid, block, 0, stream, p)
      if (strided) {
        if (grouped) { if (multi) MLD_STRIP_1(true, true, true); else MLD_STRIP_1(true, false, true); }
        else         { if (multi) MLD_STRIP_1(false, true, true); else MLD_STRIP_1(false, false, true); }
      } else {
        if (grouped) { if (multi) MLD_STRIP_1(true, true, false); else MLD_STRIP_1(true, false, false); }
        else         { if (multi) MLD_STRIP_1(false, true, false); else MLD_STRIP_1(false, false, false); }
      }
#undef MLD_STRIP_1
      return hipGetLastError();
    }
  }
  if (strided) return hipErrorInvalidValue;  // (the launcher offers strided strips to the one-chunk form only)
#define MLD_STRIP(G, Z, MU) hipLaunchKernelGGL((fc_w4_strip_kernel<LPR, WAVES, G, Z, MU>), grid, block, 0, stream, p)
  if (grouped) {
    if (zp) { if (multi) MLD_STRIP(true, true, true); else MLD_STRIP(true, true, false); }
    else    { if (multi) MLD_STRIP(true, false, true); else MLD_STRIP(true, false, false); }
  } else {
    if (zp) { if (multi) MLD_STRIP(false, true, true); else MLD_STRIP(false, true, false); }
    else    { if (multi) MLD_STRIP(false, false, true); else MLD_STRIP(false, false, false); }
  }
#undef MLD_STRIP
  return hipGetLastError();
}

template <int LPR>
hipError_t LaunchStripL(const StripParams& p, int waves, bool grouped, bool strided, dim3 grid, hipStream_t stream) {
  switch (waves) {
    case 1: return LaunchStripW<LPR, 1>(p, grouped, strided, grid, stream);
    case 2: return LaunchStripW<LPR, 2>(p, grouped, strided, grid, stream);
    case 4: return LaunchStripW<LPR, 4>(p, grouped, strided, grid, stream);
    case 8: return LaunchStripW<LPR, 8>(p, grouped, strided, grid, stream);
    default: return LaunchStripW<LPR, 16>(p, grouped, strided, grid, stream);
  }
}

// The contiguous-strip kernel serves: one token, every matrix of the launch packed in output
// groups of the same size (16, 8 or 4 slices), K a multiple of 32 channels (whole chunks).
bool StripKernelServes(const FcArgs* args, int count) {
  if (GetTuning().gemv_fast == 0) return false;
  if (args[0].params != nullptr) return false;  // runtime channel bounds: the streaming kernel
  if (args[0].m != 1) return false;
  if (DivUp(args[0].k, 4) % 8 != 0 || args[0].k % 4 != 0) return false;
  const int group = EffectiveGroup(args[0].group, DivUp(args[0].n, 4));
  if (!IsNativeGroup(group)) return false;
  // batched weights: one matrix list entry, strips of 64 channels
  if (args[0].batch_ids != nullptr && (count != 1 || group != kNativeGroup)) return false;
  for (int i = 0; i < count; ++i) {
    const int ns = DivUp(args[i].n, 4);
    if (args[i].n % 4 != 0 || ns % group != 0 || EffectiveGroup(args[i].group, ns) != group) return false;
  }
  return true;
}

// One output group over all slices (the reference's own layout) is served by the one-chunk form of
// the strip kernel, with strided rows: one token, whole strips of 64 channels, every thread exactly
// one chunk (K = 256 ... 4096 channels), no zero points, strips enough to keep K inside the
// work-groups.
bool StridedStripKernelServes(const FcArgs* args, int count) {
  const Tuning& tune = GetTuning();
  if (tune.gemv_fast == 0 || tune.gemv_one_chunk == 0 || tune.gemv_ksplit > 0 || tune.gemv_waves > 0) return false;
  if (args[0].params != nullptr || args[0].batch_ids != nullptr || args[0].m != 1) return false;
  const int ks = DivUp(args[0].k, 4);
  if (args[0].k % 32 != 0) return false;
  const int chunks = ks / 8;
  if (chunks < 8 || chunks > 128 || (chunks & (chunks - 1)) != 0) return false;
  int strips = 0;
  for (int i = 0; i < count; ++i) {
    const int ns = DivUp(args[i].n, 4);
    if (args[i].n % 64 != 0 || EffectiveGroup(args[i].group, ns) != ns || args[i].has_zero_point) return false;
    if ((size_t)ks * ns * 8 >= ((size_t)1 << 32) || ns / 2 >= (1 << 24)) return false;  // 32-bit lane offsets
    strips += ns / 16;
  }
  return strips >= 128;
}

hipError_t LaunchStrip(StreamParams& p, const FcArgs* args, int count, bool grouped, hipStream_t stream,
                       bool strided = false) {
  const Tuning& tune = GetTuning();
  // 16, 8 or 4 slices: 8, 4 or 2 lanes per row (strided: strips of 16 slices out of the one group)
  const int group = strided ? kNativeGroup : EffectiveGroup(args[0].group, p.seg[0].ns);
  const int lpr = group / 2;
  int strips = 0;
  for (int i = 0; i < count; ++i) {
    strips += p.seg[i].ns / group;
    p.seg[i].strip_end = strips;
  }
  // K stays inside the work-group when the strips alone fill the chip, and for matrices of a few
  // MB, where a second kernel for the sums costs more (2.8 us) than running on the 30-40 CUs that
  // the strips give; else it is split into power-of-two runs of at least 8 chunks (one wave) so
  // that about 256 work-groups exist.
  size_t weight_bytes = 0;
  for (int i = 0; i < count; ++i) weight_bytes += (size_t)p.ks * p.seg[i].ns * 8;
  int cps = p.chunks;
  const bool batched = p.batch_ids != nullptr;  // (no K split: a dst row's sums stay in its work-group)
  if (!batched && strips < 128 && p.chunks > 64 / lpr && weight_bytes > ((size_t)6 << 20)) {
    const int want = DivUp(256, strips);
    cps = 64 / lpr;
    while (cps * 2 * want <= p.chunks) cps *= 2;
  }
  if (tune.gemv_ksplit > 0 && !batched) cps = std::max(1, DivUp(p.chunks, tune.gemv_ksplit));
  int ksplit = DivUp(p.chunks, cps);
  if (ksplit > kGemvMaxKSplit) {
    ksplit = kGemvMaxKSplit;
    cps = DivUp(p.chunks, ksplit);
    ksplit = DivUp(p.chunks, cps);
  }
  while (ksplit > 1 && (size_t)ksplit * p.n_total > args[0].partial_floats) {
    --ksplit;
    cps = DivUp(p.chunks, ksplit);
    ksplit = DivUp(p.chunks, cps);
  }
  p.chunks_per_split = cps;
  p.ksplit = ksplit;
  int waves = 1;
  while (waves < 16 && waves * 64 / lpr < cps) waves *= 2;
  // more work-groups than CUs (several dst rows): 512 threads, so that two work-groups share a CU and
  // the second round starts while the first still streams (two c2-shaped matrices: 12.3 -> 11.4 us)
  if (batched && (long)strips * p.rows > 256) waves = std::min(waves, 8);
  if (tune.gemv_waves > 0) waves = tune.gemv_waves;
  const dim3 grid(strips, ksplit, batched ? p.rows : 1);
  StripParams sp;
  sp.batch_ids = p.batch_ids;
  sp.rows = p.rows;
  sp.src_rows = p.src_rows;
  sp.weights_batch = p.weights_batch;
  sp.act = p.act;
  sp.partial = p.partial;
  sp.ks = p.ks;
  sp.chunks = p.chunks;
  sp.chunks_per_split = p.chunks_per_split;
  sp.ksplit = p.ksplit;
  sp.group_chunks = p.group_chunks;
  sp.n_total = p.n_total;
  sp.segments = p.segments;
  sp.reserved = 0;
  sp.mask_lo = p.mask_lo;
  sp.mask_hi = p.mask_hi;
  sp.magic_lo = p.magic_lo;
  sp.magic_hi = p.magic_hi;
  for (int i = 0; i < kMaxSegments; ++i) {
    const StreamSegment& g = p.seg[i];
    sp.seg[i] = StripSegment{g.weights, g.scale, g.zero_point, g.bias, g.dst, g.n_pad, g.strip_end, g.n_off, g.row_u4};
  }
  hipError_t e;
  switch (lpr) {
    case 2: e = LaunchStripL<2>(sp, waves, grouped, strided, grid, stream); break;
    case 4: e = LaunchStripL<4>(sp, waves, grouped, strided, grid, stream); break;
    default: e = LaunchStripL<8>(sp, waves, grouped, strided, grid, stream); break;
  }
  if (e != hipSuccess || ksplit == 1) return e;
  if (grouped)
    hipLaunchKernelGGL(fc_w4_strip_reduce_kernel<true>, dim3(DivUp(p.n_total, 64)), dim3(64), 0, stream, sp);
  else
    hipLaunchKernelGGL(fc_w4_strip_reduce_kernel<false>, dim3(DivUp(p.n_total, 64)), dim3(64), 0, stream, sp);
  return hipGetLastError();
}


// ------------------------------------------------------------------------------------------
// 2..4 tokens over strips of 64 channels, one chunk per thread (the launch shapes of the one-chunk
// form above), with the multiply-accumulate on the matrix cores: v_mfma_f32_4x4x4_16B_f16 works on
// 16 independent blocks of 4 lanes.  Lane i of a block supplies row i of A = the 4 K-values of
// one of its 8 outputs (two unpacked words: exactly what the nibble trick yields), lane j supplies
// column j of B = the 4 K-values of token j, and D[i][j] arrives in lane j, register i.  The 4
// lanes of a block are 4 neighbouring 16-byte columns of one K-slice row, so they share the
// K-slice and differ in the channels: one MFMA per output index multiplies the block's 32 channels
// with up to 4 tokens, at the price of one token on the vector ALU.  Lane (row, col) then holds,
// for token col % 4, the sums of the 32 channels of its block (value 8 * i + o = lane i, output o),
// which meet across the 8 rows of a wave by the register exchanges of the one-token kernels (32 ->
// 16 -> 8 -> 4 values per lane) and across waves through LDS.
// The constant offsets of the unpacked codes (1024 + 8, 64 + 8) are removed per chunk with the
// lane's own sum of its token's activations.
// ------------------------------------------------------------------------------------------
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4v_t __attribute__((ext_vector_type(4)));

template <int WAVES, bool GROUPED, bool MULTI, bool STRIDED>
__global__ __launch_bounds__(WAVES * 64) void fc_w4_strip_tokens_kernel(StripParams p, int m) {
  constexpr int LPR = 8, STRIP = 64, MT = 4;
  __shared__ float red[WAVES][MT][STRIP];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int col = lane & 7;
  const int row = tid >> 3;  // the thread's chunk
  const int jt = col & 3;    // token slot of this lane
  const int half = col >> 2; // which 32 channels of the strip its block holds
  int strip = blockIdx.x;
  const StripSegment sg = SelectSegment<MULTI>(p, strip);
  const uint32_t mask_lo = p.mask_lo, mask_hi = p.mask_hi;
  uint32_t magic_lo = p.magic_lo, magic_hi = p.magic_hi;
  asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));  // (x & mask) | magic selects to one v_and_or_b32 that the compiler can see
  asm volatile("" : : "s"(p.act), "s"(sg.dst), "s"(sg.bias), "s"(sg.scale));
  const int ks = p.ks, n_pad = sg.n_pad;
  const u32x4* wstrip = STRIDED ? sg.weights + (size_t)strip * LPR : sg.weights + (size_t)strip * ks * LPR;
  const uint32_t row_items = STRIDED ? (uint32_t)sg.row_u4 : (uint32_t)LPR;
  const uint32_t voff = (__umul24((uint32_t)row * 8u, row_items) + (uint32_t)col) * 16u;
  const u32x4* wp = reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(wstrip) + voff);
  // this lane's token (slots beyond the launch's tokens repeat the last one; their sums are dropped)
  const u32x2* ap = reinterpret_cast<const u32x2*>(p.act) + ((size_t)row * 8 * m + min(jt, m - 1));
  u32x4 w[8];
  u32x2 a[8];
  u32x4 sv[4];
#pragma unroll
  for (int j = 0; j < 2; ++j) w[j] = __builtin_nontemporal_load(wp + (size_t)j * row_items);
#pragma unroll
  for (int j = 0; j < 8; ++j) a[j] = ap[(size_t)j * m];
  if (GROUPED) {
    const int g = row / p.group_chunks;
    const __half* sp = sg.scale + (size_t)g * n_pad + (size_t)strip * STRIP + half * 32;
#pragma unroll
    for (int i = 0; i < 4; ++i) sv[i] = *reinterpret_cast<const u32x4*>(sp + i * 8);
  }
#pragma unroll
  for (int j = 2; j < 8; ++j) w[j] = __builtin_nontemporal_load(wp + (size_t)j * row_items);

  float4v_t acc[8];
#pragma unroll
  for (int o = 0; o < 8; ++o) acc[o] = float4v_t{0.0f, 0.0f, 0.0f, 0.0f};
  float asum = 0.0f;
  const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const half4_t b = __builtin_bit_cast(half4_t, a[j]);
    asum = __builtin_amdgcn_fdot2(AsHalf2(a[j][0]), ones, asum, false);
    asum = __builtin_amdgcn_fdot2(AsHalf2(a[j][1]), ones, asum, false);
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {  // outputs 4 * hh .. + 3: words 2 * hh (inputs 0, 1) and 2 * hh + 1 (inputs 2, 3)
      const uint32_t l0 = w[j][2 * hh], l1 = w[j][2 * hh + 1];
      const uint32_t h0 = l0 >> 8, h1 = l1 >> 8;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint32_t s0 = (t & 2) ? h0 : l0, s1 = (t & 2) ? h1 : l1;
        u32x2 q;
        q[0] = (t & 1) ? ((s0 & mask_hi) | magic_hi) : ((s0 & mask_lo) | magic_lo);
        q[1] = (t & 1) ? ((s1 & mask_hi) | magic_hi) : ((s1 & mask_lo) | magic_lo);
        acc[4 * hh + t] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, q), b, acc[4 * hh + t], 0, 0, 0);
      }
    }
  }
  // value 8 * i + o: channel 32 * half + 8 * i + o of the strip (lane i of the block, its output o)
  float r[32];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int o = 0; o < 8; ++o) {
      const float centered = fmaf((o & 1) ? -72.0f : -1032.0f, asum, acc[o][i]);
      r[8 * i + o] = GROUPED ? (float)AsHalf2(sv[i][o >> 1])[o & 1] * centered : centered;
    }
  }
  float s16[16], s8[8];
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    const u32x2s x = __builtin_amdgcn_permlane32_swap(__float_as_uint(r[q]), __float_as_uint(r[q + 16]), false, false);
    s16[q] = __uint_as_float(x[0]) + __uint_as_float(x[1]);
  }
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const u32x2s x = __builtin_amdgcn_permlane16_swap(__float_as_uint(s16[q]), __float_as_uint(s16[q + 8]), false, false);
    s8[q] = __uint_as_float(x[0]) + __uint_as_float(x[1]);
  }
#pragma unroll
  for (int q = 0; q < 8; ++q)
    s8[q] += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(s8[q]), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
  const bool up8 = (lane & 8) != 0;
  const float4 mine = make_float4(up8 ? s8[4] : s8[0], up8 ? s8[5] : s8[1], up8 ? s8[6] : s8[2], up8 ? s8[7] : s8[3]);
  // lanes 32.. kept values 16.., lanes 16.. of each half values 8.., lanes 8.. of each 16 values 4..
  const int first = 32 * half + ((lane >> 5) & 1) * 16 + ((lane >> 4) & 1) * 8 + ((lane >> 3) & 1) * 4;
  *reinterpret_cast<float4*>(&red[wave][jt][first]) = mine;
  __syncthreads();
  for (int idx = tid; idx < STRIP * m; idx += WAVES * 64) {
    const int t = idx >> 6, ch = idx & 63;
    float v = 0.0f;
#pragma unroll
    for (int q = 0; q < WAVES; ++q) v += red[q][t][ch];
    const int n_out = strip * STRIP + ch;
    if (!GROUPED) v *= __half2float(sg.scale[n_out]);
    __half h = __float2half_rn(v);
    if (sg.bias) h = __hadd(h, sg.bias[n_out]);
    sg.dst[((size_t)(n_out >> 2) * m + t) * 4 + (n_out & 3)] = h;
  }
}

template <int WAVES>
hipError_t LaunchStripTokensW(const StripParams& p, int m, bool grouped, bool strided, dim3 grid, hipStream_t stream) {
  const bool multi = p.segments > 1;
  const dim3 block(WAVES * 64);
#define MLD_STRIP_T(G, MU, ST) hipLaunchKernelGGL((fc_w4_strip_tokens_kernel<WAVES, G, MU, ST>), grid, block, 0, stream, p, m)
  if (strided) {
    if (grouped) { if (multi) MLD_STRIP_T(true, true, true); else MLD_STRIP_T(true, false, true); }
    else         { if (multi) MLD_STRIP_T(false, true, true); else MLD_STRIP_T(false, false, true); }
  } else {
    if (grouped) { if (multi) MLD_STRIP_T(true, true, false); else MLD_STRIP_T(true, false, false); }
    else         { if (multi) MLD_STRIP_T(false, true, false); else MLD_STRIP_T(false, false, false); }
  }
#undef MLD_STRIP_T
  return hipGetLastError();
}

// The token form serves: 2..4 tokens, no zero points, no batched weights or runtime bounds, every
// matrix in whole strips of 64 channels packed in output groups of 16 slices (or all in the
// reference's one group: strided rows), K = 256 ... 4096 input channels in powers of two (every
// thread exactly one chunk), strips enough to keep K inside the work-groups.
bool StripTokensServes(const FcArgs* args, int count, bool* strided) {
  const Tuning& tune = GetTuning();
  if (tune.gemv_fast == 0 || tune.gemv_one_chunk == 0 || tune.gemv_ksplit > 0 || tune.gemv_waves > 0 || tune.gemv_mfma == 0) return false;
  if (args[0].params != nullptr || args[0].batch_ids != nullptr || args[0].m < 2 || args[0].m > 4) return false;
  if (args[0].k % 32 != 0) return false;
  const int ks = args[0].k / 4, chunks = ks / 8;
  if (chunks < 8 || chunks > 128 || (chunks & (chunks - 1)) != 0) return false;
  int strips = 0, native = 0, one = 0;
  for (int i = 0; i < count; ++i) {
    const int ns = DivUp(args[i].n, 4);
    if (args[i].n % 64 != 0 || args[i].has_zero_point) return false;
    const int group = EffectiveGroup(args[i].group, ns);
    if (group == kNativeGroup) ++native; else if (group == ns) ++one; else return false;
    if ((size_t)ks * ns * 8 >= ((size_t)1 << 32) || ns / 2 >= (1 << 24)) return false;  // 32-bit lane offsets
    strips += ns / 16;
  }
  if (native != count && one != count) return false;
  *strided = one == count && native != count;
  return strips >= 128;
}

hipError_t LaunchStripTokens(StreamParams& p, const FcArgs* args, int count, bool grouped, bool strided, hipStream_t stream) {
  int strips = 0;
  for (int i = 0; i < count; ++i) {
    strips += p.seg[i].ns / kNativeGroup;
    p.seg[i].strip_end = strips;
  }
  StripParams sp = {};
  sp.act = p.act;
  sp.partial = nullptr;
  sp.ks = p.ks;
  sp.chunks = p.chunks;
  sp.chunks_per_split = p.chunks;
  sp.ksplit = 1;
  sp.group_chunks = p.group_chunks;
  sp.n_total = p.n_total;
  sp.segments = p.segments;
  sp.mask_lo = p.mask_lo;
  sp.mask_hi = p.mask_hi;
  sp.magic_lo = p.magic_lo;
  sp.magic_hi = p.magic_hi;
  for (int i = 0; i < kMaxSegments; ++i) {
    const StreamSegment& g = p.seg[i];
    sp.seg[i] = StripSegment{g.weights, g.scale, g.zero_point, g.bias, g.dst, g.n_pad, g.strip_end, g.n_off, g.row_u4};
  }
  const dim3 grid(strips);
  switch (p.chunks / 8) {
    case 1: return LaunchStripTokensW<1>(sp, p.m, grouped, strided, grid, stream);
    case 2: return LaunchStripTokensW<2>(sp, p.m, grouped, strided, grid, stream);
    case 4: return LaunchStripTokensW<4>(sp, p.m, grouped, strided, grid, stream);
    case 8: return LaunchStripTokensW<8>(sp, p.m, grouped, strided, grid, stream);
    default: return LaunchStripTokensW<16>(sp, p.m, grouped, strided, grid, stream);
  }
}

// ------------------------------------------------------------------------------------------
// One token over weights packed in output groups of 2 slices (8 channels): the whole K of a strip
// of 8 channels is one contiguous run of 16-byte rows, so layers of a few thousand channels, which
// have too few 64-channel strips to occupy the chip, give every CU a strip without splitting K
// across work-groups (no second kernel for the sums).  Lane l of the work-group reads rows
// l, l + T, l + 2T, ... (T threads): every load instruction of a wave covers 1 KB of contiguous
// memory.  The rows of a thread lie in different scale groups, so with group-wise scales a row's
// sums are scaled as they are added (scale vectors come from cache: 8 lanes share one).
// K reduction: the 8 channel sums of the 64 lanes by the register exchanges of the strip kernel
// (all lanes hold rows of the same 8 channels), across waves through LDS in wave order.
// ------------------------------------------------------------------------------------------
template <int WAVES, bool GROUPED, bool ZP, bool MULTI>
__global__ __launch_bounds__(WAVES * 64) void fc_w4_rows_kernel(StripParams p) {
  constexpr int T = WAVES * 64;
  __shared__ float red[WAVES][8];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  // Work-groups go round-robin to the 8 XCDs.  The scales of 8 neighbouring strips share a 128-byte
  // line per scale group, so neighbouring strips are given to work-groups of one XCD (whose L2 then
  // fetches the line once): of every 64 work-groups, XCD x takes strips 8x .. 8x + 7.
  int strip = blockIdx.x;
  if (strip < (int)(gridDim.x & ~63u)) strip = (strip & ~63) + ((strip & 7) << 3) + ((strip >> 3) & 7);
  const StripSegment sg = SelectSegment<MULTI>(p, strip);
  struct { uint32_t mask_lo, mask_hi, magic_lo, magic_hi; } up = {p.mask_lo, p.mask_hi, p.magic_lo, p.magic_hi};
  asm volatile("" : : "s"(p.act), "s"(sg.dst), "s"(sg.bias), "s"(sg.scale));  // (fetched with the first batch of scalar loads)
  const u32x4* wstrip = sg.weights + (size_t)strip * p.ks;  // row r of the strip: K-slice r, 2 slices x 8 bytes
  const u32x2* act2 = reinterpret_cast<const u32x2*>(p.act);
  const __half* scale = sg.scale;
  const __half* zero_point = sg.zero_point;
  const int ks = p.ks, n_pad = sg.n_pad;
  const int group_shift = p.group_chunks;  // log2 of the K-slices per scale group (grouped only)
  const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};

  float acc[8], asum_all = 0.0f;
#pragma unroll
  for (int o = 0; o < 8; ++o) acc[o] = 0.0f;
  u32x4 zv_lin = {0u, 0u, 0u, 0u};
  if (ZP && !GROUPED) zv_lin = *reinterpret_cast<const u32x4*>(zero_point + (size_t)strip * 8);
  for (int r0 = tid; r0 < ks; r0 += 8 * T) {
    u32x4 w[8], sv[8], zv[8];
    u32x2 a[8];
    // small loads that come from cache first, then the eight weight loads back to back
    {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int r = r0 + T * j;
        const u32x2 v = act2[min(r, ks - 1)];
        a[j] = u32x2{r < ks ? v[0] : 0u, r < ks ? v[1] : 0u};
      }
      if (GROUPED) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const size_t so = (size_t)(min(r0 + T * j, ks - 1) >> group_shift) * n_pad + (size_t)strip * 8;
          sv[j] = *reinterpret_cast<const u32x4*>(scale + so);
          if (ZP) zv[j] = *reinterpret_cast<const u32x4*>(zero_point + so);
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) w[j] = __builtin_nontemporal_load(wstrip + min(r0 + T * j, ks - 1));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const half2_t a01 = AsHalf2(a[j][0]), a23 = AsHalf2(a[j][1]);
      float asum = __builtin_amdgcn_fdot2(a01, ones, 0.0f, false);
      asum = __builtin_amdgcn_fdot2(a23, ones, asum, false);
      float t[8];
#pragma unroll
      for (int h = 0; h < 4; h += 2) {  // words h, h + 1: inputs (0, 1) and (2, 3) of outputs 4 * (h >> 1) .. + 3
        const uint32_t lo0 = w[j][h], hi0 = lo0 >> 8, lo1 = w[j][h + 1], hi1 = lo1 >> 8;
        const int ob = 4 * (h >> 1);
        t[ob + 0] = __builtin_amdgcn_fdot2(AsHalf2(AndOr(lo0, up.mask_lo, up.magic_lo)), a01, 0.0f, false);
        t[ob + 1] = __builtin_amdgcn_fdot2(AsHalf2(AndOr(lo0, up.mask_hi, up.magic_hi)), a01, 0.0f, false);
        t[ob + 2] = __builtin_amdgcn_fdot2(AsHalf2(AndOr(hi0, up.mask_lo, up.magic_lo)), a01, 0.0f, false);
        t[ob + 3] = __builtin_amdgcn_fdot2(AsHalf2(AndOr(hi0, up.mask_hi, up.magic_hi)), a01, 0.0f, false);
        t[ob + 0] = __builtin_amdgcn_fdot2(AsHalf2(AndOr(lo1, up.mask_lo, up.magic_lo)), a23, t[ob + 0], false);
        t[ob + 1] = __builtin_amdgcn_fdot2(AsHalf2(AndOr(lo1, up.mask_hi, up.magic_hi)), a23, t[ob + 1], false);
        t[ob + 2] = __builtin_amdgcn_fdot2(AsHalf2(AndOr(hi1, up.mask_lo, up.magic_lo)), a23, t[ob + 2], false);
        t[ob + 3] = __builtin_amdgcn_fdot2(AsHalf2(AndOr(hi1, up.mask_hi, up.magic_hi)), a23, t[ob + 3], false);
      }
      if (GROUPED) {
#pragma unroll
        for (int o = 0; o < 8; ++o) {
          float centre = (o & 1) ? -72.0f : -1032.0f;  // the unpacked code carries +64 / +1024; its centre is 8
          if (ZP) centre -= (float)AsHalf2(zv[j][o >> 1])[o & 1];
          acc[o] = fmaf((float)AsHalf2(sv[j][o >> 1])[o & 1], fmaf(centre, asum, t[o]), acc[o]);
        }
      } else {
        asum_all += asum;
#pragma unroll
        for (int o = 0; o < 8; ++o) acc[o] += t[o];
      }
    }
  }
  if (!GROUPED) {
#pragma unroll
    for (int o = 0; o < 8; ++o) {
      float centre = (o & 1) ? -72.0f : -1032.0f;
      if (ZP) centre -= (float)AsHalf2(zv_lin[o >> 1])[o & 1];
      acc[o] = fmaf(centre, asum_all, acc[o]);
    }
  }
  // every lane holds sums of the same 8 channels: lane l ends with channel (l / 8) % 8
  float v = WaveStripSum<1>(acc, lane);
  const int ch = (lane >> 3) & 7;
  if (WAVES > 1) {
    if ((lane & 7) == 0) red[wave][ch] = v;
    __syncthreads();
    if (tid >= 64) return;
    v = 0.0f;
#pragma unroll
    for (int q = 0; q < WAVES; ++q) v += red[q][ch];
  }
  if ((lane & 7) != 0) return;
  const int n_out = strip * 8 + ch;
  if (!GROUPED) v *= __half2float(scale[n_out]);
  __half h = __float2half_rn(v);
  if (sg.bias) h = __hadd(h, sg.bias[n_out]);
  sg.dst[n_out] = h;
}


// The same kernel for 2..4 tokens (MT = 2 or 4 token slots, `m` of them live): a K-slice row of the
// activations holds the tokens one after the other, every unpacked weight pair feeds MT dot
// products, the MT x 8 sums of a lane are reduced token by token.  Up to 8 waves (the 1024-thread
// shape would spill its MT x 8 accumulators and MT x 8 activation pairs).
template <int WAVES, int MT, bool GROUPED, bool ZP, bool MULTI>
__global__ __launch_bounds__(WAVES * 64) void fc_w4_rows_tokens_kernel(StripParams p, int m) {
  constexpr int T = WAVES * 64;
  __shared__ float red[WAVES][MT][8];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  int strip = blockIdx.x;
  if (strip < (int)(gridDim.x & ~63u)) strip = (strip & ~63) + ((strip & 7) << 3) + ((strip >> 3) & 7);
  const StripSegment sg = SelectSegment<MULTI>(p, strip);
  struct { uint32_t mask_lo, mask_hi, magic_lo, magic_hi; } up = {p.mask_lo, p.mask_hi, p.magic_lo, p.magic_hi};
  asm volatile("" : : "s"(p.act), "s"(sg.dst), "s"(sg.bias), "s"(sg.scale));  // (fetched with the first batch of scalar loads)
  const u32x4* wstrip = sg.weights + (size_t)strip * p.ks;
  const u32x2* act2 = reinterpret_cast<const u32x2*>(p.act);
  const __half* scale = sg.scale;
  const __half* zero_point = sg.zero_point;
  const int ks = p.ks, n_pad = sg.n_pad;
  const int group_shift = p.group_chunks;
  const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};

  float acc[MT][8], asum_all[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    asum_all[t] = 0.0f;
#pragma unroll
    for (int o = 0; o < 8; ++o) acc[t][o] = 0.0f;
  }
  u32x4 zv_lin = {0u, 0u, 0u, 0u};
  if (ZP && !GROUPED) zv_lin = *reinterpret_cast<const u32x4*>(zero_point + (size_t)strip * 8);
  for (int r0 = tid; r0 < ks; r0 += 8 * T) {
    u32x4 w[8], sv[8], zv[8];
    u32x2 a[8][MT];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int r = r0 + T * j;
      const size_t base = (size_t)min(r, ks - 1) * m;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const u32x2 v = act2[base + min(t, m - 1)];
        const bool live = r < ks && t < m;
        a[j][t] = u32x2{live ? v[0] : 0u, live ? v[1] : 0u};
      }
    }
    if (GROUPED) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const size_t so = (size_t)(min(r0 + T * j, ks - 1) >> group_shift) * n_pad + (size_t)strip * 8;
        sv[j] = *reinterpret_cast<const u32x4*>(scale + so);
        if (ZP) zv[j] = *reinterpret_cast<const u32x4*>(zero_point + so);
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) w[j] = __builtin_nontemporal_load(wstrip + min(r0 + T * j, ks - 1));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      // the 8 outputs' pairs for inputs (0, 1) and for inputs (2, 3), unpacked once for all tokens
      half2_t qa[8], qb[8];
#pragma unroll
      for (int h = 0; h < 4; h += 2) {
        const uint32_t lo0 = w[j][h], hi0 = lo0 >> 8, lo1 = w[j][h + 1], hi1 = lo1 >> 8;
        const int ob = 4 * (h >> 1);
        qa[ob + 0] = AsHalf2(AndOr(lo0, up.mask_lo, up.magic_lo));
        qa[ob + 1] = AsHalf2(AndOr(lo0, up.mask_hi, up.magic_hi));
        qa[ob + 2] = AsHalf2(AndOr(hi0, up.mask_lo, up.magic_lo));
        qa[ob + 3] = AsHalf2(AndOr(hi0, up.mask_hi, up.magic_hi));
        qb[ob + 0] = AsHalf2(AndOr(lo1, up.mask_lo, up.magic_lo));
        qb[ob + 1] = AsHalf2(AndOr(lo1, up.mask_hi, up.magic_hi));
        qb[ob + 2] = AsHalf2(AndOr(hi1, up.mask_lo, up.magic_lo));
        qb[ob + 3] = AsHalf2(AndOr(hi1, up.mask_hi, up.magic_hi));
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const half2_t a01 = AsHalf2(a[j][t][0]), a23 = AsHalf2(a[j][t][1]);
        float asum = __builtin_amdgcn_fdot2(a01, ones, 0.0f, false);
        asum = __builtin_amdgcn_fdot2(a23, ones, asum, false);
        float tt[8];
#pragma unroll
        for (int o = 0; o < 8; ++o) {
          tt[o] = __builtin_amdgcn_fdot2(qa[o], a01, 0.0f, false);
          tt[o] = __builtin_amdgcn_fdot2(qb[o], a23, tt[o], false);
        }
        if (GROUPED) {
#pragma unroll
          for (int o = 0; o < 8; ++o) {
            float centre = (o & 1) ? -72.0f : -1032.0f;
            if (ZP) centre -= (float)AsHalf2(zv[j][o >> 1])[o & 1];
            acc[t][o] = fmaf((float)AsHalf2(sv[j][o >> 1])[o & 1], fmaf(centre, asum, tt[o]), acc[t][o]);
          }
        } else {
          asum_all[t] += asum;
#pragma unroll
          for (int o = 0; o < 8; ++o) acc[t][o] += tt[o];
        }
      }
    }
  }
  const int ch = (lane >> 3) & 7;
  float v[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    if (!GROUPED) {
#pragma unroll
      for (int o = 0; o < 8; ++o) {
        float centre = (o & 1) ? -72.0f : -1032.0f;
        if (ZP) centre -= (float)AsHalf2(zv_lin[o >> 1])[o & 1];
        acc[t][o] = fmaf(centre, asum_all[t], acc[t][o]);
      }
    }
    v[t] = WaveStripSum<1>(acc[t], lane);
  }
  if (WAVES > 1) {
    if ((lane & 7) == 0) {
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
  if ((lane & 7) != 0) return;
  const int n_out = strip * 8 + ch;
  const float out_scale = GROUPED ? 1.0f : __half2float(scale[n_out]);
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    if (t >= m) break;
    __half h = __float2half_rn(GROUPED ? v[t] : v[t] * out_scale);
    if (sg.bias) h = __hadd(h, sg.bias[n_out]);
    sg.dst[((size_t)(n_out >> 2) * m + t) * 4 + (n_out & 3)] = h;
  }
}

template <int WAVES, int MT>
hipError_t LaunchRowsTokensW(const StripParams& p, int m, bool grouped, dim3 grid, hipStream_t stream) {
  const bool zp = p.seg[0].zero_point != nullptr, multi = p.segments > 1;
  const dim3 block(WAVES * 64);
#define MLD_ROWS_T(G, Z, MU) hipLaunchKernelGGL((fc_w4_rows_tokens_kernel<WAVES, MT, G, Z, MU>), grid, block, 0, stream, p, m)
  if (grouped) {
    if (zp) { if (multi) MLD_ROWS_T(true, true, true); else MLD_ROWS_T(true, true, false); }
    else    { if (multi) MLD_ROWS_T(true, false, true); else MLD_ROWS_T(true, false, false); }
  } else {
    if (zp) { if (multi) MLD_ROWS_T(false, true, true); else MLD_ROWS_T(false, true, false); }
    else    { if (multi) MLD_ROWS_T(false, false, true); else MLD_ROWS_T(false, false, false); }
  }
#undef MLD_ROWS_T
  return hipGetLastError();
}
template <int WAVES>
hipError_t LaunchRowsTokens(const StripParams& p, int m, bool grouped, dim3 grid, hipStream_t stream) {
  return m <= 2 ? LaunchRowsTokensW<WAVES, 2>(p, m, grouped, grid, stream) : LaunchRowsTokensW<WAVES, 4>(p, m, grouped, grid, stream);
}

template <int WAVES>
hipError_t LaunchRowsW(const StripParams& p, bool grouped, dim3 grid, hipStream_t stream) {
  const bool zp = p.seg[0].zero_point != nullptr, multi = p.segments > 1;
  const dim3 block(WAVES * 64);
#define MLD_ROWS(G, Z, MU) hipLaunchKernelGGL((fc_w4_rows_kernel<WAVES, G, Z, MU>), grid, block, 0, stream, p)
  if (grouped) {
    if (zp) { if (multi) MLD_ROWS(true, true, true); else MLD_ROWS(true, true, false); }
    else    { if (multi) MLD_ROWS(true, false, true); else MLD_ROWS(true, false, false); }
  } else {
    if (zp) { if (multi) MLD_ROWS(false, true, true); else MLD_ROWS(false, true, false); }
    else    { if (multi) MLD_ROWS(false, false, true); else MLD_ROWS(false, false, false); }
  }
#undef MLD_ROWS
  return hipGetLastError();
}

// The row-interleaved kernels serve: 1..4 tokens, every matrix of the launch packed in output groups
// of 2 slices, scale groups of a power-of-two number of K-slices.
bool RowsKernelServes(const FcArgs* args, int count) {
  if (GetTuning().gemv_fast == 0) return false;
  if (args[0].params != nullptr) return false;  // runtime channel bounds: the streaming kernel
  if (args[0].m < 1 || args[0].m > kGemvMaxTokens || args[0].batch_ids != nullptr || args[0].k % 4 != 0) return false;
  for (int i = 0; i < count; ++i) {
    const int ns = DivUp(args[i].n, 4);
    if (args[i].n % 8 != 0 || EffectiveGroup(args[i].group, ns) != 2) return false;
  }
  if (args[0].scale_kind == kScaleBlock) {
    const int group_slices = DivUp(args[0].k, 4) / args[0].groups;
    if (group_slices < 1 || (group_slices & (group_slices - 1)) != 0) return false;
  }
  return true;
}

hipError_t LaunchRows(const StreamParams& p, const FcArgs* args, int count, bool grouped, hipStream_t stream) {
  StripParams sp;
  sp.act = p.act;
  sp.partial = nullptr;
  sp.ks = p.ks;
  sp.chunks = p.chunks;
  sp.chunks_per_split = p.chunks;
  sp.ksplit = 1;
  sp.group_chunks = 0;  // here: log2 of the K-slices per scale group
  if (grouped)
    for (int gs = p.ks / p.groups; gs > 1; gs >>= 1) ++sp.group_chunks;
  sp.n_total = p.n_total;
  sp.segments = p.segments;
  sp.reserved = 0;
  sp.mask_lo = p.mask_lo;
  sp.mask_hi = p.mask_hi;
  sp.magic_lo = p.magic_lo;
  sp.magic_hi = p.magic_hi;
  int strips = 0;
  for (int i = 0; i < kMaxSegments; ++i) {
    const StreamSegment& g = p.seg[i];
    if (i < count) strips += g.ns / 2;
    sp.seg[i] = StripSegment{g.weights, g.scale, g.zero_point, g.bias, g.dst, g.n_pad, strips, g.n_off, 0};
  }
  // eight rows per thread where K allows: all of a thread's loads are in flight at once
  const int rpt = GetTuning().gemv_rows_rpt > 0 ? GetTuning().gemv_rows_rpt : 8;
  int waves = 1;
  while (waves < 16 && waves * 64 * rpt < p.ks) waves *= 2;
  if (GetTuning().gemv_waves > 0) waves = GetTuning().gemv_waves;
  const dim3 grid(strips);
  if (p.m > 1) {  // 2..4 tokens: the token form, up to 8 waves
    switch (std::min(waves, 8)) {
      case 1: return LaunchRowsTokens<1>(sp, p.m, grouped, grid, stream);
      case 2: return LaunchRowsTokens<2>(sp, p.m, grouped, grid, stream);
      case 4: return LaunchRowsTokens<4>(sp, p.m, grouped, grid, stream);
      default: return LaunchRowsTokens<8>(sp, p.m, grouped, grid, stream);
    }
  }
  switch (waves) {
    case 1: return LaunchRowsW<1>(sp, grouped, grid, stream);
    case 2: return LaunchRowsW<2>(sp, grouped, grid, stream);
    case 4: return LaunchRowsW<4>(sp, grouped, grid, stream);
    case 8: return LaunchRowsW<8>(sp, grouped, grid, stream);
    default: return LaunchRowsW<16>(sp, grouped, grid, stream);
  }
}

}  // namespace

bool FcW4StripTokensSupported(const FcArgs& a) {
  bool strided = false;
  return FcW4StreamSupported(a) && StripTokensServes(&a, 1, &strided);
}

bool FcW4StreamSupported(const FcArgs& a) {
  if (a.weight_bits != 4 || !a.act_f16 || !a.dst_f16) return false;
  if (a.params != nullptr && (a.packed_params_offset >= 0 || a.ring_i_index >= 0 || a.ring_o_index >= 0)) return false;
  if (a.m < 1 || a.m > kGemvMaxTokens) return false;
  if (a.has_zero_point && a.zero_point == nullptr) return false;  // a scalar zero point: generic kernel
  const int ks = DivUp(a.k, 4), ns = DivUp(a.n, 4);
  if (ns % 2 != 0) return false;  // 16-byte loads need an even number of 8-byte blocks per row
  const int group = EffectiveGroup(a.group, ns);
  if (ns % group != 0 || group % 2 != 0) return false;  // ... per row of one output group
  if (a.scale_kind == kScaleScalar) return false;
  if (a.scale_kind == kScaleBlock) {
    if (a.groups <= 0 || ks % a.groups != 0) return false;
    if ((ks / a.groups) % 8 != 0) return false;  // a chunk of 8 K-slices must not straddle groups
  }
  return a.partial != nullptr;
}

hipError_t LaunchFcW4StreamFused(const FcArgs* args, int count, hipStream_t stream, const char** kernel_name) {
  if (count < 1 || count > kMaxSegments) return hipErrorInvalidValue;
  const FcArgs& a = args[0];
  StreamParams p;
  p.segments = count;
  p.act = static_cast<const __half*>(a.act);
  p.partial = a.partial;
  p.m = a.m;
  p.ks = DivUp(a.k, 4);
  p.chunks = DivUp(p.ks, 8);
  const bool grouped = a.scale_kind == kScaleBlock;
  p.groups = grouped ? a.groups : 1;
  p.group_chunks = grouped ? (p.ks / a.groups) / 8 : p.chunks;
  p.mask_lo = 0x000F000Fu;
  p.mask_hi = 0x00F000F0u;
  p.magic_lo = 0x64006400u;
  p.magic_hi = 0x54005400u;
  int total_row_u4 = 0, n_total = 0;
  size_t weight_bytes = 0;
  for (int i = 0; i < count; ++i) {
    StreamSegment& sg = p.seg[i];
    sg.weights = reinterpret_cast<const u32x4*>(args[i].weights);
    sg.scale = static_cast<const __half*>(args[i].scale);
    sg.zero_point = args[i].has_zero_point ? static_cast<const __half*>(args[i].zero_point) : nullptr;
    sg.bias = static_cast<const __half*>(args[i].bias);
    sg.dst = static_cast<__half*>(args[i].dst);
    sg.ns = DivUp(args[i].n, 4);
    sg.n_pad = sg.ns * 4;
    sg.row_u4 = sg.ns / 2;
    const int group = EffectiveGroup(args[i].group, sg.ns);
    if (sg.ns % group != 0 || group % 2 != 0) return hipErrorInvalidValue;  // whole groups of whole 16-byte items
    sg.gu4 = group / 2;
    sg.n_off = n_total;
    n_total += sg.n_pad;
    total_row_u4 += sg.row_u4;
    weight_bytes += (size_t)p.ks * sg.ns * 8;
  }
  for (int i = count; i < kMaxSegments; ++i) p.seg[i] = p.seg[0];
  p.n_total = n_total;
  p.batch_ids = a.batch_ids;
  p.rows = a.rows;
  p.src_rows = a.src_rows;
  p.weights_batch = a.weights_batch;
  p.rt_params = a.params;
  p.src_end_idx = a.src_end_ch_index;
  p.dst_end_idx = a.dst_end_ch_index;
  p.k_channels = a.k;
  if (a.params != nullptr && count != 1) return hipErrorInvalidValue;  // bounded launches are single launches
  if (a.batch_ids) {
    // One dst row per blockIdx.z, K inside the work-group.  128-byte row segments when the rows
    // together still give most CUs a work-group, else 64-byte ones.
    if (count != 1) return hipErrorInvalidValue;
    p.ksplit = 1;
    const bool wide = (long)DivUp(p.seg[0].row_u4, 8) * a.rows >= 192;
    // one token per row over output groups of 16 slices: the contiguous-strip kernel
    if (wide && StripKernelServes(args, count)) {
      if (kernel_name) *kernel_name = "fc_w4_strip_kernel";
      return LaunchStrip(p, args, count, grouped, stream);
    }
    if (kernel_name) *kernel_name = "fc_w4_stream_kernel";
    const int lpr_b = wide ? 8 : 4, rows_b = wide ? 64 : 64;
    p.chunks_per_split = DivUp(p.chunks, rows_b) * rows_b;
    p.seg[0].strip_end = DivUp(p.seg[0].row_u4, lpr_b);
    const dim3 grid_b(p.seg[0].strip_end, 1, a.rows);
    return wide ? LaunchBatchedM<8, 8>(p, grouped, grid_b, stream) : LaunchBatchedM<4, 4>(p, grouped, grid_b, stream);
  }

  if (RowsKernelServes(args, count)) {
    if (kernel_name) *kernel_name = "fc_w4_rows_kernel";
    return LaunchRows(p, args, count, grouped, stream);
  }
  bool tokens_strided = false;
  if (StripTokensServes(args, count, &tokens_strided)) {
    if (kernel_name) *kernel_name = "fc_w4_strip_tokens_kernel";
    return LaunchStripTokens(p, args, count, grouped, tokens_strided, stream);
  }
  if (StripKernelServes(args, count)) {
    if (kernel_name) *kernel_name = "fc_w4_strip_kernel";
    return LaunchStrip(p, args, count, grouped, stream);
  }
  if (StridedStripKernelServes(args, count)) {
    if (kernel_name) *kernel_name = "fc_w4_strip_kernel";
    return LaunchStrip(p, args, count, grouped, stream, true);
  }

  // Launch shape.  Aim: every thread owns one chunk (all loads in flight at once) and the
  // grid has at least ~one work-group per CU.  Narrow row segments (LPR = 8: 128 contiguous
  // bytes) keep K inside one work-group for wide layers; when the layer is too narrow for
  // that, K is split across work-groups and a second kernel adds the partials.
  // Narrow layers of a few MB take narrower strips first (LPR = 4 or 2: 64- or 32-byte
  // segments): there a second kernel costs more than the poorer coalescing.
  // Very wide launches (the fused gate / up pair) fill the chip with 256-byte segments (LPR = 16).
  const Tuning& tune = GetTuning();
  int lpr = 8, waves = 16;
  if (DivUp(total_row_u4, 16) >= 256)
    lpr = 16;
  else if (DivUp(total_row_u4, 8) < 128 && weight_bytes <= (size_t)(tune.gemv_narrow_max_mb >= 0 ? tune.gemv_narrow_max_mb : 4) << 20)
    lpr = DivUp(total_row_u4, 4) >= 64 ? 4 : 2;
  if (tune.gemv_lpr > 0) lpr = tune.gemv_lpr;
  if (lpr != 2 && lpr != 4 && lpr != 8 && lpr != 16) lpr = 8;
  // two and more tokens need the registers of a small work-group (the 1024-thread shapes spill)
  if (p.m >= 2) {
    waves = 4;
    if (lpr == 16) lpr = 8;
  }
  if (tune.gemv_waves > 0) waves = tune.gemv_waves;
  if (waves != 4 && waves != 8 && waves != 16) waves = 16;
  int strips = 0;
  for (int i = 0; i < count; ++i) {
    strips += DivUp(p.seg[i].row_u4, lpr);
    p.seg[i].strip_end = strips;
  }
  int rows = waves * 64 / lpr;
  // shrink the work-group while it would leave rows without a chunk
  while (waves > 4 && rows / 2 >= p.chunks) {
    waves /= 2;
    rows /= 2;
  }
  // only some (lanes per row, waves) pairs are compiled
  if (lpr <= 4) waves = 4;
  if (lpr == 16) waves = 16;
  rows = waves * 64 / lpr;
  int ksplit = 1;
  if (strips < 128 && count == 1) {
    ksplit = DivUp(256, strips);
    // a smaller work-group (down to 8 waves) when K does not otherwise split that far
    while (lpr == 8 && waves > 8 && DivUp(p.chunks, rows) < ksplit) {
      waves /= 2;
      rows /= 2;
    }
    const int max_split = DivUp(p.chunks, rows);
    if (ksplit > max_split) ksplit = max_split;
  }
  if (count == 1 && tune.gemv_ksplit > 0) ksplit = tune.gemv_ksplit;
  if (ksplit > kGemvMaxKSplit) ksplit = kGemvMaxKSplit;
  if (ksplit < 1) ksplit = 1;
  while (ksplit > 1 && (size_t)ksplit * p.m * p.seg[0].n_pad > a.partial_floats) --ksplit;
  // every thread row gets the same number of chunks
  p.chunks_per_split = DivUp(DivUp(p.chunks, ksplit), rows) * rows;
  p.ksplit = DivUp(p.chunks, p.chunks_per_split);
  dim3 grid(strips, p.ksplit);
  if (kernel_name) *kernel_name = "fc_w4_stream_kernel";
  hipError_t e;
  e = LaunchShape(p, lpr, waves, grouped, grid, stream);
  if (e != hipSuccess || p.ksplit == 1) return e;
  const int total = p.m * p.seg[0].n_pad;
  if (grouped)
    hipLaunchKernelGGL(fc_w4_reduce_kernel<true>, dim3(DivUp(total, 256)), dim3(256), 0, stream, p, p.seg[0].n_pad);
  else
    hipLaunchKernelGGL(fc_w4_reduce_kernel<false>, dim3(DivUp(total, 256)), dim3(256), 0, stream, p, p.seg[0].n_pad);
  return hipGetLastError();
}

bool FcW4GatedSupported(const FcArgs& gate, const FcArgs& up) {
  if (!FcW4StreamSupported(gate) || !FcW4StreamSupported(up)) return false;
  if (gate.m > 2) return false;  // the paired accumulators of more tokens would spill
  if (gate.has_zero_point || up.has_zero_point) return false;
  return gate.act == up.act && gate.m == up.m && gate.k == up.k && gate.n == up.n && gate.scale_kind == up.scale_kind &&
         gate.groups == up.groups;
}

hipError_t LaunchFcW4Gated(const FcArgs& gate, const FcArgs& up, int activation, void* dst, hipStream_t stream,
                           const char** kernel_name) {
  StreamParams p;
  p.segments = 2;
  p.act = static_cast<const __half*>(gate.act);
  p.partial = nullptr;
  p.m = gate.m;
  p.ks = DivUp(gate.k, 4);
  p.chunks = DivUp(p.ks, 8);
  p.chunks_per_split = p.chunks;
  p.ksplit = 1;
  const bool grouped = gate.scale_kind == kScaleBlock;
  p.groups = grouped ? gate.groups : 1;
  p.group_chunks = grouped ? (p.ks / gate.groups) / 8 : p.chunks;
  p.mask_lo = 0x000F000Fu;
  p.mask_hi = 0x00F000F0u;
  p.magic_lo = 0x64006400u;
  p.magic_hi = 0x54005400u;
  const FcArgs* both[2] = {&gate, &up};
  for (int i = 0; i < 2; ++i) {
    StreamSegment& sg = p.seg[i];
    sg.weights = reinterpret_cast<const u32x4*>(both[i]->weights);
    sg.scale = static_cast<const __half*>(both[i]->scale);
    sg.zero_point = nullptr;
    sg.bias = static_cast<const __half*>(both[i]->bias);
    sg.dst = static_cast<__half*>(dst);
    sg.ns = DivUp(both[i]->n, 4);
    sg.n_pad = sg.ns * 4;
    sg.row_u4 = sg.ns / 2;
    const int group = EffectiveGroup(both[i]->group, sg.ns);
    if (sg.ns % group != 0 || group % 2 != 0 || group != EffectiveGroup(gate.group, sg.ns)) return hipErrorInvalidValue;
    sg.gu4 = group / 2;
    sg.n_off = 0;
    sg.strip_end = 0;
  }
  p.seg[2] = p.seg[0];
  p.batch_ids = nullptr;
  p.rows = p.src_rows = p.weights_batch = 1;
  p.rt_params = nullptr;
  p.src_end_idx = p.dst_end_idx = -1;
  p.k_channels = gate.k;
  if (kernel_name) *kernel_name = "fc_w4_gated_stream_kernel";
  // 128-byte row segments, 8 waves: 64 rows of chunks per pass (one pass covers K = 2048); the
  // 16-wave shape would spill with the two sets of accumulators
  const dim3 grid(DivUp(p.seg[0].row_u4, 8));
  return LaunchGatedM<8, 8>(p, grouped, activation, grid, stream);
}

hipError_t LaunchFcW4Stream(const FcArgs& a, hipStream_t stream, const char** kernel_name) {
  return LaunchFcW4StreamFused(&a, 1, stream, kernel_name);
}

// ------------------------------------------------------------------------------------------
// The streaming GEMV for callers that cannot allocate: its split-K sums go to a statically
// allocated array instead of an op's workspace.  Every GPU the library runs on holds its own
// copy of the array (at its own address) until the process ends.  The array's name is only a
// host-side handle: the device address comes from hipGetSymbolAddress, once per device, and that
// pointer is what the kernels get, as they get the workspace pointer of an op.
// ------------------------------------------------------------------------------------------
namespace {
static __device__ __align__(256) float scratch[kNoAllocScratchFloats];
constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;  // guards the first call on a device from several host threads
}  // namespace

hipError_t LaunchFcW4StreamNoAlloc(FcArgs a, hipStream_t stream, const char** kernel_name) {
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  // the array that is used is the current device's: a stream of another device would launch there
  // with this device's address
  if (stream != nullptr) {
    int stream_device = device;
    e = hipStreamGetDevice(stream, &stream_device);
    if (e != hipSuccess) return e;
    if (stream_device != device) return hipErrorInvalidDevice;
  }
  float* scratch_ptr = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[device] == nullptr) {  // first call on this device, which is current
      float* ptr = nullptr;
      e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
      if (e != hipSuccess) return e;
      g_scratch_ptr[device] = ptr;
    }
    scratch_ptr = g_scratch_ptr[device];
  }
  // Nothing has to start at zero: a split launch writes every sum that its second kernel reads.
  a.partial = scratch_ptr;
  a.partial_floats = kNoAllocScratchFloats;
  if (!FcW4StreamSupported(a)) return hipErrorInvalidValue;
  return LaunchFcW4StreamFused(&a, 1, stream, kernel_name);
}

}  // namespace mldhip
