// Prefill-side kernels for gfx950: MFMA GEMMs.
//
//  fc_w4_mfma_gemm_kernel   multi-token FullyConnected over the packed uint4 I4O4 buffer: every
//                           wave dequantizes its weight operands in registers (one rounding per
//                           weight: round((u-8)*s), like the reference's fma(u, s, -8s)), then
//                           v_mfma_f32_32x32x16_f16 with fp32 accumulation; no LDS in the loop.
//  fc_w8_mfma_gemm_kernel   the same kernel over the packed uint8 I4O4 buffer (u - 128).
//  conv_int8_mfma_kernel    int8 codes x int8 weights with v_mfma_i32_32x32x32_i8 (int32
//                           accumulators, exact), tiles streamed global -> LDS without passing
//                           through registers, then the reference's rescale epilogue.
//
// Operand roles in both: the MFMA "A" operand is the weight tile (rows = output channels), "B"
// is the activation tile (columns = tokens).  In the 32x32 result a lane then holds, for one
// token, groups of 4 consecutive output channels: exactly one 4-channel slice of the
// slice-major output tensor, so a lane stores 8 (fp16) or 16 bytes and 32 lanes store
// consecutive tokens.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <type_traits>

#include "../../include/mldhip.h"
#include "gated.h"
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
typedef float float2v_t __attribute__((ext_vector_type(2)));


// One weight matrix of an int4 GEMM launch.  A launch covers up to kMaxW4Segments matrices
// that read the same activations (same K): channel tiles [tile_end of the previous, tile_end)
// belong to it.
constexpr int kMaxW4Segments = 3;
struct W4Segment {
  const uint8_t* w4;    // [Ks][Ns] blocks of 8 bytes (uint4) or 16 bytes (uint8)
  const __half* scale;  // [groups][Ns][4]
  const __half* zp;     // zero points, same shape as scale, or null
  const __half* bias;
  __half* dst;
  float* partial;  // [ksplit][Ns][m][4] fp32 sums when ksplit > 1
  int n, ns;
  int group;  // slices per output group of the packed weights (ns: one group, the rows span all of N)
  int tile_end;
  uint32_t a_bytes, s_bytes;
  int group_shift;  // log2(group) when it is a power of two, else -1
};

struct GemmParams {
  W4Segment seg[kMaxW4Segments];
  int segments;
  int m, n, k;
  int ns;        // output slices, ceil(n/4)
  int k_steps;   // K-steps
  void* dst;
  const void* bias;
  int dst_type;
  // fp16 / int4 path
  const __half* act;    // [Ks][m][4]
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
  int ksplit;       // work-groups along K per output tile (fp16 path)
  int group_shift;  // log2(group_size / 16) when that is a power of two, else -1 (not supported by the direct kernel)
  int xcd_m;        // fp16 path: the 8 XCDs form an xcd_m x (8 / xcd_m) grid over (token tiles, channel tiles)
  int gate_activation;  // gated fp16 launch: MLDHIP_GATE_*
  int dual;             // fp16 path: a work-group owns two neighbouring channel tiles
  // fp16 path, packed groups (ConvRuntimeCheckDesc::PackedGroups): blockIdx.z = weight matrix g of
  // pg_groups; its tokens are min(pg_params[pg_offset + g], pg_max) many from token
  // pg_params[pg_offset + pg_groups + g] of the one source row.  pg_groups = 0: not set.
  const int32_t* pg_params;
  int pg_offset, pg_groups, pg_max;
  // fp16 path: launch geometry worked out on the host, so that no work-group divides by a run-time
  // number in front of its first load: token tiles of the launch, the XCD rectangle (token tiles x
  // channel tiles), log2(xcd_m), ceil(2^32 / rect_m) (0 when rect_m = 1), and the 16-channel steps
  // of one wave's share of K (a multiple of the prefetch depth).
  int geo_tiles_m, geo_rect_m, geo_rect_n, geo_xm_shift;
  uint32_t geo_rect_m_magic;
  int geo_per_wave;
};

__device__ __forceinline__ half2_t AsHalf2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }
__device__ __forceinline__ uint32_t AsU32(half2_t v) { return __builtin_bit_cast(uint32_t, v); }

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
// The same with a zero activation offset and no weight zero point: the offset terms are exact
// zeros there, and adding a zero changes nothing (but possibly the sign of a zero result).
__device__ __forceinline__ float RescaleNoOffset(int acc, float ws, float src_scale) {
  const float f0 = ws * src_scale;
  return (float)acc * f0;
}
#pragma clang fp contract(fast)

// ------------------------------------------------------------------------------------------
// int8 x int8 GEMM.
//
// Both operands are stored the way the MFMA wants them: [k16][row][16 bytes], i.e. a lane's
// operand for v_mfma_i32_32x32x32_i8 (row r = lane % 32, 16 consecutive k of unit 2*step +
// lane / 32) is one aligned 16-byte item, and 64 consecutive rows of a unit are 1 KB of
// contiguous memory.  A work-group of 4 waves (2 x 2) owns 256 channels x BM tokens; each wave
// 128 x (BM / 2).  K advances in stages of 4 units (64 values of k, two MFMA steps).  A stage of
// both tiles is copied global -> LDS by buffer loads that write LDS directly (no registers, no
// ds_write); rows past the matrix and units past K are out of the buffers' range and arrive
// as zeros.  kStages stages rotate through LDS, so kStages - 1 stages of loads are in flight
// behind the one being multiplied, and there is one barrier per stage.
//
// The compiler does not know what the LDS-writing loads touch, so the LDS side is explicit
// here: operand reads are inline ds_read_b128, followed by a counter wait that is tied to the
// registers it guards.
// ------------------------------------------------------------------------------------------
constexpr int kI8Stages = 4;
constexpr int kI8Threads = 256;

template <int OFF>
__device__ __forceinline__ void DsRead128(u32x4& dst, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int N>
__device__ __forceinline__ void LdsWait(u32x4 (&f)[N]) {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+v"(f[i]));
}

// 64 lanes x 16 bytes from the buffer (a lane's offset beyond the range gives zeros) to 1 KB of
// LDS starting at `dst`, which is the same for the whole wave.
typedef __attribute__((address_space(3))) char* LdsPtr;
__device__ __forceinline__ void CopyToLds(__amdgpu_buffer_rsrc_t rsrc, LdsPtr dst, uint32_t lane_offset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dst, 16, lane_offset, 0, 0, 0);
}

// Operand read number i of one MFMA step: 4 weight items, then FM token items, 512 bytes apart.
template <int FM, int OFF_A, int OFF_B>
__device__ __forceinline__ void ReadOperand(int i, u32x4 (&a)[4], u32x4 (&b)[FM], uint32_t aa, uint32_t ab) {
  switch (i) {  // i is a constant after unrolling
    case 0: DsRead128<OFF_A + 0 * 512>(a[0], aa); break;
    case 1: DsRead128<OFF_A + 1 * 512>(a[1], aa); break;
    case 2: DsRead128<OFF_A + 2 * 512>(a[2], aa); break;
    case 3: DsRead128<OFF_A + 3 * 512>(a[3], aa); break;
    case 4: DsRead128<OFF_B + 0 * 512>(b[0], ab); break;
    case 5: if constexpr (FM > 1) DsRead128<OFF_B + 1 * 512>(b[1], ab); break;
    case 6: if constexpr (FM > 2) DsRead128<OFF_B + 2 * 512>(b[2], ab); break;
    case 7: if constexpr (FM > 2) DsRead128<OFF_B + 3 * 512>(b[3], ab); break;
  }
}

// One MFMA step on (cur_a, cur_b) with the wave's other work threaded between the MFMAs, so
// that the matrix unit never waits for it: first the 4 + FM operand reads of the next step (into
// nxt_a / nxt_b), then, if COPY, this wave's 4 + FM global -> LDS copies of a later stage.  The
// fences fix that order; an MFMA occupies the unit for 32 cycles, the other instructions issue
// in its shadow.
template <int FM, int OFF_A, int OFF_B, bool COPY, typename CopyOne>
__device__ __forceinline__ void MultiplyAndFetch(int16v_t (&acc)[4][FM], u32x4 (&cur_a)[4], u32x4 (&cur_b)[FM],
                                                 u32x4 (&nxt_a)[4], u32x4 (&nxt_b)[FM], uint32_t aa, uint32_t ab,
                                                 CopyOne&& copy_one) {
  constexpr int kReads = 4 + FM;
  constexpr int kItems = COPY ? 2 * kReads : kReads;
  constexpr int kMfmas = 4 * FM;
  constexpr int kPerSlot = (kItems + kMfmas - 1) / kMfmas;
#pragma unroll
  for (int idx = 0; idx < kMfmas; ++idx) {
    const int fn = idx / FM, fm = idx % FM;
    acc[fn][fm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(int4v_t, cur_a[fn]),
                                                        __builtin_bit_cast(int4v_t, cur_b[fm]), acc[fn][fm], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int item = idx * kPerSlot; item < (idx + 1) * kPerSlot && item < kItems; ++item) {
      if (item < kReads)
        ReadOperand<FM, OFF_A, OFF_B>(item, nxt_a, nxt_b, aa, ab);
      else
        copy_one(item - kReads);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// DST: element type of the output (MLDHIP_FLOAT16 / FLOAT32 / INT32); ZP: weights have a zero point.
template <int FM, int DST, bool ZP>
__global__ __launch_bounds__(kI8Threads) void conv_int8_mfma_kernel(GemmParams p) {
  constexpr int FN = 4;
  constexpr int BN = 2 * FN * 32;              // 256 channels
  constexpr int BM = 2 * FM * 32;              // tokens
  constexpr int kABytes = 4 * BN * 16;         // one stage of the weight tile
  constexpr int kBBytes = 4 * BM * 16;         // one stage of the token tile
  constexpr int kStageBytes = kABytes + kBBytes;
  constexpr int kLoadsPerStage = BN / 64 + BM / 64;  // per wave
  __shared__ u32x4 smem[kI8Stages * kStageBytes / 16];
  const LdsPtr lds = (LdsPtr)smem;
  const uint32_t lds_base = (uint32_t)(size_t)lds;

  // (one batch of scalar loads for the arguments, those of the epilogue included)
  asm volatile("" : : "s"(p.m), "s"(p.n), "s"(p.k), "s"(p.ns), "s"(p.k16), "s"(p.a_bytes), "s"(p.b_bytes), "s"(p.wi8), "s"(p.codes),
               "s"(p.dst), "s"(p.bias), "s"(p.params), "s"(p.wsum), "s"(p.wscale), "s"(p.wzp));
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave & 1, wm = wave >> 1;
  const int r32 = lane & 31, g2 = lane >> 5;

  // Tile order.  Work-groups go round-robin to the 8 XCDs (id % 8), each with its own L2; XCD x
  // takes the contiguous range [x*per_xcd, (x+1)*per_xcd) of a numbering that walks blocks of
  // 8 channel tiles token-tile by token-tile, so the tiles that share an L2 form a compact
  // rectangle and re-use each other's operands.
  const int tiles_n = (p.n + BN - 1) / BN;
  const int tiles_m = (p.m + BM - 1) / BM;
  const int per_xcd = (tiles_n * tiles_m + 7) / 8;
  const int tile = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (tile >= tiles_n * tiles_m) return;
  int tn, tm;
  {
    const int full = tiles_n / 8;
    if (tile < full * 8 * tiles_m) {
      const int sc = tile / (8 * tiles_m), within = tile % (8 * tiles_m);
      tn = sc * 8 + within % 8;
      tm = within / 8;
    } else {
      const int rest = tile - full * 8 * tiles_m, width = tiles_n - full * 8;
      tn = full * 8 + rest % width;
      tm = rest / width;
    }
  }
  const int n0 = tn * BN;
  const int m0 = tm * BM;

  constexpr uint32_t kOob = 0x7FFFFFF0u;
  const __amdgpu_buffer_rsrc_t rsrc_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(p.wi8), 0, p.a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(p.codes), 0, p.b_bytes, 0x00020000);

  // Copy duty of this wave: unit `wave` of every stage, all rows, 64 rows per instruction.
  // A lane's byte offset advances by one stage per copy; rows past the matrix stay parked
  // beyond the range.
  uint32_t va[BN / 64], vb[BM / 64], sa[BN / 64], sb[BM / 64];
#pragma unroll
  for (int rg = 0; rg < BN / 64; ++rg) {
    const int row = n0 + rg * 64 + lane;
    va[rg] = row < p.n ? (uint32_t)(wave * p.n + row) * 16u : kOob;
    sa[rg] = row < p.n ? (uint32_t)p.n * 64u : 0u;
  }
#pragma unroll
  for (int rg = 0; rg < BM / 64; ++rg) {
    const int row = m0 + rg * 64 + lane;
    vb[rg] = row < p.m ? (uint32_t)(wave * p.m + row) * 16u : kOob;
    sb[rg] = row < p.m ? (uint32_t)p.m * 64u : 0u;
  }
  // copy number c of a stage: weight row groups first, then token row groups
  auto copy_one = [&](int slot, int c) {
    const LdsPtr base = lds + slot * kStageBytes;
    if (c < BN / 64) {
      CopyToLds(rsrc_a, base + (wave * BN + c * 64) * 16, va[c]);
      va[c] += sa[c];
    } else {
      const int rg = c - BN / 64;
      CopyToLds(rsrc_b, base + kABytes + (wave * BM + rg * 64) * 16, vb[rg]);
      vb[rg] += sb[rg];
    }
  };

  // operand addresses inside a stage
  const uint32_t addr_a = lds_base + (uint32_t)(g2 * BN + wn * FN * 32 + r32) * 16u;
  const uint32_t addr_b = lds_base + (uint32_t)kABytes + (uint32_t)(g2 * BM + wm * FM * 32 + r32) * 16u;

  int16v_t acc[FN][FM];
#pragma unroll
  for (int fn = 0; fn < FN; ++fn)
#pragma unroll
    for (int fm = 0; fm < FM; ++fm)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[fn][fm][v] = 0;
  // Waits until at most `pending` stages of this wave's copies are still in flight, then meets
  // the other waves: after it, the stage is complete in LDS and nobody reads the slot that the
  // next copy overwrites.
  auto stage_barrier = [&]() {
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((kI8Stages - 2) * kLoadsPerStage) : "memory");
  };

  const int stages = (p.k16 + 3) / 4;
  // prologue: stages 0 .. kStages-2 in flight, stage 0 landed, its first operands requested
#pragma unroll
  for (int s = 0; s < kI8Stages - 1; ++s)
#pragma unroll
    for (int c = 0; c < kLoadsPerStage; ++c) copy_one(s, c);
  stage_barrier();
  u32x4 fa[2][FN], fb[2][FM];
#pragma unroll
  for (int i = 0; i < 4 + FM; ++i) ReadOperand<FM, 0, 0>(i, fa[0], fb[0], addr_a, addr_b);
  int slot = 0;  // slot of stage t
  for (int t = 0; t < stages; ++t) {
    const uint32_t aa = addr_a + (uint32_t)(slot * kStageBytes);
    const uint32_t ab = addr_b + (uint32_t)(slot * kStageBytes);
    // the slot of stage t-1 takes stage t + kStages - 1 (copies past K read zeros)
    const int refill = slot == 0 ? kI8Stages - 1 : slot - 1;
    LdsWait(fa[0]);
    LdsWait(fb[0]);
    __builtin_amdgcn_sched_barrier(0);
    MultiplyAndFetch<FM, 2 * BN * 16, 2 * BM * 16, true>(acc, fa[0], fb[0], fa[1], fb[1], aa, ab,
                                                         [&](int c) { copy_one(refill, c); });
    LdsWait(fa[1]);
    LdsWait(fb[1]);
    stage_barrier();  // stage t+1 complete for every wave
    slot = slot == kI8Stages - 1 ? 0 : slot + 1;
    const uint32_t na = addr_a + (uint32_t)(slot * kStageBytes);
    const uint32_t nb = addr_b + (uint32_t)(slot * kStageBytes);
    __builtin_amdgcn_sched_barrier(0);
    MultiplyAndFetch<FM, 0, 0, false>(acc, fa[1], fb[1], fa[0], fb[0], na, nb, [](int) {});
  }
  // drain the copies that ran ahead before the work-group's LDS is released
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  if constexpr (DST == MLDHIP_FLOAT16) __syncthreads();  // LDS is reused for the output tile

  // ---- epilogue ---------------------------------------------------------------------------
  // Register v of the 32x32 result belongs to channel 8*(v/4) + 4*g2 + v%4 of the MFMA's 32 and to
  // token r32: four consecutive registers are one 4-channel slice of one token.  The channel
  // constants are fetched once per slice and used for the FM token blocks.
  int mi[FM];
  float src_scale[FM], src_zp[FM], src_sum[FM];
#pragma unroll
  for (int fm = 0; fm < FM; ++fm) {
    mi[fm] = m0 + (wm * FM + fm) * 32 + r32;
    src_scale[fm] = src_zp[fm] = src_sum[fm] = 0.0f;
    if (DST != MLDHIP_INT32) {
      const float4 pr = *reinterpret_cast<const float4*>(p.params + (size_t)min(mi[fm], p.m - 1) * 4);
      src_scale[fm] = pr.x;
      src_zp[fm] = pr.y;
      src_sum[fm] = pr.z;
    }
  }
  constexpr bool has_zp = ZP;
  const float in_channels = (float)p.k;
  if constexpr (DST == MLDHIP_FLOAT16) {
    // Straight-line: every register of the tile is rescaled and staged in LDS as
    // [slice of the tile][token of the tile][4 halfs]; what lies outside the matrix is computed
    // from clamped constants and never leaves LDS.
    const bool has_bias = p.bias != nullptr;
    // the channel constants of the wave's 16 slices, all requested before any is used (one memory
    // latency instead of sixteen); the per-channel tensors are padded to whole slices
    float4 ws_all[FN * 4];
    int4v_t wsum_all[FN * 4];
    float4 wzp_all[ZP ? FN * 4 : 1];
    u32x2 bias_all[FN * 4];
#pragma unroll
    for (int g = 0; g < FN * 4; ++g) {
      const int slice_l = (wn * FN + g / 4) * 8 + (g % 4) * 2 + g2;
      const int nb = min(n0 / 4 + slice_l, p.ns - 1) * 4;  // first of 4 consecutive channels
      ws_all[g] = *reinterpret_cast<const float4*>(p.wscale + nb);
      wsum_all[g] = *reinterpret_cast<const int4v_t*>(p.wsum + nb);
      if (ZP) wzp_all[g] = *reinterpret_cast<const float4*>(p.wzp + nb);
      bias_all[g] = u32x2{0x80008000u, 0x80008000u};  // -0.0: adding it changes nothing, not even the sign of a zero
    }
    if (has_bias) {
#pragma unroll
      for (int g = 0; g < FN * 4; ++g) {
        const int slice_l = (wn * FN + g / 4) * 8 + (g % 4) * 2 + g2;
        const int nb = min(n0 / 4 + slice_l, p.ns - 1) * 4;
        bias_all[g] = *reinterpret_cast<const u32x2*>(static_cast<const __half*>(p.bias) + nb);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // symmetric activation quantization gives a zero offset for every token: then two of the
    // three products and the sum of the rescale drop out (decided per wave)
    bool all_zero_offset = !has_zp;
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) all_zero_offset = all_zero_offset && src_zp[fm] == 0.0f;
    const bool no_offset = __all(all_zero_offset);
    auto stage_tile = [&](auto no_offset_tag) {
    constexpr bool kNoOffset = decltype(no_offset_tag)::value;
#pragma unroll
    for (int fn = 0; fn < FN; ++fn) {
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        const int slice_l = (wn * FN + fn) * 8 + v4 * 2 + g2;
        const float4 ws = ws_all[fn * 4 + v4];
        const int4v_t wsum = wsum_all[fn * 4 + v4];
        const float4 wzp = ZP ? wzp_all[ZP ? fn * 4 + v4 : 0] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        const float wsc[4] = {ws.x, ws.y, ws.z, ws.w};
        const float wz[4] = {wzp.x, wzp.y, wzp.z, wzp.w};
        const u32x2 bias2 = bias_all[fn * 4 + v4];
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) {
          float r[4];
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            r[c] = kNoOffset ? RescaleNoOffset(acc[fn][fm][v4 * 4 + c], wsc[c], src_scale[fm])
                             : Rescale(acc[fn][fm][v4 * 4 + c], wsc[c], wsum[c], src_scale[fm], src_zp[fm], has_zp,
                                       wz[c], src_sum[fm], in_channels);
          }
          // two results per conversion (round to nearest even) and per bias add
          u32x2 o;
          o[0] = AsU32(__builtin_convertvector(float2v_t{r[0], r[1]}, half2_t) + AsHalf2(bias2[0]));
          o[1] = AsU32(__builtin_convertvector(float2v_t{r[2], r[3]}, half2_t) + AsHalf2(bias2[1]));
          const int token_l = (wm * FM + fm) * 32 + r32;
          reinterpret_cast<u32x2*>(smem)[slice_l * BM + token_l] = o;
        }
      }
    }
    };
    if (no_offset)
      stage_tile(std::true_type{});
    else
      stage_tile(std::false_type{});
  } else {
#pragma unroll
  for (int fn = 0; fn < FN; ++fn) {
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int nb = n0 + (wn * FN + fn) * 32 + 8 * v4 + 4 * g2;  // first of 4 consecutive channels
      const int slice = nb >> 2;
      if (slice >= p.ns) continue;
      if constexpr (DST == MLDHIP_INT32) {
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) {
          if (mi[fm] >= p.m) continue;
          int4v_t o = {acc[fn][fm][v4 * 4], acc[fn][fm][v4 * 4 + 1], acc[fn][fm][v4 * 4 + 2], acc[fn][fm][v4 * 4 + 3]};
          *reinterpret_cast<int4v_t*>(static_cast<int*>(p.dst) + ((size_t)slice * p.m + mi[fm]) * 4) = o;
        }
        continue;
      } else {
      // the per-channel tensors are padded to whole slices
      const float4 ws = *reinterpret_cast<const float4*>(p.wscale + nb);
      const int4v_t wsum = *reinterpret_cast<const int4v_t*>(p.wsum + nb);
      const float4 wzp = has_zp ? *reinterpret_cast<const float4*>(p.wzp + nb) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      const float wsc[4] = {ws.x, ws.y, ws.z, ws.w};
      const float wz[4] = {wzp.x, wzp.y, wzp.z, wzp.w};
      float bias_f[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (p.bias) {
        const float4 bv = *reinterpret_cast<const float4*>(static_cast<const float*>(p.bias) + nb);
        bias_f[0] = bv.x;
        bias_f[1] = bv.y;
        bias_f[2] = bv.z;
        bias_f[3] = bv.w;
      }
#pragma unroll
      for (int fm = 0; fm < FM; ++fm) {
        if (mi[fm] >= p.m) continue;
        const size_t o_idx = ((size_t)slice * p.m + mi[fm]) * 4;
        float r[4];
#pragma unroll
        for (int c = 0; c < 4; ++c)
          r[c] = Rescale(acc[fn][fm][v4 * 4 + c], wsc[c], wsum[c], src_scale[fm], src_zp[fm], has_zp, wz[c], src_sum[fm],
                         in_channels);
        {
          float4 o = make_float4(r[0], r[1], r[2], r[3]);
          if (p.bias) {
            o.x += bias_f[0];
            o.y += bias_f[1];
            o.z += bias_f[2];
            o.w += bias_f[3];
          }
          *reinterpret_cast<float4*>(static_cast<float*>(p.dst) + o_idx) = o;
        }
      }
      }
    }
  }
  }
  if constexpr (DST == MLDHIP_FLOAT16) {
    // The staged tile leaves as whole slice rows: BM tokens x 8 bytes contiguous in memory, 16
    // bytes per lane.  Work-groups start at different rows, so that at any moment the stores
    // of the chip are spread over the memory channels instead of all hitting the same offset
    // of their rows.
    __syncthreads();
    constexpr int kLanesPerRow = BM / 2;               // 16 bytes = 2 tokens per lane
    constexpr int kRowsPerPass = kI8Threads / kLanesPerRow;
    const int row_lane = tid % kLanesPerRow;
    const int t0 = m0 + row_lane * 2;
    const int rot = tile * 5;
    __half* dst = static_cast<__half*>(p.dst);
    for (int pass = 0; pass < BN / 4 / kRowsPerPass; ++pass) {
      const int slice_l = (pass * kRowsPerPass + tid / kLanesPerRow + rot) % (BN / 4);
      const int slice = n0 / 4 + slice_l;
      if (slice >= p.ns || t0 >= p.m) continue;
      const u32x4 v = smem[slice_l * kLanesPerRow + row_lane];
      __half* out = dst + ((size_t)slice * p.m + t0) * 4;
      // (an odd token count makes every other row start 8 bytes off a 16-byte boundary)
      if (t0 + 1 < p.m && (p.m & 1) == 0) {
        *reinterpret_cast<u32x4*>(out) = v;
      } else {
        *reinterpret_cast<u32x2*>(out) = u32x2{v[0], v[1]};
        if (t0 + 1 < p.m) *reinterpret_cast<u32x2*>(out + 4) = u32x2{v[2], v[3]};
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// int4 / int8-weight prefill GEMM without LDS in the main loop (described for uint4; the uint8
// differences are at the kernel).
//
// Work-group = WAVES waves on one output tile of 128 channels x (FM*32) tokens; the waves split
// K WAVES ways and add their fp32 tiles through LDS at the end (fixed order).  Compiled shapes:
// 32 and 64 tokens with 8 waves (two per SIMD), 128 tokens with 4 waves (one per SIMD, its 256
// accumulators in the AGPR half of the register file).  Inside a wave every
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

// {a0 a1 a2 a3}, {b0 b1 b2 b3} -> {a0 a1 b0 b1}, {a2 a3 b2 b3}, in place.
__device__ __forceinline__ void SwapRegisters(u32x4& a, u32x4& b) {
  uint32_t a2 = a[2], a3 = a[3], b0 = b[0], b1 = b[1];
  asm volatile("v_swap_b32 %0, %1" : "+v"(a2), "+v"(b0));
  asm volatile("v_swap_b32 %0, %1" : "+v"(a3), "+v"(b1));
  a[2] = a2;
  a[3] = a3;
  b[0] = b0;
  b[1] = b1;
}

// ZP: the weights have a zero-point tensor (same shape as the scales): w = (u - shift) * s - zp * s,
// one fused multiply-add per pair of weights (zp * s is formed once per channel and scale group).
// PAIR (FM even, token count even): a lane's tokens for the MFMA pair (fm, fm+1) are neighbours
// (2j, 2j+1 instead of j, j+32), so one 16-byte load brings both activation operands.
// MULTI: the launch covers more than one matrix (the single-matrix instantiation reads its
// arguments at fixed offsets instead of through a dependent scalar load).
// WB: weight bits.  8: the packed buffer holds 16-byte blocks, word i = input channel i of the
// K-slice, byte o = output channel o of the slice, u = w + 128.  A byte permute gathers byte o of
// two words into the low bytes of two halfs, 0x6400 on top makes them 1024 + u, and
// (1024 + u - 1152) * s is the weight.  Everything else is shared with the int4 form.
// GATED: seg[0] = gate, seg[1] = up, two matrices of one shape; the launch writes
// activation(gate(x)) * up(x) to seg[0].dst.  The first half of the waves works on gate, the
// second half on up, each half splitting K among its waves; the main loop is the same.  In the
// reduction the wave that adds the copies of a register adds the two halves separately and so
// holds the gate and the up value of the same slice and token.
// DUAL: the same split of the waves for an ordinary launch: the work-group owns two neighbouring
// channel tiles (2j, 2j + 1 of the launch), one per half.  The two halves read the same
// activations, so every activation tile is fetched from L2 once for 256 channels, and there are
// half as many work-groups and reduction rounds; for launches with many tiles.
enum { kModePlain = 0, kModeGated = 1, kModeDual = 2 };
// Entry `index` of the launch's matrix list, by value.  Every field of every entry sits at a fixed
// offset of the kernel arguments, so all of them are fetched by one batch of scalar loads and
// chosen with scalar selects; indexing the list with a run-time number makes the entry's loads
// wait for the round trip that produces the number.
template <bool DYNAMIC>
__device__ __forceinline__ W4Segment PickSegment(const GemmParams& p, int index) {
  W4Segment sg = p.seg[0];
  if (DYNAMIC) {
    const W4Segment s1 = p.seg[1], s2 = p.seg[2];
#define MLD_PICK(f) sg.f = index == 2 ? s2.f : (index == 1 ? s1.f : sg.f)
    MLD_PICK(w4); MLD_PICK(scale); MLD_PICK(zp); MLD_PICK(bias); MLD_PICK(dst); MLD_PICK(partial);
    MLD_PICK(n); MLD_PICK(ns); MLD_PICK(group); MLD_PICK(tile_end); MLD_PICK(a_bytes); MLD_PICK(s_bytes);
    MLD_PICK(group_shift);
#undef MLD_PICK
  }
  return sg;
}

template <int WB, int FM, int U, int WAVES, bool ZP, bool PAIR, bool MULTI, int MODE = kModePlain>
__global__ __launch_bounds__(WAVES * 64) void fc_w4_mfma_direct_kernel(GemmParams p) {
  constexpr bool GATED = MODE == kModeGated, DUAL = MODE == kModeDual;
  static_assert(WB == 4 || WB == 8, "uint4 or uint8 weights");
  static_assert(!GATED || (!ZP && !MULTI), "the gated pair is symmetric and is the whole launch");
  static_assert(!PAIR || FM % 2 == 0, "pairs of token blocks");
  constexpr uint32_t kBlk = WB == 8 ? 16u : 8u;  // bytes of one (K-slice, output slice) block
  typedef typename std::conditional<WB == 8, u32x4, u32x2>::type wblk_t;
  constexpr int BN = 128;
  constexpr int BM = FM * 32;
  static_assert(WAVES == 4 || WAVES == 8, "the reduction's LDS buffers are sized for 4 or 8 waves");
  // K reduction buffers: [phase parity][copy][register within the phase][lane], 128 KB
  constexpr int RPH = WAVES == 4 ? 16 : 8;  // accumulator registers (x 4 MFMAs) per phase
  __shared__ float4 red[2][WAVES][RPH][64];

  // One batch of scalar loads for what the prologue reads.  (Left alone, the compiler fetches
  // every argument where it is first used: seven scalar round trips, one behind the other, in
  // front of the first operand load.  Input-only operands keep the pointers' address spaces.)
  asm volatile("" : : "s"(p.m), "s"(p.ks), "s"(p.ksplit), "s"(p.xcd_m), "s"(p.pg_groups), "s"(p.group_shift),
               "s"(p.b_bytes), "s"(p.act), "s"(p.magic_lo), "s"(p.magic_hi), "s"(p.mask_lo), "s"(p.mask_hi), "s"(p.segments),
               "s"(p.geo_tiles_m), "s"(p.geo_rect_m), "s"(p.geo_rect_n), "s"(p.geo_xm_shift), "s"(p.geo_rect_m_magic),
               "s"(p.geo_per_wave));
  asm volatile("" : : "s"(p.seg[0].w4), "s"(p.seg[0].scale), "s"(p.seg[0].ns), "s"(p.seg[0].group), "s"(p.seg[0].tile_end),
               "s"(p.seg[0].a_bytes), "s"(p.seg[0].s_bytes), "s"(p.seg[0].dst), "s"(p.seg[0].bias), "s"(p.seg[0].partial));
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int i32 = lane & 31, g2 = lane >> 5;
  // XCD-aware tile order.  Work-groups go round-robin to the 8 XCDs (id % 8), each with its own
  // L2.  The XCDs form an xcd_m x (8 / xcd_m) grid over the (token tile, channel tile) plane and
  // each owns one rectangle of it: the work-groups that share an L2 then share the activation
  // tiles and the weight tiles of that rectangle, and the L2 fetches each of them once.  Inside
  // the rectangle the token tile runs fastest, so that the tiles in flight at any time reuse the
  // same few activation tiles while the weights stream through.
  const int tiles_n_all = p.seg[MULTI ? p.segments - 1 : 0].tile_end;  // channel tiles of all matrices of the launch
  const int tiles_n = DUAL ? (tiles_n_all + 1) / 2 : tiles_n_all;        // channel tiles of the grid
  // Packed groups: this work-group's matrix and the run of tokens it multiplies (else: all tokens).
  int m_lo = 0, m_hi = p.m, pg_e = 0;
  const int tiles_m = p.geo_tiles_m;  // (packed groups: the tiles of the largest group)
  if (p.pg_groups > 0) {
    pg_e = blockIdx.z;
    const int size = min(p.pg_params[p.pg_offset + pg_e], p.pg_max);
    const int off = p.pg_params[p.pg_offset + p.pg_groups + pg_e];
    if (off < 0) return;
    m_lo = off;
    m_hi = min(off + size, p.m);
  }
  const int xcd = blockIdx.x % 8, local = blockIdx.x / 8;
  const int xm = p.xcd_m;
  const int rect_m = p.geo_rect_m, rect_n = p.geo_rect_n;
  // local / rect_m by the host's reciprocal (exact: local and rect_m are below 2^16)
  const int local_n = rect_m == 1 ? local : (int)__umulhi((uint32_t)local, p.geo_rect_m_magic);
  const int local_m = local - local_n * rect_m;
  const int tm = (xcd & (xm - 1)) * rect_m + local_m;
  const int tn_grid = (xcd >> p.geo_xm_shift) * rect_n + local_n;
  if (tm >= tiles_m || tn_grid >= tiles_n) return;
  // channel tile of the launch -> matrix of the launch (return value) and tile inside it
  auto locate = [&](int& tile) {
    int seg_index = 0;
    if (MULTI && p.segments > 1 && tile >= p.seg[0].tile_end) {
      seg_index = (p.segments > 2 && tile >= p.seg[1].tile_end) ? 2 : 1;
      tile -= p.seg[seg_index - 1].tile_end;
    }
    return seg_index;
  };
  constexpr int KW = MODE != kModePlain ? WAVES / 2 : WAVES;  // waves that share one tile's K
  const int half = MODE != kModePlain ? __builtin_amdgcn_readfirstlane(wave / KW) : 0;
  int tn = DUAL ? 2 * tn_grid + half : tn_grid;
  const bool tile_ok = !DUAL || tn < tiles_n_all;  // the last pair of an odd count has one tile
  if (!tile_ok) tn = 0;
  const int si = locate(tn);
  const W4Segment sg = PickSegment<GATED || MULTI>(p, GATED ? half : (MULTI ? si : 0));
  const int slice0 = tn * (BN / 4);  // first output slice of the tile
  const int m0 = m_lo + tm * BM;
  if (m0 >= m_hi) return;  // (packed groups: a tile beyond the group's size; the whole work-group leaves)
  const int nsi = slice0 + i32;
  const bool n_ok = tile_ok && nsi < sg.ns;

  // This wave's range of 16-channel steps.  The buffer descriptors of the weights and the
  // activations end where the wave's share of K ends, so the prefetches that run past it (and
  // past K itself) read zeros without a test in the loop; a lane without an output slice or
  // a token gets an offset beyond every buffer.
  // (blockIdx.y selects the work-group's part of K; per_wave: the steps of one of the KW * ksplit
  // shares, a multiple of U)
  const int per_wave = p.geo_per_wave;
  const int t_begin = __builtin_amdgcn_readfirstlane(((int)blockIdx.y * KW + wave % KW) * per_wave);
  // Weights with output groups: the K-slice rows of a group lie one after the other (row = the
  // group's slices), the groups one after the other.  With one group the buffer ends, for this
  // wave, where its share of K ends; with several, a prefetch past the share reads other rows of
  // the buffer, which meet the zeros that the activations' descriptor returns there.
  const bool one_group = sg.group >= sg.ns;
  const uint32_t row_w = (uint32_t)sg.group * kBlk;  // bytes per K-slice row of the weights
  const uint32_t row_x = (uint32_t)p.m * 8u;   // bytes per K-slice row of the activations
  const uint32_t k_slices_end = (uint32_t)(t_begin + per_wave) * 4u;
  // (packed groups over output groups: the buffer of all matrices, see w_base)
  const uint32_t w_end = one_group ? (uint32_t)min((uint64_t)sg.a_bytes, (uint64_t)k_slices_end * row_w)
                                   : sg.a_bytes * (uint32_t)max(p.pg_groups, 1);
  const uint32_t x_end = min((uint64_t)p.b_bytes, (uint64_t)k_slices_end * row_x);

  constexpr uint32_t kOob = 0x7FFFFFF0u;
  // packed groups: matrix pg_e of the batched buffers (weights one matrix after the other, or, with
  // output groups, the matrices of a group one after the other; scales [group][matrix][Ns][4])
  const uint8_t* w_base = sg.w4 + (one_group ? (size_t)pg_e * sg.a_bytes : 0);
  const __half* s_base = sg.scale + (size_t)pg_e * sg.ns * 4;
  const __half* z_base = (ZP ? sg.zp : sg.scale) + (size_t)pg_e * sg.ns * 4;
  const uint32_t s_bytes = sg.s_bytes - (uint32_t)pg_e * (uint32_t)sg.ns * 8u;
  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(w_base), 0, w_end, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_x =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half*>(p.act), 0, x_end, 0x00020000);
  // Second descriptors, one K-slice row further: the loads of rows 2q and 2q+1 share an offset.
  // (Base and size go through readfirstlane so that the descriptors stay in scalar registers.)
  auto uniform_ptr = [](const void* ptr, uint32_t add) {
    const uint64_t v = reinterpret_cast<uint64_t>(ptr) + add;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<void*>(((uint64_t)hi << 32) | lo);
  };
  const uint32_t w1_bytes = __builtin_amdgcn_readfirstlane(w_end > row_w ? w_end - row_w : 0u);
  const uint32_t x1_bytes = __builtin_amdgcn_readfirstlane(x_end > row_x ? x_end - row_x : 0u);
  const __amdgpu_buffer_rsrc_t rsrc_w1 = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(w_base, row_w), 0, w1_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_x1 = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.act, row_x), 0, x1_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_s =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half*>(s_base), 0, s_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_z =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half*>(z_base), 0, s_bytes, 0x00020000);

  // Per-lane byte offsets of the next step to fetch; each fetch advances them by one step.
  // Only the per-lane offset takes part in the range check of a buffer load, so the whole
  // address lives there.
  const uint32_t step_w = 4u * row_w, step_x = 4u * row_x;
  // (the slice's output group and its place inside it: a shift where the group size allows)
  const uint32_t nsi_group = sg.group_shift >= 0 ? (uint32_t)nsi >> sg.group_shift : (uint32_t)(nsi / sg.group);
  const uint32_t nsi_in_group = (uint32_t)nsi - nsi_group * (uint32_t)sg.group;
  const uint32_t col_w = one_group ? (uint32_t)nsi * kBlk
                                   : ((nsi_group * (uint32_t)max(p.pg_groups, 1) + (uint32_t)pg_e) * (uint32_t)p.ks * (uint32_t)sg.group +
                                      nsi_in_group) * kBlk;
  uint32_t vw0 = n_ok ? ((uint32_t)t_begin * 4u + (uint32_t)g2 * 2u) * row_w + col_w : kOob;
  const uint32_t vs = n_ok ? (uint32_t)nsi * 8u : kOob;
  // token of this lane in MFMA token block fm
  auto token = [&](int fm) { return PAIR ? m0 + (fm / 2) * 64 + 2 * i32 + (fm & 1) : m0 + fm * 32 + i32; };
  constexpr int NX = PAIR ? FM / 2 : FM;  // activation load items per K-slice row
  uint32_t vx[NX];
#pragma unroll
  for (int i = 0; i < NX; ++i) {
    const int mi = token(PAIR ? 2 * i : i);
    vx[i] = mi < m_hi ? ((uint32_t)t_begin * 4u + (uint32_t)g2 * 2u) * row_x + (uint32_t)mi * 8u : kOob;
  }
  const uint32_t group_bytes = (uint32_t)sg.ns * 8u * (uint32_t)max(p.pg_groups, 1);  // one scale group: [matrices][Ns][4] halfs

  wblk_t rw[U][2];
  u32x2 rsc[U], rzp[U], rx[U][NX][2];
  u32x4 rxp[U][NX][2];  // PAIR: {token 2j: 4 halfs, token 2j+1: 4 halfs} per K-slice row
  auto load_step = [&](int t, bool with_scale, wblk_t (&w)[2], u32x2& sc, u32x2& zpv, u32x2 (&x)[NX][2],
                       u32x4 (&xp)[NX][2]) {
    // The scales (and zero points) of a pair of steps (t - 1, t), t odd, which share a group
    // because a group holds an even number of steps.  They travel with the odd step: by then
    // both users of the previous pair are done with the registers.  First in the stage, so
    // that waiting for them holds back as few younger loads as possible.
    if (with_scale) {
      sc = __builtin_amdgcn_raw_buffer_load_b64(rsrc_s, vs + (uint32_t)(t >> p.group_shift) * group_bytes, 0, 0);
      if (ZP) zpv = __builtin_amdgcn_raw_buffer_load_b64(rsrc_z, vs + (uint32_t)(t >> p.group_shift) * group_bytes, 0, 0);
    }
    if constexpr (WB == 8) {
      w[0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, vw0, 0, 0);
      w[1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w1, vw0, 0, 0);
    } else {
      w[0] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, vw0, 0, 0);
      w[1] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w1, vw0, 0, 0);
    }
    vw0 += step_w;
#pragma unroll
    for (int i = 0; i < NX; ++i) {
      if (PAIR) {
        xp[i][0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, vx[i], 0, 0);
        xp[i][1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_x1, vx[i], 0, 0);
      } else {
        x[i][0] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_x, vx[i], 0, 0);
        x[i][1] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_x1, vx[i], 0, 0);
      }
      vx[i] += step_x;
    }
  };

  float16_t acc[4][FM];
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4)
#pragma unroll
    for (int fm = 0; fm < FM; ++fm)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t4][fm][v] = 0.0f;

  // The exponent patterns are parked in vector registers: (x & mask) | magic then selects to one
  // v_and_or_b32 (the instruction reads at most one scalar register) without inline asm, so the
  // compiler sees every vector write near the MFMAs and can place the wait states it needs (as
  // fast as the asm form: same-box runs agree within 2 %).
  uint32_t magic_lo = p.magic_lo, magic_hi = p.magic_hi;
  asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));
  const half2_t off_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f};
  const half2_t off_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
  const half2_t off_w8 = {(_Float16)-1152.0f, (_Float16)-1152.0f};

  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    load_step(t_begin + u, u % 2 == 1, rw[u], rsc[u & ~1], rzp[u & ~1], rx[u], rxp[u]);
    __builtin_amdgcn_sched_barrier(0);
  }
  if constexpr (FM == 1) {
  // 32-token tiles: four weight words per MFMA keep the vector ALU busier than the matrix pipe
  // whatever the order (two waves per SIMD fill each other's gaps), and the plain loop is the
  // faster one there.
    for (int tt = 0; tt < per_wave; tt += U) {
  #pragma unroll
      for (int u = 0; u < U; ++u) {
        const int t = t_begin + tt + u;
        // consume stage u
        const wblk_t wr[2] = {rw[u][0], rw[u][1]};
        const u32x2 scr = rsc[u & ~1];
        u32x4 blk = {0u, 0u, 0u, 0u}, blk8 = blk;
        if constexpr (WB == 4) {
          blk = u32x4{wr[0][0], wr[0][1], wr[1][0], wr[1][1]};
          blk8 = u32x4{blk[0] >> 8, blk[1] >> 8, blk[2] >> 8, blk[3] >> 8};
        }
        const half2_t sc01 = AsHalf2(scr[0]), sc23 = AsHalf2(scr[1]);
        half2_t zp01 = {(_Float16)0.0f, (_Float16)0.0f}, zp23 = zp01;
        if (ZP) {
          zp01 = AsHalf2(rzp[u & ~1][0]);
          zp23 = AsHalf2(rzp[u & ~1][1]);
        }
        if (PAIR) {
          // The two 16-byte loads of a token pair hold {token 2j, token 2j+1} of K-slice rows 2q
          // and 2q+1; exchanging the inner halves makes each of them one token's operand.
  #pragma unroll
          for (int i = 0; i < NX; ++i) {
            SwapRegisters(rxp[u][i][0], rxp[u][i][1]);
          }
        }
  #pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) {
          const half2_t sp = (t4 & 2) ? sc23 : sc01;
          const half2_t s2 = (t4 & 1) ? __builtin_shufflevector(sp, sp, 1, 1) : __builtin_shufflevector(sp, sp, 0, 0);
          const half2_t off = WB == 8 ? off_w8 : ((t4 & 1) ? off_hi : off_lo);
          // zero point: (u - shift) * s - zp * s in one fused step, so that a fractional zero point
          // costs one extra rounding of zp * s and not a rounding of shift + zp to an integer
          half2_t mzs = {(_Float16)0.0f, (_Float16)0.0f};
          if (ZP) {
            const half2_t zq = (t4 & 2) ? zp23 : zp01;
            mzs = -(((t4 & 1) ? __builtin_shufflevector(zq, zq, 1, 1) : __builtin_shufflevector(zq, zq, 0, 0)) * s2);
          }
          u32x4 aop;
  #pragma unroll
          for (int wd = 0; wd < 4; ++wd) {
            uint32_t bits;
            if constexpr (WB == 8) {
              // bytes t4 of the words of input channels 2*wd, 2*wd + 1 -> the low bytes of two halfs
              const uint32_t sel = 0x0c000c00u | (uint32_t)t4 | ((uint32_t)(4 + t4) << 16);
              bits = __builtin_amdgcn_perm(wr[wd >> 1][2 * (wd & 1) + 1], wr[wd >> 1][2 * (wd & 1)], sel) | magic_lo;
            } else {
              const uint32_t x = (t4 & 2) ? blk8[wd] : blk[wd];
              bits = (t4 & 1) ? ((x & p.mask_hi) | magic_hi) : ((x & p.mask_lo) | magic_lo);
            }
            const half2_t centred = AsHalf2(bits) + off;  // exact: u - shift
            aop[wd] = AsU32(ZP ? __builtin_elementwise_fma(centred, s2, mzs) : centred * s2);
          }
  #pragma unroll
          for (int fm = 0; fm < FM; ++fm) {
            const u32x4 bop = PAIR ? rxp[u][fm / 2][fm & 1]
                                   : u32x4{rx[u][PAIR ? 0 : fm][0][0], rx[u][PAIR ? 0 : fm][0][1], rx[u][PAIR ? 0 : fm][1][0],
                                           rx[u][PAIR ? 0 : fm][1][1]};
            acc[t4][fm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, aop),
                                                                 __builtin_bit_cast(half8_t, bop), acc[t4][fm], 0, 0, 0);
          }
        }
        // refill stage u with step t + U; the fences keep the loads of a stage together and in
        // program order, so that waiting for one stage leaves the younger ones in flight
        __builtin_amdgcn_sched_barrier(0);
        load_step(t + U, u % 2 == 1, rw[u], rsc[u & ~1], rzp[u & ~1], rx[u], rxp[u]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  } else {
    // The loop is software-pipelined by one weight operand: while the FM MFMAs of output-channel phase
    // t4 run, the vector ALU dequantizes the operand of phase t4 + 1 (at t4 = 3: phase 0 of the next
    // stage), 4 / FM words behind every MFMA.  A wave issues in order, and an MFMA that waits for the
    // matrix pipe holds back whatever follows it, so a run of MFMAs followed by a run of vector
    // instructions serialises the two; placed between the MFMAs, the vector instructions issue in the
    // 32 cycles each MFMA occupies the pipe.  The scheduling groups at the end of a step ask for that order.
    struct Stage {
      u32x4 blk, blk8;   // WB == 4: the stage's 32 weights, and the same shifted by 8 bits
      wblk_t w0, w1;     // WB == 8: the two blocks
      half2_t sc01, sc23, zp01, zp23;
    };
    auto open_stage = [&](int u) {
      Stage st;
      st.w0 = rw[u][0];
      st.w1 = rw[u][1];
      st.blk = st.blk8 = u32x4{0u, 0u, 0u, 0u};
      if constexpr (WB == 4) {
        st.blk = u32x4{rw[u][0][0], rw[u][0][1], rw[u][1][0], rw[u][1][1]};
        st.blk8 = u32x4{st.blk[0] >> 8, st.blk[1] >> 8, st.blk[2] >> 8, st.blk[3] >> 8};
      }
      const u32x2 scr = rsc[u & ~1];
      st.sc01 = AsHalf2(scr[0]);
      st.sc23 = AsHalf2(scr[1]);
      st.zp01 = st.zp23 = half2_t{(_Float16)0.0f, (_Float16)0.0f};
      if (ZP) {
        st.zp01 = AsHalf2(rzp[u & ~1][0]);
        st.zp23 = AsHalf2(rzp[u & ~1][1]);
      }
      return st;
    };
    // word wd (input channels 2 wd, 2 wd + 1 of the step's 8) of the operand of phase t4
    auto dequant_word = [&](const Stage& st, int t4, int wd) -> uint32_t {
      const half2_t sp = (t4 & 2) ? st.sc23 : st.sc01;
      const half2_t s2 = (t4 & 1) ? __builtin_shufflevector(sp, sp, 1, 1) : __builtin_shufflevector(sp, sp, 0, 0);
      const half2_t off = WB == 8 ? off_w8 : ((t4 & 1) ? off_hi : off_lo);
      // zero point: (u - shift) * s - zp * s in one fused step, so that a fractional zero point
      // costs one extra rounding of zp * s and not a rounding of shift + zp to an integer
      half2_t mzs = {(_Float16)0.0f, (_Float16)0.0f};
      if (ZP) {
        const half2_t zq = (t4 & 2) ? st.zp23 : st.zp01;
        mzs = -(((t4 & 1) ? __builtin_shufflevector(zq, zq, 1, 1) : __builtin_shufflevector(zq, zq, 0, 0)) * s2);
      }
      uint32_t bits;
      if constexpr (WB == 8) {
        // bytes t4 of the words of input channels 2*wd, 2*wd + 1 -> the low bytes of two halfs
        const uint32_t sel = 0x0c000c00u | (uint32_t)t4 | ((uint32_t)(4 + t4) << 16);
        const wblk_t& wr = (wd >> 1) ? st.w1 : st.w0;
        bits = __builtin_amdgcn_perm(wr[2 * (wd & 1) + 1], wr[2 * (wd & 1)], sel) | magic_lo;
      } else {
        const uint32_t x = (t4 & 2) ? st.blk8[wd] : st.blk[wd];
        bits = (t4 & 1) ? ((x & p.mask_hi) | magic_hi) : ((x & p.mask_lo) | magic_lo);
      }
      const half2_t centred = AsHalf2(bits) + off;  // exact: u - shift
      return AsU32(ZP ? __builtin_elementwise_fma(centred, s2, mzs) : centred * s2);
    };
    // vector instructions per MFMA of a step: 13-14 per phase (3 per word, the scale broadcast, the shifts of a new stage)
    constexpr int kValuPerMfma = FM >= 4 ? 4 : (FM == 2 ? 8 : 16);
    Stage cur = open_stage(0);
    u32x4 aop;
  #pragma unroll
    for (int wd = 0; wd < 4; ++wd) aop[wd] = dequant_word(cur, 0, wd);
    __builtin_amdgcn_sched_barrier(0);
    for (int tt = 0; tt < per_wave; tt += U) {
  #pragma unroll
      for (int u = 0; u < U; ++u) {
        const int t = t_begin + tt + u;
        if (PAIR) {
          // The two 16-byte loads of a token pair hold {token 2j, token 2j+1} of K-slice rows 2q
          // and 2q+1; exchanging the inner halves makes each of them one token's operand.
  #pragma unroll
          for (int i = 0; i < NX; ++i) {
            SwapRegisters(rxp[u][i][0], rxp[u][i][1]);
          }
        }
        Stage nxt = cur;
  #pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) {
          // the operand that follows this one: the next phase of this stage, or phase 0 of the next
          // stage (after the last step: of a stage that was fetched beyond the range and holds zeros)
          if (t4 == 3) nxt = open_stage((u + 1) % U);
          const int t4n = (t4 + 1) & 3;
          u32x4 anext;
  #pragma unroll
          for (int fm = 0; fm < FM; ++fm) {
            const u32x4 bop = PAIR ? rxp[u][fm / 2][fm & 1]
                                   : u32x4{rx[u][PAIR ? 0 : fm][0][0], rx[u][PAIR ? 0 : fm][0][1], rx[u][PAIR ? 0 : fm][1][0],
                                           rx[u][PAIR ? 0 : fm][1][1]};
            acc[t4][fm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, aop),
                                                                 __builtin_bit_cast(half8_t, bop), acc[t4][fm], 0, 0, 0);
          }
  #pragma unroll
          for (int wd = 0; wd < 4; ++wd) anext[wd] = dequant_word(nxt, t4n, wd);
          aop = anext;
        }
        cur = nxt;
        // the order of the step's instructions: one MFMA, then its share of the vector instructions
  #pragma unroll
        for (int i = 0; i < 4 * FM; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, kValuPerMfma, 0);
        }
        // refill stage u with step t + U; the fences keep the loads of a stage together and in
        // program order, so that waiting for one stage leaves the younger ones in flight
        __builtin_amdgcn_sched_barrier(0);
        load_step(t + U, u % 2 == 1, rw[u], rsc[u & ~1], rzp[u & ~1], rx[u], rxp[u]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // K-split reduction, spread over all waves.  The tile goes through LDS in phases of RPH
  // accumulator registers per lane (x 4 MFMAs): every wave writes its copy, then wave w adds the
  // WAVES copies of registers w, w + WAVES, ... in a fixed order and stores that part of the
  // output.  Two buffers alternate, so one barrier per phase is enough: a wave that writes
  // phase p + 2 has passed the barrier of phase p + 1, which every wave reaches only after its
  // reads of phase p.  In the 32x32 result, register v of lane (g2, i32) belongs to output slice
  // 8*(v/4) + 4*g2 + v%4 and token i32, and the four MFMAs hold the slice's four channels: one
  // 8-byte store.
  // GATED: copies 0 .. KW-1 are gate's, the others up's; the two sums are rounded to fp16 (+ bias)
  // as the two FullyConnected nodes would store them, then combined in fp32.  DUAL: the two sums
  // belong to the two tiles of the work-group.
  int tile_b = 2 * tn_grid + 1;  // DUAL: the second tile
  const bool tile_b_ok = DUAL && tile_b < tiles_n_all;
  if (!tile_b_ok) tile_b = 0;
  int tile_a = DUAL ? 2 * tn_grid : tn;
  const int seg_a = DUAL ? locate(tile_a) : si, seg_b = DUAL ? locate(tile_b) : 0;
  const W4Segment sga = PickSegment<!GATED && MULTI>(p, GATED ? 0 : (MULTI ? seg_a : 0));
  const W4Segment sgb = PickSegment<GATED || MULTI>(p, GATED ? 1 : (MULTI ? seg_b : 0));
  const int slice0_a = DUAL ? tile_a * (BN / 4) : slice0, slice0_b = tile_b * (BN / 4);
  // one slice of four channels of one token: the K-split partial sums, or the fp16 result
  auto store = [&](const W4Segment& sgx, int slice, int mi, const float4& sum) {
    if (p.ksplit > 1) {
      // this work-group's share of K: fp32 sums for the second pass
      *reinterpret_cast<float4*>(sgx.partial + (((size_t)blockIdx.y * sgx.ns + slice) * p.m + mi) * 4) = sum;
      return;
    }
    __half h[4] = {__float2half_rn(sum.x), __float2half_rn(sum.y), __float2half_rn(sum.z), __float2half_rn(sum.w)};
    if (sgx.bias) {
#pragma unroll
      for (int t4 = 0; t4 < 4; ++t4) h[t4] = __hadd(h[t4], sgx.bias[slice * 4 + t4]);
    }
    u32x2 o;
    o[0] = (uint32_t)__half_as_ushort(h[0]) | ((uint32_t)__half_as_ushort(h[1]) << 16);
    o[1] = (uint32_t)__half_as_ushort(h[2]) | ((uint32_t)__half_as_ushort(h[3]) << 16);
    *reinterpret_cast<u32x2*>(sgx.dst + ((size_t)slice * p.m + mi) * 4) = o;
  };
  static_assert(16 % RPH == 0 && RPH % WAVES == 0, "phases tile the 16 registers, waves tile a phase");
#pragma unroll
  for (int fm = 0; fm < FM; ++fm) {
    const int mi = token(fm);
#pragma unroll
    for (int ph = 0; ph < 16 / RPH; ++ph) {
      const int buf = (fm * (16 / RPH) + ph) & 1;
#pragma unroll
      for (int j = 0; j < RPH; ++j) {
        const int v = ph * RPH + j;
        red[buf][wave][j][lane] = make_float4(acc[0][fm][v], acc[1][fm][v], acc[2][fm][v], acc[3][fm][v]);
      }
      LdsBarrier();
#pragma unroll
      for (int q = 0; q < RPH / WAVES; ++q) {
        const int j = q * WAVES + wave;
        float4 sum = red[buf][0][j][lane];
#pragma unroll
        for (int c = 1; c < KW; ++c) {
          const float4 o = red[buf][c][j][lane];
          sum.x += o.x;
          sum.y += o.y;
          sum.z += o.z;
          sum.w += o.w;
        }
        const int v = ph * RPH + j;
        const int slice_l = 8 * (v >> 2) + 4 * g2 + (v & 3);  // slice inside the tile
        if constexpr (MODE != kModePlain) {
          float4 sum_b = red[buf][KW][j][lane];
#pragma unroll
          for (int c = KW + 1; c < WAVES; ++c) {
            const float4 o = red[buf][c][j][lane];
            sum_b.x += o.x;
            sum_b.y += o.y;
            sum_b.z += o.z;
            sum_b.w += o.w;
          }
          if (DUAL) {
            if (mi < m_hi && slice0_a + slice_l < sga.ns) store(sga, slice0_a + slice_l, mi, sum);
            if (mi < m_hi && tile_b_ok && slice0_b + slice_l < sgb.ns) store(sgb, slice0_b + slice_l, mi, sum_b);
          } else if (mi < m_hi && slice0 + slice_l < sga.ns) {
            const int slice = slice0 + slice_l;
            const float g[4] = {sum.x, sum.y, sum.z, sum.w}, up[4] = {sum_b.x, sum_b.y, sum_b.z, sum_b.w};
            __half h[4];
#pragma unroll
            for (int t4 = 0; t4 < 4; ++t4) {
              __half hg = __float2half_rn(g[t4]), hu = __float2half_rn(up[t4]);
              if (sga.bias) hg = __hadd(hg, sga.bias[slice * 4 + t4]);
              if (sgb.bias) hu = __hadd(hu, sgb.bias[slice * 4 + t4]);
              h[t4] = __float2half_rn(GatedActivation(p.gate_activation, __half2float(hg), __half2float(hu)));
            }
            u32x2 o;
            o[0] = (uint32_t)__half_as_ushort(h[0]) | ((uint32_t)__half_as_ushort(h[1]) << 16);
            o[1] = (uint32_t)__half_as_ushort(h[2]) | ((uint32_t)__half_as_ushort(h[3]) << 16);
            *reinterpret_cast<u32x2*>(sga.dst + ((size_t)slice * p.m + mi) * 4) = o;
          }
        } else if (mi < m_hi && slice0 + slice_l < sg.ns) {
          store(sg, slice0 + slice_l, mi, sum);
        }
      }
    }
  }
}

template <int WB, int FM, int U, int WAVES, bool PAIR, int MODE>
void LaunchDirectW(bool zp, dim3 grid, hipStream_t stream, const GemmParams& p) {
  const dim3 block(WAVES * 64);
  if (zp && p.segments > 1)
    hipLaunchKernelGGL((fc_w4_mfma_direct_kernel<WB, FM, U, WAVES, true, PAIR, true, MODE>), grid, block, 0, stream, p);
  else if (zp)
    hipLaunchKernelGGL((fc_w4_mfma_direct_kernel<WB, FM, U, WAVES, true, PAIR, false, MODE>), grid, block, 0, stream, p);
  else if (p.segments > 1)
    hipLaunchKernelGGL((fc_w4_mfma_direct_kernel<WB, FM, U, WAVES, false, PAIR, true, MODE>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((fc_w4_mfma_direct_kernel<WB, FM, U, WAVES, false, PAIR, false, MODE>), grid, block, 0, stream, p);
}
// DUAL_OK: the two-tile mode is compiled for this shape.
template <int FM, int U, int WAVES, bool PAIR, bool DUAL_OK>
void LaunchDirect(int weight_bits, bool zp, dim3 grid, hipStream_t stream, const GemmParams& p) {
  if (p.gate_activation != 0) {  // gated pair: symmetric weights
    if (weight_bits == 8)
      hipLaunchKernelGGL((fc_w4_mfma_direct_kernel<8, FM, U, WAVES, false, PAIR, false, kModeGated>), grid,
                         dim3(WAVES * 64), 0, stream, p);
    else
      hipLaunchKernelGGL((fc_w4_mfma_direct_kernel<4, FM, U, WAVES, false, PAIR, false, kModeGated>), grid,
                         dim3(WAVES * 64), 0, stream, p);
    return;
  }
  if constexpr (DUAL_OK) {
    if (p.dual) {
      if (weight_bits == 8)
        LaunchDirectW<8, FM, U, WAVES, PAIR, kModeDual>(zp, grid, stream, p);
      else
        LaunchDirectW<4, FM, U, WAVES, PAIR, kModeDual>(zp, grid, stream, p);
      return;
    }
  }
  if (weight_bits == 8)
    LaunchDirectW<8, FM, U, WAVES, PAIR, kModePlain>(zp, grid, stream, p);
  else
    LaunchDirectW<4, FM, U, WAVES, PAIR, kModePlain>(zp, grid, stream, p);
}

// ------------------------------------------------------------------------------------------
// int4-weight GEMM for many tokens with both operands shared through LDS.
//
// Work-group = 4 waves (2 x 2) on 256 channels x 256 tokens, each wave 128 x 128 (its 256
// accumulators in the AGPR half of the register file), K in stages of 32 input channels (two MFMA
// steps).  Per stage and work-group:
//  - weights: 64 slices x 8 K-slice rows of 8-byte blocks.  Thread (slice = lane, K-slice pair = wave)
//    loads its two blocks four stages ahead, dequantizes them once for the whole work-group (the
//    direct kernel dequantizes every weight once per 128-token tile) into the four A operands of
//    MFMAs t = 0..3 (rows = channels 4 * slice + t) and writes them to LDS as
//    [MFMA step][K half][t][slice][16 bytes]: a lane's operand read is one aligned 16-byte item and a
//    wave's read covers consecutive items.  Two slots: the stage being multiplied and the next one.
//  - activations: 8 K-slice rows x 256 tokens x 8 bytes, copied global -> LDS by loads that write
//    LDS directly, in the tensor's own order ([row][token][4 halfs], 2 KB per row).  A lane's B
//    operand (8 consecutive input channels of one token) is the two 8-byte items of rows 2q, 2q + 1:
//    one ds_read2st64_b64.  Four slots, three stages of copies in flight.
// One barrier per stage, between its two MFMA steps: step 0 runs next to the reads of step 1, the
// copies and loads of later stages and the dequantization of the next stage, step 1 next to the
// operand reads of the next stage's step 0.  The LDS side is inline asm: the compiler does not know
// what the LDS-writing loads touch and would wait for all of them in front of any LDS access it sees.
// ------------------------------------------------------------------------------------------
constexpr int kTlThreads = 256;
constexpr int kTlASlot = 16384, kTlBSlot = 16384;  // bytes of one stage of either tile
constexpr int kTlBBase = 2 * kTlASlot;            // the activation slots follow the two weight slots

template <int OFF>
__device__ __forceinline__ void DsWrite128(uint32_t addr, const u32x4& v) {
  asm volatile("ds_write_b128 %0, %1 offset:%2" : : "v"(addr), "v"(v), "n"(OFF) : "memory");
}
// two 8-byte items, 512 * O0 and 512 * O1 bytes behind addr
template <int O0, int O1>
__device__ __forceinline__ void DsRead2x64(u32x4& dst, uint32_t addr) {
  asm volatile("ds_read2st64_b64 %0, %1 offset0:%2 offset1:%3" : "=v"(dst) : "v"(addr), "n"(O0), "n"(O1));
}

template <bool ZP>
__global__ __launch_bounds__(kTlThreads) void fc_w4_mfma_tiled_kernel(GemmParams p) {
  __shared__ u32x4 smem[(2 * kTlASlot + 4 * kTlBSlot) / 16];
  const LdsPtr lds = (LdsPtr)smem;
  const uint32_t lds_base = (uint32_t)(size_t)lds;
  asm volatile("" : : "s"(p.m), "s"(p.ks), "s"(p.group_shift), "s"(p.b_bytes), "s"(p.act), "s"(p.magic_lo), "s"(p.magic_hi),
               "s"(p.mask_lo), "s"(p.mask_hi));
  asm volatile("" : : "s"(p.seg[0].w4), "s"(p.seg[0].scale), "s"(p.seg[0].ns), "s"(p.seg[0].group), "s"(p.seg[0].a_bytes),
               "s"(p.seg[0].s_bytes), "s"(p.seg[0].dst), "s"(p.seg[0].bias), "s"(p.seg[0].group_shift));
  const W4Segment sg = p.seg[0];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave & 1, wm = wave >> 1;
  const int r32 = lane & 31, g2 = lane >> 5;

  // Tile order: XCD x (work-groups go round-robin to the 8 XCDs) takes a contiguous range of a
  // numbering that walks blocks of 8 channel tiles token tile by token tile, so that the tiles
  // which share an L2 form a compact rectangle.
  const int tiles_n = (sg.ns + 63) / 64;
  const int tiles_m = (p.m + 255) / 256;
  const int per_xcd = (tiles_n * tiles_m + 7) / 8;
  const int tile = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (tile >= tiles_n * tiles_m) return;
  int tn, tm;
  {
    const int full = tiles_n / 8;
    if (tile < full * 8 * tiles_m) {
      const int sc = tile / (8 * tiles_m), within = tile % (8 * tiles_m);
      tn = sc * 8 + within % 8;
      tm = within / 8;
    } else {
      const int rest = tile - full * 8 * tiles_m, width = tiles_n - full * 8;
      tn = full * 8 + rest % width;
      tm = rest / width;
    }
  }
  const int slice0 = tn * 64;
  const int m0 = tm * 256;

  constexpr uint32_t kOob = 0x7FFFFFF0u;
  const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(sg.w4), 0, sg.a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<__half*>(p.act), 0, p.b_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(const_cast<__half*>(sg.scale), 0, sg.s_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_z =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half*>(ZP ? sg.zp : sg.scale), 0, sg.s_bytes, 0x00020000);

  // Weight duty: slice `lane` of the tile, K-slice rows 2 * wave and 2 * wave + 1 of every stage.
  // (Rows past K are beyond the buffer with one output group and read zeros; with several they are
  // rows of other groups, finite values that meet the zeros the activations' descriptor returns.)
  const int nsi = slice0 + lane;
  const bool n_ok = nsi < sg.ns;
  const bool one_group = sg.group >= sg.ns;
  const uint32_t row_w = (uint32_t)sg.group * 8u;
  const uint32_t nsi_group = sg.group_shift >= 0 ? (uint32_t)nsi >> sg.group_shift : (uint32_t)(nsi / sg.group);
  const uint32_t nsi_in_group = (uint32_t)nsi - nsi_group * (uint32_t)sg.group;
  const uint32_t col_w = one_group ? (uint32_t)nsi * 8u : (nsi_group * (uint32_t)p.ks * (uint32_t)sg.group + nsi_in_group) * 8u;
  uint32_t vw = n_ok ? (uint32_t)(2 * wave) * row_w + col_w : kOob;
  const uint32_t step_w = 8u * row_w;
  const uint32_t vs = n_ok ? (uint32_t)nsi * 8u : kOob;
  const uint32_t group_bytes = (uint32_t)sg.ns * 8u;
  const uint32_t addr_w = lds_base + (uint32_t)((wave * 4) * 64 + lane) * 16u;

  // Copy duty: rows 2 * wave, 2 * wave + 1 of every stage, two halves of 128 tokens (a lane moves a
  // pair of tokens; the token count is even, so a pair is inside the row or past it).
  const uint32_t row_x = (uint32_t)p.m * 8u, step_x = 8u * row_x;
  uint32_t vb[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int tok = m0 + (c & 1) * 128 + 2 * lane;
    vb[c] = tok < p.m ? (uint32_t)(2 * wave + (c >> 1)) * row_x + (uint32_t)tok * 8u : kOob;
  }
  auto copy_one = [&](int slot, int c) {
    CopyToLds(rsrc_x, lds + kTlBBase + slot * kTlBSlot + ((2 * wave + (c >> 1)) * 256 + (c & 1) * 128) * 8, vb[c]);
    vb[c] += step_x;
  };

  // operand addresses (slot, MFMA step and operand number go into the instructions' offsets)
  const uint32_t addr_a = lds_base + (uint32_t)((g2 * 4) * 64 + wn * 32 + r32) * 16u;
  const uint32_t addr_b0 = lds_base + (uint32_t)kTlBBase + (uint32_t)((2 * g2) * 256 + wm * 128 + r32) * 8u;
  const uint32_t addr_b1 = addr_b0 + 256u;  // token blocks 1 and 3

  // the registers of four stages of weights in flight
  u32x2 wq[4][2], wsc[4], wzp[4];
  auto load_w = [&](int set, int t) {
    const uint32_t so = vs + (uint32_t)((2 * t) >> p.group_shift) * group_bytes;
    wsc[set] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_s, so, 0, 0);
    if (ZP) wzp[set] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_z, so, 0, 0);
    wq[set][0] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, vw, 0, 0);
    wq[set][1] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, vw + row_w, 0, 0);
    vw += step_w;
  };
  constexpr int kLw = ZP ? 4 : 3;  // loads of one stage of weights

  uint32_t magic_lo = p.magic_lo, magic_hi = p.magic_hi;
  asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));
  const half2_t off_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f};
  const half2_t off_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
  // word wd (input channels 2 wd, 2 wd + 1 of the 8) of the operand of MFMA t4, from register set `set`
  auto dequant_word = [&](int set, int t4, int wd) -> uint32_t {
    const uint32_t sp = (t4 & 2) ? wsc[set][1] : wsc[set][0];
    const half2_t sph = AsHalf2(sp);
    const half2_t s2 = (t4 & 1) ? __builtin_shufflevector(sph, sph, 1, 1) : __builtin_shufflevector(sph, sph, 0, 0);
    half2_t mzs = {(_Float16)0.0f, (_Float16)0.0f};
    if (ZP) {
      const half2_t zq = AsHalf2((t4 & 2) ? wzp[set][1] : wzp[set][0]);
      mzs = -(((t4 & 1) ? __builtin_shufflevector(zq, zq, 1, 1) : __builtin_shufflevector(zq, zq, 0, 0)) * s2);
    }
    const uint32_t raw = wq[set][wd >> 1][wd & 1];
    const uint32_t x = (t4 & 2) ? raw >> 8 : raw;
    const uint32_t bits = (t4 & 1) ? ((x & p.mask_hi) | magic_hi) : ((x & p.mask_lo) | magic_lo);
    const half2_t centred = AsHalf2(bits) + ((t4 & 1) ? off_hi : off_lo);  // exact: u - 8
    return AsU32(ZP ? __builtin_elementwise_fma(centred, s2, mzs) : centred * s2);
  };

  float16_t acc[4][4];
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4)
#pragma unroll
    for (int fm = 0; fm < 4; ++fm)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t4][fm][v] = 0.0f;

  // Waits until the activation copies of the next stage have landed (the loads issued behind them
  // stay in flight: two more stages of copies and three of weights) and this wave's LDS writes are
  // done, then meets the other waves.
  auto stage_barrier = [&]() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(8 + 3 * kLw) : "memory");
  };

  // Prologue, in the order the loop continues: weights 0, then (copies s, weights s + 1) for s = 0, 1, 2.
  const int stages = (p.ks + 7) / 8;
  load_w(0, 0);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int s0 = 0; s0 < 3; ++s0) {
#pragma unroll
    for (int c = 0; c < 4; ++c) copy_one(s0, c);
    __builtin_amdgcn_sched_barrier(0);
    load_w(s0 + 1, s0 + 1);
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4) {
    u32x4 aop;
#pragma unroll
    for (int wd = 0; wd < 4; ++wd) aop[wd] = dequant_word(0, t4, wd);
    switch (t4) {
      case 0: DsWrite128<0 * 1024>(addr_w, aop); break;
      case 1: DsWrite128<1 * 1024>(addr_w, aop); break;
      case 2: DsWrite128<2 * 1024>(addr_w, aop); break;
      default: DsWrite128<3 * 1024>(addr_w, aop); break;
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  stage_barrier();
  u32x4 fa[2][4], fb[2][4];
  DsRead128<0 * 1024>(fa[0][0], addr_a);
  DsRead128<1 * 1024>(fa[0][1], addr_a);
  DsRead128<2 * 1024>(fa[0][2], addr_a);
  DsRead128<3 * 1024>(fa[0][3], addr_a);
  DsRead2x64<0, 4>(fb[0][0], addr_b0);
  DsRead2x64<0, 4>(fb[0][1], addr_b1);
  DsRead2x64<1, 5>(fb[0][2], addr_b0);
  DsRead2x64<1, 5>(fb[0][3], addr_b1);

  // Stage t, t % 4 = S known at compile time: every slot, register set and offset is a constant.
  auto stage = [&](auto tag, int t) {
    constexpr int S = decltype(tag)::value;
    constexpr int SA = S & 1, SB = S;                  // slots of this stage
    constexpr int NA = (S + 1) & 1, NB = (S + 1) & 3;  // slots of the next stage
    constexpr int RB = (S + 3) & 3;                    // activation slot that takes stage t + 3
    constexpr int NW = (S + 1) & 3;                    // register set of the next stage's weights
    LdsWait(fa[0]);
    LdsWait(fb[0]);
    __builtin_amdgcn_sched_barrier(0);
    u32x4 aop = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int idx = 0; idx < 16; ++idx) {
      const int t4 = idx / 4, fm = idx % 4;
      acc[t4][fm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, fa[0][t4]),
                                                           __builtin_bit_cast(half8_t, fb[0][fm]), acc[t4][fm], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      // the operands of step 1, the copies of stage t + 3, the weights of stage t + 4
      switch (idx) {
        case 0: DsRead128<SA * kTlASlot + 8192 + 0 * 1024>(fa[1][0], addr_a); break;
        case 1: DsRead128<SA * kTlASlot + 8192 + 1 * 1024>(fa[1][1], addr_a); break;
        case 2: DsRead128<SA * kTlASlot + 8192 + 2 * 1024>(fa[1][2], addr_a); break;
        case 3: DsRead128<SA * kTlASlot + 8192 + 3 * 1024>(fa[1][3], addr_a); break;
        case 4: DsRead2x64<SB * 32 + 16 + 0, SB * 32 + 16 + 4>(fb[1][0], addr_b0); break;
        case 5: DsRead2x64<SB * 32 + 16 + 0, SB * 32 + 16 + 4>(fb[1][1], addr_b1); break;
        case 6: DsRead2x64<SB * 32 + 16 + 1, SB * 32 + 16 + 5>(fb[1][2], addr_b0); break;
        case 7: DsRead2x64<SB * 32 + 16 + 1, SB * 32 + 16 + 5>(fb[1][3], addr_b1); break;
        case 8: copy_one(RB, 0); break;
        case 9: copy_one(RB, 1); break;
        case 10: copy_one(RB, 2); break;
        case 11: copy_one(RB, 3); break;
        case 12: load_w(S, t + 4); break;
        default: break;
      }
      // one word of the next stage's weights; every fourth completes an operand
      aop[idx % 4] = dequant_word(NW, idx / 4, idx % 4);
      if (idx % 4 == 3) {
        switch (idx / 4) {
          case 0: DsWrite128<NA * kTlASlot + 0 * 1024>(addr_w, aop); break;
          case 1: DsWrite128<NA * kTlASlot + 1 * 1024>(addr_w, aop); break;
          case 2: DsWrite128<NA * kTlASlot + 2 * 1024>(addr_w, aop); break;
          default: DsWrite128<NA * kTlASlot + 3 * 1024>(addr_w, aop); break;
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    LdsWait(fa[1]);
    LdsWait(fb[1]);
    stage_barrier();  // stage t + 1 is complete in LDS for every wave
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int idx = 0; idx < 16; ++idx) {
      const int t4 = idx / 4, fm = idx % 4;
      acc[t4][fm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, fa[1][t4]),
                                                           __builtin_bit_cast(half8_t, fb[1][fm]), acc[t4][fm], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      switch (idx) {  // step 0 of the next stage
        case 0: DsRead128<NA * kTlASlot + 0 * 1024>(fa[0][0], addr_a); break;
        case 1: DsRead128<NA * kTlASlot + 1 * 1024>(fa[0][1], addr_a); break;
        case 2: DsRead128<NA * kTlASlot + 2 * 1024>(fa[0][2], addr_a); break;
        case 3: DsRead128<NA * kTlASlot + 3 * 1024>(fa[0][3], addr_a); break;
        case 4: DsRead2x64<NB * 32 + 0, NB * 32 + 4>(fb[0][0], addr_b0); break;
        case 5: DsRead2x64<NB * 32 + 0, NB * 32 + 4>(fb[0][1], addr_b1); break;
        case 6: DsRead2x64<NB * 32 + 1, NB * 32 + 5>(fb[0][2], addr_b0); break;
        case 7: DsRead2x64<NB * 32 + 1, NB * 32 + 5>(fb[0][3], addr_b1); break;
        default: break;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // (stages past K, up to the next multiple of four, multiply zeros)
  for (int t = 0; t < stages; t += 4) {
    stage(std::integral_constant<int, 0>{}, t);
    stage(std::integral_constant<int, 1>{}, t + 1);
    stage(std::integral_constant<int, 2>{}, t + 2);
    stage(std::integral_constant<int, 3>{}, t + 3);
  }
  // the copies and reads that ran ahead land before the work-group's LDS is released
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");

  // Register v of lane (g2, r32) belongs to slice 8 * (v / 4) + 4 * g2 + v % 4 of the wave's 32 and to
  // token r32 of the block; the four MFMAs hold the slice's four channels: one 8-byte store.
  // (the bias of the lane's 16 slices is requested before any of it is used: one memory latency)
  u32x2 bias_all[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) bias_all[v] = u32x2{0x80008000u, 0x80008000u};  // -0.0: adding it changes nothing
  if (sg.bias) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int slice = min(slice0 + wn * 32 + 8 * (v >> 2) + 4 * g2 + (v & 3), sg.ns - 1);
      bias_all[v] = *reinterpret_cast<const u32x2*>(sg.bias + (size_t)slice * 4);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int slice = slice0 + wn * 32 + 8 * (v >> 2) + 4 * g2 + (v & 3);
    if (slice >= sg.ns) continue;
    const u32x2 bias2 = bias_all[v];
#pragma unroll
    for (int fm = 0; fm < 4; ++fm) {
      const int mi = m0 + wm * 128 + fm * 32 + r32;
      if (mi >= p.m) continue;
      u32x2 o;
      o[0] = AsU32(__builtin_convertvector(float2v_t{acc[0][fm][v], acc[1][fm][v]}, half2_t) + AsHalf2(bias2[0]));
      o[1] = AsU32(__builtin_convertvector(float2v_t{acc[2][fm][v], acc[3][fm][v]}, half2_t) + AsHalf2(bias2[1]));
      *reinterpret_cast<u32x2*>(sg.dst + ((size_t)slice * p.m + mi) * 4) = o;
    }
  }
}

// Second pass of a K split across work-groups: adds the parts in a fixed order, converts, adds
// the bias.  One thread per (slice, token).
__global__ __launch_bounds__(256) void fc_w4_splitk_reduce_kernel(GemmParams p) {
  // items of all matrices of the launch, matrix after matrix (the list entries by value: fixed
  // argument offsets, one batch of scalar loads)
  uint32_t idx = blockIdx.x * 256u + threadIdx.x;
  const uint32_t m = (uint32_t)p.m;
  const uint32_t items0 = (uint32_t)p.seg[0].ns * m, items1 = (uint32_t)p.seg[1].ns * m;
  int si = 0;
  if (p.segments > 1 && idx >= items0) {
    idx -= items0;
    si = 1;
    if (p.segments > 2 && idx >= items1) {
      idx -= items1;
      si = 2;
    }
  }
  const W4Segment sg = PickSegment<true>(p, si);
  const uint32_t items = (uint32_t)sg.ns * m;
  if (idx >= items) return;
  const float4* part = reinterpret_cast<const float4*>(sg.partial) + idx;
  // the shares are added in their order, four loads in flight at a time
  float4 sum = part[0];
  const int ksplit = p.ksplit;
  for (int s0 = 1; s0 < ksplit; s0 += 4) {
    float4 o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = part[(size_t)min(s0 + j, ksplit - 1) * items];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (s0 + j < ksplit) {
        sum.x += o[j].x;
        sum.y += o[j].y;
        sum.z += o[j].z;
        sum.w += o[j].w;
      }
    }
  }
  __half h[4] = {__float2half_rn(sum.x), __float2half_rn(sum.y), __float2half_rn(sum.z), __float2half_rn(sum.w)};
  if (sg.bias) {
    const __half* bias = sg.bias + (idx / m) * 4;
#pragma unroll
    for (int c = 0; c < 4; ++c) h[c] = __hadd(h[c], bias[c]);
  }
  u32x2 o2;
  o2[0] = (uint32_t)__half_as_ushort(h[0]) | ((uint32_t)__half_as_ushort(h[1]) << 16);
  o2[1] = (uint32_t)__half_as_ushort(h[2]) | ((uint32_t)__half_as_ushort(h[3]) << 16);
  reinterpret_cast<u32x2*>(sg.dst)[idx] = o2;
}

// Token tile of the int4 GEMM in blocks of 32 tokens.  64 tokens when that still yields a
// work-group for half the CUs, else 32 (more work-groups beat a K split across them).  128 tokens (one wave per SIMD, every
// dequantized weight feeds four MFMAs) when the launch fills the chip anyway and the rounds of
// 256 work-groups come out cheaper: a 128-token tile takes about 1.85 x the time of a 64-token
// one.
int W4TokenBlocks(int m, int n) {
  const long tiles_n = DivUp(n, 128);
  const long tiles64 = tiles_n * DivUp(m, 64), tiles128 = tiles_n * DivUp(m, 128);
  if (m % 2 == 0 && tiles128 >= 256 && 1.85 * DivUp(tiles128, 256L) < (double)DivUp(tiles64, 256L)) return 4;
  return (m > 32 && tiles64 >= 128) ? 2 : 1;
}
// K split across work-groups: doubled while the grid stays within the CU count and every wave
// keeps at least 24 steps of 16 channels (below that the partial sums and the second kernel
// cost more than the idle CUs: 2048 x 2048 at 128 tokens 10.9 -> 8.5 us without a split).
int W4KSplit(int m, int k, int n) {
  if (W4TokenBlocks(m, n) == 4) return 1;
  const long tiles = (long)DivUp(n, 128) * DivUp(m, W4TokenBlocks(m, n) * 32);
  const int steps = DivUp(k, 16);
  int s = 1;
  while (s < 8 && tiles * s * 2 <= 256 && steps / (8 * s * 2) >= 24) s *= 2;
  return s;
}

// Shape of the XCD grid over the (token tile, channel tile) plane: xcd_m x (8 / xcd_m), every XCD
// owning a rectangle of rect_m x rect_n tiles.  Picks the shape with the smallest estimate of
// rounds of 32 tiles per XCD plus the time its L2 needs to fetch the rectangle's activation and
// weight tiles once (activations that do not stay resident, above 2 MB, count once per round).
int W4XcdGrid(int tiles_m, int tiles_n, int bm, int k, int groups) {
  const double act_tile = 2.0 * bm * k, weight_tile = 64.0 * k + 256.0 * groups;  // bytes
  const double tile_us = 2.0 * bm * 128 * k / 4.0e6;  // one CU at 4 TFLOP/s
  int best = 8;
  double best_us = 0;
  for (int xm = 8; xm >= 1; xm /= 2) {
    const int rect_m = DivUp(tiles_m, xm), rect_n = DivUp(tiles_n, 8 / xm);
    const double rounds = rect_m * (double)rect_n / 32.0;
    const double act_bytes = rect_m * act_tile;
    const double refetch = act_bytes > 2.0e6 ? std::max(1.0, rounds) : 1.0;
    const double us = rounds * tile_us + (act_bytes * refetch + rect_n * weight_tile) / 1.5e6;
    if (xm == 8 || us < best_us) {
      best = xm;
      best_us = us;
    }
  }
  return best;
}

template <int FM>
hipError_t LaunchConvInt8Tile(const GemmParams& p, hipStream_t stream) {
  const int tiles = DivUp(p.n, 256) * DivUp(p.m, 2 * FM * 32);
  const dim3 grid(DivUp(tiles, 8) * 8), block(kI8Threads);
  const bool zp = p.wzp != nullptr;
  if (p.dst_type == MLDHIP_INT32)
    hipLaunchKernelGGL((conv_int8_mfma_kernel<FM, MLDHIP_INT32, false>), grid, block, 0, stream, p);
  else if (p.dst_type == MLDHIP_FLOAT32 && zp)
    hipLaunchKernelGGL((conv_int8_mfma_kernel<FM, MLDHIP_FLOAT32, true>), grid, block, 0, stream, p);
  else if (p.dst_type == MLDHIP_FLOAT32)
    hipLaunchKernelGGL((conv_int8_mfma_kernel<FM, MLDHIP_FLOAT32, false>), grid, block, 0, stream, p);
  else if (zp)
    hipLaunchKernelGGL((conv_int8_mfma_kernel<FM, MLDHIP_FLOAT16, true>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((conv_int8_mfma_kernel<FM, MLDHIP_FLOAT16, false>), grid, block, 0, stream, p);
  return hipGetLastError();
}

// What the matrix-core kernel can run at all (any token count).
bool DirectGemmShapeOk(const FcArgs& a) {
  if ((a.weight_bits != 4 && a.weight_bits != 8) || !a.act_f16 || !a.dst_f16) return false;
  if (a.scale_kind == kScaleScalar) return false;
  if (a.has_zero_point && a.zero_point == nullptr) return false;  // a scalar zero point: generic kernel
  if (a.m < 1) return false;
  // 32-bit buffer offsets
  const size_t block_bytes = a.weight_bits == 8 ? 16 : 8;
  if ((size_t)DivUp(a.k, 4) * DivUp(a.n, 4) * block_bytes >= 0x7FFFFFF0u || (size_t)DivUp(a.k, 4) * a.m * 8 >= 0x7FFFFFF0u)
    return false;
  if (a.scale_kind == kScaleBlock) {
    // an MFMA step of 16 input channels must not straddle scale groups
    if (a.groups <= 0 || a.k % a.groups != 0 || (a.k / a.groups) % 16 != 0) return false;
    const int steps_per_group = (a.k / a.groups) / 16;
    if (steps_per_group & (steps_per_group - 1)) return false;  // the kernel finds the group by a shift
    if (steps_per_group < 2) return false;                      // and loads the scales once per two steps
  }
  return true;
}

// gate_activation != 0: args = {gate, up}, one output (gated_dst) of activation(gate) * up.
hipError_t LaunchDirectGemm(const FcArgs* args, int count, int gate_activation, void* gated_dst, hipStream_t stream,
                            const char** kernel_name) {
  if (count < 1 || count > kMaxW4Segments) return hipErrorInvalidValue;
  const bool gated = gate_activation != 0;
  if (gated && count != 2) return hipErrorInvalidValue;
  const FcArgs& a = args[0];
  // packed groups: one launch plane per weight matrix, token tiles sized for the largest group
  const bool packed = a.params != nullptr && a.packed_params_offset >= 0;
  if (packed && (count != 1 || gated || a.weights_batch < 1 || a.packed_max_group_size < 1)) return hipErrorInvalidValue;
  GemmParams p = {};
  p.gate_activation = gate_activation;
  p.segments = count;
  p.m = a.m;
  p.k = a.k;
  p.ks = DivUp(a.k, 4);
  p.dst_type = MLDHIP_FLOAT16;
  p.act = static_cast<const __half*>(a.act);
  p.groups = a.scale_kind == kScaleBlock ? a.groups : 1;
  p.mask_lo = 0x000F000Fu;
  p.mask_hi = 0x00F000F0u;
  p.magic_lo = 0x64006400u;
  p.magic_hi = 0x54005400u;
  p.b_bytes = (uint32_t)((size_t)p.ks * p.m * 8);
  p.group_size = a.scale_kind == kScaleBlock ? a.k / a.groups : a.k;
  p.group_shift = -1;
  if (a.scale_kind != kScaleBlock) {
    p.group_shift = 30;  // one group
  } else {
    const int spg = p.group_size / 16;
    for (int sh = 0; sh < 30; ++sh)
      if ((1 << sh) == spg) p.group_shift = sh;
  }
  int n_total = 0, tiles_n = 0;
  for (int i = 0; i < count; ++i) {
    W4Segment& sg = p.seg[i];
    sg.w4 = args[i].weights;
    sg.scale = static_cast<const __half*>(args[i].scale);
    sg.zp = args[i].has_zero_point ? static_cast<const __half*>(args[i].zero_point) : nullptr;
    sg.bias = static_cast<const __half*>(args[i].bias);
    sg.dst = static_cast<__half*>(gated ? gated_dst : args[i].dst);
    sg.partial = args[i].partial;
    sg.n = args[i].n;
    sg.ns = DivUp(args[i].n, 4);
    sg.group = EffectiveGroup(args[i].group, sg.ns);
    if (sg.ns % sg.group != 0) return hipErrorInvalidValue;  // whole groups only
    if (args[i].weight_bits != a.weight_bits) return hipErrorInvalidValue;
    sg.group_shift = -1;
    for (int sh = 0; sh < 30; ++sh)
      if ((1 << sh) == sg.group) sg.group_shift = sh;
    sg.a_bytes = (uint32_t)((size_t)p.ks * sg.ns * (a.weight_bits == 8 ? 16 : 8));
    sg.s_bytes = (uint32_t)((size_t)p.groups * sg.ns * 8 * (packed ? a.weights_batch : 1));
    if (gated) {
      tiles_n = DivUp(args[i].n, 128);  // a tile holds the same 128 channels of both matrices
      if (args[i].n != a.n) return hipErrorInvalidValue;
    } else {
      tiles_n += DivUp(args[i].n, 128);
    }
    sg.tile_end = tiles_n;
    n_total += args[i].n;
  }
  if (gated) n_total = a.n;  // one set of channel tiles, each with twice the work
  for (int i = count; i < kMaxW4Segments; ++i) p.seg[i] = p.seg[0];
  if (kernel_name)
    *kernel_name = gated ? (a.weight_bits == 8 ? "fc_w8_gated_mfma_gemm_kernel" : "fc_w4_gated_mfma_gemm_kernel")
                         : (a.weight_bits == 8 ? "fc_w8_mfma_gemm_kernel" : "fc_w4_mfma_gemm_kernel");
  const Tuning& tune = GetTuning();
  // the geometry the work-groups would otherwise divide out: waves = waves of the work-group that
  // share one tile's K (all of them, or half in the gated and two-tile modes)
  auto set_geometry = [&p](int tiles_m, int tiles_n_grid, int fm, bool halves) {
    const int xn = 8 / p.xcd_m;
    p.geo_tiles_m = tiles_m;
    p.geo_rect_m = DivUp(tiles_m, p.xcd_m);
    p.geo_rect_n = DivUp(tiles_n_grid, xn);
    p.geo_xm_shift = p.xcd_m == 8 ? 3 : (p.xcd_m == 4 ? 2 : (p.xcd_m == 2 ? 1 : 0));
    p.geo_rect_m_magic = p.geo_rect_m > 1 ? (uint32_t)((((uint64_t)1 << 32) + p.geo_rect_m - 1) / p.geo_rect_m) : 0u;
    const int waves = fm == 4 ? 4 : 8, kw = halves ? waves / 2 : waves, prefetch = 4;
    const int shares = kw * p.ksplit, steps_total = DivUp(p.k, 16);
    p.geo_per_wave = DivUp(DivUp(steps_total, shares), prefetch) * prefetch;
  };
  // Many tokens over one uint4 matrix: both operands shared through LDS, 256 x 256 tiles.  Both
  // kernels run into the same limit on large launches (the chip lowers its clock under dense MFMA
  // work on random data) and finish within a few percent of each other, so the tile counts decide:
  // the large tiles are taken where they fill one round of the 256 CUs and the 128 x 128 tiles of
  // the direct kernel would leave its last round half empty (1024 x 4096 x 14336: 131 against 155 us).
  {
    const bool tiled_ok = !gated && !packed && count == 1 && a.weight_bits == 4 && a.m % 2 == 0 && p.group_size % 32 == 0;
    const long tiles = (long)DivUp(a.n, 256) * DivUp(a.m, 256);
    const long small_tiles_last = ((long)DivUp(a.n, 128) * DivUp(a.m, 128)) % 256;
    bool tiled = tiled_ok && a.m >= 1024 && tiles >= 208 && tiles <= 256 && small_tiles_last >= 1 && small_tiles_last <= 160;
    if (tune.gemm_tiled >= 0) tiled = tiled_ok && tune.gemm_tiled != 0;
    if (tiled) {
      if (kernel_name) *kernel_name = "fc_w4_mfma_tiled_kernel";
      const dim3 grid((unsigned)DivUp(tiles, 8L) * 8u), block(kTlThreads);
      if (p.seg[0].zp != nullptr)
        hipLaunchKernelGGL((fc_w4_mfma_tiled_kernel<true>), grid, block, 0, stream, p);
      else
        hipLaunchKernelGGL((fc_w4_mfma_tiled_kernel<false>), grid, block, 0, stream, p);
      return hipGetLastError();
    }
  }
  if (packed) {
    p.pg_params = a.params;
    p.pg_offset = a.packed_params_offset;
    p.pg_groups = a.weights_batch;
    p.pg_max = std::min(a.packed_max_group_size, a.m);
    p.ksplit = 1;
    // token tiles of 32, 64 or (groups of hundreds of tokens) 128 tokens; a group starts at any token,
    // so the tiles are read token by token (no 16-byte token pairs)
    int fm = p.pg_max <= 32 ? 1 : (p.pg_max >= 256 ? 4 : 2);
    if (tune.gemm_fm == 1 || tune.gemm_fm == 2 || tune.gemm_fm == 4) fm = tune.gemm_fm;
    const int tiles_m = DivUp(p.pg_max, fm * 32);
    p.xcd_m = 1;  // few token tiles per matrix: the XCDs share the channel tiles
    if (tune.gemm_xcd_m == 1 || tune.gemm_xcd_m == 2 || tune.gemm_xcd_m == 4 || tune.gemm_xcd_m == 8) p.xcd_m = tune.gemm_xcd_m;
    const dim3 grid(8 * DivUp(tiles_m, p.xcd_m) * DivUp(tiles_n, 8 / p.xcd_m), 1, a.weights_batch);
    if (grid.x / 8 >= (1u << 16)) return hipErrorInvalidValue;  // (the reciprocal of rect_m is exact below 2^16)
    set_geometry(tiles_m, tiles_n, fm, false);
    const bool zp = p.seg[0].zp != nullptr;
    if (fm == 4)
      LaunchDirect<4, 4, 4, false, false>(a.weight_bits, zp, grid, stream, p);
    else if (fm == 2)
      LaunchDirect<2, 4, 8, false, false>(a.weight_bits, zp, grid, stream, p);
    else
      LaunchDirect<1, 4, 8, false, false>(a.weight_bits, zp, grid, stream, p);
    return hipGetLastError();
  }
  // token tile and K split follow the launch as a whole (all channels of all matrices)
  int fm = W4TokenBlocks(a.m, n_total);
  if (tune.gemm_fm > 0) fm = tune.gemm_fm == 1 ? 1 : (tune.gemm_fm == 4 && a.m % 2 == 0 ? 4 : 2);
  p.ksplit = 1;
  if (fm == W4TokenBlocks(a.m, n_total)) p.ksplit = W4KSplit(a.m, a.k, n_total);
  if (tune.gemm_ksplit > 0) p.ksplit = tune.gemm_ksplit;
  if (gated) p.ksplit = 1;  // the epilogue needs whole sums
  for (int i = 0; i < count; ++i)
    while (p.ksplit > 1 && (size_t)p.ksplit * p.seg[i].ns * 4 * a.m > args[i].partial_floats) p.ksplit /= 2;
  const int tiles_m = DivUp(a.m, fm * 32);
  const bool pair = a.m % 2 == 0 && tune.gemm_no_pair <= 0;
  // Two channel tiles per work-group when the rounds of 256 work-groups come out cheaper: a
  // two-tile work-group takes 1.87 x the time of a one-tile one, and a last round filled to the
  // fraction f costs 0.45 + 0.55 f of a full one (fitted to same-box timings of 14 shapes).
  const bool dual_ok = !gated && pair && fm >= 2 && p.ksplit == 1;
  auto rounds = [](long work_groups) {
    const double r = work_groups / 256.0, whole = std::floor(r), f = r - whole;
    return whole + (f > 0.0 ? 0.45 + 0.55 * f : 0.0);
  };
  p.dual = dual_ok && 1.87 * rounds((long)DivUp(tiles_n, 2) * tiles_m) < 0.97 * rounds((long)tiles_n * tiles_m);
  if (tune.gemm_dual >= 0) p.dual = dual_ok && tune.gemm_dual != 0;
  if (p.dual) tiles_n = DivUp(tiles_n, 2);
  p.xcd_m = W4XcdGrid(tiles_m, tiles_n, fm * 32, a.k, p.groups);
  if (tune.gemm_xcd_m > 0) p.xcd_m = tune.gemm_xcd_m;
  if (p.xcd_m != 1 && p.xcd_m != 2 && p.xcd_m != 4 && p.xcd_m != 8) p.xcd_m = 8;
  const dim3 grid(8 * DivUp(tiles_m, p.xcd_m) * DivUp(tiles_n, 8 / p.xcd_m), p.ksplit);
  if (grid.x / 8 >= (1u << 16)) return hipErrorInvalidValue;  // (the reciprocal of rect_m is exact below 2^16)
  set_geometry(tiles_m, tiles_n, fm, gated || p.dual);
  const bool zp = p.seg[0].zp != nullptr;
  if (fm == 4)
    LaunchDirect<4, 4, 4, true, true>(a.weight_bits, zp, grid, stream, p);
  else if (fm == 2 && pair)
    LaunchDirect<2, 4, 8, true, true>(a.weight_bits, zp, grid, stream, p);
  else if (fm == 2)
    LaunchDirect<2, 4, 8, false, false>(a.weight_bits, zp, grid, stream, p);
  else
    LaunchDirect<1, 4, 8, false, false>(a.weight_bits, zp, grid, stream, p);
  if (p.ksplit > 1) {
    size_t items = 0;
    for (int i = 0; i < count; ++i) items += (size_t)p.seg[i].ns * a.m;
    hipLaunchKernelGGL(fc_w4_splitk_reduce_kernel, dim3((unsigned)DivUp((long)items, 256L)), dim3(256), 0, stream, p);
  }
  return hipGetLastError();
}

}  // namespace

bool FcW4MfmaSupported(const FcArgs& a) { return a.m > kGemvMaxTokens && DirectGemmShapeOk(a); }

// Packed groups on the matrix cores: batched weights in the one-group layout, no channel bounds.
bool FcW4MfmaPackedSupported(const FcArgs& a) {
  if (a.params == nullptr || a.packed_params_offset < 0 || a.batch_ids != nullptr) return false;
  if (a.src_end_ch_index >= 0 || a.dst_end_ch_index >= 0) return false;
  // 32-bit offsets into the scale tensor of all matrices and, with output groups, into their weights
  if ((size_t)(a.scale_kind == kScaleBlock ? a.groups : 1) * a.weights_batch * DivUp(a.n, 4) * 8 >= 0x7FFFFFF0u) return false;
  if ((size_t)a.weights_batch * DivUp(a.k, 4) * DivUp(a.n, 4) * (a.weight_bits == 8 ? 16 : 8) >= 0x7FFFFFF0u) return false;
  return DirectGemmShapeOk(a);
}

hipError_t LaunchFcW4MfmaFused(const FcArgs* args, int count, hipStream_t stream, const char** kernel_name) {
  return LaunchDirectGemm(args, count, 0, nullptr, stream, kernel_name);
}

hipError_t LaunchFcW4Mfma(const FcArgs& a, hipStream_t stream, const char** kernel_name) {
  return LaunchFcW4MfmaFused(&a, 1, stream, kernel_name);
}

bool FcW4MfmaGatedSupported(const FcArgs& gate, const FcArgs& up) {
  if (!DirectGemmShapeOk(gate) || !DirectGemmShapeOk(up)) return false;
  if (gate.weight_bits != up.weight_bits) return false;
  // uint8 pairs of a few tokens are better served by their two streaming GEMVs and the host's
  // elementwise node than by a 32-token tile
  if (gate.weight_bits == 8 && gate.m <= kGemvMaxTokens) return false;
  if (gate.has_zero_point || up.has_zero_point) return false;
  return gate.act == up.act && gate.m == up.m && gate.k == up.k && gate.n == up.n && gate.scale_kind == up.scale_kind &&
         gate.groups == up.groups;
}

hipError_t LaunchFcW4MfmaGated(const FcArgs& gate, const FcArgs& up, int activation, void* dst, hipStream_t stream,
                               const char** kernel_name) {
  const FcArgs both[2] = {gate, up};
  return LaunchDirectGemm(both, 2, activation, dst, stream, kernel_name);
}

size_t FcW4MfmaWorkspaceFloats(int max_tokens, int k, int n) {
  size_t need = 0;
  for (int m = kGemvMaxTokens + 1; m <= max_tokens; ++m) {
    const int s = W4KSplit(m, k, n);
    if (s > 1) need = std::max(need, (size_t)s * DivUp(n, 4) * 4 * m);
  }
  return need;
}

hipError_t LaunchConvInt8(const ConvInt8Args& a, hipStream_t stream, const char** kernel_name) {
  GemmParams p = {};
  p.m = a.m;
  p.n = a.n;
  p.k = a.k;
  p.ns = DivUp(a.n, 4);
  p.k16 = DivUp(a.k, 16);
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
  // token tile: the largest of 256 / 128 / 64 that still gives most CUs a work-group
  auto tiles = [&](int bm) { return (long)DivUp(p.n, 256) * DivUp(p.m, bm); };
  if (GetTuning().gemm_i8_fm > 0) {  // tuning override: token tile in blocks of 64
    const int fm = GetTuning().gemm_i8_fm;
    if (fm == 4) return LaunchConvInt8Tile<4>(p, stream);
    if (fm == 2) return LaunchConvInt8Tile<2>(p, stream);
    if (fm == 1) return LaunchConvInt8Tile<1>(p, stream);
  }
  if (tiles(256) >= 200) return LaunchConvInt8Tile<4>(p, stream);
  if (tiles(128) >= 200) return LaunchConvInt8Tile<2>(p, stream);
  return LaunchConvInt8Tile<1>(p, stream);
}

}  // namespace mldhip
