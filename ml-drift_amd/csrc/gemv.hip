// Decode-side FullyConnected kernels for gfx950: HBM-streaming GEMV over the reference's
// packed I4O4 weight buffers.
//
//  fc_generic_kernel   any weight width / scale kind / zero point / tensor type, fp32 math.
//  fc_int8_math_kernel int8 activations x uint8/uint4 weights -> int32 (bit-exact).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

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

// Work-group geometry of both kernels: x = output slice inside a strip of kSl, y = K lane.
// Narrow strips and many K lanes: a 14336-channel layer is 224 work-groups, and a lane's K loop
// is short enough to unroll, so that several loads are in flight per thread.
constexpr int kSl = 8;
constexpr int kKl = 32;

// ------------------------------------------------------------------------------------------
// Generic kernel.
// ------------------------------------------------------------------------------------------
struct GenericParams {
  const void* act;
  const uint8_t* weights;
  const void* scale;
  const void* zero_point;
  const void* bias;
  void* dst;
  int m, ks, ns;
  int wgroup;  // output group size of the packed weights (slices)
  int scale_kind, groups, group_slices;
  float scalar_scale, scalar_zero_point;
  int has_zero_point;
  // batched weights by runtime ids (fully_connected.cc:654-665, 804-822; fully_connected_util.cc:
  // 279-290): blockIdx.z = dst row; m = tokens per row
  const int32_t* batch_ids;
  int rows, src_rows, weights_batch;
  // runtime channel bounds (common/task/gpu_operation.h:384-412): device values, index < 0 = not set
  const int32_t* params;
  int src_end_ch_index, dst_end_ch_index;
  int k_channels;
  // packed groups (fully_connected_util.cc:263-277; fully_connected.cc:706-710, 810-816): blockIdx.z =
  // weight matrix g; its tokens are params[off + g] many from token params[off + weights_batch + g]
  int packed_params_offset, packed_max_group_size;
  // ringed weights (fully_connected.cc:411-441, 676-706; uint8 only): 1 = ring over the input channels
  // of an I4O4 buffer of w_ks K-slices, 2 = ring over the output channels of an O4I4 buffer; the
  // offset is params[ring_index] modulo ring_size
  int ring_kind, ring_index, ring_size, w_ks;
};

// K-slices the loop covers and dst slices that are written, with runtime channel bounds
// (fully_connected.cc:750-755, 795; fully_connected_util.cc:231-243 with
// ConvRuntimeCheckDesc::GetRuntimeEndSlice, common/task/gpu_operation.cc:1832-1836).  The source
// bound does not apply to group-wise scales: that loop runs over all groups (fully_connected.cc:784-794).
__device__ __forceinline__ int RuntimeSrcEndSlices(const int32_t* params, int index, int k_channels, int ks, bool block) {
  if (params == nullptr || index < 0 || block) return ks;
  const int end_ch = min(params[index], k_channels);
  return min(max((end_ch + 3) / 4, 0), ks);
}
__device__ __forceinline__ int RuntimeDstEndSlice(const int32_t* params, int index, int ns) {
  if (params == nullptr || index < 0) return ns;
  return min(max(((params[index] + 31) / 32) * 32 / 4, 0), ns);
}

template <typename ActT, typename DstT, int WBITS, int TB>
__global__ __launch_bounds__(256) void fc_generic_kernel(GenericParams p) {
  __shared__ float red[kKl][kSl][TB * 4];
  const int tx = threadIdx.x, ty = threadIdx.y;
  const int ds = blockIdx.x * kSl + tx;
  const int tok0 = blockIdx.y * TB;
  const ActT* act = static_cast<const ActT*>(p.act);
  const ActT* scale = static_cast<const ActT*>(p.scale);
  const ActT* zp = static_cast<const ActT*>(p.zero_point);
  const float shift = WBITS == 8 ? 128.0f : 8.0f;
  // Row of the launch: its weight matrix, its source row (one shared row is broadcast) and the
  // token strides of the two tensors.  An id outside the batch is clamped into it (the reference
  // reads whatever lies there).
  const int row = blockIdx.z;
  int wb = p.batch_ids ? p.batch_ids[row] : 0;
  wb = min(max(wb, 0), p.weights_batch - 1);
  size_t act_stride = (size_t)p.src_rows * p.m, dst_stride = (size_t)p.rows * p.m;
  size_t act_tok0 = (size_t)min(row, p.src_rows - 1) * p.m, dst_tok0 = (size_t)row * p.m;
  int tok_count = p.m;  // tokens of this row: tok0 + t < tok_count
  if (p.packed_params_offset >= 0) {
    // one row of p.m tokens; this work-group's matrix owns tok_count of them from token dst_tok0 on
    wb = row;
    const int size = p.params[p.packed_params_offset + row];
    const int offset = p.params[p.packed_params_offset + p.weights_batch + row];
    tok_count = min(min(size, p.packed_max_group_size), p.m - offset);
    act_stride = dst_stride = (size_t)p.m;
    act_tok0 = dst_tok0 = (size_t)max(offset, 0);
    if (offset < 0 || tok0 >= tok_count) return;  // (the whole work-group: no barrier is left waiting)
  }
  const uint8_t* weights = p.weights;  // (matrix wb: through the block index)

  float acc[TB][4];
#pragma unroll
  for (int t = 0; t < TB; ++t)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[t][c] = 0.0f;

  const int ks_end = RuntimeSrcEndSlices(p.params, p.src_end_ch_index, p.k_channels, p.ks, p.scale_kind == kScaleBlock);
  const int ns_end = RuntimeDstEndSlice(p.params, p.dst_end_ch_index, p.ns);
  // ring start: ((offset % ring_size) + ring_size) % ring_size (fully_connected.cc:678-679, 699-700)
  int ring_off = 0;
  if (WBITS == 8 && p.ring_kind != 0) ring_off = ((p.params[p.ring_index] % p.ring_size) + p.ring_size) % p.ring_size;
  if (ds < ns_end) {
    float s[4], z[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      s[c] = p.scalar_scale;
      z[c] = p.has_zero_point ? p.scalar_zero_point : 0.0f;
    }
    if (p.scale_kind == kScaleLinear) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        s[c] = LoadF(scale, ((size_t)wb * p.ns + ds) * 4 + c);
        if (zp) z[c] = LoadF(zp, ((size_t)wb * p.ns + ds) * 4 + c);
      }
    }
#pragma unroll 4
    for (int ks = ty; ks < ks_end; ks += kKl) {
      if (p.scale_kind == kScaleBlock) {
        int g = ks / p.group_slices;
        if (g >= p.groups) g = p.groups - 1;
        const size_t sidx = (((size_t)g * p.weights_batch + wb) * p.ns + ds) * 4;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          s[c] = LoadF(scale, sidx + c);
          if (zp) z[c] = LoadF(zp, sidx + c);
        }
      }
      const size_t blk = BatchedBlockIndex(ks, ds, wb, p.weights_batch, p.ks, p.ns, p.wgroup);
      float wf[4][4];
      if (WBITS == 8 && p.ring_kind != 0) {
        // four 4-byte reads with addresses of their own (ReadRingedWeightsAsFloat, fully_connected.cc:443-471)
        const uint32_t* w32 = reinterpret_cast<const uint32_t*>(weights);
        uint32_t w[4];
        if (p.ring_kind == 1) {
          // rows of 4 output channels: a = (i >> 2) * dst_stride + (i & 3) + ring_i_base, dst_stride =
          // 4 * Ns, ring_i_base = dst_s * 4 + w_batch_id * ring_size * Ns (fully_connected.cc:424-441, 701-706)
          const size_t base = (size_t)wb * p.ring_size * p.ns + (size_t)ds * 4;
          int ij = (ks * 4 + ring_off) % p.ring_size;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            w[i] = w32[base + (size_t)(ij >> 2) * p.ns * 4 + (ij & 3)];
            ij = ij + 1 >= p.ring_size ? ij + 1 - p.ring_size : ij + 1;
          }
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int c = 0; c < 4; ++c) wf[i][c] = ((float)((w[i] >> (8 * c)) & 0xFFu) - (shift + z[c])) * s[c];
        } else {
          // rows of 4 input channels: a = src_s * ring_size + o + w_batch_id * ring_size * Ks
          // (fully_connected.cc:411-422, 680-697); scale and zero point belong to the dst channel
          const size_t base = ((size_t)wb * p.ks + ks) * p.ring_size;
          int oc = (ds * 4 + ring_off) % p.ring_size;
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            w[c] = w32[base + oc];
            oc = oc + 1 >= p.ring_size ? oc + 1 - p.ring_size : oc + 1;
          }
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int c = 0; c < 4; ++c) wf[i][c] = ((float)((w[c] >> (8 * i)) & 0xFFu) - (shift + z[c])) * s[c];
        }
      } else if (WBITS == 8) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(weights + blk * 16);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int c = 0; c < 4; ++c)
            wf[i][c] = ((float)((w[i] >> (8 * c)) & 0xFFu) - (shift + z[c])) * s[c];
      } else {
        const u32x2 w = *reinterpret_cast<const u32x2*>(weights + blk * 8);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int c = 0; c < 4; ++c)
            wf[i][c] = ((float)((w[i >> 1] >> (16 * (i & 1) + 4 * c)) & 0xFu) - (shift + z[c])) * s[c];
      }
#pragma unroll
      for (int t = 0; t < TB; ++t) {
        const int tok = tok0 + t;
        if (tok < tok_count) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float a = LoadF(act, ((size_t)ks * act_stride + act_tok0 + tok) * 4 + i);
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
  if (ty == 0 && ds < ns_end) {
    DstT* dst = static_cast<DstT*>(p.dst);
    const DstT* bias = static_cast<const DstT*>(p.bias);
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      const int tok = tok0 + t;
      if (tok >= tok_count) continue;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        float r = 0.0f;
#pragma unroll
        for (int q = 0; q < kKl; ++q) r += red[q][tx][t * 4 + c];
        StoreOut(dst, ((size_t)ds * dst_stride + dst_tok0 + tok) * 4 + c, r, bias, (size_t)ds * 4 + c);
      }
    }
  }
}

template <typename ActT, typename DstT, int WBITS>
hipError_t LaunchGenericT(const GenericParams& p, hipStream_t stream) {
  constexpr int TB = 4;
  dim3 grid(DivUp(p.ns, kSl), DivUp(p.m, TB), p.rows);
  if (p.packed_params_offset >= 0) grid = dim3(DivUp(p.ns, kSl), DivUp(std::min(p.m, p.packed_max_group_size), TB), p.weights_batch);
  dim3 block(kSl, kKl);
  hipLaunchKernelGGL((fc_generic_kernel<ActT, DstT, WBITS, TB>), grid, block, 0, stream, p);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// int8-math kernel: same thread layout as the generic kernel, int32 accumulators.
// ------------------------------------------------------------------------------------------
template <int WBITS, int TB>
__global__ __launch_bounds__(256) void fc_int8_math_kernel(const int8_t* __restrict__ act,
                                                           const uint8_t* __restrict__ weights,
                                                           int32_t* __restrict__ dst, int m, int ks_n,
                                                           int ns, int k_channels, FcBatchRows batch) {
  __shared__ int red[kKl][kSl][TB * 4];
  const int tx = threadIdx.x, ty = threadIdx.y;
  const int ds = blockIdx.x * kSl + tx;
  const int tok0 = blockIdx.y * TB;
  // batched weights: blockIdx.z = dst row (one row, matrix 0, for a plain launch)
  const int row = blockIdx.z;
  int wb = batch.ids ? batch.ids[row] : 0;
  wb = min(max(wb, 0), batch.weights_batch - 1);
  size_t act_stride = (size_t)batch.src_rows * m, dst_stride = (size_t)batch.rows * m;
  size_t act_tok0 = (size_t)min(row, batch.src_rows - 1) * m, dst_tok0 = (size_t)row * m;
  int tok_count = m;  // tokens of this row: tok0 + t < tok_count
  if (batch.packed_params_offset >= 0) {
    // packed groups (fully_connected_util.cc:263-277; fully_connected.cc:706-710, 810-816): one row of m
    // tokens; this plane's matrix owns tok_count of them from token dst_tok0 on
    wb = row;
    const int size = batch.params[batch.packed_params_offset + row];
    const int offset = batch.params[batch.packed_params_offset + batch.weights_batch + row];
    tok_count = min(min(size, batch.packed_max_group_size), m - offset);
    act_stride = dst_stride = (size_t)m;
    act_tok0 = dst_tok0 = (size_t)max(offset, 0);
    if (offset < 0 || tok0 >= tok_count) return;  // (the whole work-group: no barrier is left waiting)
  }
  int acc[TB][4];
#pragma unroll
  for (int t = 0; t < TB; ++t)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[t][c] = 0;
  const int ks_end = RuntimeSrcEndSlices(batch.params, batch.src_end_ch_index, k_channels, ks_n, false);
  const int ns_end = RuntimeDstEndSlice(batch.params, batch.dst_end_ch_index, ns);
  if (ds < ns_end) {
#pragma unroll 4
    for (int ks = ty; ks < ks_end; ks += kKl) {
      const size_t blk = BatchedBlockIndex(ks, ds, wb, batch.weights_batch, ks_n, ns, batch.group);
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
        if (tok >= tok_count) continue;
        const int v = *reinterpret_cast<const int*>(act + ((size_t)ks * act_stride + act_tok0 + tok) * 4);
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
  if (ty == 0 && ds < ns_end) {
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      const int tok = tok0 + t;
      if (tok >= tok_count) continue;
#pragma unroll
      for (int c = 0; c < 4; ++c)
      {
        int r = 0;
#pragma unroll
        for (int q = 0; q < kKl; ++q) r += red[q][tx][t * 4 + c];
        dst[((size_t)ds * dst_stride + dst_tok0 + tok) * 4 + c] = r;
      }
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
  p.wgroup = a.group;
  p.scale_kind = a.scale_kind;
  p.groups = a.groups;
  p.group_slices = a.scale_kind == kScaleBlock ? (p.ks / a.groups > 0 ? p.ks / a.groups : 1) : p.ks;
  p.scalar_scale = a.scalar_scale;
  p.scalar_zero_point = a.scalar_zero_point;
  p.has_zero_point = a.has_zero_point;
  p.batch_ids = a.batch_ids;
  p.rows = a.rows;
  p.src_rows = a.src_rows;
  p.weights_batch = a.weights_batch;
  p.params = a.params;
  p.src_end_ch_index = a.src_end_ch_index;
  p.dst_end_ch_index = a.dst_end_ch_index;
  p.k_channels = a.k;
  p.packed_params_offset = a.params ? a.packed_params_offset : -1;
  p.packed_max_group_size = a.packed_max_group_size;
  p.ring_kind = a.params && a.ring_i_index >= 0 ? 1 : (a.params && a.ring_o_index >= 0 ? 2 : 0);
  p.ring_index = p.ring_kind == 1 ? a.ring_i_index : a.ring_o_index;
  p.ring_size = a.ring_size;
  p.w_ks = DivUp(a.weights_k > 0 ? a.weights_k : a.k, 4);
  if (p.ring_kind != 0 && (a.weight_bits != 8 || a.ring_size < 1 || a.packed_params_offset >= 0 ||
                           EffectiveGroup(a.group, p.ns) != p.ns))
    return hipErrorInvalidValue;
  if (p.ring_kind == 1 && (a.ring_size > 4 * p.w_ks || (a.weights_batch > 1 && a.ring_size != 4 * p.w_ks)))
    return hipErrorInvalidValue;
  if (p.ring_kind == 2 && a.ring_size % 4 != 0) return hipErrorInvalidValue;
  if (p.packed_params_offset >= 0 && (a.batch_ids != nullptr || a.packed_max_group_size < 1 || a.weights_batch < 1))
    return hipErrorInvalidValue;
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

hipError_t LaunchFcInt8Math(const int8_t* act, const uint8_t* weights, int32_t* dst, int m, int k,
                            int n, int weight_bits, hipStream_t stream, const char** kernel_name,
                            const FcBatchRows& batch) {
  constexpr int TB = 4;
  const int ks = DivUp(k, 4), ns = DivUp(n, 4);
  dim3 grid(DivUp(ns, kSl), DivUp(m, TB), batch.ids ? batch.rows : 1);
  if (batch.packed_params_offset >= 0) {
    if (batch.ids != nullptr || batch.params == nullptr || batch.packed_max_group_size < 1 || batch.weights_batch < 1)
      return hipErrorInvalidValue;
    grid = dim3(DivUp(ns, kSl), DivUp(std::min(m, batch.packed_max_group_size), TB), batch.weights_batch);
  }
  dim3 block(kSl, kKl);
  if (kernel_name) *kernel_name = "fc_int8_math_kernel";
  if (weight_bits == 8)
    hipLaunchKernelGGL((fc_int8_math_kernel<8, TB>), grid, block, 0, stream, act, weights, dst, m, ks, ns, k, batch);
  else
    hipLaunchKernelGGL((fc_int8_math_kernel<4, TB>), grid, block, 0, stream, act, weights, dst, m, ks, ns, k, batch);
  return hipGetLastError();
}

}  // namespace mldhip
