// Internal launch interface between the C-ABI layer (api.cpp) and the HIP kernels.
#ifndef MLDHIP_KERNELS_H_
#define MLDHIP_KERNELS_H_

#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

namespace mldhip {

inline int DivUp(int a, int b) { return (a + b - 1) / b; }

// The I4O4 weights layout with output groups (WeightsDescription::output_group_size, in 4-channel
// slices): [output group][K-slice][slice inside the group] blocks of 4 x 4 elements.  The
// reference's FullyConnected uses one group (group = ns); groups of 16 slices make the share of
// every 64-channel strip one contiguous run of K rows of 128 bytes.
// Index of block (K-slice ks, output slice s); group = 0 stands for one group.
__host__ __device__ inline size_t BlockIndex(int ks, int s, int ks_total, int ns, int group) {
  const int g = group > 0 && group < ns ? group : ns;
  return ((size_t)(s / g) * ks_total + ks) * g + s % g;
}
// Batched weights (matrix b of `batch` matrices): the reference packs them as the height of the
// OHWI shape, and a spatial position lies between the output group and the K-slice
// ([Og][HW][Is][G] blocks, weights_conversion.cc:139-185); with one output group that is one matrix
// after the other, which is what fully_connected.cc:493-496 reads.
__host__ __device__ inline size_t BatchedBlockIndex(int ks, int s, int b, int batch, int ks_total, int ns, int group) {
  const int g = group > 0 && group < ns ? group : ns;
  return (((size_t)(s / g) * batch + b) * ks_total + ks) * g + s % g;
}
inline int EffectiveGroup(int group, int ns) { return group > 0 && group < ns ? group : ns; }
// Output group size (slices) of the layout mldhip_fc_int4_weights_desc asks for: 16 (64-channel
// strips, 128-byte rows).  The kernels also read groups of 8 and 4 slices (narrower strips, more of
// them), which measured slower on every layer width tried (the rows fall below a cache line).
constexpr int kNativeGroup = 16;
inline bool IsNativeGroup(int group) { return group == 4 || group == 8 || group == 16; }
inline int NativeGroupFor(int o) {
  const int ns = DivUp(o, 4);
  return (o % 4 == 0 && ns % kNativeGroup == 0) ? kNativeGroup : ns;
}

enum ScaleKind { kScaleScalar = 0, kScaleLinear = 1, kScaleBlock = 2 };

// Runtime channel bounds (ConvRuntimeCheckDesc, common/task/gpu_operation.h:384-412) from the values a
// kernel has read out of "params": K-slices the loop covers, src_end_slices = (min(end_ch, channels) +
// 3) / 4 (fully_connected.cc:750-755), and dst slices that are written, min(round_up(end_ch, 32) / 4,
// slices) (GetRuntimeEndSlice, common/task/gpu_operation.cc:1832-1836; fully_connected_util.cc:231-243).
__host__ __device__ inline int SrcEndSlices(int end_ch, int k_channels, int ks) {
  const int c = end_ch < k_channels ? end_ch : k_channels;
  const int s = (c + 3) / 4;
  return s < 0 ? 0 : (s > ks ? ks : s);
}
__host__ __device__ inline int DstEndSlice(int end_ch, int ns) {
  const int s = ((end_ch + 31) / 32) * 32 / 4;
  return s < 0 ? 0 : (s > ns ? ns : s);
}

// One FullyConnected launch.  Tensors are slice-major: act [Ks][m][4], dst [Ns][m][4].
struct FcArgs {
  const void* act = nullptr;
  const uint8_t* weights = nullptr;  // I4O4 blocks: [Ks][Ns] x (16 B for uint8, 8 B for uint4)
  const void* scale = nullptr;       // linear: Ns*4; block: [groups][Ns][4]; tensor type
  const void* zero_point = nullptr;  // same shape as scale
  const void* bias = nullptr;        // Ns*4, dst type
  void* dst = nullptr;
  int m = 0, k = 0, n = 0;
  bool act_f16 = true;   // activations / scale / zero-point element type
  bool dst_f16 = true;   // output / bias element type
  int weight_bits = 4;
  int group = 0;  // output group size of the packed weights in slices; 0 = one group (the reference's FC layout)
  int scale_kind = kScaleLinear;
  int groups = 1;
  float scalar_scale = 1.0f;
  bool has_zero_point = false;
  float scalar_zero_point = 0.0f;
  // private workspace of the op (split-K partial sums)
  float* partial = nullptr;
  size_t partial_floats = 0;
  // Batched weights selected by a runtime tensor of ids (the reference's
  // CreateFullyConnectedWeightsBatchIds): dst row y (of `rows`, m tokens each) = FC of src row
  // min(y, src_rows - 1) with weight matrix batch_ids[y] of `weights_batch`.  The packed buffer
  // holds the matrices of an output group one after the other (BatchedBlockIndex), scales are
  // [groups][weights_batch][Ns][4].
  // Plain launches: batch_ids = nullptr, rows = src_rows = weights_batch = 1.
  const int32_t* batch_ids = nullptr;
  int rows = 1, src_rows = 1, weights_batch = 1;
  // Runtime channel bounds (ConvRuntimeCheckDesc): int32 values in device memory, read by the
  // kernel; an index < 0 = not set.  Served by the unspecialised kernels.
  const int32_t* params = nullptr;
  int src_end_ch_index = -1, dst_end_ch_index = -1;
  // Packed groups (ConvRuntimeCheckDesc::PackedGroups, common/task/gpu_operation.h:396-406): the
  // tokens of the one source row are sorted by weight matrix; params[offset + g] tokens starting at
  // token params[offset + weights_batch + g] are multiplied with matrix g.  offset < 0 = not set.
  int packed_params_offset = -1, packed_max_group_size = 0;
  // Ringed weights (fully_connected.cc:411-441, 676-706; uint8, one output group, the unspecialised
  // kernel): the offset is params[ring_*_index] modulo ring_size.  ring_i: k = src channels, the
  // I4O4 buffer holds weights_k input channels; ring_o: n = dst channels, the O4I4 buffer holds
  // ring_size output channels.
  int ring_o_index = -1, ring_i_index = -1, ring_size = 0;
  int weights_k = 0;  // input channels of the weights buffer (ring_i); 0 = k
};

// Split-K workspace sizing for the streaming GEMV.
constexpr int kGemvMaxTokens = 4;
constexpr int kGemvMaxKSplit = 32;

hipError_t LaunchFcGeneric(const FcArgs& a, hipStream_t stream, const char** kernel_name);
// Ringed uint8 weights with the ring over the input channels, 1..4 tokens per row, up to 16 tokens per
// launch: walks the ring's own K-slice rows (aligned 16-byte blocks) and shifts the activations.
bool FcW8RingSupported(const FcArgs& a);
hipError_t LaunchFcW8Ring(const FcArgs& a, hipStream_t stream, const char** kernel_name);
size_t FcW8RingWorkspaceFloats(int max_tokens, int o);
bool FcW4StreamSupported(const FcArgs& a);
// 2..4 tokens over wide layers in whole strips, one chunk per thread: the matrix-core token form of the strip kernel.
bool FcW4StripTokensSupported(const FcArgs& a);
hipError_t LaunchFcW4Stream(const FcArgs& a, hipStream_t stream, const char** kernel_name);
// Up to 3 FCs that read the same activations (same m, k, scale grouping) as one launch.
hipError_t LaunchFcW4StreamFused(const FcArgs* args, int count, hipStream_t stream, const char** kernel_name);

// The same launch with the split-K sums in the library's statically allocated scratch array
// (kNoAllocScratchFloats floats per device) instead of a.partial: allocates nothing.
constexpr size_t kNoAllocScratchFloats = (size_t)512 * 1024;  // 2 MiB
constexpr int kNoAllocMaxChannels = 65536;                    // leaves room for an 8-way K split
hipError_t LaunchFcW4StreamNoAlloc(FcArgs a, hipStream_t stream, const char** kernel_name);

// dst = activation(gate(x)) * up(x) for a pair of int4 layers of one shape on the streaming GEMV
// (1..2 tokens).
bool FcW4GatedSupported(const FcArgs& gate, const FcArgs& up);
hipError_t LaunchFcW4Gated(const FcArgs& gate, const FcArgs& up, int activation, void* dst, hipStream_t stream,
                           const char** kernel_name);

// The int4 streaming GEMV for 1..16 tokens on the matrix cores (per-channel scales, wide layers).
bool FcW4MfmaStreamSupported(const FcArgs& a);
hipError_t LaunchFcW4MfmaStream(const FcArgs& a, hipStream_t stream, const char** kernel_name);

// Streaming GEMV over uint8 weights (1..4 tokens, fp32 or fp16 tensors of one type).
bool FcW8StreamSupported(const FcArgs& a);
hipError_t LaunchFcW8Stream(const FcArgs& a, hipStream_t stream, const char** kernel_name);
// One token over uint8 weights in output groups of one slice (fp32 or fp16 tensors of one type).
bool FcW8RowsSupported(const FcArgs& a);
hipError_t LaunchFcW8Rows(const FcArgs& a, hipStream_t stream, const char** kernel_name);

// Batched weights selected by runtime ids, for the integer-math launches (the same fields as in
// FcArgs): dst row y of `rows` (m tokens each) = source row min(y, src_rows - 1) x matrix ids[y].
struct FcBatchRows {
  const int32_t* ids = nullptr;
  int rows = 1, src_rows = 1, weights_batch = 1;
  int group = 0;  // output group size of the packed weights (0 = one group)
  // runtime channel bounds, as in FcArgs (the tiled kernel only)
  const int32_t* params = nullptr;
  int src_end_ch_index = -1, dst_end_ch_index = -1;
  // packed groups, as in FcArgs (the tiled kernel only): one launch plane per matrix
  int packed_params_offset = -1, packed_max_group_size = 0;
};

// int8 activations x uint8/uint4 weights -> int32 (no scales).
hipError_t LaunchFcInt8Math(const int8_t* act, const uint8_t* weights, int32_t* dst, int m, int k,
                            int n, int weight_bits, hipStream_t stream, const char** kernel_name,
                            const FcBatchRows& batch = FcBatchRows());
// The same for 1..4 tokens as an HBM-streaming kernel.
bool FcInt8MathStreamSupported(int m, int k, int n, int weight_bits);
hipError_t LaunchFcInt8MathStream(const int8_t* act, const uint8_t* weights, int32_t* dst, int m, int k, int n,
                                  int weight_bits, hipStream_t stream, const char** kernel_name,
                                  const FcBatchRows& batch = FcBatchRows());

// Process-wide overrides of the launch heuristics, set through mldhip_set_tuning (tests and
// tuning runs); -1 = leave the choice to the heuristic.  Read at launch, never from the environment.
struct Tuning {
  int force_generic = -1;       // 1: every FullyConnected launch takes the unspecialised kernels
  int gemv_mfma = -1;           // 1: one token also runs on the matrix-core GEMV
  int gemv_fast = -1;           // 0: never take the contiguous-strip GEMV (grouped layout)
  int fc_group = -1;            // output group size that mldhip_fc_int4_weights_desc returns where it divides the slices
  int gemv_lpr = -1, gemv_waves = -1, gemv_ksplit = -1, gemv_narrow_max_mb = -1;
  int gemv_rows_rpt = -1;       // rows per thread the row-interleaved GEMV sizes its work-groups for
  int gemv_one_chunk = -1;      // 0: never take the one-chunk form of the contiguous-strip GEMV
  int gemm_fm = -1, gemm_ksplit = -1, gemm_no_pair = -1, gemm_dual = -1, gemm_xcd_m = -1;
  int gemm_i8_fm = -1;
  int gemm_tiled = -1;          // 1 / 0: always / never take the LDS-tiled int4 GEMM where it can run
};
Tuning& GetTuning();

struct QuantArgs {
  const void* src = nullptr;
  void* codes = nullptr;
  float* params = nullptr;
  int tokens = 0, channels = 0, batch = 1;
  int width = 1, height = 1;  // tokens = height * width * batch (the W4C4 types address by column)
  bool src_f16 = true;
  int packed_type = 2;  // PackedType (common/data_type.h:48-58)
  bool symmetric = false;
  bool calculate_sum = false;
  bool nearest_even = false;  // round-to-nearest-even codes instead of the reference's floor(v + 0.5)
};
hipError_t LaunchQuantize(const QuantArgs& a, hipStream_t stream, const char** kernel_name);

struct ConvInt8Args {
  const int8_t* codes = nullptr;    // [ceil(k/16)][m][16]
  const int8_t* weights = nullptr;  // [ceil(k/16)][n][16]
  const float* params = nullptr;    // [m][4]
  const int32_t* weights_sum = nullptr;
  const float* weights_scale = nullptr;
  const float* weights_zero_point = nullptr;
  const void* bias = nullptr;
  void* dst = nullptr;
  int m = 0, k = 0, n = 0;
  int dst_type = 1;  // MLDHIP_FLOAT16 / FLOAT32 / INT32
};
hipError_t LaunchConvInt8(const ConvInt8Args& a, hipStream_t stream, const char** kernel_name);

// Multi-token FullyConnected with uint4 or uint8 weights on the MFMA units (fp16 tensors).
bool FcW4MfmaSupported(const FcArgs& a);
bool FcW4MfmaPackedSupported(const FcArgs& a);  // packed groups: launched through LaunchFcW4Mfma
hipError_t LaunchFcW4Mfma(const FcArgs& a, hipStream_t stream, const char** kernel_name);
// Up to 3 FCs that read the same activations (same m, k, scale grouping) as one launch.
hipError_t LaunchFcW4MfmaFused(const FcArgs* args, int count, hipStream_t stream, const char** kernel_name);
// fp32 workspace the MFMA path wants for token counts up to max_tokens (K split across
// work-groups); 0 when it never splits.
size_t FcW4MfmaWorkspaceFloats(int max_tokens, int k, int n);
// dst = activation(gate(x)) * up(x) on the matrix-core kernel (symmetric weights; uint4 at any token
// count, uint8 above the GEMV token counts).
bool FcW4MfmaGatedSupported(const FcArgs& gate, const FcArgs& up);
hipError_t LaunchFcW4MfmaGated(const FcArgs& gate, const FcArgs& up, int activation, void* dst, hipStream_t stream,
                               const char** kernel_name);

}  // namespace mldhip

#endif  // MLDHIP_KERNELS_H_
