/*
 * mldhip — MI355X (gfx950) implementation of ML Drift's quantized fully-connected path.
 *
 * C-ABI boundary.  Everything here is `extern "C"`, plain pointers and sizes.  Each entry
 * point names the reference interface it stands in for (paths relative to the reference
 * checkout, ml_drift/...).
 *
 * Conventions
 *  - Return value: an absl::StatusCode number (0 OK, 3 INVALID_ARGUMENT, 9
 *    FAILED_PRECONDITION, 11 OUT_OF_RANGE, 12 UNIMPLEMENTED, 13 INTERNAL), the same codes
 *    the reference's absl::Status carries.  mldhip_last_error() gives the message of the
 *    last failure on the calling thread.  No exception crosses this boundary.
 *  - Device pointers are caller-owned (the reference's tensors belong to its
 *    InferenceContext; external weights "must be valid during life of InferenceContext",
 *    common/gpu_model.h:83-96).  An op owns only its metadata and a small private
 *    device workspace, allocated by the create call (no launch allocates, so a first launch
 *    may be recorded under stream capture).  Bound buffers must be 16-byte aligned (the kernels
 *    use 128-bit loads and stores); mldhip_op_set_src / _set_dst reject others.
 *  - Launches are asynchronous on the caller's hipStream_t (passed as void*).  Handles
 *    are not thread-safe; creation functions are re-entrant.
 *  - Weight shapes are OHWI with H = W = 1 for ops; the host packers accept any H, W.
 *  - Activation / output tensors are buffers in the reference's default physical layout
 *    PhysicalLayout1D::kDCHWBC4 = [ceil(C/4)][tokens][4] with tokens = (y*W+x)*B+b
 *    (common/task/tensor_desc.cc:1604-1609, 1857-1860).
 */
#ifndef MLDHIP_H_
#define MLDHIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* absl::StatusCode numerics */
enum {
  MLDHIP_OK = 0,
  MLDHIP_INVALID_ARGUMENT = 3,
  MLDHIP_NOT_FOUND = 5,
  MLDHIP_FAILED_PRECONDITION = 9,
  MLDHIP_OUT_OF_RANGE = 11,
  MLDHIP_UNIMPLEMENTED = 12,
  MLDHIP_INTERNAL = 13
};

/* DataType, common/data_type.h:25-48 (same numbers) */
enum {
  MLDHIP_FLOAT16 = 1,
  MLDHIP_FLOAT32 = 2,
  MLDHIP_UINT8 = 5,
  MLDHIP_INT8 = 6,
  MLDHIP_INT32 = 10,
  MLDHIP_UINT4 = 15
};

/* PackedType, common/data_type.h:50-60 (same numbers; the ones this path produces) */
enum {
  MLDHIP_PACKED_UINT8C4 = 1,
  MLDHIP_PACKED_INT8C4 = 2,
  MLDHIP_PACKED_UINT8W4C4 = 3,
  MLDHIP_PACKED_INT8W4C4 = 4,
  MLDHIP_PACKED_INT8C16 = 5,
  MLDHIP_PACKED_UINT8C16 = 6,
  MLDHIP_PACKED_INT4C32 = 7,
  MLDHIP_PACKED_UINT4C32 = 8
};

/* WeightsLayout, common/task/weights_layout.h:27-42 (same order) */
enum {
  MLDHIP_LAYOUT_UNKNOWN = 0,
  MLDHIP_LAYOUT_OSPATIAL_IOGROUP_I4O4 = 1,
  MLDHIP_LAYOUT_OSPATIAL_IOGROUP_O4I4 = 2,
  MLDHIP_LAYOUT_2D_YSPATIALIO_XOGROUP_I4O4 = 6,
  MLDHIP_LAYOUT_CUSTOM_GROUPS = 7
};

/* CalculationsPrecision, common/precision.h:24-33 */
enum { MLDHIP_PRECISION_F32 = 0, MLDHIP_PRECISION_F32_F16 = 1, MLDHIP_PRECISION_F16 = 2 };

/* Axis ids for custom group lists (Axis::kOutputChannels, kHeight, kWidth, kInputChannels) */
enum { MLDHIP_AXIS_O = 0, MLDHIP_AXIS_H = 1, MLDHIP_AXIS_W = 2, MLDHIP_AXIS_I = 3 };

#define MLDHIP_MAX_CUSTOM_GROUPS 8

/* WeightsDescription, common/task/weights_layout.h:44-93 (the fields this path uses).
 * For MLDHIP_LAYOUT_CUSTOM_GROUPS the list is fastest-varying first and a size <= 0 means
 * "the rest of that axis" (common/task/weights_conversion.cc:285-331). */
typedef struct {
  int32_t type;              /* MLDHIP_UINT8 / MLDHIP_UINT4 / MLDHIP_INT8 */
  int32_t layout;            /* MLDHIP_LAYOUT_* */
  int32_t output_group_size; /* OGroup size, for the OGroup layouts */
  int32_t n_groups;          /* custom groups only */
  int32_t group_axis[MLDHIP_MAX_CUSTOM_GROUPS];
  int32_t group_size[MLDHIP_MAX_CUSTOM_GROUPS];
} mldhip_weights_desc;

const char* mldhip_last_error(void);
const char* mldhip_version(void);

/* Overrides a launch heuristic of this library for the whole process (tests and tuning runs;
 * the reference keeps its counterpart, the work-group size argument of
 * CreateFullyConnectedExternalWeights, common/kernels/fully_connected.h:155-161, per call).
 * value -1 restores the heuristic.  Knobs: force_generic, gemv_mfma, gemv_fast, gemv_one_chunk,
 * fc_group, gemv_lpr, gemv_waves, gemv_ksplit, gemv_rows_rpt, gemv_narrow_max_mb, gemm_fm,
 * gemm_ksplit, gemm_no_pair, gemm_dual, gemm_xcd_m, gemm_i8_fm, gemm_tiled.  MLDHIP_NOT_FOUND for an unknown
 * name.  A test and tuning aid, not part of the op contract: the state is one set of plain
 * integers per process, read without synchronisation at every launch (and by
 * mldhip_fc_int4_weights_desc for fc_group), so it must not be changed while another thread
 * creates or launches ops; a product build never calls it. */
int mldhip_set_tuning(const char* name, int value);

/* ------------------------------------------------------------------------------------ */
/* Weight descriptions and host packers ("weights rearrangement")                         */
/* ------------------------------------------------------------------------------------ */

/* GetFullyConnectedInt8WeightsDesc / GetFullyConnectedInt4WeightsDesc
 * (common/kernels/fully_connected.h:185-192, .cc:1218-1246): the layout this device's
 * FullyConnected wants the builder to pack the weights in (the reference picks per GPU too:
 * buffers or textures).  uint8: kOSpatialIOGroupI4O4 (buffer storage), output_group_size =
 * ceil(o/4), exactly the reference's choice.  uint4: the same layout enum with
 * output_group_size = 16 slices when o is a multiple of 64 (else ceil(o/4)): the reference's
 * packers produce it from this description as they do any group size
 * (common/task/weights_conversion.cc:139-185, 631-708), and the K rows of every 64-channel
 * strip then lie one after the other in memory, which is what lets the decode GEMV stream at
 * the rate of a plain copy on this device.  mldhip_fc_create takes either group size. */
int mldhip_fc_int8_weights_desc(int o, int i, mldhip_weights_desc* desc);
int mldhip_fc_int4_weights_desc(int o, int i, mldhip_weights_desc* desc);
/* The reference's own GetFullyConnectedInt4WeightsDesc choice (one output group,
 * output_group_size = ceil(o/4)), for weights that were packed for the reference's kernel. */
int mldhip_fc_int4_weights_desc_reference(int o, int i, mldhip_weights_desc* desc);
/* The layout for an op that only ever runs one token per launch (the FullyConnected nodes of a
 * decode graph, where a builder keeps a second packed copy of the weights for the prefill graph):
 * as mldhip_fc_int4_weights_desc, except that layers of fewer than 8192 output channels, which
 * have too few 64-channel strips to occupy the chip, take output groups of 2 slices (8 channels,
 * 16-byte K rows): every CU then streams the whole K of a strip and no second kernel adds partial
 * sums.  Ops over this layout run any number of tokens, but more than one token is served by the
 * slower general kernels. */
int mldhip_fc_int4_weights_desc_decode(int o, int i, mldhip_weights_desc* desc);
/* The same for uint8 weights: output groups of one slice, the layout FullyConnectedOI reads
 * (linear_i4o4 = dst_s * src_slices + src_s, common/kernels/fully_connected_oi.cc:122-133): the K
 * rows of 4 channels are one contiguous run that one work-group streams. */
int mldhip_fc_int8_weights_desc_decode(int o, int i, mldhip_weights_desc* desc);

/* The weights layout the int8 x int8 MFMA convolution asks for, the counterpart of the
 * conv_weights_desc that SelectConvolutionInt8 returns to the builder
 * (common/gpu_model_builder.cc:1383-1407): signed int8, custom groups {I:16, O:rest, I:rest},
 * i.e. [ceil(i/16)][o][16]. */
int mldhip_conv_int8_weights_desc(int o, int i, mldhip_weights_desc* desc);

/* GetTotalElementsCountForLayout (common/task/weights_conversion.cc:1015-1076) and the byte
 * size of the packed buffer (elements * bits / 8). */
int mldhip_total_elements(const mldhip_weights_desc* desc, int o, int h, int w, int i,
                          size_t* elements);
int mldhip_packed_bytes(const mldhip_weights_desc* desc, int o, int h, int w, int i,
                        size_t* bytes);

/* RearrangeWeightsInt8AsUint8 / RearrangeWeightsInt8AsUint4
 * (common/task/weights_conversion.h, .cc:1495-1523): int8-held values + shift, reordered to
 * desc->layout, padding elements = pad.  The reference calls them with (128, 128u) and
 * (8, 8u) (weights_conversion.cc:1679-1684). */
int mldhip_rearrange_int8_as_uint8(const int8_t* weights, int o, int h, int w, int i,
                                   const mldhip_weights_desc* desc, uint8_t* dst,
                                   size_t dst_bytes, int shift, unsigned pad);
int mldhip_rearrange_int8_as_uint4(const int8_t* weights, int o, int h, int w, int i,
                                   const mldhip_weights_desc* desc, uint8_t* dst,
                                   size_t dst_bytes, int shift, unsigned pad);

/* RearrangeWeights(Tensor<OHWI,kInt8>) (common/task/weights_conversion.cc:1351-1423):
 * signed int8, pad 0; layouts I4O4, O4I4, 2D twin and custom groups. */
int mldhip_rearrange_int8(const int8_t* weights, int o, int h, int w, int i,
                          const mldhip_weights_desc* desc, int8_t* dst, size_t dst_bytes);

/* RearrangeWeightsUInt4Packed (common/task/weights_conversion.cc:1604-1620): input is
 * nibble-packed two's-complement OHWI (IHWO when swap_dims), low nibble = even element;
 * also writes weights_sum_i[o] = sum_i w[o,i].  sum_len may exceed o (padding sums stay
 * as given beyond o, entries < o are overwritten).  Layouts other than the two I4O4 ones
 * return MLDHIP_UNIMPLEMENTED like the reference. */
int mldhip_rearrange_uint4_packed(const uint8_t* weights, int o, int h, int w, int i,
                                  const mldhip_weights_desc* desc, uint8_t* dst,
                                  size_t dst_bytes, int32_t* weights_sum_i, size_t sum_len,
                                  unsigned pad, int swap_dims);

/* GetWeightsAccumulatedInputChannels (common/task/weights_conversion.cc:1584-1602) */
int mldhip_weights_sum_i(const int8_t* weights, int o, int h, int w, int i, int32_t* sum);

/* ScaleOrZeroPointToTensorDesc (common/task/tensor_desc.cc:2245-2257, 267-292): float
 * scales OHWI(o,1,1,groups) -> the tensor the kernels read: groups == 1: linear, ceil(o/4)*4
 * values; else [groups][ceil(o/4)][4]; element type dst_type (FLOAT16 or FLOAT32),
 * zero padded.  dst_bytes must be groups*ceil(o/4)*4*sizeof(type). */
int mldhip_scale_to_tensor(const float* scale, int o, int groups, int dst_type, void* dst,
                           size_t dst_bytes);

/* The same for batched weights, scale_zp_shape OHWI(o, batch, 1, groups) (OHIToHOIO4,
 * common/task/tensor_desc.cc:267-292, as the HWC tensor of :294-311): scale[o][batch][groups]
 * -> [groups][batch][ceil(o/4)][4]. */
int mldhip_scale_to_tensor_batched(const float* scale, int o, int batch, int groups, int dst_type,
                                   void* dst, size_t dst_bytes);

/* ------------------------------------------------------------------------------------ */
/* Checkpoint files -> the buffers of a quantized FullyConnected (host side)              */
/* ------------------------------------------------------------------------------------ */

/* One linear layer as the LLM sample stores it on disk (samples/llm/extract_weights_hf.py writes
 * these files, samples/llm/llm_file_tensor_loader.cc reads them): `<weights_name>` holds int8
 * [o][i] values, or two's-complement nibbles with the low nibble first;
 * `<base_name>.weight_quantized_scale` holds fp32 scales [o] or [o][i / group] (or an int32
 * group-size header followed by int8 / int16 values of scale * 1024);
 * `<base_name>.weight_quantized_zp`, if present, holds zero points in the same two formats,
 * in units of the dequantized weight.  File names are appended to `directory` as they are
 * (the directory string ends in a separator, as in the reference). */
typedef struct {
  mldhip_weights_desc weights; /* GetFullyConnectedInt4WeightsDesc / ...Int8WeightsDesc of (o, i) */
  int o, i;
  int weight_bits;             /* 4 or 8 */
  int group_size;              /* input channels per scale; i for per-channel scales */
  int scale_i;                 /* i / group_size: the scale / zero-point shape is OHWI(o, 1, 1, scale_i) */
  int has_zero_point;          /* the zero-point file exists */
  size_t weights_bytes;        /* bytes of the packed weight buffer */
  size_t scale_elements;       /* elements of the scale (and zero-point) tensor: scale_i * ceil(o/4) * 4 */
} mldhip_checkpoint_fc;

/* What LlmWeightsLoader::GetWeightsInt4 / GetWeightsInt8 (samples/llm/llm_weights_loader.cc:29-117)
 * find out before they load: the weights description, the quantization group size
 * (LlmFileTensorLoader::GetQuantizationIGroupSize, llm_file_tensor_loader.cc:399-452: derived
 * from the size of the scale file; a missing or unrecognised file means per-channel) and
 * whether a zero-point file exists.  MLDHIP_NOT_FOUND when the weights file cannot be opened. */
int mldhip_checkpoint_fc_probe(const char* directory, const char* weights_name,
                               const char* base_name, int o, int i, int weight_bits,
                               mldhip_checkpoint_fc* info);

/* LoadInt4Weights (fast path, llm_file_tensor_loader.cc:350-395) / LoadInt8Weights (:262-302),
 * LoadScale (:454-467) and LoadZeroPoint (:469-496) into caller-provided host buffers, ready to
 * upload and bind as "weights", "weights_scale", "weights_zero_point" (and the weights_sum_i of
 * the int8 x int8 route): packed weights in info->weights layout, scale and zero-point tensors
 * of ScaleOrZeroPointToTensorDesc in `tensor_type` (FLOAT16 / FLOAT32), zero point = file value
 * / scale (0 where the scale is 0), weights_sum_i[o] int32.  `swap_dims`: the weights file is
 * [i][o].  `zero_point` may be null when info->has_zero_point is 0; `scale_bytes` is the size of
 * each of the two tensor buffers.  As in the reference, a file shorter than the shape reads as
 * zeros beyond its end. */
int mldhip_checkpoint_fc_read(const char* directory, const char* weights_name,
                              const char* base_name, const mldhip_checkpoint_fc* info,
                              int swap_dims, int tensor_type, uint8_t* weights,
                              size_t weights_bytes, void* scale, void* zero_point,
                              size_t scale_bytes, int32_t* weights_sum_i);

/* ------------------------------------------------------------------------------------ */
/* Operations (node executors)                                                            */
/* ------------------------------------------------------------------------------------ */

typedef struct mldhip_op mldhip_op;

/* IsFullyConnectedRecommended (common/kernels/fully_connected.cc:998-1011) restated for
 * this device: returns 1 when `tokens` is small enough for the streaming GEMV kernels,
 * 0 when the MFMA GEMM kernels are used.  mldhip_fc_create serves both ranges. */
int mldhip_fc_is_recommended(int precision, int tokens);

/* CreateFullyConnectedExternalWeights (common/kernels/fully_connected.h:155-161,
 * .cc:1078-1172) and, for larger token counts, the WeightsConverter + float ConvGeneric
 * pair the builder would emit instead (common/gpu_model_builder.cc:1110-1276), fused into
 * one MFMA kernel.
 *
 * src objects, in the reference's registration order (fully_connected.cc:359-360,
 * 1160-1170; fully_connected_util.cc:409-487):
 *   0 "src_tensor"            activations [ceil(i/4)][tokens][4], src_type
 *   1 "weights"               packed buffer per `weights`
 *   2 "weights_scale"         present iff scale_o*scale_i > 1
 *   3 "weights_zero_point"    present iff has_zero_point_tensor
 *   4 "biases"                present iff has_bias, ceil(o/4)*4 values of dst_type
 *   5 "params"                present iff a runtime channel bound or a ring offset is set (int32, see below)
 * (absent objects do not take an index).  dst 0 "dst_tensor": [ceil(o/4)][tokens][4].
 *
 * Zero points (fully_connected_util.cc:91-99: w = u*s - s*(shift + zp)) are taken by every
 * kernel, whole (the builder converts them from int32, common/gpu_model_builder.cc:1917-1935) or
 * fractional.
 *
 * src_type INT8 selects the integer-math variant (fully_connected.cc:543-621, 874-903):
 * no scales, dst_type must be INT32. */
typedef struct {
  int32_t precision;  /* MLDHIP_PRECISION_*; F32 <=> fp32 tensors, otherwise fp16 tensors.  F16 is
                         computed like F32_F16 (fp32 accumulation of fp16 products): at least as
                         accurate as the reference's all-fp16 arithmetic
                         (common/kernels/fully_connected_util.cc:167-203), not bit-identical to it */
  int32_t src_type;   /* MLDHIP_FLOAT32 / MLDHIP_FLOAT16 / MLDHIP_INT8 */
  int32_t dst_type;   /* MLDHIP_FLOAT32 / MLDHIP_FLOAT16 / MLDHIP_INT32 */
  int32_t o, i;       /* ExternalWeights::shape = OHWI(o,1,1,i) */
  mldhip_weights_desc weights; /* ExternalWeights::desc */
  int32_t scale_o, scale_i;    /* ExternalWeights::scale_zp_shape (o, i); (1,1) = scalar */
  float scalar_scale;          /* used when scale_o*scale_i == 1 */
  int32_t has_zero_point_tensor;
  int32_t has_scalar_zero_point;
  float scalar_zero_point;
  int32_t has_bias;
  int32_t max_tokens; /* upper bound for mldhip_op_set_shape's b*h*w */
  /* ConvRuntimeCheckDesc (common/task/gpu_operation.h:384-412), read when has_runtime_check != 0;
   * an index < 0 means "not set".  With a channel bound set, the op takes one more src object,
   * "params" (int32 values in device memory, registered last, as the reference's tests bind it:
   * common/kernels/tests/fully_connected_test_util.cc:1195-1204), read at launch on the device:
   *   src_end_ch = min(params[src_end_ch_index], i): the K loop stops after ceil(src_end_ch / 4)
   *     slices (fully_connected.cc:750-755, 795; not applied with group-wise scales, whose loop runs
   *     over all groups, :784-794);
   *   dst slices from min(round_up(params[dst_end_ch_index], 32) / 4, ceil(o/4)) on are not
   *     written (fully_connected_util.cc:231-243, fully_connected.cc:644-652).
   * Ringed weights (ring_o_offset_index / ring_i_offset_index >= 0, ring_size > 0; uint8 weights in
   * one output group): the weights buffer is a ring along one axis (a key / value cache bound as
   * weights) whose start is read at launch, offset = params[index] taken modulo ring_size
   * (fully_connected.cc:676-706).
   *   ring_i_offset_index, kOSpatialIOGroupI4O4 (GetRingedIAddresses, fully_connected.cc:424-441):
   *     `i` is the ring's length in input channels, the src tensor has `src_channels` channels, and
   *     src channel c meets weights row (c + offset) % ring_size; composes with src_end_ch_index.
   *   ring_o_offset_index, kOSpatialIOGroupO4I4 (GetRingedOAddresses, fully_connected.cc:411-422):
   *     `o` is the ring's length in output channels (= ring_size, a multiple of 4), the dst tensor has
   *     `dst_channels` channels, and dst channel c is weights row (c + offset) % ring_size; scales,
   *     zero points and biases belong to the dst channel.
   *   With batched weights every matrix is a ring of its own (ring_batch_offset, ring_i_base,
   *   fully_connected.cc:690-706).
   * As in the reference (fully_connected.cc:1087-1097), INVALID_ARGUMENT for weights of fewer than 8
   * bits ("Unsupported WeightsDescription type for ringed weights.") and for the 2D texture layouts
   * ("Unsupported WeightsDescription layout for ringed weights.").  The integer-math variant does not
   * apply a ring in the reference (fully_connected.cc:543-621 reads linear_i4o4) and returns
   * UNIMPLEMENTED here. */
  int32_t has_runtime_check;
  int32_t src_end_ch_index, dst_end_ch_index;
  int32_t ring_o_offset_index, ring_i_offset_index, ring_size;
  /* ConvRuntimeCheckDesc::PackedGroups (common/task/gpu_operation.h:396-406), read when
   * has_runtime_check != 0 and packed_num_groups > 0: the grouped FullyConnected of a
   * mixture-of-experts prefill (MakeConvWithPackedGroups, common/gpu_model_builder_moe_util.cc:119-230).
   * ExternalWeights::shape = OHWI(o, packed_num_groups, 1, i): the matrices packed with the op's
   * WeightsDescription and the scales [scale_i][packed_num_groups][ceil(o/4)][4], both as for
   * mldhip_fc_batch_ids_create (the two ops of a layer read the same buffers).  The source is one row of tokens sorted by matrix; matrix g multiplies
   * the params[packed_params_offset + g] tokens that start at token
   * params[packed_params_offset + packed_num_groups + g] (fully_connected_util.cc:263-277), at most
   * packed_max_group_size of them; dst tokens that belong to no group are not written.  "params" is
   * the last src object; mldhip_op_set_shape(op, 1, 1, tokens). */
  int32_t packed_params_offset, packed_num_groups, packed_max_group_size;
  /* Channels of the src / dst tensors where they differ from the weights' i / o: ringed weights
   * only (ring_i: src_channels, ring_o: dst_channels); 0 = the weights' own. */
  int32_t src_channels, dst_channels;
} mldhip_fc_desc;

int mldhip_fc_create(const mldhip_fc_desc* desc, mldhip_op** op);

/* CreateFullyConnectedWeightsBatchIds (common/kernels/fully_connected.cc:1174-1216): the
 * FullyConnected of a mixture-of-experts layer (common/gpu_model_builder_moe_util.cc:232-291).
 * ExternalWeights::shape = OHWI(o, weights_batch, 1, i): `weights_batch` matrices, packed as the
 * rearrange functions pack OHWI(o, weights_batch, 1, i) with the op's WeightsDescription: one
 * matrix after the other when the description has one output group (what the reference's kernel
 * reads, fully_connected.cc:493-496), else the matrices of an output group one after the other
 * ([o / (4 * group)][weights_batch][ceil(i/4)][group] blocks, weights_conversion.cc:139-185);
 * scale_zp_shape = OHWI(scale_o, weights_batch, 1, scale_i), as a tensor
 * [scale_i][weights_batch][ceil(o/4)][4] (mldhip_scale_to_tensor_batched).  Row y of the dst
 * tensor (h rows of w tokens; mldhip_op_set_shape(op, 1, h, w)) is the FullyConnected of source
 * row min(y, source rows - 1) with matrix batch_ids[y] (fully_connected.cc:654-665, 804-822;
 * fully_connected_util.cc:279-290); the source has h rows, or one row that every dst row reads
 * when `shared_src` is set (fully_connected_test.cc:241-250).  An id outside [0, weights_batch)
 * is clamped into the range.
 * src objects: 0 "src_tensor", 1 "batch_ids" (int32 [h]), 2 "weights", then "weights_scale",
 * "weights_zero_point", "biases" as for mldhip_fc_create (fully_connected.cc:1203-1213).
 * With src_type INT8 / dst_type INT32 the integer-math variant runs over the batched weights (no
 * scale objects).  desc->max_tokens bounds h*w; the tensors have batch 1. */
int mldhip_fc_batch_ids_create(const mldhip_fc_desc* desc, int weights_batch, int shared_src, mldhip_op** op);

/* CreateQuantization (common/kernels/quantize_and_dequantize.h:57-73, .cc:693-842).
 * src 0 "src_tensor" [ceil(c/4)][tokens][4] (FLOAT16 or FLOAT32);
 * dst 0 "dst_tensor": codes, the tensor of GetShapeForPackedType (common/util.cc:262-277) as a
 *       buffer (quantize_and_dequantize.cc:461-653); tokens = (y * w + x) * b + batch element:
 *       C4   [ceil(c/4)][tokens][4] bytes;
 *       C16  [ceil(c/16)][tokens][16] bytes (4 slices x 4 channels);
 *       C32  [ceil(c/32)][tokens][16] bytes: 4-bit codes, channel j of the 32 in nibble j (low
 *            nibble first, two's complement for INT4C32); code range 16 (scale abs_max / 7);
 *       W4C4 [ceil(c/4)][h][ceil(w/4)][b][16] bytes: 4 columns x 4 channels, columns at or beyond
 *            w repeat column w - 1 (set the shape with mldhip_op_set_shape);
 *       slices that pad the last C16 / C32 group repeat the last slice, as in the reference's
 *       kernel (they meet zero weights in the convolution);
 * dst 1 "dst_params": fp32 [tokens][4] = (inv_scale, offset, sum, 0), the BHWC(b,h,w,2|3)
 *       fp32 tensor the builder allocates (common/gpu_model_builder.cc:1285-1289). */
typedef struct {
  int32_t src_type;
  int32_t packed_type; /* MLDHIP_PACKED_* */
  int32_t channels;
  int32_t calculate_sum;
  int32_t symmetric;
  int32_t max_tokens;
  /* 0 (the reference's kernel): codes by floor(x * scale + zero point + 0.5), asymmetric
   * int((x - min) * scale + 0.5) (quantize_and_dequantize.cc:424-434).  1: round-to-nearest-even of
   * the scaled value, rint(x * scale) + zero point and rint((x - min) * scale); no counterpart in the
   * reference.  The two differ by one code where the scaled value lies (within fp32 rounding of the
   * reference's sum) half way between two codes. */
  int32_t round_to_nearest_even;
} mldhip_quant_desc;

int mldhip_quantization_create(const mldhip_quant_desc* desc, mldhip_op** op);

/* GetConvolutionInt8SrcType (common/selectors/convolution_selector.cc:384-400) for this
 * device: the packed activation type the int8 convolution reads (MLDHIP_PACKED_INT8C16). */
int mldhip_conv_int8_src_type(void);

/* CreateConvGenericInt8ExternalWeights (common/kernels/conv_generic.cc:4237-4265) for 1x1
 * kernels with CreateDequantization (common/kernels/quantize_and_dequantize.h:76-81,
 * .cc:867-964) linked as its epilogue, as the builder wires them
 * (common/gpu_model_builder.cc:1325-1431).  src objects in node-input order (:1414-1424):
 *   0 "src_tensor"          codes, src_packed_type
 *   1 "weights"             per `weights` (mldhip_conv_int8_weights_desc)
 *   2 "params_tensor"       fp32 [tokens][4] from the quantization op
 *   3 "weights_sum"         int32, ceil(o/4)*4
 *   4 "weights_scale"       fp32, ceil(o/4)*4
 *   5 "weights_zero_point"  fp32, present iff has_zero_point
 *   6 "biases"              dst_type, present iff has_bias (the builder's separate Add)
 * dst 0 "dst_tensor" [ceil(o/4)][tokens][4]; dst_type INT32 returns the raw accumulators
 * (no epilogue; only objects 0 and 1 are bound). */
typedef struct {
  int32_t src_packed_type;
  int32_t dst_type; /* MLDHIP_FLOAT16 / MLDHIP_FLOAT32 / MLDHIP_INT32 */
  int32_t o, i;
  mldhip_weights_desc weights;
  int32_t has_zero_point;
  int32_t has_bias;
  int32_t max_tokens;
} mldhip_conv_int8_desc;

int mldhip_conv_int8_create(const mldhip_conv_int8_desc* desc, mldhip_op** op);

/* Introspection of the object lists, in registration order (GPUOperation::src_tensors_names_,
 * dst_tensors_names_, common/task/gpu_operation.h:97-274). */
int mldhip_op_src_count(const mldhip_op* op);
int mldhip_op_dst_count(const mldhip_op* op);
const char* mldhip_op_src_name(const mldhip_op* op, int index);
const char* mldhip_op_dst_name(const mldhip_op* op, int index);

/* ClOperation::SetSrcTensor / SetDstTensor (cl/cl_operation.cc:66-82): bind a device buffer
 * to the index-th src / dst object.  `bytes` is checked against what the current shape
 * needs at launch. */
int mldhip_op_set_src(mldhip_op* op, int index, const void* device_ptr, size_t bytes);
int mldhip_op_set_dst(mldhip_op* op, int index, void* device_ptr, size_t bytes);

/* Runtime shape of the activation tensor, BHW (channels are fixed at creation); the
 * counterpart of UpdateParams -> BindArguments + GetGridSize (cl/cl_operation.cc:59-64,
 * common/kernels/fully_connected.cc:944-979).  b*h*w must be <= max_tokens. */
int mldhip_op_set_shape(mldhip_op* op, int b, int h, int w);

/* ClOperation::AddToQueue (cl/cl_operation.cc:84-88): enqueue on `stream` (hipStream_t). */
int mldhip_op_launch(mldhip_op* op, void* stream);

/* One launch for up to 3 FullyConnected ops that read the same "src_tensor" (same binding, same
 * shape, same K and scale grouping) and are served by the same int4 kernel (streaming GEMV at a
 * few tokens, MFMA GEMM beyond), e.g. the
 * q / k / v projections or the gate / up projections of a decoder layer, which the reference
 * emits as separate nodes over one input (samples/llm/gemma3_model_builder.cc:1115-1128).
 * Results are those of launching the ops one by one (bit for bit, except that a fused MFMA launch
 * may split K across work-groups differently, which changes the fp32 summation order).  Returns
 * FAILED_PRECONDITION (and
 * launches nothing) when the ops cannot share a launch; the caller then launches them singly. */
int mldhip_fc_launch_fused(mldhip_op* const* ops, int count, void* stream);

/* The MLP step after the gate and up projections of a decoder layer,
 * dst = activation(gate(x)) * up(x), in the same launch as the two projections
 * (samples/llm/gemma3_model_builder.cc:1054-1090 CreateGeluTanhMulOp over the two Linear nodes of
 * :1141-1147; samples/llm/qwen3_model_builder.cc:850-883 CreateSiluMulOp).  `gate` and `up` are
 * FullyConnected ops bound to the same src_tensor with the same shape; their results are rounded
 * to fp16 (+ biases) as the two nodes would store them and combined in fp32 in the operation
 * order of the sample's elementwise kernel; their own dst tensors are not written.  dst:
 * [ceil(o/4)][tokens][4] halfs.  Served for fp16 tensors and symmetric weights: int4 at 1..2
 * tokens by the streaming GEMV pair, int4 at more tokens and int8 above 4 tokens by the
 * matrix-core GEMM (half of a work-group's waves on gate, half on up, combined where the K
 * reduction ends).  MLDHIP_FAILED_PRECONDITION otherwise:
 * launch the two ops (mldhip_fc_launch_fused) and the host framework's elementwise node
 * instead. */
enum { MLDHIP_GATE_GELU_TANH = 1, MLDHIP_GATE_SILU = 2 };
int mldhip_fc_launch_gated(mldhip_op* gate, mldhip_op* up, int activation, void* dst,
                           size_t dst_bytes, void* stream);

/* No counterpart in the reference.  For callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid it): the int4 decode
 * FullyConnected of mldhip_op_launch (fp16 tensors, 1..4 tokens, symmetric uint4 weights,
 * per-channel scales or scale groups of whole multiples of 32 input channels, optional bias)
 * without an op object: the buffers are passed directly and the split-K sums, which an op keeps in
 * the workspace that its create call allocates, go to an array of 2 MiB that the library holds
 * statically on every GPU it runs on (until the process ends).  Calls no hipMalloc / hipFree.
 * Runs the streaming GEMV kernels (fc_w4_strip_kernel / fc_w4_rows_kernel / fc_w4_stream_kernel), with
 * the results mldhip_op_launch gives wherever it takes the same kernel (one token always; at 2..4
 * tokens mldhip_op_launch prefers the matrix-core GEMV for per-channel layers of 8192 channels and
 * more, whose sums are added in another order).  The current device must be the stream's device.
 * Limits: o <= 65536 (MLDHIP_OUT_OF_RANGE beyond), an even number of 4-channel slices,
 * output_group_size = any even number of slices that divides ceil(o/4) (the reference's one group,
 * 16, the decode layout's 2, ...).  All calls on one GPU share
 * that GPU's array: calls that overlap in time on one GPU (different streams) race; calls on
 * one stream are ordered.  The array needs no clearing between calls.
 *   src [ceil(i/4)][tokens][4] halfs, weights packed uint4, weights_scale [scale_groups][ceil(o/4)][4]
 *   halfs, biases ceil(o/4)*4 halfs or null, dst [ceil(o/4)][tokens][4] halfs. */
int mldhip_fc_int4_decode_noalloc(const void* src, const void* weights, const void* weights_scale,
                                  const void* biases, void* dst, int o, int i, int scale_groups,
                                  int output_group_size, int tokens, void* stream);

/* Name of the kernel the last launch used, and the algorithmic bytes / flops of one launch
 * at the current shape (GPUOperation::flops_/read_size_/write_size_,
 * common/task/gpu_operation.h:190-195). */
const char* mldhip_op_kernel_name(const mldhip_op* op);
int mldhip_op_cost(const mldhip_op* op, uint64_t* bytes, uint64_t* flops);

void mldhip_op_destroy(mldhip_op* op);

#ifdef __cplusplus
}
#endif
#endif /* MLDHIP_H_ */
