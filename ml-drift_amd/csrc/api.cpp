// C-ABI layer: argument validation, op objects (the node executors), kernel dispatch.
#include <algorithm>
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <string>
#include <vector>

#include "../../include/mldhip.h"
#include "kernels.h"
#include "packer.h"

using namespace mldhip;

namespace {
thread_local std::string g_error;
}  // namespace

namespace mldhip {
// Records the calling thread's error message (mldhip_last_error) and returns `code`.
int Fail(int code, const std::string& msg) {
  g_error = msg;
  return code;
}
Tuning& GetTuning() {
  static Tuning tuning;
  return tuning;
}
}  // namespace mldhip

namespace {
using mldhip::Fail;

int HipFail(hipError_t e, const char* what) {
  return Fail(MLDHIP_INTERNAL, std::string(what) + ": " + hipGetErrorString(e));
}

size_t TypeBytes(int type) {
  switch (type) {
    case MLDHIP_FLOAT16: return 2;
    case MLDHIP_FLOAT32: return 4;
    case MLDHIP_INT32: return 4;
    case MLDHIP_UINT8:
    case MLDHIP_INT8: return 1;
    default: return 0;
  }
}

int WeightBits(int type) {
  if (type == MLDHIP_UINT4) return 4;
  if (type == MLDHIP_UINT8 || type == MLDHIP_INT8) return 8;
  return 0;
}

int CheckShape(int o, int h, int w, int i) {
  if (o <= 0 || h <= 0 || w <= 0 || i <= 0) return Fail(MLDHIP_INVALID_ARGUMENT, "weights shape must be positive");
  return MLDHIP_OK;
}

bool IsOGroupLayout(int layout) {
  return layout == MLDHIP_LAYOUT_OSPATIAL_IOGROUP_I4O4 || layout == MLDHIP_LAYOUT_OSPATIAL_IOGROUP_O4I4 ||
         layout == MLDHIP_LAYOUT_2D_YSPATIALIO_XOGROUP_I4O4;
}

int CheckDesc(const mldhip_weights_desc* d) {
  if (!d) return Fail(MLDHIP_INVALID_ARGUMENT, "null WeightsDescription");
  if (IsOGroupLayout(d->layout)) {
    if (d->output_group_size <= 0) return Fail(MLDHIP_INVALID_ARGUMENT, "output_group_size must be positive");
    return MLDHIP_OK;
  }
  if (d->layout == MLDHIP_LAYOUT_CUSTOM_GROUPS) {
    if (d->n_groups <= 0 || d->n_groups > MLDHIP_MAX_CUSTOM_GROUPS)
      return Fail(MLDHIP_INVALID_ARGUMENT, "custom groups: bad group count");
    for (int g = 0; g < d->n_groups; ++g)
      if (d->group_axis[g] < 0 || d->group_axis[g] > 3)
        return Fail(MLDHIP_INVALID_ARGUMENT, "custom groups: bad axis");
    return MLDHIP_OK;
  }
  return Fail(MLDHIP_UNIMPLEMENTED, "Unsupported layout");
}

}  // namespace

struct mldhip_op {
  enum Kind { kFc, kQuant, kConvInt8 } kind = kFc;
  std::vector<std::string> src_names, dst_names;
  std::vector<const void*> src_ptr;
  std::vector<size_t> src_bytes;
  std::vector<void*> dst_ptr;
  std::vector<size_t> dst_bytes;
  int b = 1, h = 1, w = 1;
  int max_tokens = 1;
  mldhip_fc_desc fc{};
  mldhip_quant_desc q{};
  mldhip_conv_int8_desc cv{};
  int idx_scale = -1, idx_zp = -1, idx_bias = -1;
  // FullyConnected with batched weights selected by a runtime tensor of ids
  int idx_weights = 1, idx_ids = -1;
  int idx_params = -1;  // runtime channel bounds
  int weights_batch = 1;  // ExternalWeights::shape.h
  int src_c = 0, dst_c = 0;  // channels of the src / dst tensors (the weights' i / o unless the weights are ringed)
  int shared_src = 0;     // the source tensor has one row that every dst row reads
  float* partial = nullptr;
  size_t partial_floats = 0;
  const char* last_kernel = "";
  // bytes every object needs at the current shape (kept up to date by create and set_shape, so that
  // a launch checks its bindings without touching the heap)
  std::vector<size_t> need_src, need_dst;

  void AddSrc(const char* name) {
    src_names.emplace_back(name);
    src_ptr.push_back(nullptr);
    src_bytes.push_back(0);
  }
  void AddDst(const char* name) {
    dst_names.emplace_back(name);
    dst_ptr.push_back(nullptr);
    dst_bytes.push_back(0);
  }
  int Tokens() const { return b * h * w; }
};

extern "C" {

static void UpdateRequiredSizes(mldhip_op* op);

const char* mldhip_last_error(void) { return g_error.c_str(); }
const char* mldhip_version(void) { return "mldhip 0.1 (gfx950)"; }

// ---------------------------------------------------------------------------------------
// weight descriptions and packers
// ---------------------------------------------------------------------------------------

static int FcDesc(int o, int i, int type, bool native_groups, mldhip_weights_desc* desc) {
  if (!desc) return Fail(MLDHIP_INVALID_ARGUMENT, "null desc");
  if (o <= 0 || i <= 0) return Fail(MLDHIP_INVALID_ARGUMENT, "weights shape must be positive");
  std::memset(desc, 0, sizeof(*desc));
  desc->type = type;
  desc->layout = MLDHIP_LAYOUT_OSPATIAL_IOGROUP_I4O4;
  const int ns = DivUp(o, 4);
  // uint4 weights: output groups of 16, 8 or 4 slices, so that the K rows of a strip of channels
  // lie one after the other in memory
  desc->output_group_size = ns;
  if (native_groups) {
    desc->output_group_size = NativeGroupFor(o);
    const int forced = GetTuning().fc_group;
    if (forced > 0 && o % 4 == 0 && ns % forced == 0 && (IsNativeGroup(forced) || forced == ns)) desc->output_group_size = forced;
  }
  return MLDHIP_OK;
}

int mldhip_fc_int8_weights_desc(int o, int i, mldhip_weights_desc* desc) {
  return FcDesc(o, i, MLDHIP_UINT8, false, desc);
}
int mldhip_fc_int4_weights_desc(int o, int i, mldhip_weights_desc* desc) {
  return FcDesc(o, i, MLDHIP_UINT4, true, desc);
}
int mldhip_fc_int4_weights_desc_reference(int o, int i, mldhip_weights_desc* desc) {
  return FcDesc(o, i, MLDHIP_UINT4, false, desc);
}
int mldhip_fc_int8_weights_desc_decode(int o, int i, mldhip_weights_desc* desc) {
  if (int rc = FcDesc(o, i, MLDHIP_UINT8, false, desc)) return rc;
  // output groups of one slice (what FullyConnectedOI reads), which the one-token kernel reads with
  // the whole K of 4 channels inside a work-group
  if (o > 4 && GetTuning().fc_group <= 0) desc->output_group_size = 1;
  return MLDHIP_OK;
}
int mldhip_fc_int4_weights_desc_decode(int o, int i, mldhip_weights_desc* desc) {
  if (int rc = FcDesc(o, i, MLDHIP_UINT4, true, desc)) return rc;
  // fewer than 128 strips of 64 channels: strips of 8 channels (output groups of 2 slices), which the
  // one-token kernel reads with the whole K inside a work-group
  if (o % 8 == 0 && o / 64 < 128 && GetTuning().fc_group <= 0) desc->output_group_size = 2;
  return MLDHIP_OK;
}

int mldhip_set_tuning(const char* name, int value) {
  if (!name) return Fail(MLDHIP_INVALID_ARGUMENT, "null name");
  Tuning& t = GetTuning();
  const struct { const char* name; int* field; } knobs[] = {
      {"force_generic", &t.force_generic}, {"gemv_mfma", &t.gemv_mfma}, {"gemv_fast", &t.gemv_fast},
      {"fc_group", &t.fc_group}, {"gemv_rows_rpt", &t.gemv_rows_rpt},
      {"gemv_one_chunk", &t.gemv_one_chunk},
      {"gemv_lpr", &t.gemv_lpr}, {"gemv_waves", &t.gemv_waves}, {"gemv_ksplit", &t.gemv_ksplit},
      {"gemv_narrow_max_mb", &t.gemv_narrow_max_mb}, {"gemm_fm", &t.gemm_fm}, {"gemm_ksplit", &t.gemm_ksplit},
      {"gemm_no_pair", &t.gemm_no_pair}, {"gemm_dual", &t.gemm_dual}, {"gemm_xcd_m", &t.gemm_xcd_m},
      {"gemm_i8_fm", &t.gemm_i8_fm}, {"gemm_tiled", &t.gemm_tiled}};
  for (const auto& k : knobs)
    if (std::strcmp(name, k.name) == 0) {
      *k.field = value;
      return MLDHIP_OK;
    }
  return Fail(MLDHIP_NOT_FOUND, std::string("unknown tuning knob: ") + name);
}

int mldhip_conv_int8_weights_desc(int o, int i, mldhip_weights_desc* desc) {
  if (!desc) return Fail(MLDHIP_INVALID_ARGUMENT, "null desc");
  if (o <= 0 || i <= 0) return Fail(MLDHIP_INVALID_ARGUMENT, "weights shape must be positive");
  std::memset(desc, 0, sizeof(*desc));
  desc->type = MLDHIP_INT8;
  desc->layout = MLDHIP_LAYOUT_CUSTOM_GROUPS;
  desc->output_group_size = 1;
  desc->n_groups = 3;
  desc->group_axis[0] = MLDHIP_AXIS_I;
  desc->group_size[0] = 16;
  desc->group_axis[1] = MLDHIP_AXIS_O;
  desc->group_size[1] = 0;
  desc->group_axis[2] = MLDHIP_AXIS_I;
  desc->group_size[2] = 0;
  return MLDHIP_OK;
}

int mldhip_total_elements(const mldhip_weights_desc* desc, int o, int h, int w, int i, size_t* elements) {
  if (!elements) return Fail(MLDHIP_INVALID_ARGUMENT, "null output");
  if (int rc = CheckDesc(desc)) return rc;
  if (int rc = CheckShape(o, h, w, i)) return rc;
  const PackShape sh{o, h, w, i};
  *elements = desc->layout == MLDHIP_LAYOUT_CUSTOM_GROUPS
                  ? CustomTotalElements(sh, desc->group_axis, desc->group_size, desc->n_groups)
                  : TotalElements(sh, desc->layout, desc->output_group_size);
  return MLDHIP_OK;
}

int mldhip_packed_bytes(const mldhip_weights_desc* desc, int o, int h, int w, int i, size_t* bytes) {
  size_t elements = 0;
  if (int rc = mldhip_total_elements(desc, o, h, w, i, &elements)) return rc;
  const int bits = WeightBits(desc->type);
  if (!bits) return Fail(MLDHIP_INVALID_ARGUMENT, "Unsupported WeightsDescription type");
  *bytes = (elements * bits + 7) / 8;
  return MLDHIP_OK;
}

static int CheckPackArgs(const void* weights, const mldhip_weights_desc* desc, const void* dst, int o, int h,
                         int w, int i, size_t dst_bytes, int bits) {
  if (!weights || !dst) return Fail(MLDHIP_INVALID_ARGUMENT, "null buffer");
  if (int rc = CheckDesc(desc)) return rc;
  if (int rc = CheckShape(o, h, w, i)) return rc;
  size_t elements = 0;
  if (int rc = mldhip_total_elements(desc, o, h, w, i, &elements)) return rc;
  if (dst_bytes < (elements * bits + 7) / 8)
    return Fail(MLDHIP_INVALID_ARGUMENT, "destination span is smaller than the layout needs");
  return MLDHIP_OK;
}

int mldhip_rearrange_int8_as_uint8(const int8_t* weights, int o, int h, int w, int i,
                                   const mldhip_weights_desc* desc, uint8_t* dst, size_t dst_bytes, int shift,
                                   unsigned pad) {
  if (int rc = CheckPackArgs(weights, desc, dst, o, h, w, i, dst_bytes, 8)) return rc;
  if (!IsOGroupLayout(desc->layout)) return Fail(MLDHIP_UNIMPLEMENTED, "Unsupported layout");
  RearrangeU8(reinterpret_cast<const uint8_t*>(weights), PackShape{o, h, w, i}, desc->layout,
              desc->output_group_size, (uint8_t)pad, shift, dst);
  return MLDHIP_OK;
}

int mldhip_rearrange_int8_as_uint4(const int8_t* weights, int o, int h, int w, int i,
                                   const mldhip_weights_desc* desc, uint8_t* dst, size_t dst_bytes, int shift,
                                   unsigned pad) {
  if (int rc = CheckPackArgs(weights, desc, dst, o, h, w, i, dst_bytes, 4)) return rc;
  if (!IsOGroupLayout(desc->layout)) return Fail(MLDHIP_UNIMPLEMENTED, "Unsupported layout");
  RearrangeInt8AsUint4(weights, PackShape{o, h, w, i}, desc->layout, desc->output_group_size, shift, pad, dst);
  return MLDHIP_OK;
}

int mldhip_rearrange_int8(const int8_t* weights, int o, int h, int w, int i, const mldhip_weights_desc* desc,
                          int8_t* dst, size_t dst_bytes) {
  if (int rc = CheckPackArgs(weights, desc, dst, o, h, w, i, dst_bytes, 8)) return rc;
  const PackShape sh{o, h, w, i};
  if (desc->layout == MLDHIP_LAYOUT_CUSTOM_GROUPS) {
    RearrangeCustomI8(weights, sh, desc->group_axis, desc->group_size, desc->n_groups, 0, dst);
  } else {
    RearrangeU8(reinterpret_cast<const uint8_t*>(weights), sh, desc->layout, desc->output_group_size, 0, 0,
                reinterpret_cast<uint8_t*>(dst));
  }
  return MLDHIP_OK;
}

int mldhip_rearrange_uint4_packed(const uint8_t* weights, int o, int h, int w, int i,
                                  const mldhip_weights_desc* desc, uint8_t* dst, size_t dst_bytes,
                                  int32_t* weights_sum_i, size_t sum_len, unsigned pad, int swap_dims) {
  if (!desc) return Fail(MLDHIP_INVALID_ARGUMENT, "null WeightsDescription");
  if (desc->layout != MLDHIP_LAYOUT_OSPATIAL_IOGROUP_I4O4 &&
      desc->layout != MLDHIP_LAYOUT_2D_YSPATIALIO_XOGROUP_I4O4)
    return Fail(MLDHIP_UNIMPLEMENTED, "Unsupported layout");
  if (int rc = CheckPackArgs(weights, desc, dst, o, h, w, i, dst_bytes, 4)) return rc;
  if (!weights_sum_i) return Fail(MLDHIP_INVALID_ARGUMENT, "null weights_sum_i");
  RearrangeUint4Packed(weights, PackShape{o, h, w, i}, desc->layout, desc->output_group_size, dst, weights_sum_i,
                       sum_len, pad, swap_dims != 0);
  return MLDHIP_OK;
}

int mldhip_weights_sum_i(const int8_t* weights, int o, int h, int w, int i, int32_t* sum) {
  if (!weights || !sum) return Fail(MLDHIP_INVALID_ARGUMENT, "null buffer");
  if (int rc = CheckShape(o, h, w, i)) return rc;
  WeightsSumI(weights, PackShape{o, h, w, i}, sum);
  return MLDHIP_OK;
}

static uint16_t FloatToHalfBits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const int32_t exp = (int32_t)((x >> 23) & 0xFF) - 127 + 15;
  uint32_t man = x & 0x7FFFFFu;
  if (((x >> 23) & 0xFF) == 0xFF) return (uint16_t)(sign | 0x7C00u | (man ? 0x200u : 0u));
  if (exp >= 31) return (uint16_t)(sign | 0x7C00u);
  if (exp <= 0) {
    if (exp < -10) return (uint16_t)sign;
    man |= 0x800000u;
    const int shift = 14 - exp;
    uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) ++q;
    return (uint16_t)(sign | q);
  }
  uint32_t q = ((uint32_t)exp << 10) | (man >> 13);
  const uint32_t rem = man & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1))) ++q;
  return (uint16_t)(sign | q);
}

int mldhip_scale_to_tensor_batched(const float* scale, int o, int batch, int groups, int dst_type, void* dst,
                                   size_t dst_bytes) {
  if (!scale || !dst) return Fail(MLDHIP_INVALID_ARGUMENT, "null buffer");
  if (o <= 0 || groups <= 0 || batch <= 0) return Fail(MLDHIP_INVALID_ARGUMENT, "bad scale shape");
  if (dst_type != MLDHIP_FLOAT16 && dst_type != MLDHIP_FLOAT32)
    return Fail(MLDHIP_INVALID_ARGUMENT, "scale tensor type must be FLOAT16 or FLOAT32");
  const int os = DivUp(o, 4);
  const size_t count = (size_t)groups * batch * os * 4;
  if (dst_bytes < count * TypeBytes(dst_type)) return Fail(MLDHIP_INVALID_ARGUMENT, "destination too small");
  for (int g = 0; g < groups; ++g)
    for (int b = 0; b < batch; ++b)
      for (int oc = 0; oc < os * 4; ++oc) {
        const float v = oc < o ? scale[((size_t)oc * batch + b) * groups + g] : 0.0f;
        const size_t idx = ((size_t)g * batch + b) * os * 4 + oc;
        if (dst_type == MLDHIP_FLOAT32)
          static_cast<float*>(dst)[idx] = v;
        else
          static_cast<uint16_t*>(dst)[idx] = FloatToHalfBits(v);
      }
  return MLDHIP_OK;
}

int mldhip_scale_to_tensor(const float* scale, int o, int groups, int dst_type, void* dst, size_t dst_bytes) {
  return mldhip_scale_to_tensor_batched(scale, o, 1, groups, dst_type, dst, dst_bytes);
}

// ---------------------------------------------------------------------------------------
// ops
// ---------------------------------------------------------------------------------------

int mldhip_fc_is_recommended(int precision, int tokens) {
  (void)precision;
  return tokens <= kGemvMaxTokens ? 1 : 0;
}

static int AllocWorkspace(mldhip_op* op, int n, bool ring_i = false) {
  if (op->partial) return MLDHIP_OK;
  // A host without a GPU can still create and inspect ops (object lists, validation); they cannot
  // be launched there, so they need no workspace.
  int devices = 0;
  if (hipGetDeviceCount(&devices) != hipSuccess || devices == 0) {
    (void)hipGetLastError();
    return MLDHIP_OK;
  }
  const int n_pad = DivUp(n, 4) * 4;
  op->partial_floats = std::max((size_t)kGemvMaxKSplit * kGemvMaxTokens * n_pad,
                                FcW4MfmaWorkspaceFloats(op->fc.max_tokens, op->fc.i, op->fc.o));
  // (the ring over the input channels: partial sums of the parts of its window)
  if (ring_i) op->partial_floats = FcW8RingWorkspaceFloats(op->fc.max_tokens, op->fc.o);
  hipError_t e = hipMalloc(reinterpret_cast<void**>(&op->partial), op->partial_floats * sizeof(float));
  if (e != hipSuccess) return HipFail(e, "hipMalloc(workspace)");
  return MLDHIP_OK;
}

static int CreateFc(const mldhip_fc_desc* d, bool batch_ids, int weights_batch, int shared_src, mldhip_op** out) {
  if (!d || !out) return Fail(MLDHIP_INVALID_ARGUMENT, "null argument");
  *out = nullptr;
  if (batch_ids && weights_batch < 1) return Fail(MLDHIP_INVALID_ARGUMENT, "weights_batch must be positive");
  if (d->o <= 0 || d->i <= 0) return Fail(MLDHIP_INVALID_ARGUMENT, "weights shape must be positive");
  if (d->max_tokens <= 0) return Fail(MLDHIP_INVALID_ARGUMENT, "max_tokens must be positive");
  const mldhip_weights_desc& wd = d->weights;
  if (wd.type != MLDHIP_UINT8 && wd.type != MLDHIP_UINT4) {
    if (wd.type == MLDHIP_FLOAT16 || wd.type == MLDHIP_FLOAT32)
      return Fail(MLDHIP_UNIMPLEMENTED, "float weights are outside the quantized path");
    return Fail(MLDHIP_INVALID_ARGUMENT, "Unsupported WeightsDescription type.");
  }
  // Ringed weights: refused where the reference refuses them (fully_connected.cc:1087-1097: types under
  // 8 bits, layouts that are not linear = the 2D texture layouts, weights_layout.cc:167-171)
  const bool ring_i = d->has_runtime_check && d->ring_i_offset_index >= 0;
  const bool ring_o = d->has_runtime_check && d->ring_o_offset_index >= 0;
  if (ring_i || ring_o) {
    if (wd.type == MLDHIP_UINT4) return Fail(MLDHIP_INVALID_ARGUMENT, "Unsupported WeightsDescription type for ringed weights.");
    if (wd.layout == MLDHIP_LAYOUT_2D_YSPATIALIO_XOGROUP_I4O4)
      return Fail(MLDHIP_INVALID_ARGUMENT, "Unsupported WeightsDescription layout for ringed weights.");
    if (ring_i && ring_o) return Fail(MLDHIP_INVALID_ARGUMENT, "ring_o_offset_index and ring_i_offset_index exclude each other");
    if (d->ring_size < 1) return Fail(MLDHIP_INVALID_ARGUMENT, "ringed weights need a positive ring_size");
    // the reference's address arithmetic is written for these two (fully_connected.cc:411-441: "kOSpatialIOGroupO4I4 ->
    // kBIOI4", "kOSpatialIOGroupI4O4 -> kBIOI4O4")
    if (wd.layout != (ring_i ? MLDHIP_LAYOUT_OSPATIAL_IOGROUP_I4O4 : MLDHIP_LAYOUT_OSPATIAL_IOGROUP_O4I4))
      return Fail(MLDHIP_UNIMPLEMENTED, "ring_i_offset_index reads kOSpatialIOGroupI4O4 weights, ring_o_offset_index kOSpatialIOGroupO4I4");
    if (wd.output_group_size != DivUp(d->o, 4))
      return Fail(MLDHIP_UNIMPLEMENTED, "ringed weights are read in one output group (output_group_size = ceil(o / 4))");
    if (d->src_type == MLDHIP_INT8)
      return Fail(MLDHIP_UNIMPLEMENTED, "the integer-math FullyConnected does not apply a ring (nor does the reference's)");
    if (d->packed_num_groups > 0) return Fail(MLDHIP_UNIMPLEMENTED, "ringed weights with packed groups are not supported");
    if (ring_i && (d->ring_size > DivUp(d->i, 4) * 4 || ((batch_ids && weights_batch > 1) && d->ring_size != d->i)))
      return Fail(MLDHIP_INVALID_ARGUMENT, "ring_size exceeds the weights' input channels (batched weights: must equal them)");
    if (ring_o && (d->ring_size != d->o || d->o % 4 != 0))
      return Fail(MLDHIP_INVALID_ARGUMENT, "ring_o_offset_index: ring_size must equal the weights' output channels, a multiple of 4");
  } else if (wd.layout != MLDHIP_LAYOUT_OSPATIAL_IOGROUP_I4O4) {
    if (wd.layout == MLDHIP_LAYOUT_2D_YSPATIALIO_XOGROUP_I4O4)
      return Fail(MLDHIP_UNIMPLEMENTED, "texture weight layouts are not supported; use the buffer layout");
    if (wd.layout == MLDHIP_LAYOUT_OSPATIAL_IOGROUP_O4I4)
      return Fail(MLDHIP_UNIMPLEMENTED, "kOSpatialIOGroupO4I4 weights are served as ringed weights only; use kOSpatialIOGroupI4O4");
    return Fail(MLDHIP_INVALID_ARGUMENT, "Unsupported WeightsDescription layout");
  }
  if (!ring_i && d->src_channels > 0 && d->src_channels != d->i)
    return Fail(MLDHIP_INVALID_ARGUMENT, "src_channels differs from the weights' input channels without ring_i_offset_index");
  if (!ring_o && d->dst_channels > 0 && d->dst_channels != d->o)
    return Fail(MLDHIP_INVALID_ARGUMENT, "dst_channels differs from the weights' output channels without ring_o_offset_index");
  // channels of the tensors: the weights' own, except along a ringed axis
  const int src_c = ring_i && d->src_channels > 0 ? d->src_channels : d->i;
  const int dst_c = ring_o && d->dst_channels > 0 ? d->dst_channels : d->o;
  {
    const int ns = DivUp(d->o, 4);
    // One output group is the layout of FullyConnected (fully_connected.cc:1073-1086); groups of one
    // slice are the layout FullyConnectedOI reads (linear_i4o4 = dst_s * src_slices + src_s,
    // fully_connected_oi.cc:122-133); any other whole number of groups is addressed the same way.
    // Batched weights: as the packers lay out an OHWI shape whose height is the batch (the matrices
    // of an output group one after the other; with one group, one matrix after the other).
    const bool whole_groups = wd.output_group_size > 0 && ns % wd.output_group_size == 0;
    if (wd.output_group_size != ns && !whole_groups)
      return Fail(MLDHIP_INVALID_ARGUMENT, "Unsupported WeightsDescription output_group_size.");
  }
  if (d->precision < MLDHIP_PRECISION_F32 || d->precision > MLDHIP_PRECISION_F16)
    return Fail(MLDHIP_INVALID_ARGUMENT, "bad precision");
  const bool int8_math = d->src_type == MLDHIP_INT8;
  if (int8_math) {
    if (d->dst_type != MLDHIP_INT32) return Fail(MLDHIP_INVALID_ARGUMENT, "int8 source needs an int32 destination");
    if (d->scale_o * d->scale_i > 1 || d->has_zero_point_tensor || d->has_bias)
      return Fail(MLDHIP_INVALID_ARGUMENT, "int8-math FullyConnected takes no scale, zero point or bias");
  } else {
    const int tensor_type = d->precision == MLDHIP_PRECISION_F32 ? MLDHIP_FLOAT32 : MLDHIP_FLOAT16;
    if (d->src_type != tensor_type || d->dst_type != tensor_type)
      return Fail(MLDHIP_INVALID_ARGUMENT, "tensor types do not match the calculations precision");
    if (d->scale_o < 1 || d->scale_i < 1) return Fail(MLDHIP_INVALID_ARGUMENT, "bad scale_zp_shape");
    if (d->scale_o != 1 && d->scale_o != dst_c)
      return Fail(MLDHIP_INVALID_ARGUMENT, "scale_zp_shape.o must be 1 or the output channel count");
    if (d->scale_o == 1 && d->scale_i != 1)
      return Fail(MLDHIP_INVALID_ARGUMENT, "group-wise scales need one row per output channel");
    if (d->scale_i > 1 && (d->scale_i > src_c / 4 || (src_c % (4 * d->scale_i)) != 0))
      return Fail(MLDHIP_INVALID_ARGUMENT, "input channels must split into scale groups of whole 4-channel slices");
    if (d->has_zero_point_tensor && d->scale_o * d->scale_i == 1)
      return Fail(MLDHIP_INVALID_ARGUMENT, "a zero-point tensor needs a scale tensor of the same shape");
  }
  bool runtime_bounds = false, packed_groups = false;
  if (d->has_runtime_check) {
    runtime_bounds = d->src_end_ch_index >= 0 || d->dst_end_ch_index >= 0 || ring_i || ring_o;
    if (d->packed_num_groups > 0) {
      if (batch_ids) return Fail(MLDHIP_INVALID_ARGUMENT, "packed groups and batch ids exclude each other");
      if (d->packed_params_offset < 0 || d->packed_max_group_size < 1)
        return Fail(MLDHIP_INVALID_ARGUMENT, "packed groups need a params offset >= 0 and a positive max_group_size");
      packed_groups = true;
      weights_batch = d->packed_num_groups;
    }
  }
  mldhip_op* op = new (std::nothrow) mldhip_op();
  if (!op) return Fail(MLDHIP_INTERNAL, "out of memory");
  op->kind = mldhip_op::kFc;
  op->fc = *d;
  if (!d->has_runtime_check)
    op->fc.src_end_ch_index = op->fc.dst_end_ch_index = op->fc.ring_i_offset_index = op->fc.ring_o_offset_index = -1;
  op->src_c = src_c;
  op->dst_c = dst_c;
  if (!packed_groups) op->fc.packed_num_groups = 0;
  if (packed_groups) op->weights_batch = weights_batch;
  op->max_tokens = d->max_tokens;
  op->AddSrc("src_tensor");
  if (batch_ids) {  // registered before the weights objects (fully_connected.cc:1203-1208)
    op->idx_ids = (int)op->src_names.size();
    op->AddSrc("batch_ids");
    op->weights_batch = weights_batch;
    op->shared_src = shared_src ? 1 : 0;
  }
  op->idx_weights = (int)op->src_names.size();
  op->AddSrc("weights");
  if (!int8_math && d->scale_o * d->scale_i > 1) {
    op->idx_scale = (int)op->src_names.size();
    op->AddSrc("weights_scale");
    if (d->has_zero_point_tensor) {
      op->idx_zp = (int)op->src_names.size();
      op->AddSrc("weights_zero_point");
    }
  }
  if (d->has_bias) {
    op->idx_bias = (int)op->src_names.size();
    op->AddSrc("biases");
  }
  if (runtime_bounds || packed_groups) {
    op->idx_params = (int)op->src_names.size();
    op->AddSrc("params");
  }
  op->AddDst("dst_tensor");
  // split-K workspace of the fp16 streaming and matrix-core kernels: allocated here, so that no
  // launch allocates (a first launch may be under stream capture)
  if (!int8_math && (d->src_type == MLDHIP_FLOAT16 || ring_i)) {
    if (int rc = AllocWorkspace(op, d->o, ring_i)) {
      delete op;
      return rc;
    }
  }
  UpdateRequiredSizes(op);
  *out = op;
  return MLDHIP_OK;
}

int mldhip_fc_create(const mldhip_fc_desc* d, mldhip_op** out) { return CreateFc(d, false, 1, 0, out); }

int mldhip_fc_batch_ids_create(const mldhip_fc_desc* d, int weights_batch, int shared_src, mldhip_op** out) {
  return CreateFc(d, true, weights_batch, shared_src, out);
}

int mldhip_quantization_create(const mldhip_quant_desc* d, mldhip_op** out) {
  if (!d || !out) return Fail(MLDHIP_INVALID_ARGUMENT, "null argument");
  *out = nullptr;
  if (d->src_type != MLDHIP_FLOAT16 && d->src_type != MLDHIP_FLOAT32)
    return Fail(MLDHIP_INVALID_ARGUMENT, "source must be FLOAT16 or FLOAT32");
  if (d->packed_type < MLDHIP_PACKED_UINT8C4 || d->packed_type > MLDHIP_PACKED_UINT4C32)
    return Fail(MLDHIP_INVALID_ARGUMENT, "unknown packed type");
  if (d->channels <= 0 || d->max_tokens <= 0) return Fail(MLDHIP_INVALID_ARGUMENT, "bad shape");
  if (d->round_to_nearest_even != 0 && d->round_to_nearest_even != 1)
    return Fail(MLDHIP_INVALID_ARGUMENT, "round_to_nearest_even must be 0 or 1");
  mldhip_op* op = new (std::nothrow) mldhip_op();
  if (!op) return Fail(MLDHIP_INTERNAL, "out of memory");
  op->kind = mldhip_op::kQuant;
  op->q = *d;
  op->max_tokens = d->max_tokens;
  op->AddSrc("src_tensor");
  op->AddDst("dst_tensor");
  op->AddDst("dst_params");
  UpdateRequiredSizes(op);
  *out = op;
  return MLDHIP_OK;
}

int mldhip_conv_int8_src_type(void) { return MLDHIP_PACKED_INT8C16; }

int mldhip_conv_int8_create(const mldhip_conv_int8_desc* d, mldhip_op** out) {
  if (!d || !out) return Fail(MLDHIP_INVALID_ARGUMENT, "null argument");
  *out = nullptr;
  if (d->o <= 0 || d->i <= 0 || d->max_tokens <= 0) return Fail(MLDHIP_INVALID_ARGUMENT, "bad shape");
  if (d->src_packed_type != MLDHIP_PACKED_INT8C16)
    return Fail(MLDHIP_UNIMPLEMENTED, "the int8 convolution reads kInt8C16 activations");
  mldhip_weights_desc want;
  mldhip_conv_int8_weights_desc(d->o, d->i, &want);
  const mldhip_weights_desc& wd = d->weights;
  bool same = wd.type == want.type && wd.layout == want.layout && wd.n_groups == want.n_groups;
  for (int g = 0; same && g < want.n_groups; ++g)
    same = wd.group_axis[g] == want.group_axis[g] && wd.group_size[g] == want.group_size[g];
  if (!same)
    return Fail(MLDHIP_INVALID_ARGUMENT,
                "weights must be in the layout mldhip_conv_int8_weights_desc returns (convert them first)");
  if (d->dst_type != MLDHIP_FLOAT16 && d->dst_type != MLDHIP_FLOAT32 && d->dst_type != MLDHIP_INT32)
    return Fail(MLDHIP_INVALID_ARGUMENT, "bad destination type");
  mldhip_op* op = new (std::nothrow) mldhip_op();
  if (!op) return Fail(MLDHIP_INTERNAL, "out of memory");
  op->kind = mldhip_op::kConvInt8;
  op->cv = *d;
  op->max_tokens = d->max_tokens;
  op->AddSrc("src_tensor");
  op->AddSrc("weights");
  if (d->dst_type != MLDHIP_INT32) {
    op->AddSrc("params_tensor");
    op->AddSrc("weights_sum");
    op->AddSrc("weights_scale");
    if (d->has_zero_point) {
      op->idx_zp = (int)op->src_names.size();
      op->AddSrc("weights_zero_point");
    }
    if (d->has_bias) {
      op->idx_bias = (int)op->src_names.size();
      op->AddSrc("biases");
    }
  }
  op->AddDst("dst_tensor");
  UpdateRequiredSizes(op);
  *out = op;
  return MLDHIP_OK;
}

int mldhip_op_src_count(const mldhip_op* op) { return op ? (int)op->src_names.size() : 0; }
int mldhip_op_dst_count(const mldhip_op* op) { return op ? (int)op->dst_names.size() : 0; }
const char* mldhip_op_src_name(const mldhip_op* op, int index) {
  if (!op || index < 0 || index >= (int)op->src_names.size()) return nullptr;
  return op->src_names[index].c_str();
}
const char* mldhip_op_dst_name(const mldhip_op* op, int index) {
  if (!op || index < 0 || index >= (int)op->dst_names.size()) return nullptr;
  return op->dst_names[index].c_str();
}

int mldhip_op_set_src(mldhip_op* op, int index, const void* device_ptr, size_t bytes) {
  if (!op) return Fail(MLDHIP_INVALID_ARGUMENT, "null op");
  if (index < 0 || index >= (int)op->src_ptr.size()) return Fail(MLDHIP_OUT_OF_RANGE, "src index out of range");
  if (!device_ptr) return Fail(MLDHIP_INVALID_ARGUMENT, "null device pointer");
  if (reinterpret_cast<uintptr_t>(device_ptr) % 16 != 0)
    return Fail(MLDHIP_INVALID_ARGUMENT, "src object '" + op->src_names[index] + "' is not 16-byte aligned");
  op->src_ptr[index] = device_ptr;
  op->src_bytes[index] = bytes;
  return MLDHIP_OK;
}

int mldhip_op_set_dst(mldhip_op* op, int index, void* device_ptr, size_t bytes) {
  if (!op) return Fail(MLDHIP_INVALID_ARGUMENT, "null op");
  if (index < 0 || index >= (int)op->dst_ptr.size()) return Fail(MLDHIP_OUT_OF_RANGE, "dst index out of range");
  if (!device_ptr) return Fail(MLDHIP_INVALID_ARGUMENT, "null device pointer");
  if (reinterpret_cast<uintptr_t>(device_ptr) % 16 != 0)
    return Fail(MLDHIP_INVALID_ARGUMENT, "dst object '" + op->dst_names[index] + "' is not 16-byte aligned");
  op->dst_ptr[index] = device_ptr;
  op->dst_bytes[index] = bytes;
  return MLDHIP_OK;
}

int mldhip_op_set_shape(mldhip_op* op, int b, int h, int w) {
  if (!op) return Fail(MLDHIP_INVALID_ARGUMENT, "null op");
  if (b <= 0 || h <= 0 || w <= 0) return Fail(MLDHIP_INVALID_ARGUMENT, "shape must be positive");
  if ((long long)b * h * w > op->max_tokens) return Fail(MLDHIP_OUT_OF_RANGE, "b*h*w exceeds max_tokens");
  if (op->idx_ids >= 0 && b != 1) return Fail(MLDHIP_UNIMPLEMENTED, "batched weights: the tensors have batch 1");
  op->b = b;
  op->h = h;
  op->w = w;
  UpdateRequiredSizes(op);
  return MLDHIP_OK;
}

// Sizes (bytes) every object needs at the current shape, in object order.
static void RequiredSizes(const mldhip_op* op, std::vector<size_t>* src, std::vector<size_t>* dst) {
  const size_t m = (size_t)op->Tokens();
  src->assign(op->src_ptr.size(), 0);
  dst->assign(op->dst_ptr.size(), 0);
  if (op->kind == mldhip_op::kFc) {
    const mldhip_fc_desc& d = op->fc;
    // tensor slices, and the slices of the weights' own shape (they differ along a ringed axis)
    const size_t ks = DivUp(op->src_c, 4), ns = DivUp(op->dst_c, 4);
    const size_t wks = DivUp(d.i, 4), wns = DivUp(d.o, 4);
    const size_t wbatch = (size_t)op->weights_batch;
    // batched weights: h rows of w tokens; a shared source has one row
    (*src)[0] = ks * (op->shared_src ? (size_t)op->w : m) * 4 * TypeBytes(d.src_type);
    if (op->idx_ids >= 0) (*src)[op->idx_ids] = (size_t)op->h * sizeof(int32_t);
    (*src)[op->idx_weights] = wbatch * wks * wns * 16 * WeightBits(d.weights.type) / 8;
    const size_t tb = TypeBytes(d.src_type);
    if (op->idx_scale >= 0) (*src)[op->idx_scale] = (size_t)d.scale_i * wbatch * ns * 4 * tb;
    if (op->idx_zp >= 0) (*src)[op->idx_zp] = (size_t)d.scale_i * wbatch * ns * 4 * tb;
    if (op->idx_bias >= 0) (*src)[op->idx_bias] = ns * 4 * TypeBytes(d.dst_type);
    if (op->idx_params >= 0) {
      int values = std::max(std::max(d.src_end_ch_index, d.dst_end_ch_index), std::max(d.ring_i_offset_index, d.ring_o_offset_index)) + 1;
      if (d.packed_num_groups > 0) values = std::max(values, d.packed_params_offset + 2 * d.packed_num_groups);
      (*src)[op->idx_params] = (size_t)values * sizeof(int32_t);
    }
    (*dst)[0] = ns * m * 4 * TypeBytes(d.dst_type);
  } else if (op->kind == mldhip_op::kQuant) {
    const mldhip_quant_desc& d = op->q;
    const size_t s = DivUp(d.channels, 4);
    (*src)[0] = s * m * 4 * TypeBytes(d.src_type);
    // GetShapeForPackedType (common/util.cc:262-277): 16 bytes per element of the packed tensor
    switch (d.packed_type) {
      case MLDHIP_PACKED_INT8C16:
      case MLDHIP_PACKED_UINT8C16: (*dst)[0] = (size_t)DivUp((int)s, 4) * m * 16; break;
      case MLDHIP_PACKED_INT4C32:
      case MLDHIP_PACKED_UINT4C32: (*dst)[0] = (size_t)DivUp((int)s, 8) * m * 16; break;
      case MLDHIP_PACKED_INT8W4C4:
      case MLDHIP_PACKED_UINT8W4C4: (*dst)[0] = s * op->h * DivUp(op->w, 4) * op->b * 16; break;
      default: (*dst)[0] = s * m * 4;
    }
    (*dst)[1] = m * 4 * sizeof(float);
  } else {
    const mldhip_conv_int8_desc& d = op->cv;
    const size_t k16 = DivUp(d.i, 16), ns = DivUp(d.o, 4);
    (*src)[0] = k16 * m * 16;
    (*src)[1] = k16 * (size_t)d.o * 16;
    if (d.dst_type != MLDHIP_INT32) {
      (*src)[2] = m * 4 * sizeof(float);
      (*src)[3] = ns * 4 * sizeof(int32_t);
      (*src)[4] = ns * 4 * sizeof(float);
      if (op->idx_zp >= 0) (*src)[op->idx_zp] = ns * 4 * sizeof(float);
      if (op->idx_bias >= 0) (*src)[op->idx_bias] = ns * 4 * TypeBytes(d.dst_type);
    }
    (*dst)[0] = ns * m * 4 * TypeBytes(d.dst_type);
  }
}

static void UpdateRequiredSizes(mldhip_op* op) { RequiredSizes(op, &op->need_src, &op->need_dst); }

static int CheckBindings(const mldhip_op* op) {
  const std::vector<size_t>&need_src = op->need_src, &need_dst = op->need_dst;
  for (size_t i = 0; i < need_src.size(); ++i) {
    if (!op->src_ptr[i]) return Fail(MLDHIP_FAILED_PRECONDITION, "src object '" + op->src_names[i] + "' is not bound");
    if (op->src_bytes[i] < need_src[i])
      return Fail(MLDHIP_INVALID_ARGUMENT, "src object '" + op->src_names[i] + "' is smaller than the shape needs (" +
                                               std::to_string(op->src_bytes[i]) + " < " + std::to_string(need_src[i]) + ")");
  }
  for (size_t i = 0; i < need_dst.size(); ++i) {
    if (!op->dst_ptr[i]) return Fail(MLDHIP_FAILED_PRECONDITION, "dst object '" + op->dst_names[i] + "' is not bound");
    if (op->dst_bytes[i] < need_dst[i])
      return Fail(MLDHIP_INVALID_ARGUMENT, "dst object '" + op->dst_names[i] + "' is smaller than the shape needs (" +
                                               std::to_string(op->dst_bytes[i]) + " < " + std::to_string(need_dst[i]) + ")");
  }
  return MLDHIP_OK;
}

// The launch arguments of a floating-point FC op at its current bindings and shape.
static int BuildFcArgs(mldhip_op* op, FcArgs* out) {
  const mldhip_fc_desc& d = op->fc;
  FcArgs a;
  a.act = op->src_ptr[0];
  a.weights = static_cast<const uint8_t*>(op->src_ptr[op->idx_weights]);
  a.scale = op->idx_scale >= 0 ? op->src_ptr[op->idx_scale] : nullptr;
  a.zero_point = op->idx_zp >= 0 ? op->src_ptr[op->idx_zp] : nullptr;
  a.bias = op->idx_bias >= 0 ? op->src_ptr[op->idx_bias] : nullptr;
  a.dst = op->dst_ptr[0];
  a.m = op->Tokens();
  if (op->idx_ids >= 0) {
    a.batch_ids = static_cast<const int32_t*>(op->src_ptr[op->idx_ids]);
    a.rows = op->h;
    a.src_rows = op->shared_src ? 1 : op->h;
    a.weights_batch = op->weights_batch;
    a.m = op->w;  // tokens per row
  }
  a.k = op->src_c;
  a.n = op->dst_c;
  a.weights_k = d.i;
  a.act_f16 = d.src_type == MLDHIP_FLOAT16;
  a.dst_f16 = d.dst_type == MLDHIP_FLOAT16;
  a.weight_bits = WeightBits(d.weights.type);
  a.group = d.weights.output_group_size;
  a.scale_kind = d.scale_o * d.scale_i == 1 ? kScaleScalar : (d.scale_i == 1 ? kScaleLinear : kScaleBlock);
  a.groups = d.scale_i;
  a.scalar_scale = d.scalar_scale;
  a.has_zero_point = d.has_zero_point_tensor || d.has_scalar_zero_point;
  a.scalar_zero_point = d.has_scalar_zero_point ? d.scalar_zero_point : 0.0f;
  a.partial = op->partial;
  a.partial_floats = op->partial_floats;
  if (op->idx_params >= 0) {
    a.params = static_cast<const int32_t*>(op->src_ptr[op->idx_params]);
    a.src_end_ch_index = d.src_end_ch_index;
    a.dst_end_ch_index = d.dst_end_ch_index;
    a.ring_i_index = d.ring_i_offset_index;
    a.ring_o_index = d.ring_o_offset_index;
    a.ring_size = d.ring_size;
    if (d.packed_num_groups > 0) {
      a.packed_params_offset = d.packed_params_offset;
      a.packed_max_group_size = d.packed_max_group_size;
      a.weights_batch = op->weights_batch;
    }
  }
  *out = a;
  return MLDHIP_OK;
}

int mldhip_op_launch(mldhip_op* op, void* stream_ptr) {
  if (!op) return Fail(MLDHIP_INVALID_ARGUMENT, "null op");
  if (int rc = CheckBindings(op)) return rc;
  hipStream_t stream = static_cast<hipStream_t>(stream_ptr);
  hipError_t e = hipSuccess;
  if (op->kind == mldhip_op::kFc) {
    const mldhip_fc_desc& d = op->fc;
    if (d.src_type == MLDHIP_INT8) {
      const int bits = WeightBits(d.weights.type);
      FcBatchRows batch;
      int tokens = op->Tokens();
      if (op->idx_ids >= 0) {  // batched weights: h rows of w tokens
        batch.ids = static_cast<const int32_t*>(op->src_ptr[op->idx_ids]);
        batch.rows = op->h;
        batch.src_rows = op->shared_src ? 1 : op->h;
        batch.weights_batch = op->weights_batch;
        tokens = op->w;
      }
      batch.group = d.weights.output_group_size;
      if (op->idx_params >= 0) {
        batch.params = static_cast<const int32_t*>(op->src_ptr[op->idx_params]);
        batch.src_end_ch_index = d.src_end_ch_index;
        batch.dst_end_ch_index = d.dst_end_ch_index;
        if (d.packed_num_groups > 0) {  // one launch plane per matrix over the one row of tokens
          batch.packed_params_offset = d.packed_params_offset;
          batch.packed_max_group_size = d.packed_max_group_size;
          batch.weights_batch = op->weights_batch;
        }
      }
      const int8_t* act = static_cast<const int8_t*>(op->src_ptr[0]);
      const uint8_t* weights = static_cast<const uint8_t*>(op->src_ptr[op->idx_weights]);
      int32_t* dst = static_cast<int32_t*>(op->dst_ptr[0]);
      const int group = EffectiveGroup(batch.group, DivUp(d.o, 4));
      if (GetTuning().force_generic <= 0 && op->idx_params < 0 && FcInt8MathStreamSupported(tokens, d.i, d.o, bits) &&
          (bits == 8 || group % 2 == 0))
        e = LaunchFcInt8MathStream(act, weights, dst, tokens, d.i, d.o, bits, stream, &op->last_kernel, batch);
      else
        e = LaunchFcInt8Math(act, weights, dst, tokens, d.i, d.o, bits, stream, &op->last_kernel, batch);
    } else {
      FcArgs a;
      if (int rc = BuildFcArgs(op, &a)) return rc;
      // Runtime channel bounds at 1..4 tokens run on the streaming GEMVs (which stop their K loop at the
      // bound and skip the dst strips beyond it); ringed weights, packed groups off the matrix cores and
      // bounds at more tokens on the unspecialised kernel.
      const bool bounded = a.params != nullptr;
      const bool bounded_stream = bounded && a.packed_params_offset < 0 && a.ring_i_index < 0 && a.ring_o_index < 0 &&
                                  (FcW4StreamSupported(a) || FcW8StreamSupported(a));
      const bool force_generic = GetTuning().force_generic > 0 || (bounded && !bounded_stream);
      // ringed weights over the input channels at a few tokens: the kernel that walks the ring's rows
      if (GetTuning().force_generic <= 0 && FcW8RingSupported(a)) {
        e = LaunchFcW8Ring(a, stream, &op->last_kernel);
      } else
      // packed groups: the matrix-core GEMM with one launch plane per matrix where it serves the shape
      if (GetTuning().force_generic <= 0 && FcW4MfmaPackedSupported(a)) {
        e = LaunchFcW4Mfma(a, stream, &op->last_kernel);
      } else
      // batched weights by runtime ids: the streaming GEMVs, else the unspecialised kernel
      if (a.batch_ids != nullptr) {
        if (!force_generic && FcW4StreamSupported(a))
          e = LaunchFcW4Stream(a, stream, &op->last_kernel);
        else if (!force_generic && FcW8StreamSupported(a))
          e = LaunchFcW8Stream(a, stream, &op->last_kernel);
        else
          e = LaunchFcGeneric(a, stream, &op->last_kernel);
      } else
      // 2..16 tokens on wide per-channel layers: the matrix-core GEMV (one token streams faster
      // on the vector-ALU kernel; the tuning knob gemv_mfma = 1 forces the matrix-core one there too)
      if (!force_generic && a.m >= 2 && a.m <= 4 && FcW4StripTokensSupported(a)) {
        e = LaunchFcW4Stream(a, stream, &op->last_kernel);  // (2..4 tokens in whole strips: the token form of the strip kernel)
      } else if (!force_generic && (a.m >= 2 || GetTuning().gemv_mfma > 0 || !FcW4StreamSupported(a)) &&
          FcW4MfmaStreamSupported(a)) {
        e = LaunchFcW4MfmaStream(a, stream, &op->last_kernel);
      } else if (!force_generic && FcW4StreamSupported(a)) {
        e = LaunchFcW4Stream(a, stream, &op->last_kernel);
      } else if (!force_generic && FcW4MfmaSupported(a)) {
        e = LaunchFcW4Mfma(a, stream, &op->last_kernel);
      } else if (!force_generic && FcW8RowsSupported(a)) {
        e = LaunchFcW8Rows(a, stream, &op->last_kernel);
      } else if (!force_generic && FcW8StreamSupported(a)) {
        e = LaunchFcW8Stream(a, stream, &op->last_kernel);
      } else {
        e = LaunchFcGeneric(a, stream, &op->last_kernel);
      }
    }
  } else if (op->kind == mldhip_op::kQuant) {
    const mldhip_quant_desc& d = op->q;
    QuantArgs a;
    a.src = op->src_ptr[0];
    a.codes = op->dst_ptr[0];
    a.params = static_cast<float*>(op->dst_ptr[1]);
    a.tokens = op->Tokens();
    a.channels = d.channels;
    a.batch = op->b;
    a.width = op->w;
    a.height = op->h;
    a.src_f16 = d.src_type == MLDHIP_FLOAT16;
    a.packed_type = d.packed_type;
    a.symmetric = d.symmetric != 0;
    a.calculate_sum = d.calculate_sum != 0;
    a.nearest_even = d.round_to_nearest_even != 0;
    e = LaunchQuantize(a, stream, &op->last_kernel);
  } else {
    const mldhip_conv_int8_desc& d = op->cv;
    ConvInt8Args a;
    a.codes = static_cast<const int8_t*>(op->src_ptr[0]);
    a.weights = static_cast<const int8_t*>(op->src_ptr[1]);
    if (d.dst_type != MLDHIP_INT32) {
      a.params = static_cast<const float*>(op->src_ptr[2]);
      a.weights_sum = static_cast<const int32_t*>(op->src_ptr[3]);
      a.weights_scale = static_cast<const float*>(op->src_ptr[4]);
      a.weights_zero_point = op->idx_zp >= 0 ? static_cast<const float*>(op->src_ptr[op->idx_zp]) : nullptr;
      a.bias = op->idx_bias >= 0 ? op->src_ptr[op->idx_bias] : nullptr;
    }
    a.dst = op->dst_ptr[0];
    a.m = op->Tokens();
    a.k = d.i;
    a.n = d.o;
    a.dst_type = d.dst_type;
    e = LaunchConvInt8(a, stream, &op->last_kernel);
  }
  if (e != hipSuccess) return HipFail(e, "kernel launch");
  return MLDHIP_OK;
}

int mldhip_fc_launch_fused(mldhip_op* const* ops, int count, void* stream_ptr) {
  if (!ops || count < 1) return Fail(MLDHIP_INVALID_ARGUMENT, "no ops");
  if (count > 3) return Fail(MLDHIP_FAILED_PRECONDITION, "at most 3 ops per fused launch");
  FcArgs args[3];
  bool stream_ok = true, mfma_ok = true;
  for (int i = 0; i < count; ++i) {
    mldhip_op* op = ops[i];
    if (!op) return Fail(MLDHIP_INVALID_ARGUMENT, "null op");
    if (op->kind != mldhip_op::kFc || op->fc.src_type == MLDHIP_INT8 || op->idx_ids >= 0 || op->idx_params >= 0)
      return Fail(MLDHIP_FAILED_PRECONDITION, "fused launch takes floating-point FullyConnected ops without batched weights or runtime channel bounds");
    if (int rc = CheckBindings(op)) return rc;
    if (int rc = BuildFcArgs(op, &args[i])) return rc;
    const FcArgs &a = args[i], &f = args[0];
    stream_ok = stream_ok && FcW4StreamSupported(a);
    mfma_ok = mfma_ok && FcW4MfmaSupported(a);
    if (a.act != f.act || a.m != f.m || a.k != f.k || a.scale_kind != f.scale_kind || a.groups != f.groups ||
        a.has_zero_point != f.has_zero_point || a.weight_bits != f.weight_bits)
      return Fail(MLDHIP_FAILED_PRECONDITION, "op " + std::to_string(i) + " does not read the same tensor with the same K, weight type and scale groups as op 0");
  }
  if (!stream_ok && !mfma_ok)
    return Fail(MLDHIP_FAILED_PRECONDITION, "the ops are not all served by the same kernel at this shape");
  const char* name = nullptr;
  hipStream_t stream = static_cast<hipStream_t>(stream_ptr);
  hipError_t e = stream_ok ? LaunchFcW4StreamFused(args, count, stream, &name) : LaunchFcW4MfmaFused(args, count, stream, &name);
  if (e != hipSuccess) return HipFail(e, "fused launch");
  for (int i = 0; i < count; ++i) ops[i]->last_kernel = name;
  return MLDHIP_OK;
}

int mldhip_fc_launch_gated(mldhip_op* gate, mldhip_op* up, int activation, void* dst, size_t dst_bytes,
                           void* stream_ptr) {
  if (!gate || !up || !dst) return Fail(MLDHIP_INVALID_ARGUMENT, "null argument");
  if (activation != MLDHIP_GATE_GELU_TANH && activation != MLDHIP_GATE_SILU)
    return Fail(MLDHIP_INVALID_ARGUMENT, "unknown gate activation");
  mldhip_op* ops[2] = {gate, up};
  FcArgs args[2];
  for (int i = 0; i < 2; ++i) {
    if (ops[i]->kind != mldhip_op::kFc || ops[i]->fc.src_type == MLDHIP_INT8 || ops[i]->idx_ids >= 0 || ops[i]->idx_params >= 0)
      return Fail(MLDHIP_FAILED_PRECONDITION, "gated launch takes floating-point FullyConnected ops without batched weights or runtime channel bounds");
    if (int rc = CheckBindings(ops[i])) return rc;
    if (int rc = BuildFcArgs(ops[i], &args[i])) return rc;
  }
  const bool gemv = FcW4GatedSupported(args[0], args[1]);
  if (!gemv && !FcW4MfmaGatedSupported(args[0], args[1]))
    return Fail(MLDHIP_FAILED_PRECONDITION,
                "gate and up are not a pair of fp16 FullyConnected ops over one tensor with one shape and weight "
                "type, symmetric weights and scale groups the gated kernels serve (int8 weights: above 4 tokens)");
  const size_t need = (size_t)DivUp(args[0].n, 4) * 4 * args[0].m * sizeof(uint16_t);
  if (dst_bytes < need) return Fail(MLDHIP_INVALID_ARGUMENT, "dst is too small for the gated output");
  if (reinterpret_cast<uintptr_t>(dst) % 16 != 0) return Fail(MLDHIP_INVALID_ARGUMENT, "dst is not 16-byte aligned");
  const char* name = nullptr;
  hipStream_t stream = static_cast<hipStream_t>(stream_ptr);
  // 1..2 tokens: the streaming GEMV pair; more: the matrix-core GEMM with the gated epilogue
  hipError_t e = gemv ? LaunchFcW4Gated(args[0], args[1], activation, dst, stream, &name)
                      : LaunchFcW4MfmaGated(args[0], args[1], activation, dst, stream, &name);
  if (e != hipSuccess) return HipFail(e, "gated launch");
  gate->last_kernel = up->last_kernel = name;
  return MLDHIP_OK;
}

int mldhip_fc_int4_decode_noalloc(const void* src, const void* weights, const void* weights_scale, const void* biases,
                                  void* dst, int o, int i, int scale_groups, int output_group_size, int tokens,
                                  void* stream_ptr) {
  if (!src || !weights || !weights_scale || !dst) return Fail(MLDHIP_INVALID_ARGUMENT, "null device pointer");
  if (o <= 0 || i <= 0) return Fail(MLDHIP_INVALID_ARGUMENT, "weights shape must be positive");
  if (o > kNoAllocMaxChannels)
    return Fail(MLDHIP_OUT_OF_RANGE, "more output channels than the static scratch array serves (65536)");
  if (tokens < 1 || tokens > kGemvMaxTokens)
    return Fail(MLDHIP_OUT_OF_RANGE, "the allocation-free entry point serves 1..4 tokens");
  const int ns = DivUp(o, 4), ks = DivUp(i, 4);
  if (ns % 2 != 0) return Fail(MLDHIP_UNIMPLEMENTED, "an odd number of 4-channel output slices is not served here");
  if (scale_groups < 1 || ks % scale_groups != 0 || (scale_groups > 1 && (ks / scale_groups) % 8 != 0))
    return Fail(MLDHIP_INVALID_ARGUMENT, "scale groups must be whole multiples of 32 input channels");
  // whole groups of an even number of slices (16-byte items of the packed rows), as the streaming kernels read them
  if (output_group_size < 1 || ns % output_group_size != 0 || output_group_size % 2 != 0)
    return Fail(MLDHIP_INVALID_ARGUMENT, "Unsupported WeightsDescription output_group_size.");
  const void* ptrs[5] = {src, weights, weights_scale, biases, dst};
  for (const void* ptr : ptrs)
    if (reinterpret_cast<uintptr_t>(ptr) % 16 != 0) return Fail(MLDHIP_INVALID_ARGUMENT, "a buffer is not 16-byte aligned");
  FcArgs a;
  a.act = src;
  a.weights = static_cast<const uint8_t*>(weights);
  a.scale = weights_scale;
  a.bias = biases;
  a.dst = dst;
  a.m = tokens;
  a.k = i;
  a.n = o;
  a.act_f16 = a.dst_f16 = true;
  a.weight_bits = 4;
  a.group = output_group_size;
  a.scale_kind = scale_groups == 1 ? kScaleLinear : kScaleBlock;
  a.groups = scale_groups;
  const char* name = nullptr;
  hipError_t e = LaunchFcW4StreamNoAlloc(a, static_cast<hipStream_t>(stream_ptr), &name);
  if (e != hipSuccess) return HipFail(e, "allocation-free launch");
  return MLDHIP_OK;
}

const char* mldhip_op_kernel_name(const mldhip_op* op) { return op ? op->last_kernel : ""; }

int mldhip_op_cost(const mldhip_op* op, uint64_t* bytes, uint64_t* flops) {
  if (!op) return Fail(MLDHIP_INVALID_ARGUMENT, "null op");
  std::vector<size_t> need_src, need_dst;
  RequiredSizes(op, &need_src, &need_dst);
  // batched weights: only the matrices the ids select are read
  // (common/gpu_model_builder_moe_util.cc:268-283)
  if (op->kind == mldhip_op::kFc && op->idx_ids >= 0 && op->h < op->weights_batch) {
    const int objects[3] = {op->idx_weights, op->idx_scale, op->idx_zp};
    for (int idx : objects)
      if (idx >= 0) need_src[idx] = need_src[idx] / op->weights_batch * op->h;
  }
  uint64_t total = 0;
  for (size_t v : need_src) total += v;
  for (size_t v : need_dst) total += v;
  if (bytes) *bytes = total;
  if (flops) {
    const uint64_t m = (uint64_t)op->Tokens();
    if (op->kind == mldhip_op::kFc)
      *flops = 2 * m * (uint64_t)op->src_c * (uint64_t)op->dst_c;
    else if (op->kind == mldhip_op::kConvInt8)
      *flops = 2 * m * (uint64_t)op->cv.i * (uint64_t)op->cv.o;
    else
      *flops = 5 * m * (uint64_t)op->q.channels;
  }
  return MLDHIP_OK;
}

void mldhip_op_destroy(mldhip_op* op) {
  if (!op) return;
  if (op->partial) (void)hipFree(op->partial);
  delete op;
}

}  // extern "C"
