// Checkpoint files of the reference's LLM sample -> the buffers a quantized FullyConnected op
// binds (host side only; nothing here touches the GPU).
//
// Follows samples/llm/llm_weights_loader.cc:29-117 (GetWeightsInt4 / GetWeightsInt8: which files
// make up one linear layer) and samples/llm/llm_file_tensor_loader.cc:
//   :54-97   ReadScaleOrZeroPointInt     header (int32 group size) + int8 / int16 values / 1024
//   :111-131 IsGroupedQuantization        which of the two scale formats a file is
//   :134-148 LoadScaleOrZeroPoint         raw fp32 otherwise
//   :244-260 LoadInt4Packed, :202-212 LoadInt8    raw weight bytes (a short file leaves zeros)
//   :262-302 LoadInt8Weights, :350-395 LoadInt4WeightsFast   packing + weights_sum_i
//   :399-452 GetQuantizationIGroupSize    group size from the size of the scale file
//   :454-496 LoadScale, LoadZeroPoint     zero point file / scale, 0 where the scale is 0
// The files themselves are what samples/llm/extract_weights_hf.py writes: `<name>` = int8 [o][i]
// or two's-complement nibbles, low nibble first; `<base>.weight_quantized_scale` = fp32 [o] or
// [o][i / block].
#include <cstdio>
#include <cstring>
#include <new>
#include <string>
#include <vector>

#include "../../include/mldhip.h"

namespace mldhip {
int Fail(int code, const std::string& msg);  // api.cpp: sets the thread's error string
}

namespace {

int FailWith(int code, const std::string& msg) { return mldhip::Fail(code, msg); }

long FileSize(const std::string& path) {
  FILE* f = std::fopen(path.c_str(), "rb");
  if (!f) return -1;
  std::fseek(f, 0, SEEK_END);
  const long n = std::ftell(f);
  std::fclose(f);
  return n;
}

// Reads up to `bytes` bytes; what the file does not hold stays zero (the reference reads into a
// zero-initialised vector and does not look at the stream state).  False: cannot open.
bool ReadPrefix(const std::string& path, size_t offset, void* dst, size_t bytes) {
  FILE* f = std::fopen(path.c_str(), "rb");
  if (!f) return false;
  std::memset(dst, 0, bytes);
  if (offset == 0 || std::fseek(f, (long)offset, SEEK_SET) == 0) {
    const size_t got = std::fread(dst, 1, bytes, f);
    (void)got;
  }
  std::fclose(f);
  return true;
}

bool ReadHeader(const std::string& path, int32_t* group_size) {
  *group_size = 0;
  return ReadPrefix(path, 0, group_size, sizeof(int32_t));
}

// llm_file_tensor_loader.cc:399-452
int QuantizationIGroupSize(const std::string& scale_path, int o, int i) {
  const long scale_size = FileSize(scale_path);
  if (scale_size < 4) return i;
  if (scale_size % 4 == 0) {
    const long elements = scale_size / 4;
    if (elements > 0 && elements % o == 0) {
      const long scale_i = elements / o;
      if (i % scale_i == 0) return (int)(i / scale_i);
    }
  }
  int32_t group_size = 0;
  if (!ReadHeader(scale_path, &group_size)) return i;
  if (group_size > 0 && group_size <= i && i % group_size == 0) {
    const long elements = (long)o * (i / group_size);
    if (scale_size == 4 + elements || scale_size == 4 + elements * 2) return group_size;
  }
  return i;
}

// llm_file_tensor_loader.cc:111-148, 54-97.  `count` = o * scale_i values, [o][scale_i].
// Returns false when the file cannot be used (the reference returns an empty tensor).
bool LoadScaleOrZeroPoint(const std::string& path, size_t count, std::vector<float>* out) {
  out->assign(count, 0.0f);
  const long size = FileSize(path);
  bool grouped = false;
  if (size >= 4) {
    int32_t group_size = 0;
    if (ReadHeader(path, &group_size) && group_size > 0 && group_size < 65536) {
      const size_t rest = (size_t)size - 4;
      grouped = rest == count || rest == count * 2;
    }
  }
  if (!grouped) return ReadPrefix(path, 0, out->data(), count * sizeof(float));
  const size_t bytes_per = ((size_t)size - 4) / count;
  if (bytes_per == 1) {
    std::vector<int8_t> raw(count);
    if (!ReadPrefix(path, 4, raw.data(), count)) return false;
    for (size_t k = 0; k < count; ++k) (*out)[k] = raw[k] / 1024.0f;
  } else if (bytes_per == 2) {
    std::vector<int16_t> raw(count);
    if (!ReadPrefix(path, 4, raw.data(), count * 2)) return false;
    for (size_t k = 0; k < count; ++k) (*out)[k] = raw[k] / 1024.0f;
  } else {
    return false;
  }
  return true;
}

std::string Join(const char* directory, const std::string& name) { return std::string(directory) + name; }

}  // namespace

extern "C" int mldhip_checkpoint_fc_probe(const char* directory, const char* weights_name, const char* base_name,
                                          int o, int i, int weight_bits, mldhip_checkpoint_fc* info) {
  if (!directory || !weights_name || !base_name || !info) return FailWith(MLDHIP_INVALID_ARGUMENT, "null argument");
  if (o <= 0 || i <= 0) return FailWith(MLDHIP_INVALID_ARGUMENT, "bad weights shape");
  if (weight_bits != 4 && weight_bits != 8) return FailWith(MLDHIP_INVALID_ARGUMENT, "weight_bits must be 4 or 8");
  std::memset(info, 0, sizeof(*info));
  const int rc = weight_bits == 4 ? mldhip_fc_int4_weights_desc(o, i, &info->weights)
                                  : mldhip_fc_int8_weights_desc(o, i, &info->weights);
  if (rc != MLDHIP_OK) return rc;
  if (FileSize(Join(directory, weights_name)) < 0)
    return FailWith(MLDHIP_NOT_FOUND, std::string("Failed to load weights: ") + weights_name);
  info->o = o;
  info->i = i;
  info->weight_bits = weight_bits;
  const std::string base(base_name);
  info->group_size = QuantizationIGroupSize(Join(directory, base + ".weight_quantized_scale"), o, i);
  info->scale_i = i / info->group_size;
  info->has_zero_point = FileSize(Join(directory, base + ".weight_quantized_zp")) >= 0 ? 1 : 0;
  if (int rc2 = mldhip_packed_bytes(&info->weights, o, 1, 1, i, &info->weights_bytes)) return rc2;
  info->scale_elements = (size_t)info->scale_i * ((o + 3) / 4) * 4;
  return MLDHIP_OK;
}

static int ReadFc(const char* directory, const char* weights_name, const char* base_name, const mldhip_checkpoint_fc* info,
                  int swap_dims, int tensor_type, uint8_t* weights, size_t weights_bytes, void* scale, void* zero_point,
                  size_t scale_bytes, int32_t* weights_sum_i) {
  if (!directory || !weights_name || !base_name || !info || !weights || !scale || !weights_sum_i)
    return FailWith(MLDHIP_INVALID_ARGUMENT, "null argument");
  if (tensor_type != MLDHIP_FLOAT16 && tensor_type != MLDHIP_FLOAT32)
    return FailWith(MLDHIP_INVALID_ARGUMENT, "tensor_type must be FLOAT16 or FLOAT32");
  if (info->has_zero_point && !zero_point) return FailWith(MLDHIP_INVALID_ARGUMENT, "zero_point buffer missing");
  const int o = info->o, i = info->i;
  if (o <= 0 || i <= 0 || info->scale_i <= 0) return FailWith(MLDHIP_INVALID_ARGUMENT, "info was not filled by the probe");
  if (weights_bytes < info->weights_bytes) return FailWith(MLDHIP_INVALID_ARGUMENT, "weights buffer too small");
  const size_t elem = tensor_type == MLDHIP_FLOAT16 ? 2 : 4;
  if (scale_bytes < info->scale_elements * elem) return FailWith(MLDHIP_INVALID_ARGUMENT, "scale buffer too small");
  const size_t count = (size_t)o * i;

  // ---- weights + weights_sum_i
  const std::string w_path = Join(directory, weights_name);
  if (info->weight_bits == 4) {
    // LoadInt4Packed: an odd element count yields no data
    if (count % 2 != 0) return FailWith(MLDHIP_NOT_FOUND, std::string("Failed to load weights: ") + weights_name);
    std::vector<uint8_t> raw(count / 2);
    if (!ReadPrefix(w_path, 0, raw.data(), raw.size()))
      return FailWith(MLDHIP_NOT_FOUND, std::string("Failed to load weights: ") + weights_name);
    for (int c = 0; c < o; ++c) weights_sum_i[c] = 0;
    if (int rc = mldhip_rearrange_uint4_packed(raw.data(), o, 1, 1, i, &info->weights, weights, weights_bytes,
                                               weights_sum_i, (size_t)o, 8u, swap_dims))
      return rc;
  } else {
    std::vector<int8_t> raw(count);
    if (!ReadPrefix(w_path, 0, raw.data(), raw.size()))
      return FailWith(MLDHIP_NOT_FOUND, std::string("Failed to load weights: ") + weights_name);
    if (swap_dims) {  // the file is [i][o]
      std::vector<int8_t> t(count);
      for (int c = 0; c < o; ++c)
        for (int k = 0; k < i; ++k) t[(size_t)c * i + k] = raw[(size_t)k * o + c];
      raw.swap(t);
    }
    if (int rc = mldhip_rearrange_int8_as_uint8(raw.data(), o, 1, 1, i, &info->weights, weights, weights_bytes, 128, 128u))
      return rc;
    if (int rc = mldhip_weights_sum_i(raw.data(), o, 1, 1, i, weights_sum_i)) return rc;
  }

  // ---- scale (LoadScale) and zero point (LoadZeroPoint: file value / scale)
  const std::string base(base_name);
  const size_t s_count = (size_t)o * info->scale_i;
  std::vector<float> s_host, z_host;
  const std::string s_name = base + ".weight_quantized_scale";
  if (!LoadScaleOrZeroPoint(Join(directory, s_name), s_count, &s_host))
    return FailWith(MLDHIP_NOT_FOUND, "Failed to load scale: " + s_name);
  if (int rc = mldhip_scale_to_tensor(s_host.data(), o, info->scale_i, tensor_type, scale, scale_bytes)) return rc;
  if (info->has_zero_point) {
    if (!LoadScaleOrZeroPoint(Join(directory, base + ".weight_quantized_zp"), s_count, &z_host))
      z_host.assign(s_count, 0.0f);
    for (size_t k = 0; k < s_count; ++k) z_host[k] = s_host[k] == 0.0f ? 0.0f : z_host[k] / s_host[k];
    if (int rc = mldhip_scale_to_tensor(z_host.data(), o, info->scale_i, tensor_type, zero_point, scale_bytes)) return rc;
  }
  return MLDHIP_OK;
}

extern "C" int mldhip_checkpoint_fc_read(const char* directory, const char* weights_name, const char* base_name,
                                         const mldhip_checkpoint_fc* info, int swap_dims, int tensor_type,
                                         uint8_t* weights, size_t weights_bytes, void* scale, void* zero_point,
                                         size_t scale_bytes, int32_t* weights_sum_i) {
  try {  // (the staging buffers are as large as the layer: no exception may cross the C boundary)
    return ReadFc(directory, weights_name, base_name, info, swap_dims, tensor_type, weights, weights_bytes, scale, zero_point,
                  scale_bytes, weights_sum_i);
  } catch (const std::bad_alloc&) {
    return FailWith(MLDHIP_INTERNAL, "out of host memory while reading the layer");
  }
}
