/*
 * TEST INFRASTRUCTURE ONLY — CPU oracle for ML Drift's quantized fully-connected path.
 *
 * This is a plain-C restatement of the reference's algorithms (host weight packers, the
 * generated FullyConnected kernel, per-token quantization, the int32->float rescale
 * epilogue).  It exists so that tests, the smoke check and the cpu_baseline leg of the
 * benchmark have something to compare the HIP product against.  Nothing in the product
 * library links, loads or calls it.
 *
 * Every function cites the reference file:line it follows (paths relative to the
 * reference checkout, ml_drift/...).
 *
 * Parity pinning status (which independent evidence fixes each function) is listed in the
 * header comment of mld_oracle.c.
 */
#ifndef MLD_ORACLE_H_
#define MLD_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- enums (numeric values chosen to match the product C-ABI) ---- */
enum {
  MLDO_LAYOUT_OSPATIAL_IOGROUP_I4O4 = 1, /* WeightsLayout::kOSpatialIOGroupI4O4 */
  MLDO_LAYOUT_OSPATIAL_IOGROUP_O4I4 = 2, /* WeightsLayout::kOSpatialIOGroupO4I4 */
  MLDO_LAYOUT_2D_YSPATIALIO_XOGROUP_I4O4 = 6 /* k2DYIsSpatialIOAndXIsOGroupI4O4 */
};
enum { MLDO_PREC_F32 = 0, MLDO_PREC_F32F16 = 1, MLDO_PREC_F16 = 2 };
enum { MLDO_SCALE_SCALAR = 0, MLDO_SCALE_LINEAR = 1, MLDO_SCALE_BLOCK = 2 };
enum {
  MLDO_PACKED_UINT8C4 = 1,
  MLDO_PACKED_INT8C4 = 2,
  MLDO_PACKED_UINT8W4C4 = 3,
  MLDO_PACKED_INT8W4C4 = 4,
  MLDO_PACKED_INT8C16 = 5,
  MLDO_PACKED_UINT8C16 = 6,
  MLDO_PACKED_INT4C32 = 7,
  MLDO_PACKED_UINT4C32 = 8
};
enum { MLDO_AXIS_O = 0, MLDO_AXIS_H = 1, MLDO_AXIS_W = 2, MLDO_AXIS_I = 3 };

/* ---- IEEE binary16 helpers (round-to-nearest-even) ---- */
uint16_t mldo_f32_to_f16(float v);
float mldo_f16_to_f32(uint16_t h);
void mldo_convert_f32_f16(const float* src, uint16_t* dst, size_t n);
void mldo_convert_f16_f32(const uint16_t* src, float* dst, size_t n);

/* ---- tensor layout: logical BHWC <-> physical slice-major buffer [S][tokens][4] ---- */
void mldo_bhwc_to_slices(const void* src, int tokens, int channels, int elem_size, void* dst);
void mldo_slices_to_bhwc(const void* src, int tokens, int channels, int elem_size, void* dst);

/* ---- weight packers ---- */
size_t mldo_total_elements(int layout, int o, int h, int w, int i, int out_group_size);
int mldo_rearrange_u8(const uint8_t* src, int o, int h, int w, int i, int layout,
                      int out_group_size, uint8_t pad, uint8_t* dst);
int mldo_rearrange_u8_reshape(const uint8_t* src, int o, int h, int w, int i, int layout,
                              int out_group_size, uint8_t pad, uint8_t* dst);
int mldo_rearrange_i8(const int8_t* src, int o, int h, int w, int i, int layout,
                      int out_group_size, int8_t* dst);
int mldo_int8_as_uint8(const int8_t* src, int o, int h, int w, int i, int layout,
                       int out_group_size, int shift, unsigned pad, uint8_t* dst);
int mldo_int8_as_uint4(const int8_t* src, int o, int h, int w, int i, int layout,
                       int out_group_size, int shift, unsigned pad, uint8_t* dst);
int mldo_uint4_packed(const uint8_t* src, int o, int h, int w, int i, int layout,
                      int out_group_size, uint8_t* dst, int32_t* sum_i, size_t sum_len,
                      unsigned pad, int swap_dims);
void mldo_weights_sum_i(const int8_t* src, int o, int h, int w, int i, int32_t* sum);
size_t mldo_custom_total_elements(int o, int h, int w, int i, const int* axes,
                                  const int* sizes, int n_groups);
void mldo_rearrange_custom_i8(const int8_t* src, int o, int h, int w, int i, const int* axes,
                              const int* sizes, int n_groups, int8_t pad, int8_t* dst);
void mldo_scale_to_hoio4(const float* scale_ohwi, int o, int h, int i, float* dst);

/* ---- FullyConnected ---- */
typedef struct {
  int m, k, n;        /* tokens, input channels, output channels */
  int precision;      /* MLDO_PREC_* ; tensors are fp32 for F32, fp16 otherwise */
  int weight_bits;    /* 8 or 4 (packed uint8/uint4, I4O4, out_group_size = ceil(n/4)) */
  int scale_kind;     /* MLDO_SCALE_* */
  int groups;         /* scale_zp_shape.i for MLDO_SCALE_BLOCK, else 1 */
  int has_zero_point;
  int has_bias;
  int use_fma;        /* fc::UseFMA: true for AMD+OpenCL */
  int wg_y;           /* K-split across work-group y (1 = sequential) */
  float scalar_scale;
  float scalar_zero_point;
  int threads;        /* OpenMP threads, <=0: runtime default */
} mldo_fc_params;

/* Returns the path taken: 0 = one output channel at a time, 1 = eight channels at a time (x86-64
 * with AVX2, FMA and F16C, detected at run time; F32_F16 precision without zero point, wg_y = 1).
 * The two are bit-identical; mldo_set_fast_path(0) forces path 0. */
int mldo_fc_kernel(const mldo_fc_params* p, const void* act, const uint8_t* weights,
                   const void* scale, const void* zero_point, const void* bias, void* dst);
void mldo_set_fast_path(int enabled);
void mldo_fc_int8_kernel(int m, int k, int n, int weight_bits, const int8_t* act,
                         const uint8_t* weights, int32_t* dst);
void mldo_fc_reference_f32(int m, int k, int n, const float* src, const float* weights,
                           const float* bias, float* dst);
void mldo_fc_reference_i8(int m, int k, int n, const int8_t* src, const int8_t* weights,
                          int32_t* dst);
void mldo_make_weights_from_int8(int n, int k, const int8_t* w, const float* scale,
                                 const float* zero_point, int scale_o, int scale_i,
                                 float* dst);

/* ---- per-token quantization and the int32 -> float rescale epilogue ---- */
void mldo_quantize(int tokens, int channels, int batch, int src_is_f16, const void* src,
                   int packed_type, int symmetric, int calculate_sum, void* codes,
                   float* params);
/* every packed type; the tensor is BHWC(batch, height, width, channels), tokens = (y*W + x)*B + b */
void mldo_quantize_packed(int height, int width, int batch, int channels, int src_is_f16,
                          const void* src, int packed_type, int symmetric, int calculate_sum,
                          void* codes, float* params);
void mldo_dequantize(int tokens, int n, int k, const int32_t* acc, const float* params,
                     const int32_t* weights_sum, const float* weights_scale,
                     const float* weights_zero_point, const void* bias, int dst_is_f16,
                     void* dst);
void mldo_dequantize_weights(int n, int k, int weight_bits, const uint8_t* weights,
                             int scale_kind, int groups, const uint16_t* scale,
                             const uint16_t* zero_point, uint16_t* dst_ohwi);

#ifdef __cplusplus
}
#endif
#endif /* MLD_ORACLE_H_ */
