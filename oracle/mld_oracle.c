/*
 * TEST INFRASTRUCTURE ONLY — CPU oracle for ML Drift's quantized fully-connected path.
 * See mld_oracle.h.  Never linked into, loaded by or called from the product library.
 *
 * Citations are relative to the reference checkout (ml_drift/...).
 *
 * How each function is pinned (independent of this file's own formulas):
 *   packers (mldo_rearrange_*, mldo_int8_as_*, mldo_uint4_packed, mldo_weights_sum_i)
 *     - the literal golden vectors of common/task/weights_conversion_test.cc:50-479
 *       (base, zero-init of sums, 2D twin, N padding, K "double pad", swap_dims),
 *     - the reference's own equivalence tests (packed-input path == int8 path, :183-262),
 *     - two formulations here (explicit loop vs pad+6-D transpose) compared on ragged shapes,
 *     - brute force: unpack every (o,i) with the kernel's nibble order and compare to w+shift.
 *   mldo_rearrange_custom_i8: reference tests :1196-1270 state that group lists
 *       {O4,I4,O4,I*,W*,H*,O*} and {I4,O4,O4,I*,W*,H*,O*} equal I4O4 / O4I4 with group 4.
 *   mldo_fc_kernel / mldo_fc_reference_f32: known answers {20.5,15.5}, {91.0,26.8},
 *       {509.0,-121.4}, all-8.0 (common/kernels/tests/fully_connected_test_util.cc:49-249,
 *       1541-1614); kernel restatement vs textbook reference within the reference's own
 *       tolerance rule on unaligned shapes (K=171, N=533).
 *   mldo_fc_int8_kernel: exact equality with the closed-form integer dot product
 *       (the reference's own check, fully_connected_test_util.cc:1446-1448).
 *   mldo_quantize: the CPU mirrors inside the reference tests
 *       (tests/quantize_and_dequantize_test_util.cc:165-202, 633-673), their edge rows
 *       (all-zero row, +-65504 row, C=237 and C=64) and the round-trip invariant.
 *   mldo_dequantize: the algebra in quantize_and_dequantize.cc:844-866 checked against a
 *       float FullyConnected of the dequantised operands.
 *   fp16 conversion: exhaustive round trip of all 65536 half patterns and numpy's float16.
 */
#include "mld_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline int div_up(int a, int b) { return (a + b - 1) / b; }
static inline int align_n(int a, int b) { return div_up(a, b) * b; }

/* ------------------------------------------------------------------------------------ */
/* binary16                                                                               */
/* ------------------------------------------------------------------------------------ */

/* double -> half, round to nearest even, one rounding. */
static uint16_t d2h(double d) {
  uint64_t b;
  memcpy(&b, &d, sizeof b);
  const uint16_t sign = (uint16_t)((b >> 48) & 0x8000u);
  const int e = (int)((b >> 52) & 0x7FF);
  uint64_t m = b & 0xFFFFFFFFFFFFFull;
  if (e == 0x7FF) return (uint16_t)(sign | 0x7C00u | (m ? 0x200u : 0u));
  if (e == 0) return sign; /* double subnormal: far below half's range */
  const int E = e - 1023;
  if (E > 15) return (uint16_t)(sign | 0x7C00u);
  m |= 1ull << 52;
  int shift = 42;
  uint32_t base = 0;
  if (E >= -14) {
    base = (uint32_t)(E + 15) << 10; /* mantissa's hidden bit is added below and carries */
  } else {
    shift += -14 - E;
  }
  if (shift >= 54) return sign;
  uint64_t q = m >> shift;
  const uint64_t rem = m & ((1ull << shift) - 1);
  const uint64_t half = 1ull << (shift - 1);
  if (rem > half || (rem == half && (q & 1))) q++;
  uint32_t bits = (E >= -14) ? base + (uint32_t)q - 0x400u : (uint32_t)q;
  if (bits >= 0x7C00u) bits = 0x7C00u;
  return (uint16_t)(sign | bits);
}

uint16_t mldo_f32_to_f16(float v) { return d2h((double)v); }

float mldo_f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t e = (h >> 10) & 0x1Fu;
  const uint32_t m = h & 0x3FFu;
  float out;
  if (e == 0) {
    out = (float)m * 5.9604644775390625e-08f; /* m * 2^-24 */
    uint32_t bits;
    memcpy(&bits, &out, 4);
    bits |= sign;
    memcpy(&out, &bits, 4);
    return out;
  }
  uint32_t bits;
  if (e == 31) {
    bits = sign | 0x7F800000u | (m << 13);
  } else {
    bits = sign | ((e + 112u) << 23) | (m << 13);
  }
  memcpy(&out, &bits, 4);
  return out;
}

/* common/task/weights_conversion.cc:40-44 (ConvertF32F16), checked by its test :43-48 */
void mldo_convert_f32_f16(const float* src, uint16_t* dst, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = mldo_f32_to_f16(src[i]);
}
void mldo_convert_f16_f32(const uint16_t* src, float* dst, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = mldo_f16_to_f32(src[i]);
}

/* Arithmetic "in type T": values are carried as float, rounded to half after each
 * operation when T is half.  For + and * one float operation followed by a rounding to
 * half equals a correctly rounded half operation (24 >= 2*11+2 bits). */
static inline float rt(float x, int is_half) {
  return is_half ? mldo_f16_to_f32(mldo_f32_to_f16(x)) : x;
}
static inline float t_mul(float a, float b, int is_half) { return rt(a * b, is_half); }
static inline float t_add(float a, float b, int is_half) { return rt(a + b, is_half); }
static inline float t_fma(float a, float b, float c, int is_half) {
  if (!is_half) return fmaf(a, b, c);
  return mldo_f16_to_f32(d2h(fma((double)a, (double)b, (double)c)));
}

/* ------------------------------------------------------------------------------------ */
/* tensor layout                                                                          */
/* ------------------------------------------------------------------------------------ */

/* Buffer storage, PhysicalLayout1D::kDCHWBC4: index (((s*H+y)*W+x)*B+b)*4+c
 * (common/task/tensor_desc.cc:1604-1609, 1857-1860).  "tokens" is the flattened (y,x,b)
 * index (y*W+x)*B+b; channels beyond C are zero (UploadData zero-fills). */
void mldo_bhwc_to_slices(const void* src, int tokens, int channels, int elem_size, void* dst) {
  const int slices = div_up(channels, 4);
  const char* s = (const char*)src;
  char* d = (char*)dst;
  memset(d, 0, (size_t)slices * tokens * 4 * elem_size);
  for (int t = 0; t < tokens; ++t)
    for (int c = 0; c < channels; ++c)
      memcpy(d + ((size_t)((c / 4) * tokens + t) * 4 + c % 4) * elem_size,
             s + ((size_t)t * channels + c) * elem_size, elem_size);
}

void mldo_slices_to_bhwc(const void* src, int tokens, int channels, int elem_size, void* dst) {
  const char* s = (const char*)src;
  char* d = (char*)dst;
  for (int t = 0; t < tokens; ++t)
    for (int c = 0; c < channels; ++c)
      memcpy(d + ((size_t)t * channels + c) * elem_size,
             s + ((size_t)((c / 4) * tokens + t) * 4 + c % 4) * elem_size, elem_size);
}

/* ------------------------------------------------------------------------------------ */
/* weight packers                                                                         */
/* ------------------------------------------------------------------------------------ */

/* common/task/weights_conversion.cc:1015-1034 (GetTotalElementsCountForLayout) */
size_t mldo_total_elements(int layout, int o, int h, int w, int i, int g) {
  switch (layout) {
    case MLDO_LAYOUT_OSPATIAL_IOGROUP_I4O4:
    case MLDO_LAYOUT_OSPATIAL_IOGROUP_O4I4:
      return (size_t)align_n(i, 4) * align_n(o, 4 * g) * h * w;
    case MLDO_LAYOUT_2D_YSPATIALIO_XOGROUP_I4O4:
      return (size_t)div_up(i, 4) * align_n(div_up(o, 4), g) * 16 * h * w;
    default:
      return 0;
  }
}

/* Explicit-loop formulation.
 *   I4O4: common/task/weights_conversion.cc:139-185 (RearrangeWeightsToOHWIOGroupI4O4)
 *   2D twin: same element order with the o-group loop moved inside the i-slice loop
 *            (weights_conversion.cc:730-737)
 *   O4I4: perm {0,3,4,1,2,5} of dims [Og][G][4o][HW][Is][4i] (weights_conversion.cc:1374-1376)
 */
static int rearrange_generic(const uint8_t* src, int O, int H, int W, int I, int layout,
                             int G, uint8_t pad, uint8_t* dst) {
  const int dst_slices = div_up(O, 4), src_slices = div_up(I, 4);
  const int dst_groups = div_up(dst_slices, G);
  uint8_t* p = dst;
#define SRC_AT(oc, y, x, ic) \
  (((oc) < O && (ic) < I) ? src[(((size_t)(oc) * H + (y)) * W + (x)) * I + (ic)] : pad)
  if (layout == MLDO_LAYOUT_OSPATIAL_IOGROUP_I4O4) {
    for (int d = 0; d < dst_groups; ++d)
      for (int y = 0; y < H; ++y)
        for (int x = 0; x < W; ++x)
          for (int s = 0; s < src_slices; ++s)
            for (int dg = 0; dg < G; ++dg)
              for (int ic = 4 * s; ic < 4 * s + 4; ++ic)
                for (int j = 0; j < 4; ++j) *p++ = SRC_AT(4 * (d * G + dg) + j, y, x, ic);
    return 0;
  }
  if (layout == MLDO_LAYOUT_2D_YSPATIALIO_XOGROUP_I4O4) {
    for (int y = 0; y < H; ++y)
      for (int x = 0; x < W; ++x)
        for (int s = 0; s < src_slices; ++s)
          for (int d = 0; d < dst_groups; ++d)
            for (int dg = 0; dg < G; ++dg)
              for (int ic = 4 * s; ic < 4 * s + 4; ++ic)
                for (int j = 0; j < 4; ++j) *p++ = SRC_AT(4 * (d * G + dg) + j, y, x, ic);
    return 0;
  }
  if (layout == MLDO_LAYOUT_OSPATIAL_IOGROUP_O4I4) {
    for (int d = 0; d < dst_groups; ++d)
      for (int y = 0; y < H; ++y)
        for (int x = 0; x < W; ++x)
          for (int s = 0; s < src_slices; ++s)
            for (int dg = 0; dg < G; ++dg)
              for (int j = 0; j < 4; ++j)
                for (int ic = 4 * s; ic < 4 * s + 4; ++ic)
                  *p++ = SRC_AT(4 * (d * G + dg) + j, y, x, ic);
    return 0;
  }
#undef SRC_AT
  return -1;
}

int mldo_rearrange_u8(const uint8_t* src, int o, int h, int w, int i, int layout, int g,
                      uint8_t pad, uint8_t* dst) {
  return rearrange_generic(src, o, h, w, i, layout, g, pad, dst);
}

/* weights_conversion.cc:1351-1423 (signed int8, pad value 0) */
int mldo_rearrange_i8(const int8_t* src, int o, int h, int w, int i, int layout, int g,
                      int8_t* dst) {
  return rearrange_generic((const uint8_t*)src, o, h, w, i, layout, g, 0, (uint8_t*)dst);
}

/* Second formulation: constant-pad then 6-D transpose, as in
 * common/task/weights_conversion.cc:46-87 (Reshape) with the perms of :1439-1445. */
int mldo_rearrange_u8_reshape(const uint8_t* src, int O, int H, int W, int I, int layout,
                              int G, uint8_t pad, uint8_t* dst) {
  size_t perm[6];
  if (layout == MLDO_LAYOUT_OSPATIAL_IOGROUP_I4O4) {
    const size_t p[6] = {0, 3, 4, 1, 5, 2};
    memcpy(perm, p, sizeof p);
  } else if (layout == MLDO_LAYOUT_2D_YSPATIALIO_XOGROUP_I4O4) {
    const size_t p[6] = {3, 4, 0, 1, 5, 2};
    memcpy(perm, p, sizeof p);
  } else if (layout == MLDO_LAYOUT_OSPATIAL_IOGROUP_O4I4) {
    const size_t p[6] = {0, 3, 4, 1, 2, 5};
    memcpy(perm, p, sizeof p);
  } else {
    return -1;
  }
  const size_t dst_groups = (size_t)div_up(O, G * 4), src_groups = (size_t)div_up(I, 4);
  const size_t PO = dst_groups * G * 4, PI = src_groups * 4, HW = (size_t)H * W;
  uint8_t* padded = (uint8_t*)malloc(PO * HW * PI);
  memset(padded, pad, PO * HW * PI);
  for (int oc = 0; oc < O; ++oc)
    for (size_t sp = 0; sp < HW; ++sp)
      memcpy(padded + ((size_t)oc * HW + sp) * PI, src + ((size_t)oc * HW + sp) * I, (size_t)I);
  const size_t dims[6] = {dst_groups, (size_t)G, 4, HW, src_groups, 4};
  size_t in_stride[6];
  in_stride[5] = 1;
  for (int a = 4; a >= 0; --a) in_stride[a] = in_stride[a + 1] * dims[a + 1];
  size_t od[6], idx[6] = {0, 0, 0, 0, 0, 0};
  for (int a = 0; a < 6; ++a) od[a] = dims[perm[a]];
  const size_t total = PO * HW * PI;
  for (size_t n = 0; n < total; ++n) {
    size_t off = 0;
    for (int a = 0; a < 6; ++a) off += idx[a] * in_stride[perm[a]];
    dst[n] = padded[off];
    for (int a = 5; a >= 0; --a) {
      if (++idx[a] < od[a]) break;
      idx[a] = 0;
    }
  }
  free(padded);
  return 0;
}

/* weights_conversion.cc:1495-1508 (RearrangeWeightsInt8AsUint8) */
int mldo_int8_as_uint8(const int8_t* src, int o, int h, int w, int i, int layout, int g,
                       int shift, unsigned pad, uint8_t* dst) {
  const size_t n = (size_t)o * h * w * i;
  uint8_t* u = (uint8_t*)malloc(n ? n : 1);
  for (size_t e = 0; e < n; ++e) u[e] = (uint8_t)(src[e] + shift);
  const int rc = rearrange_generic(u, o, h, w, i, layout, g, (uint8_t)pad, dst);
  free(u);
  return rc;
}

/* weights_conversion.cc:1510-1523 (RearrangeWeightsInt8AsUint4): dst[e] = v[2e] | v[2e+1]<<4 */
int mldo_int8_as_uint4(const int8_t* src, int o, int h, int w, int i, int layout, int g,
                       int shift, unsigned pad, uint8_t* dst) {
  const size_t total = mldo_total_elements(layout, o, h, w, i, g);
  uint8_t* u = (uint8_t*)malloc(total ? total : 1);
  const int rc = mldo_int8_as_uint8(src, o, h, w, i, layout, g, shift, pad, u);
  if (rc == 0)
    for (size_t e = 0; e < total / 2; ++e) dst[e] = (uint8_t)((u[2 * e + 1] << 4) | u[2 * e]);
  free(u);
  return rc;
}

static inline uint8_t nib(uint8_t v, int msb) { return msb ? (uint8_t)(v >> 4) : (uint8_t)(v & 0xF); }

/* weights_conversion.cc:631-708 and :711-788 (already nibble-packed two's-complement
 * input, ^0x88 flip, optional swap_dims, per-output-channel sums). */
int mldo_uint4_packed(const uint8_t* src, int O, int H, int W, int I, int layout, int G,
                      uint8_t* dst, int32_t* sum_i, size_t sum_len, unsigned pad_value,
                      int swap_dims) {
  if (layout != MLDO_LAYOUT_OSPATIAL_IOGROUP_I4O4 &&
      layout != MLDO_LAYOUT_2D_YSPATIALIO_XOGROUP_I4O4)
    return -1; /* UnimplementedError("Unsupported layout"), weights_conversion.cc:1617 */
  const int dst_slices = div_up(O, 4), src_slices = div_up(I, 4);
  const int dst_groups = div_up(dst_slices, G);
  const long df = swap_dims ? 1 : (long)H * W * I;
  for (int k = 0; k < O; ++k) sum_i[k] = 0;
  const uint8_t double_pad = (uint8_t)(pad_value | pad_value << 4);
  const uint8_t pad = (uint8_t)(pad_value ^ 0x8);
  uint8_t* p = dst;
  const int two_d = layout == MLDO_LAYOUT_2D_YSPATIALIO_XOGROUP_I4O4;
  /* outer order: I4O4 = d,y,x,s ; 2D = y,x,s,d */
  const int n_outer = dst_groups * H * W * src_slices;
  for (int it = 0; it < n_outer; ++it) {
    int d, y, x, s, r = it;
    if (!two_d) {
      s = r % src_slices; r /= src_slices;
      x = r % W; r /= W;
      y = r % H; r /= H;
      d = r;
    } else {
      d = r % dst_groups; r /= dst_groups;
      s = r % src_slices; r /= src_slices;
      x = r % W; r /= W;
      y = r;
    }
    for (int dg = 0; dg < G; ++dg) {
      const int d_ch = 4 * (d * G + dg);
      const int diff = O - d_ch;
      for (int s_ch = 4 * s; s_ch < 4 * s + 4; ++s_ch) {
        if (s_ch >= I) {
          *p++ = double_pad;
          *p++ = double_pad;
          continue;
        }
        long f = swap_dims ? (((long)s_ch * H + y) * W + x) * O + d_ch
                           : (((long)d_ch * H + y) * W + x) * I + s_ch;
        uint8_t v[4];
        for (int j = 0; j < 4; ++j) {
          v[j] = diff > j ? nib(src[f >> 1], (int)(f & 1)) : pad;
          f += df;
        }
        *p++ = (uint8_t)(((v[1] << 4) | v[0]) ^ 0x88);
        *p++ = (uint8_t)(((v[3] << 4) | v[2]) ^ 0x88);
        for (int j = 0; j < 4; ++j)
          if ((size_t)(d_ch + j) < sum_len) sum_i[d_ch + j] += (v[j] ^ 0x8) - 8;
      }
    }
  }
  return 0;
}

/* weights_conversion.cc:1584-1602 (GetWeightsAccumulatedInputChannels) */
void mldo_weights_sum_i(const int8_t* src, int O, int H, int W, int I, int32_t* sum) {
  const size_t per_o = (size_t)H * W * I;
  for (int o = 0; o < O; ++o) {
    int32_t s = 0;
    for (size_t e = 0; e < per_o; ++e) s += src[(size_t)o * per_o + e];
    sum[o] = s;
  }
}

/* weights_conversion.cc:1038-1063 for WeightsLayout::kCustomGroups */
size_t mldo_custom_total_elements(int o, int h, int w, int i, const int* axes, const int* sizes,
                                  int n_groups) {
  int shape[4] = {o, h, w, i};
  int total[4] = {1, 1, 1, 1};
  for (int g = 0; g < n_groups; ++g) {
    int sz = sizes[g];
    if (sz <= 0) sz = div_up(shape[axes[g]], total[axes[g]]);
    total[axes[g]] *= sz;
  }
  return (size_t)total[0] * total[1] * total[2] * total[3];
}

/* weights_conversion.cc:285-331 (RearrangeWeightsToCustom): mixed-radix order, the first
 * listed group is the fastest-varying one; size <= 0 means "the rest of that axis". */
void mldo_rearrange_custom_i8(const int8_t* src, int O, int H, int W, int I, const int* axes,
                              const int* sizes_in, int n_groups, int8_t pad, int8_t* dst) {
  int shape[4] = {O, H, W, I};
  int total[4] = {1, 1, 1, 1};
  int* sizes = (int*)malloc(sizeof(int) * (n_groups + 1));
  int* coord = (int*)calloc(n_groups + 1, sizeof(int));
  for (int g = 0; g < n_groups; ++g) {
    int sz = sizes_in[g];
    if (sz <= 0) sz = div_up(shape[axes[g]], total[axes[g]]);
    sizes[g] = sz;
    total[axes[g]] *= sz;
  }
  const size_t n = (size_t)total[0] * total[1] * total[2] * total[3];
  for (size_t e = 0; e < n; ++e) {
    int c[4] = {0, 0, 0, 0}, prev[4] = {1, 1, 1, 1};
    for (int g = 0; g < n_groups; ++g) {
      if (coord[g] == sizes[g]) {
        coord[g] = 0;
        ++coord[g + 1];
      }
      const int a = axes[g];
      c[a] = coord[g] * prev[a] + c[a];
      prev[a] *= sizes[g];
    }
    dst[e] = (c[0] < O && c[3] < I) ? src[(((size_t)c[0] * H + c[1]) * W + c[2]) * I + c[3]] : pad;
    ++coord[0];
  }
  free(sizes);
  free(coord);
}

/* common/task/tensor_desc.cc:267-292 (OHIToHOIO4): dst HWC(h, ceil(o/4), 4*i),
 * dst[b][o_slice][i*4+ch]; as a slice-major buffer that is [i][o_slice][4] per b. */
void mldo_scale_to_hoio4(const float* s, int O, int Hh, int I, float* dst) {
  const int os = div_up(O, 4);
  for (int b = 0; b < Hh; ++b)
    for (int i = 0; i < I; ++i)
      for (int sl = 0; sl < os; ++sl)
        for (int ch = 0; ch < 4; ++ch) {
          const int oc = sl * 4 + ch;
          const float v = oc < O ? s[((size_t)oc * Hh + b) * I + i] : 0.0f;
          dst[((size_t)b * os + sl) * (4 * I) + i * 4 + ch] = v;
        }
}

/* ------------------------------------------------------------------------------------ */
/* FullyConnected: restatement of the generated kernel                                    */
/* ------------------------------------------------------------------------------------ */

static inline float load_t(const void* p, size_t idx, int is_half) {
  return is_half ? mldo_f16_to_f32(((const uint16_t*)p)[idx]) : ((const float*)p)[idx];
}
static inline void store_t(void* p, size_t idx, float v, int is_half) {
  if (is_half)
    ((uint16_t*)p)[idx] = mldo_f32_to_f16(v);
  else
    ((float*)p)[idx] = v;
}

/* Unpack one I4O4 block at linear index `blk` into u[i][o].
 * uint8: 16 bytes, byte (i*4+o)          (common/task/util.cc:619-636)
 * uint4:  8 bytes, nibble (i*4+o), low nibble first (common/task/util.cc:772-790) */
static inline void unpack_block(const uint8_t* w, size_t blk, int bits, int u[4][4]) {
  if (bits == 8) {
    const uint8_t* b = w + blk * 16;
    for (int e = 0; e < 16; ++e) u[e / 4][e % 4] = b[e];
  } else {
    const uint8_t* b = w + blk * 8;
    for (int e = 0; e < 16; ++e) u[e / 4][e % 4] = (b[e / 2] >> (4 * (e & 1))) & 0xF;
  }
}

/* One work-item of common/kernels/fully_connected.cc:623-942 for (dst_s, token, y-lane):
 * accumulates K-slices src_s = y, y+wg_y, ... (or scale groups, when block-quantized,
 * :784-797), dequantizing with fc::WeightsScaleAddBias (fully_connected_util.cc:142-165)
 * and accumulating with fc::AccumulateFloat (:167-203). */
static void fc_partial(const mldo_fc_params* p, const void* act, const uint8_t* weights,
                       const void* scale, const void* zp, int dst_s, int tok, int y,
                       float r[4]) {
  const int is_half = p->precision != MLDO_PREC_F32;     /* Type */
  const int acc_half = p->precision == MLDO_PREC_F16;    /* AccType */
  const int ks = div_up(p->k, 4), ns = div_up(p->n, 4);
  const float shift = p->weight_bits == 8 ? 128.0f : 8.0f; /* fully_connected_util.cc:35-45 */
  float w_scale[4] = {0, 0, 0, 0}, w_bias[4] = {0, 0, 0, 0};
  r[0] = r[1] = r[2] = r[3] = 0.0f;

  const int block = p->scale_kind == MLDO_SCALE_BLOCK;
  const int outer_n = block ? p->groups : ks;
  const int group_slices = block ? ks / p->groups : 1; /* src_slices / src_groups, fully_connected.cc:366-369 */

  if (!block) {
    for (int c = 0; c < 4; ++c) {
      float s, z = 0.0f;
      if (p->scale_kind == MLDO_SCALE_SCALAR) { /* fully_connected_util.cc:124-140 */
        s = rt(p->scalar_scale, is_half);
        if (p->has_zero_point) z = rt(p->scalar_zero_point, is_half);
      } else { /* :102-122 */
        s = load_t(scale, (size_t)dst_s * 4 + c, is_half);
        if (p->has_zero_point) z = load_t(zp, (size_t)dst_s * 4 + c, is_half);
      }
      w_scale[c] = s;
      const float sh = p->has_zero_point ? t_add(shift, z, is_half) : shift;
      w_bias[c] = t_mul(-s, sh, is_half);
    }
  }
  for (int outer = y; outer < outer_n; outer += p->wg_y) {
    if (block) { /* fully_connected_util.cc:80-100: tensor (x=o_slice, y=0, s=group) */
      for (int c = 0; c < 4; ++c) {
        const size_t idx = ((size_t)outer * ns + dst_s) * 4 + c;
        const float s = load_t(scale, idx, is_half);
        const float z = p->has_zero_point ? load_t(zp, idx, is_half) : 0.0f;
        w_scale[c] = s;
        const float sh = p->has_zero_point ? t_add(shift, z, is_half) : shift;
        w_bias[c] = t_mul(-s, sh, is_half);
      }
    }
    for (int sub = 0; sub < group_slices; ++sub) {
      const int src_s = block ? outer * group_slices + sub : outer;
      float v[4];
      for (int c = 0; c < 4; ++c) v[c] = load_t(act, ((size_t)src_s * p->m + tok) * 4 + c, is_half);
      int u[4][4];
      unpack_block(weights, (size_t)src_s * ns + dst_s, p->weight_bits, u); /* :492 linear_i4o4 */
      float wf[4][4];
      for (int i = 0; i < 4; ++i)
        for (int c = 0; c < 4; ++c) {
          const float q = (float)u[i][c]; /* exact in half as well (<= 255) */
          wf[i][c] = p->use_fma ? t_fma(q, w_scale[c], w_bias[c], is_half)
                                : t_add(t_mul(q, w_scale[c], is_half), w_bias[c], is_half);
        }
      for (int c = 0; c < 4; ++c) {
        if (p->precision == MLDO_PREC_F32F16) {
          /* r += float(v.x*w0 + v.y*w1 + v.z*w2 + v.w*w3), the sum in half */
          float t = t_mul(v[0], wf[0][c], 1);
          t = t_add(t, t_mul(v[1], wf[1][c], 1), 1);
          t = t_add(t, t_mul(v[2], wf[2][c], 1), 1);
          t = t_add(t, t_mul(v[3], wf[3][c], 1), 1);
          r[c] = r[c] + t;
        } else {
          for (int i = 0; i < 4; ++i)
            r[c] = p->use_fma ? t_fma(v[i], wf[i][c], r[c], acc_half)
                              : t_add(r[c], t_mul(v[i], wf[i][c], acc_half), acc_half);
        }
      }
    }
  }
}

/* One (dst slice, token) of the kernel on the scalar path: the wg_y partial sums, the work-group
 * tree reduction, the conversion and the bias. */
static void fc_slice_token(const mldo_fc_params* q, const void* act, const uint8_t* weights,
                           const void* scale, const void* zp, const void* bias, void* dst,
                           int dst_s, int tok) {
  const int is_half = q->precision != MLDO_PREC_F32;
  const int acc_half = q->precision == MLDO_PREC_F16;
  const int wg_y = q->wg_y;
  float part[64][4];
  for (int y = 0; y < wg_y; ++y) fc_partial(q, act, weights, scale, zp, dst_s, tok, y, part[y]);
  /* work-group tree reduction, fully_connected_util.cc:321-354 */
  for (int stride = wg_y / 2; stride > 0; stride /= 2)
    for (int y = 0; y < stride; ++y)
      for (int c = 0; c < 4; ++c) part[y][c] = t_add(part[y][c], part[y + stride][c], acc_half);
  /* fully_connected_util.cc:356-407: convert to dst type, then add bias in dst type */
  for (int c = 0; c < 4; ++c) {
    float res = rt(part[0][c], is_half);
    if (q->has_bias) res = t_add(res, load_t(bias, (size_t)dst_s * 4 + c, is_half), is_half);
    store_t(dst, ((size_t)dst_s * q->m + tok) * 4 + c, res, is_half);
  }
}

/* ---- the same operation sequence, eight output channels at a time (x86-64 AVX2 + FMA + F16C) ----
 *
 * Serves F32_F16 precision without zero point, wg_y = 1, per-channel or group-wise scales.  Every
 * half operation of the scalar path (a float operation followed by a rounding to half) becomes one
 * vector float operation followed by vcvtps2ph / vcvtph2ps, which rounds to nearest even like
 * d2h(); the operations and their order per output channel are those of fc_partial(), so the
 * results are bit-identical (tests compare the two paths).  The one place where the scalar path
 * rounds once from a wider type, the fused q * scale + bias of the dequantization, is exact in
 * float here: the path is taken only when bias = -shift * scale holds exactly for every scale
 * (shift is a power of two, so this fails only where shift * scale leaves half's range), and then
 * q * scale + bias = (q - shift) * scale has at most 8 + 11 significant bits. */
#if defined(__x86_64__)
#include <immintrin.h>
#define MLDO_AVX2 __attribute__((target("avx2,fma,f16c")))

static int g_fast_path_enabled = 1;

MLDO_AVX2 static inline __m256 rt8(__m256 x) {
  return _mm256_cvtph_ps(_mm256_cvtps_ph(x, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
}

/* all scales s (n_values halves) have -shift * s representable in half */
static int scales_dequant_exactly(const uint16_t* scale, size_t n_values, float shift) {
  for (size_t i = 0; i < n_values; ++i) {
    const float s = mldo_f16_to_f32(scale[i]);
    const float b = -s * shift;
    if (!(mldo_f16_to_f32(mldo_f32_to_f16(b)) == b)) return 0; /* also false for NaN */
  }
  return 1;
}

/* Two adjacent dst slices (8 channels) x one K-slice: the four rows wf[i] of dequantized weights. */
MLDO_AVX2 static inline void dequant_pair(const uint8_t* weights, size_t blk, int bits, __m256 s,
                                          __m256 b, int use_fma, __m256 wf[4]) {
  __m128i a0, a1; /* the 16 codes (i*4+o) of slice s and of slice s+1, one per byte */
  if (bits == 8) {
    a0 = _mm_loadu_si128((const __m128i*)(weights + blk * 16));
    a1 = _mm_loadu_si128((const __m128i*)(weights + blk * 16 + 16));
  } else {
    const __m128i raw = _mm_loadu_si128((const __m128i*)(weights + blk * 8));
    const __m128i m4 = _mm_set1_epi8(0x0F);
    const __m128i lo = _mm_and_si128(raw, m4);
    const __m128i hi = _mm_and_si128(_mm_srli_epi16(raw, 4), m4);
    a0 = _mm_unpacklo_epi8(lo, hi); /* low nibble first, common/task/util.cc:772-790 */
    a1 = _mm_unpackhi_epi8(lo, hi);
  }
  const __m128i i01 = _mm_unpacklo_epi32(a0, a1); /* [i=0: slice s, slice s+1][i=1: ...] */
  const __m128i i23 = _mm_unpackhi_epi32(a0, a1);
  const __m128i rows[4] = {i01, _mm_srli_si128(i01, 8), i23, _mm_srli_si128(i23, 8)};
  for (int i = 0; i < 4; ++i) {
    const __m256 q = _mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(rows[i]));
    wf[i] = use_fma ? rt8(_mm256_fmadd_ps(q, s, b)) : rt8(_mm256_add_ps(rt8(_mm256_mul_ps(q, s)), b));
  }
}

/* dst slices [s0, s0 + 2*units) of token `tok`; act_f: the token's activations as float [k4]. */
MLDO_AVX2 static inline __attribute__((always_inline)) void fc_pairs_avx2(const mldo_fc_params* p, const float* act_f, const uint8_t* weights,
                                    const uint16_t* scale, const uint16_t* bias, uint16_t* dst, int s0,
                                    int units, int tok) {
  const int ks = div_up(p->k, 4), ns = div_up(p->n, 4);
  const int block = p->scale_kind == MLDO_SCALE_BLOCK;
  const int outer_n = block ? p->groups : 1;
  const int group_slices = block ? ks / p->groups : ks;
  const __m256 neg_shift = _mm256_set1_ps(p->weight_bits == 8 ? -128.0f : -8.0f);
  __m256 acc[4], sc[4], bi[4];
  for (int u = 0; u < units; ++u) acc[u] = _mm256_setzero_ps();
  for (int outer = 0; outer < outer_n; ++outer) {
    for (int u = 0; u < units; ++u) {
      const size_t idx = ((size_t)outer * ns + s0 + 2 * u) * 4;
      sc[u] = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(scale + idx)));
      bi[u] = rt8(_mm256_mul_ps(sc[u], neg_shift)); /* t_mul(-s, shift) */
    }
    for (int sub = 0; sub < group_slices; ++sub) {
      const int src_s = outer * group_slices + sub;
      const __m256 v0 = _mm256_broadcast_ss(act_f + src_s * 4 + 0);
      const __m256 v1 = _mm256_broadcast_ss(act_f + src_s * 4 + 1);
      const __m256 v2 = _mm256_broadcast_ss(act_f + src_s * 4 + 2);
      const __m256 v3 = _mm256_broadcast_ss(act_f + src_s * 4 + 3);
      for (int u = 0; u < units; ++u) {
        __m256 wf[4];
        dequant_pair(weights, (size_t)src_s * ns + s0 + 2 * u, p->weight_bits, sc[u], bi[u], p->use_fma, wf);
        /* r += float(v.x*w0 + v.y*w1 + v.z*w2 + v.w*w3), the sum in half */
        __m256 t = rt8(_mm256_mul_ps(v0, wf[0]));
        t = rt8(_mm256_add_ps(t, rt8(_mm256_mul_ps(v1, wf[1]))));
        t = rt8(_mm256_add_ps(t, rt8(_mm256_mul_ps(v2, wf[2]))));
        t = rt8(_mm256_add_ps(t, rt8(_mm256_mul_ps(v3, wf[3]))));
        acc[u] = _mm256_add_ps(acc[u], t);
      }
    }
  }
  for (int u = 0; u < units; ++u) {
    __m256 res = rt8(acc[u]);
    const int s = s0 + 2 * u;
    if (p->has_bias)
      res = rt8(_mm256_add_ps(res, _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(bias + (size_t)s * 4)))));
    const __m128i h = _mm256_cvtps_ph(res, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
    /* dst is [Ns][M][4]: the two slices of the pair are M*4 halves apart */
    _mm_storel_epi64((__m128i*)(dst + ((size_t)s * p->m + tok) * 4), h);
    _mm_storel_epi64((__m128i*)(dst + ((size_t)(s + 1) * p->m + tok) * 4), _mm_srli_si128(h, 8));
  }
}

/* the full chunk of four pairs with the pair loop unrolled, the tail chunk as it comes */
MLDO_AVX2 static void fc_chunk_avx2(const mldo_fc_params* p, const float* act_f, const uint8_t* weights,
                                    const uint16_t* scale, const uint16_t* bias, uint16_t* dst, int s0,
                                    int units, int tok) {
  if (units == 4)
    fc_pairs_avx2(p, act_f, weights, scale, bias, dst, s0, 4, tok);
  else
    fc_pairs_avx2(p, act_f, weights, scale, bias, dst, s0, units, tok);
}

static int fast_path_serves(const mldo_fc_params* p, const void* scale) {
  if (!g_fast_path_enabled || p->precision != MLDO_PREC_F32F16 || p->wg_y != 1 || p->has_zero_point) return 0;
  if (p->weight_bits != 4 && p->weight_bits != 8) return 0;
  if (p->scale_kind != MLDO_SCALE_LINEAR && p->scale_kind != MLDO_SCALE_BLOCK) return 0;
  if (p->scale_kind == MLDO_SCALE_BLOCK && (p->groups <= 0 || div_up(p->k, 4) % p->groups)) return 0;
  if (!__builtin_cpu_supports("avx2") || !__builtin_cpu_supports("fma") || !__builtin_cpu_supports("f16c")) return 0;
  const size_t n_scales = (size_t)div_up(p->n, 4) * 4 * (p->scale_kind == MLDO_SCALE_BLOCK ? p->groups : 1);
  return scales_dequant_exactly((const uint16_t*)scale, n_scales, p->weight_bits == 8 ? 128.0f : 8.0f);
}
#else
static int g_fast_path_enabled = 0;
#endif

void mldo_set_fast_path(int enabled) { g_fast_path_enabled = enabled; }

int mldo_fc_kernel(const mldo_fc_params* p, const void* act, const uint8_t* weights,
                   const void* scale, const void* zp, const void* bias, void* dst) {
  const int ns = div_up(p->n, 4);
  mldo_fc_params q = *p;
  q.wg_y = p->wg_y > 0 ? p->wg_y : 1;
#ifdef _OPENMP
  const int nthreads = p->threads > 0 ? p->threads : omp_get_max_threads();
#endif
#if defined(__x86_64__)
  if (fast_path_serves(&q, scale)) {
    const int ks4 = div_up(p->k, 4) * 4;
    float* act_f = (float*)malloc((size_t)p->m * ks4 * sizeof(float));
    for (int tok = 0; tok < p->m; ++tok)
      for (int c = 0; c < ks4; ++c)
        act_f[(size_t)tok * ks4 + c] = mldo_f16_to_f32(((const uint16_t*)act)[((size_t)(c / 4) * p->m + tok) * 4 + c % 4]);
    const int pairs = ns / 2;           /* an odd last slice goes through the scalar path */
    const int chunks = div_up(pairs, 4); /* 8 slices: one 64-byte line of uint4 blocks per K-slice */
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(nthreads)
#endif
    for (int ch = 0; ch < chunks; ++ch) {
      const int units = pairs - ch * 4 < 4 ? pairs - ch * 4 : 4;
      for (int tok = 0; tok < p->m; ++tok)
        fc_chunk_avx2(&q, act_f + (size_t)tok * ks4, weights, (const uint16_t*)scale, (const uint16_t*)bias,
                      (uint16_t*)dst, ch * 8, units, tok);
    }
    if (ns & 1)
      for (int tok = 0; tok < p->m; ++tok) fc_slice_token(&q, act, weights, scale, zp, bias, dst, ns - 1, tok);
    free(act_f);
    return 1;
  }
#endif
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(nthreads)
#endif
  for (int dst_s = 0; dst_s < ns; ++dst_s)
    for (int tok = 0; tok < p->m; ++tok) fc_slice_token(&q, act, weights, scale, zp, bias, dst, dst_s, tok);
  return 0;
}

static inline int32_t sat_add32(int32_t a, int64_t b) {
  int64_t s = (int64_t)a + b;
  if (s > INT32_MAX) s = INT32_MAX;
  if (s < INT32_MIN) s = INT32_MIN;
  return (int32_t)s;
}
/* dot_acc_sat_4x8packed_su_int(a signed, b unsigned, acc) */
static inline int32_t dot_su(uint32_t a, uint32_t b, int32_t acc) {
  int64_t d = 0;
  for (int j = 0; j < 4; ++j) d += (int64_t)(int8_t)(a >> (8 * j)) * (int64_t)(uint8_t)(b >> (8 * j));
  return sat_add32(acc, d);
}

/* int8-math FullyConnected: common/kernels/fully_connected.cc:543-621 (bit transposes of
 * the I4O4 block into four packed words, one per output), fully_connected_util.cc:205-229
 * (packed dot accumulate, then r -= sum(act) * shift).  act is int8 [Ks][M][4]; dst int32
 * [Ns][M][4]. */
void mldo_fc_int8_kernel(int m, int k, int n, int bits, const int8_t* act, const uint8_t* weights,
                         int32_t* dst) {
  const int ks = div_up(k, 4), ns = div_up(n, 4);
  const int shift = bits == 8 ? 128 : 8;
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
  for (int dst_s = 0; dst_s < ns; ++dst_s) {
    for (int tok = 0; tok < m; ++tok) {
      int32_t r[4] = {0, 0, 0, 0}, r_sum = 0;
      for (int src_s = 0; src_s < ks; ++src_s) {
        uint32_t v;
        memcpy(&v, act + ((size_t)src_s * m + tok) * 4, 4);
        const size_t blk = (size_t)src_s * ns + dst_s;
        uint32_t w0, w1, w2, w3;
        if (bits == 4) {
          uint32_t wx, wy;
          memcpy(&wx, weights + blk * 8, 4);
          memcpy(&wy, weights + blk * 8 + 4, 4);
          uint32_t t = (wy ^ (wx >> 16)) & 0x0000FFFFu;
          uint32_t t0 = wx ^ (t << 16);
          uint32_t t1 = wy ^ t;
          t = (t1 ^ (t0 >> 8)) & 0x00FF00FFu;
          t1 ^= t;
          t0 ^= (t << 8);
          w0 = t0 & 0x0F0F0F0Fu;
          w1 = (t0 >> 4) & 0x0F0F0F0Fu;
          w2 = t1 & 0x0F0F0F0Fu;
          w3 = (t1 >> 4) & 0x0F0F0F0Fu;
        } else {
          uint32_t wx, wy, wz, ww;
          memcpy(&wx, weights + blk * 16, 4);
          memcpy(&wy, weights + blk * 16 + 4, 4);
          memcpy(&wz, weights + blk * 16 + 8, 4);
          memcpy(&ww, weights + blk * 16 + 12, 4);
          uint32_t t = (wz ^ (wx >> 16)) & 0x0000FFFFu;
          w2 = wz ^ t;
          w0 = wx ^ (t << 16);
          t = (ww ^ (wy >> 16)) & 0x0000FFFFu;
          w3 = ww ^ t;
          w1 = wy ^ (t << 16);
          t = (w1 ^ (w0 >> 8)) & 0x00FF00FFu;
          w1 ^= t;
          w0 ^= (t << 8);
          t = (w3 ^ (w2 >> 8)) & 0x00FF00FFu;
          w3 ^= t;
          w2 ^= (t << 8);
        }
        r[0] = dot_su(v, w0, r[0]);
        r[1] = dot_su(v, w1, r[1]);
        r[2] = dot_su(v, w2, r[2]);
        r[3] = dot_su(v, w3, r[3]);
        r_sum = dot_su(v, 0x01010101u, r_sum);
      }
      for (int c = 0; c < 4; ++c)
        dst[((size_t)dst_s * m + tok) * 4 + c] = (int32_t)((uint32_t)r[c] - (uint32_t)r_sum * (uint32_t)shift);
    }
  }
}

/* common/task/testing_ref_ops.cc:961-988 (FullyConnectedReference, float): src BHWC [m][k],
 * weights OHWI [n][k], sum starts at the bias and accumulates in float, in k order. */
void mldo_fc_reference_f32(int m, int k, int n, const float* src, const float* weights,
                           const float* bias, float* dst) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
  for (int d = 0; d < n; ++d)
    for (int t = 0; t < m; ++t) {
      float sum = bias ? bias[d] : 0.0f;
      for (int s = 0; s < k; ++s) sum += src[(size_t)t * k + s] * weights[(size_t)d * k + s];
      dst[(size_t)t * n + d] = sum;
    }
}

/* common/task/testing_ref_ops.cc:1069-1098 (FullyConnectedReference, int8 x int8 -> int32) */
void mldo_fc_reference_i8(int m, int k, int n, const int8_t* src, const int8_t* weights,
                          int32_t* dst) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
  for (int d = 0; d < n; ++d)
    for (int t = 0; t < m; ++t) {
      int32_t sum = 0;
      for (int s = 0; s < k; ++s) sum += (int32_t)src[(size_t)t * k + s] * (int32_t)weights[(size_t)d * k + s];
      dst[(size_t)t * n + d] = sum;
    }
}

/* common/task/testing_ref_ops.cc:2715-2742 (MakeWeightsFromInt8, OHWI scale/zero-point):
 * W[o,i] = (q[o,i] - zp[og,ig]) * s[og,ig]; zero_point may be NULL (= 0). */
void mldo_make_weights_from_int8(int n, int k, const int8_t* w, const float* scale,
                                 const float* zero_point, int scale_o, int scale_i, float* dst) {
  const int ig = k / scale_i, og = n / scale_o;
  for (int i = 0; i < k; ++i)
    for (int o = 0; o < n; ++o) {
      const size_t sidx = (size_t)(o / og) * scale_i + (i / ig);
      const float z = zero_point ? zero_point[sidx] : 0.0f;
      dst[(size_t)o * k + i] = ((float)w[(size_t)o * k + i] - z) * scale[sidx];
    }
}

/* ------------------------------------------------------------------------------------ */
/* per-token quantization                                                                 */
/* ------------------------------------------------------------------------------------ */

static inline int f2i_trunc(float v) { /* Convert<int4>: truncation; NaN -> 0 */
  if (v != v) return 0;
  if (v >= 2147483520.0f) return INT32_MAX;
  if (v <= -2147483648.0f) return INT32_MIN;
  return (int)v;
}

/* common/kernels/quantize_and_dequantize.cc:212-691 (GetCode) with the constants of
 * :757-788.  src is the slice-major buffer [S][tokens][4] (fp16 or fp32); params are the
 * fp32 tensor the builder allocates (common/gpu_model_builder.cc:1285-1289), stored as
 * [tokens][4] = (inv_scale, offset, sum, 0).  `batch` is the tensor's B: the min/max
 * search of the asymmetric variant starts from the element (b, y=0, x=0, c=0) (:288).
 * tokens are the flattened (y, x, b) index (y*W + x)*B + b.
 * Code range (:757, 779-803): range = 2^bits (8-bit types 256, C32 types 16), dst_range = range-1,
 * symmetric half range = range/2 - 1, zero point = range/2, rounding offset range/2 + 0.5, the
 * unsigned cap kMaxHalf / (range/2), asymmetric middle (range/2)/(range-1).
 * codes, as bytes in memory (:461-653, dst tensor of GetShapeForPackedType, common/util.cc:262-277,
 * in buffer layout [slice][y][x][b][4 elements]):
 *   C4   [S][tokens][4] one byte per channel;
 *   W4C4 [S][H][ceil(W/4)][B][4 x][4 channels]: element (x/4, y, s) of an int32x4 tensor holds the
 *        char4 of x, x+1, x+2, x+3; positions at or beyond W repeat column W-1 (x_clamped, :284);
 *   C16  [ceil(S/4)][tokens][4 slices][4 channels];
 *   C32  [ceil(S/8)][tokens][16 bytes]: channel j of the 32 in nibble j (two's complement for the
 *        signed type), i.e. byte j/2, low nibble first;
 *   slices at or beyond S inside the last C16 / C32 group repeat slice S-1 (s_clamped, :407). */
void mldo_quantize_packed(int height, int width, int batch, int channels, int src_is_f16, const void* src,
                          int packed_type, int symmetric, int calculate_sum, void* codes, float* params) {
  const int tokens = height * width * batch;
  const int slices = div_up(channels, 4);
  const int is_signed = packed_type == MLDO_PACKED_INT8C4 || packed_type == MLDO_PACKED_INT8C16 ||
                        packed_type == MLDO_PACKED_INT8W4C4 || packed_type == MLDO_PACKED_INT4C32;
  const int c16 = packed_type == MLDO_PACKED_INT8C16 || packed_type == MLDO_PACKED_UINT8C16;
  const int c32 = packed_type == MLDO_PACKED_INT4C32 || packed_type == MLDO_PACKED_UINT4C32;
  const int w4 = packed_type == MLDO_PACKED_INT8W4C4 || packed_type == MLDO_PACKED_UINT8W4C4;
  const int range = c32 ? 16 : 256;
  const int dst_range = range - 1;
  const float half_range = (float)(range / 2 - 1), zero_point = (float)(range / 2);
  const float kMinNormalHalf = 6.103515625e-05f, kMaxHalf = 65504.0f;
  const int width4 = div_up(width, 4);
  uint8_t* out = (uint8_t*)codes;
  uint8_t* row = (uint8_t*)malloc((size_t)slices * 4); /* the token's codes, one byte per channel */
  for (int t = 0; t < tokens; ++t) {
    float inv_scale = 0.0f, scale = 0.0f, offset = 0.0f, min_value = 0.0f;
    if (symmetric) {
      float abs_max = 0.0f;
      for (int c = 0; c < channels; ++c) {
        const float v = fabsf(load_t(src, ((size_t)(c / 4) * tokens + t) * 4 + c % 4, src_is_f16));
        if (v > abs_max) abs_max = v;
      }
      if (abs_max > 0.0f) { /* :363-377 */
        const float min_scale = src_is_f16 ? kMinNormalHalf : 1.0e-30f;
        inv_scale = fmaxf(min_scale, abs_max / half_range);
        if (!is_signed && src_is_f16) inv_scale = fminf(inv_scale, kMaxHalf / zero_point);
        scale = 1.0f / inv_scale;
        if (!is_signed) offset = -inv_scale * zero_point;
      }
    } else {
      const int b = batch > 0 ? t % batch : 0;
      min_value = load_t(src, (size_t)b * 4, src_is_f16); /* Read(0,0,0).x of batch b */
      float max_value = min_value;
      for (int c = 0; c < channels; ++c) {
        const float v = load_t(src, ((size_t)(c / 4) * tokens + t) * 4 + c % 4, src_is_f16);
        if (v < min_value) min_value = v;
        if (v > max_value) max_value = v;
      }
      const float src_range = rt(max_value - min_value, src_is_f16); /* subtraction in SrcType, :392 */
      offset = min_value;
      scale = (float)dst_range / src_range;
      inv_scale = src_range / (float)dst_range;
      if (is_signed) {
        const float middle = zero_point / (float)dst_range; /* :786-787 */
        const float prod = src_range * middle;
        offset = offset + prod;
      }
    }
    int sum = 0;
    for (int s = 0; s < slices; ++s) {
      for (int c = 0; c < 4; ++c) {
        const float x = load_t(src, ((size_t)s * tokens + t) * 4 + c, src_is_f16);
        int q;
        if (symmetric) { /* :423-429 */
          float v = x * scale;
          v = v + (zero_point + 0.5f);
          v = floorf(v);
          v = fminf((float)dst_range, fmaxf(0.0f, v));
          q = f2i_trunc(v);
        } else { /* :431-437 */
          float v = (x - min_value) * scale;
          v = v + 0.5f;
          q = f2i_trunc(v);
          if (q > dst_range) q = dst_range;
          if (q < 0) q = 0;
        }
        if (is_signed) q -= (dst_range + 1) / 2;
        if (calculate_sum && s * 4 + c < channels) sum += q; /* :442-459 */
        row[s * 4 + c] = (uint8_t)q;
      }
    }
    if (c16) {
      for (int s = 0; s < div_up(slices, 4) * 4; ++s) {
        const int sc = s < slices ? s : slices - 1;
        memcpy(out + ((size_t)(s / 4) * tokens + t) * 16 + (s % 4) * 4, row + sc * 4, 4);
      }
    } else if (c32) {
      for (int g = 0; g < div_up(slices, 8); ++g) {
        uint8_t* d = out + ((size_t)g * tokens + t) * 16;
        memset(d, 0, 16);
        for (int j = 0; j < 32; ++j) {
          const int s = g * 8 + j / 4, sc = s < slices ? s : slices - 1;
          d[j / 2] |= (uint8_t)((row[sc * 4 + j % 4] & 15u) << (4 * (j & 1)));
        }
      }
    } else if (w4) {
      const int b = t % batch, x = (t / batch) % width, y = t / (batch * width);
      for (int s = 0; s < slices; ++s) {
        /* column x, and the columns beyond the width when x is the last one */
        for (int xx = x; xx < (x == width - 1 ? width4 * 4 : x + 1); ++xx)
          memcpy(out + ((((size_t)s * height + y) * width4 + xx / 4) * batch + b) * 16 + (xx % 4) * 4, row + s * 4, 4);
      }
    } else {
      for (int s = 0; s < slices; ++s) memcpy(out + ((size_t)s * tokens + t) * 4, row + s * 4, 4);
    }
    params[(size_t)t * 4 + 0] = inv_scale;
    params[(size_t)t * 4 + 1] = offset;
    params[(size_t)t * 4 + 2] = calculate_sum ? (float)sum : 0.0f;
    params[(size_t)t * 4 + 3] = 0.0f;
  }
  free(row);
}

void mldo_quantize(int tokens, int channels, int batch, int src_is_f16, const void* src,
                   int packed_type, int symmetric, int calculate_sum, void* codes, float* params) {
  const int b = batch > 0 ? batch : 1;
  mldo_quantize_packed(1, tokens / b, b, channels, src_is_f16, src, packed_type, symmetric, calculate_sum, codes,
                       params);
}

/* common/kernels/quantize_and_dequantize.cc:867-964 (CreateDequantization), fused after the
 * int8 convolution; an optional bias is a separate Add node in the destination type
 * (common/gpu_model_builder.cc:1427-1429).  acc int32 [Ns][tokens][4], params [tokens][4],
 * weights_sum / scale / zero_point padded to Ns*4; dst [Ns][tokens][4] fp16 or fp32. */
void mldo_dequantize(int tokens, int n, int k, const int32_t* acc, const float* params,
                     const int32_t* weights_sum, const float* weights_scale,
                     const float* weights_zero_point, const void* bias, int dst_is_f16, void* dst) {
  const int ns = div_up(n, 4);
  for (int s = 0; s < ns; ++s)
    for (int t = 0; t < tokens; ++t)
      for (int c = 0; c < 4; ++c) {
        const size_t idx = ((size_t)s * tokens + t) * 4 + c;
        const float src_scale = params[(size_t)t * 4 + 0];
        const float src_zp = params[(size_t)t * 4 + 1];
        const float ws = weights_scale[s * 4 + c];
        float res = (float)acc[idx];
        const float f0 = ws * src_scale;
        res = res * f0;
        const float f1 = ws * src_zp;
        const float f2 = f1 * (float)weights_sum[s * 4 + c];
        res = res + f2;
        if (weights_zero_point) {
          const float wzp = weights_zero_point[s * 4 + c];
          const float src_sum = params[(size_t)t * 4 + 2];
          const float g0 = src_scale * wzp;
          const float g1 = g0 * src_sum;
          res = res + g1;
          const float g2 = src_zp * wzp;
          const float g3 = g2 * (float)k;
          res = res + g3;
        }
        res = rt(res, dst_is_f16);
        if (bias) res = t_add(res, load_t(bias, (size_t)s * 4 + c, dst_is_f16), dst_is_f16);
        store_t(dst, idx, res, dst_is_f16);
      }
}

/* common/kernels/conv_weights_converter.cc:202-211, 248-290: w_f = q*s + (-s*(shift+zp)) in
 * the destination type (fp16 here), written back in plain OHWI order [n][k]. */
void mldo_dequantize_weights(int n, int k, int bits, const uint8_t* weights, int scale_kind,
                             int groups, const uint16_t* scale, const uint16_t* zero_point,
                             uint16_t* dst) {
  const int ks = div_up(k, 4), ns = div_up(n, 4);
  const float shift = bits == 8 ? 128.0f : 8.0f;
  const int group_slices = scale_kind == MLDO_SCALE_BLOCK ? ks / groups : ks;
  for (int src_s = 0; src_s < ks; ++src_s)
    for (int dst_s = 0; dst_s < ns; ++dst_s) {
      int u[4][4];
      unpack_block(weights, (size_t)src_s * ns + dst_s, bits, u);
      const int g = scale_kind == MLDO_SCALE_BLOCK ? src_s / group_slices : 0;
      for (int c = 0; c < 4; ++c) {
        const size_t sidx = ((size_t)g * ns + dst_s) * 4 + c;
        const float s = mldo_f16_to_f32(scale[sidx]);
        const float z = zero_point ? mldo_f16_to_f32(zero_point[sidx]) : 0.0f;
        const float sh = zero_point ? t_add(shift, z, 1) : shift;
        const float b = t_mul(-s, sh, 1);
        for (int i = 0; i < 4; ++i) {
          const int oc = dst_s * 4 + c, ic = src_s * 4 + i;
          if (oc < n && ic < k)
            dst[(size_t)oc * k + ic] = mldo_f32_to_f16(t_add(t_mul((float)u[i][c], s, 1), b, 1));
        }
      }
    }
}
