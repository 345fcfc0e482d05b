// Host-side weight packers ("weights rearrangement") of the quantized fully-connected path.
//
// Every destination element is produced from a closed-form source index, block by block,
// so the loops parallelise over blocks (OpenMP) instead of walking one output pointer.
// Layouts (reference: common/task/weights_layout.h, common/task/weights_conversion.cc):
//   OSpatialIOGroupI4O4   [Og][HW][Is][G][4i][4o]
//   OSpatialIOGroupO4I4   [Og][HW][Is][G][4o][4i]
//   2D Y=spatial*I, X=OGroup  [HW][Is][Og][G][4i][4o]
//   custom groups         mixed radix, first listed group fastest
#include "packer.h"

#include <cstring>
#include <vector>

namespace mldhip {
namespace {

inline int DivUpI(int a, int b) { return (a + b - 1) / b; }

struct BlockGeom {
  int dst_slices, src_slices, dst_groups, G, HW;
  int layout;
  // index of the first element of block (d, sp, s, dg); a block is 16 elements
  size_t BlockBase(int d, int sp, int s, int dg) const {
    if (layout == kLayout2D) return ((((size_t)sp * src_slices + s) * dst_groups + d) * G + dg) * 16;
    return ((((size_t)d * HW + sp) * src_slices + s) * G + dg) * 16;
  }
  // position of (ii, oo) inside the block
  int Inner(int ii, int oo) const { return layout == kLayoutO4I4 ? oo * 4 + ii : ii * 4 + oo; }
};

bool MakeGeom(const PackShape& sh, int layout, int group, BlockGeom* g) {
  if (layout != kLayoutI4O4 && layout != kLayoutO4I4 && layout != kLayout2D) return false;
  if (group <= 0) return false;
  g->layout = layout;
  g->G = group;
  g->HW = sh.h * sh.w;
  g->dst_slices = DivUpI(sh.o, 4);
  g->src_slices = DivUpI(sh.i, 4);
  g->dst_groups = DivUpI(g->dst_slices, group);
  return true;
}

// Generic element fetch + store over all blocks.  Fetch(oc, sp, ic) is only called in range.
template <typename T, typename Fetch>
void FillBlocks(const PackShape& sh, const BlockGeom& g, T pad, T* dst, Fetch fetch) {
  const long n_outer = (long)g.dst_groups * g.HW * g.src_slices;
#pragma omp parallel for schedule(static)
  for (long outer = 0; outer < n_outer; ++outer) {
    const int s = (int)(outer % g.src_slices);
    const int sp = (int)((outer / g.src_slices) % g.HW);
    const int d = (int)(outer / ((long)g.src_slices * g.HW));
    for (int dg = 0; dg < g.G; ++dg) {
      T* blk = dst + g.BlockBase(d, sp, s, dg);
      const int o0 = 4 * (d * g.G + dg), i0 = 4 * s;
      for (int ii = 0; ii < 4; ++ii)
        for (int oo = 0; oo < 4; ++oo) {
          const int oc = o0 + oo, ic = i0 + ii;
          blk[g.Inner(ii, oo)] = (oc < sh.o && ic < sh.i) ? fetch(oc, sp, ic) : pad;
        }
    }
  }
}

}  // namespace

size_t TotalElements(const PackShape& sh, int layout, int group) {
  const int i4 = DivUpI(sh.i, 4) * 4;
  switch (layout) {
    case kLayoutI4O4:
    case kLayoutO4I4:
      return (size_t)i4 * (DivUpI(sh.o, 4 * group) * 4 * group) * sh.h * sh.w;
    case kLayout2D:
      return (size_t)DivUpI(sh.i, 4) * (DivUpI(DivUpI(sh.o, 4), group) * group) * 16 * sh.h * sh.w;
    default:
      return 0;
  }
}

size_t CustomTotalElements(const PackShape& sh, const int* axes, const int* sizes, int n) {
  const int shape[4] = {sh.o, sh.h, sh.w, sh.i};
  int total[4] = {1, 1, 1, 1};
  for (int g = 0; g < n; ++g) {
    int sz = sizes[g];
    if (sz <= 0) sz = DivUpI(shape[axes[g]], total[axes[g]]);
    total[axes[g]] *= sz;
  }
  return (size_t)total[0] * total[1] * total[2] * total[3];
}

bool RearrangeU8(const uint8_t* src, const PackShape& sh, int layout, int group, uint8_t pad,
                 int add, uint8_t* dst) {
  BlockGeom g;
  if (!MakeGeom(sh, layout, group, &g)) return false;
  const size_t per_o = (size_t)g.HW * sh.i;
  FillBlocks<uint8_t>(sh, g, pad, dst, [&](int oc, int sp, int ic) {
    return (uint8_t)(src[(size_t)oc * per_o + (size_t)sp * sh.i + ic] + add);
  });
  return true;
}

bool RearrangeInt8AsUint4(const int8_t* src, const PackShape& sh, int layout, int group, int shift,
                          unsigned pad, uint8_t* dst) {
  const size_t total = TotalElements(sh, layout, group);
  if (total == 0) return false;
  std::vector<uint8_t> wide(total);
  if (!RearrangeU8(reinterpret_cast<const uint8_t*>(src), sh, layout, group, (uint8_t)pad, shift,
                   wide.data()))
    return false;
  const long n = (long)(total / 2);
#pragma omp parallel for schedule(static)
  for (long e = 0; e < n; ++e) dst[e] = (uint8_t)((wide[2 * e + 1] << 4) | wide[2 * e]);
  return true;
}

bool RearrangeUint4Packed(const uint8_t* src, const PackShape& sh, int layout, int group,
                          uint8_t* dst, int32_t* sum_i, size_t sum_len, unsigned pad_value,
                          bool swap_dims) {
  if (layout != kLayoutI4O4 && layout != kLayout2D) return false;
  BlockGeom g;
  if (!MakeGeom(sh, layout, group, &g)) return false;
  const uint8_t out_pad = (uint8_t)(pad_value & 0xF);  // nibble stored for a padded element
  const size_t per_o = (size_t)g.HW * sh.i;
  auto nibble = [&](int oc, int sp, int ic) -> uint8_t {
    const size_t f = swap_dims ? ((size_t)ic * g.HW + sp) * sh.o + oc
                               : (size_t)oc * per_o + (size_t)sp * sh.i + ic;
    const uint8_t byte = src[f >> 1];
    return (uint8_t)(((f & 1) ? (byte >> 4) : (byte & 0xF)) ^ 0x8);  // two's complement -> +8
  };
  const long n_outer = (long)g.dst_groups * g.HW * g.src_slices;
#pragma omp parallel for schedule(static)
  for (long outer = 0; outer < n_outer; ++outer) {
    const int s = (int)(outer % g.src_slices);
    const int sp = (int)((outer / g.src_slices) % g.HW);
    const int d = (int)(outer / ((long)g.src_slices * g.HW));
    for (int dg = 0; dg < g.G; ++dg) {
      uint8_t* blk = dst + g.BlockBase(d, sp, s, dg) / 2;
      const int o0 = 4 * (d * g.G + dg), i0 = 4 * s;
      for (int ii = 0; ii < 4; ++ii) {
        uint8_t v[4];
        for (int oo = 0; oo < 4; ++oo) {
          const int oc = o0 + oo, ic = i0 + ii;
          v[oo] = (oc < sh.o && ic < sh.i) ? nibble(oc, sp, ic) : out_pad;
        }
        blk[ii * 2 + 0] = (uint8_t)(v[0] | (v[1] << 4));
        blk[ii * 2 + 1] = (uint8_t)(v[2] | (v[3] << 4));
      }
    }
  }
  // Per-output-channel sums over everything the channel owns (all spatial positions and
  // input channels); entries beyond o are left untouched.
  const long n_o = (long)sh.o;
#pragma omp parallel for schedule(static)
  for (long oc = 0; oc < n_o; ++oc) {
    if ((size_t)oc >= sum_len) continue;
    int32_t acc = 0;
    for (int sp = 0; sp < g.HW; ++sp)
      for (int ic = 0; ic < sh.i; ++ic) acc += (int32_t)nibble((int)oc, sp, ic) - 8;
    sum_i[oc] = acc;
  }
  return true;
}

void WeightsSumI(const int8_t* src, const PackShape& sh, int32_t* sum) {
  const size_t per_o = (size_t)sh.h * sh.w * sh.i;
  const long n_o = sh.o;
#pragma omp parallel for schedule(static)
  for (long oc = 0; oc < n_o; ++oc) {
    int32_t acc = 0;
    const int8_t* row = src + (size_t)oc * per_o;
    for (size_t e = 0; e < per_o; ++e) acc += row[e];
    sum[oc] = acc;
  }
}

void RearrangeCustomI8(const int8_t* src, const PackShape& sh, const int* axes, const int* sizes_in,
                       int n, int8_t pad, int8_t* dst) {
  const int shape[4] = {sh.o, sh.h, sh.w, sh.i};
  int sizes[16];
  int total[4] = {1, 1, 1, 1};
  for (int g = 0; g < n; ++g) {
    int sz = sizes_in[g];
    if (sz <= 0) sz = DivUpI(shape[axes[g]], total[axes[g]]);
    sizes[g] = sz;
    total[axes[g]] *= sz;
  }
  const long count = (long)total[0] * total[1] * total[2] * total[3];
#pragma omp parallel for schedule(static)
  for (long e = 0; e < count; ++e) {
    long rem = e;
    int coord[4] = {0, 0, 0, 0}, radix[4] = {1, 1, 1, 1};
    for (int g = 0; g < n; ++g) {
      const int digit = (int)(rem % sizes[g]);
      rem /= sizes[g];
      coord[axes[g]] += digit * radix[axes[g]];
      radix[axes[g]] *= sizes[g];
    }
    const bool in = coord[0] < sh.o && coord[1] < sh.h && coord[2] < sh.w && coord[3] < sh.i;
    dst[e] = in ? src[(((size_t)coord[0] * sh.h + coord[1]) * sh.w + coord[2]) * sh.i + coord[3]] : pad;
  }
}

}  // namespace mldhip
