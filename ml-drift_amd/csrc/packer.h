// Host-side weight packers; see packer.cpp.
#ifndef MLDHIP_PACKER_H_
#define MLDHIP_PACKER_H_

#include <stddef.h>
#include <stdint.h>

namespace mldhip {

enum { kLayoutI4O4 = 1, kLayoutO4I4 = 2, kLayout2D = 6, kLayoutCustom = 7 };

struct PackShape {
  int o, h, w, i;
};

size_t TotalElements(const PackShape& sh, int layout, int group);
size_t CustomTotalElements(const PackShape& sh, const int* axes, const int* sizes, int n);

// dst[e] = src[...] + add (mod 256), padding elements = pad.
bool RearrangeU8(const uint8_t* src, const PackShape& sh, int layout, int group, uint8_t pad,
                 int add, uint8_t* dst);
bool RearrangeInt8AsUint4(const int8_t* src, const PackShape& sh, int layout, int group, int shift,
                          unsigned pad, uint8_t* dst);
bool RearrangeUint4Packed(const uint8_t* src, const PackShape& sh, int layout, int group,
                          uint8_t* dst, int32_t* sum_i, size_t sum_len, unsigned pad_value,
                          bool swap_dims);
void WeightsSumI(const int8_t* src, const PackShape& sh, int32_t* sum);
void RearrangeCustomI8(const int8_t* src, const PackShape& sh, const int* axes, const int* sizes,
                       int n, int8_t pad, int8_t* dst);

}  // namespace mldhip

#endif  // MLDHIP_PACKER_H_
