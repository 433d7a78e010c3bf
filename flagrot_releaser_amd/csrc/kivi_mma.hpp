// Pieces shared by the two matrix-pipe decode kernels over KIVI-style pages (head dim 128: kivi_decode.hip, head dim
// 256: kivi_decode_wide.hip): packed-fp16 helpers, global loads through the global address space, and the strip
// geometry (a strip row serves 128 channels = 64 fp16 pairs; the 256-d kernel works through its head in two halves).
#pragma once
#include "fr_common.hpp"

namespace frkv {
namespace mma {
using namespace fr;

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

DEVI float dot2(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), c, false);
}
DEVI float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }
DEVI uint32_t pk_mul(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, a) * __builtin_bit_cast(half2_t, b));
}
DEVI uint32_t pk_fma(uint32_t a, uint32_t b, uint32_t c) {      // a * b + c per half, one rounding
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b),
                                                                __builtin_bit_cast(half2_t, c)));
}
DEVI uint32_t pack_rn(float a, float b) {
  half2_t v = {static_cast<_Float16>(a), static_cast<_Float16>(b)};
  return __builtin_bit_cast(uint32_t, v);
}
DEVI float ror8(float v) {      // the value of the lane 8 further in its row of 16 (row_ror:8)
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true));
}
// page and ring words: read once per launch and never written by it -- loaded with the non-temporal hint, which keeps
// streamed lines from displacing each other in the caches (a kernel that only reads a launch's pages is 11 % faster with it)
template <class T> DEVI T gload(const uint8_t* p) {
  typedef const __attribute__((address_space(1))) T* gp;
  return __builtin_nontemporal_load((gp)(p));
}
constexpr uint32_t X256 = 0x5C005C00u;                                         // fp16 pair (256, 256)
// fp16 pattern of the value scale (8.0) above which a 32-token group takes the rescaled form of its value products: up
// to there the plain form loses at most 2^-13 * 8 = 1e-3 of a token's weight per instruction, which is what the rescaled
// form leaves at a scale of 700 (unit-variance data has scales around 1.4 and reaches 2.5 in a few per cent of the groups)
constexpr uint32_t WIDE_SCALE = 0x4800u;
constexpr int GT = 8;                           // query heads per workgroup (a whole GQA group of up to 8)
constexpr int QROW = 68;                        // words per row of the query strips and tables: 64 + 4 pad (conflict-free 128-bit rows)
constexpr int PROW = 40;                        // fp16 per row of the p and code-byte strips: 32 + 8 pad

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

}  // namespace mma
}  // namespace frkv
