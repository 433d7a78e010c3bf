// The quantiser of the KIVI-style pages, shared by the 128-d and the 256-d kernels (kivi_write.hip, kivi_wide.hip).
// Include from translation units compiled with -ffp-contract=off: every operation rounds on its own, as the
// reference's (integrations/vllm_flagrot/csrc/kivi.cu:94-128).
#pragma once
#include "fr_common.hpp"

namespace frkv {
using namespace fr;

DEVI float kv_scale(float mn, float mx) { return (mx - mn) * (1.0f / 3.0f); }
// fp32 -> E4M3 byte (1 sign, 4 exponent bits of bias 7, 3 mantissa bits, no infinities; kivi.cu:113-121): nearest even,
// saturating at +-448.  Below 2^-6 the grid is m 2^-9 (pattern = m, and m = 8 is the pattern of 2^-6); above, the fp32
// mantissa is rounded to 3 bits in place (a carry moves into the exponent, never past 448 = 1.75 2^8).
DEVI uint32_t e4m3_bits(float x) {
  const float a = fminf(fabsf(x), 448.f);
  uint32_t code;
  if (a < 0.015625f) code = static_cast<uint32_t>(rintf(a * 512.f));
  else {
    uint32_t b = __float_as_uint(a);
    b += 0x7FFFFu + ((b >> 20) & 1u);
    code = (b >> 20) - (120u << 3);
  }
  return code | ((__float_as_uint(x) >> 24) & 0x80u);
}
DEVI float e4m3_value(uint32_t b) {
  const uint32_t e = (b >> 3) & 15u, m = b & 7u;
  const float a = e == 0 ? static_cast<float>(m) * 0.001953125f : __uint_as_float(((e + 120u) << 23) | (m << 20));
  return (b & 0x80u) ? -a : a;
}
template <bool F8> DEVI void kv_params(float& mn, float& s) {         // the (min, scale) the codes are computed from
  if (F8) { mn = e4m3_value(e4m3_bits(mn)); s = e4m3_value(e4m3_bits(s)); }
}
DEVI int kv_code(float x, float mn, float s) {
  const float d = s == 0.f ? 1.f : s;
  float q = (x - mn) / d;
  q = fminf(fmaxf(q, 0.f), 3.f);
  return static_cast<int>(rintf(q));
}
DEVI float kv_rec(int code, float mn, float s) { return static_cast<float>(code) * s + mn; }

}  // namespace frkv
