// Exact fp16 unpacking of FlagRot page codes (gfx950), shared by the decode and the multi-query prefill kernels.
//
// A 32-bit word of eight 4-bit fields f0..f7 (or, INT2, the 2-bit fields at bit 4 n of a pre-shifted word) becomes
// four fp16 pairs (f0,f4) (f1,f5) (f2,f6) (f3,f7): the field is or-ed into the mantissa of 1024.0 (exact), then
// -(1024 + zero point) is added with one packed fp16 add, which is exact too: the pairs hold code - zero point.
#pragma once
#include "fr_common.hpp"

namespace fr {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

DEVI half2_t as_h2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
DEVI uint32_t pk_add(uint32_t a, uint32_t b) { return __builtin_bit_cast(uint32_t, as_h2(a) + as_h2(b)); }
DEVI uint32_t pk_mul(uint32_t a, uint32_t b) { return __builtin_bit_cast(uint32_t, as_h2(a) * as_h2(b)); }

template <int QM> struct Unpack;
// MAGIC (the fp16 pattern of 1024.0 twice) is kept in a register the compiler cannot constant-fold, so that
// (w & mask) | MAGIC is a single v_and_or_b32 (one literal per instruction).
struct Consts { uint32_t magic; };
DEVI Consts make_consts() {
  Consts c;
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(c.magic));
  return c;
}
template <> struct Unpack<QM_ASYM4> {
  static DEVI void run(uint32_t w, const uint32_t (&nz)[4], const Consts& c, uint32_t (&x)[4]) {
    x[0] = pk_add((w & 0x000F000Fu) | c.magic, nz[0]);
    x[1] = pk_add(((w >> 4) & 0x000F000Fu) | c.magic, nz[1]);
    x[2] = pk_add(((w >> 8) & 0x000F000Fu) | c.magic, nz[2]);
    x[3] = pk_add(((w >> 12) & 0x000F000Fu) | c.magic, nz[3]);
  }
};
template <> struct Unpack<QM_ASYM2> {
  static DEVI void run(uint32_t w, const uint32_t (&nz)[4], const Consts& c, uint32_t (&x)[4]) {  // fields at bits 0, 2, 8, 10 (+16)
    x[0] = pk_add((w & 0x00030003u) | c.magic, nz[0]);
    x[1] = pk_add(((w >> 2) & 0x00030003u) | c.magic, nz[1]);
    x[2] = pk_add(((w >> 8) & 0x00030003u) | c.magic, nz[2]);
    x[3] = pk_add(((w >> 10) & 0x00030003u) | c.magic, nz[3]);
  }
};
template <> struct Unpack<QM_SYM4> {  // sign-magnitude bytes s0000mmm -> exact signed fp16
  static DEVI uint32_t pair(uint32_t bytes02, const Consts& c) {  // bytes at bits 0..7 and 16..23
    const uint32_t m = pk_add((bytes02 & 0x00070007u) | c.magic, 0xE400E400u);
    return m ^ ((bytes02 & 0x00800080u) << 8);
  }
  static DEVI void run(uint32_t w, const uint32_t (&)[4], const Consts& c, uint32_t (&x)[4]) {
    const uint32_t a = w & 0x87878787u;                                   // A_i in byte i
    const uint32_t b = ((w << 4) | (w >> 28)) & 0x87878787u;              // B_i in byte i
    x[0] = pair(a, c); x[1] = pair(b, c); x[2] = pair(a >> 8, c); x[3] = pair(b >> 8, c);
  }
};
// Denormal form: a code field masked IN PLACE inside the low 10 bits of an fp16 half is a denormal whose value is
// code * 2^(position - 24), exactly; v_dot2_f32_f16 takes denormal inputs at full precision.  The four pairs come out as
// (f0,f4) (f1,f5) (f2,f6) (f3,f7) like above, but pairs 1 and 3 carry the factor 2^SH (SH = field width) and every pair the
// factor 2^-24: the other operand of the contraction is pre-scaled by 2^-SH in those slots, the sum by 2^24, and the zero
// point is removed through sums of that other operand (sum(c - z) q = sum c q - z sum q).
template <int QM> struct UnpackD;
template <> struct UnpackD<QM_ASYM4> {
  static constexpr int SH = 4;
  static DEVI void run(uint32_t w, uint32_t (&x)[4]) {
    const uint32_t t = w >> 8;
    x[0] = w & 0x000F000Fu; x[1] = w & 0x00F000F0u; x[2] = t & 0x000F000Fu; x[3] = t & 0x00F000F0u;
  }
};
template <> struct UnpackD<QM_ASYM2> {   // fields at bits 0, 2, 8, 10 (+16) of the word
  static constexpr int SH = 2;
  static constexpr int HI = 4;             // run_hi: the fields 4 bits higher (the other group / sub-vector of the word)
  static DEVI void run(uint32_t w, uint32_t (&x)[4]) {
    const uint32_t t = w >> 8;
    x[0] = w & 0x00030003u; x[1] = w & 0x000C000Cu; x[2] = t & 0x00030003u; x[3] = t & 0x000C000Cu;
  }
  // still inside the 10 mantissa bits: every pair carries the extra factor 2^HI, which the caller folds into the
  // scale of the sum instead of shifting the word first
  static DEVI void run_hi(uint32_t w, uint32_t (&x)[4]) {
    const uint32_t t = w >> 8;
    x[0] = w & 0x00300030u; x[1] = w & 0x00C000C0u; x[2] = t & 0x00300030u; x[3] = t & 0x00C000C0u;
  }
};
template <> struct UnpackD<QM_SYM4> {    // sign-magnitude bytes s....mmm -> signed denormals (no extra factor)
  static constexpr int SH = 0;
  // A byte doubled into both bytes of an fp16 half has its magnitude bits in the mantissa (low copy) and its sign bit
  // on the sign (high copy): one byte permute and one mask per pair.
  static DEVI uint32_t pair(uint32_t w, uint32_t sel) { return __builtin_amdgcn_perm(w, w, sel) & 0x80078007u; }
  static DEVI void run(uint32_t w, uint32_t (&x)[4]) {
    const uint32_t b = __builtin_amdgcn_alignbit(w, w, 28);               // B_i (magnitude, sign) in byte i like A_i
    x[0] = pair(w, 0x02020000u); x[1] = pair(b, 0x02020000u); x[2] = pair(w, 0x03030101u); x[3] = pair(b, 0x03030101u);
  }
  // Key side: the odd bytes are left where they are.  Bits 8..10 of an fp16 half are the top two mantissa bits and the
  // lowest exponent bit, and a pattern below 2^11 still reads code * 2^(position - 24) (exponent field 0 and 1 share one
  // scale), the byte's bit 7 is the half's sign already: one mask per pair, the pairs carrying 2^8 (KODD) that the query
  // operand is divided by.  7 instructions per word.  (Not for the value side: there the factor would sit on p.)
  static constexpr int KODD = 8;
  static DEVI void run_k(uint32_t w, uint32_t (&x)[4]) {
    const uint32_t b = __builtin_amdgcn_alignbit(w, w, 28);
    x[0] = pair(w, 0x02020000u); x[1] = pair(b, 0x02020000u); x[2] = w & 0x87008700u; x[3] = b & 0x87008700u;
  }
};
// the key words of a format, and the power of two element (isB, i) of a lane's four comes out of them with (group g)
template <int QM> DEVI void unpack_key(uint32_t w, uint32_t (&x)[4]) {
  if constexpr (QM == QM_SYM4) UnpackD<QM>::run_k(w, x); else UnpackD<QM>::run(w, x);
}
template <int QM> DEVI float key_field_factor(int isB, int g, int i) {
  if constexpr (QM == QM_SYM4) return (i & 1) ? static_cast<float>(1 << UnpackD<QM>::KODD) : 1.f;
  else return (isB ? static_cast<float>(1 << UnpackD<QM>::SH) : 1.f) * ((QM == QM_ASYM2 && (g & 1)) ? 16.f : 1.f);
}
// fp16 pattern of -(1024 + z)
DEVI uint32_t negz16(uint32_t z) { return 0xE400u | z; }

}  // namespace fr
