// Shared device helpers of the FlagRot gfx950 kernels: bf16 / fp16 bit conversions, half-wave (32-lane) exchange,
// the Sylvester butterflies in the reference's fp32 association, the group quantisers and the page layout offsets.
//
// A head row of 128 dims is held by one half wave (32 lanes of a 64-wide wavefront), 4 consecutive dims per lane
// (d = 4 * l + i).  Every arithmetic helper here is written so that each product, sum and quotient is rounded
// separately; translation units that include this header for a bit-exact writer are compiled with
// -ffp-contract=off.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define DEVI __device__ __forceinline__

namespace fr {

constexpr float kC32 = 0.17677669529663687f;   // fp32(1 / sqrt(32))
constexpr float kC128 = 0.08838834764831845f;  // fp32(1 / sqrt(128))

enum Fmt : int { FMT_INT4 = 4, FMT_INT4A = 5, FMT_KONLY = 6, FMT_KONLYA = 7, FMT_INT2A = 8, FMT_KONLYA2 = 9 };
enum Kind : int { KIND_KONLY = 6, KIND_KONLYA = 10, KIND_KONLYA2 = 11 };
// quantiser mode: 0 symmetric INT4 (sign-magnitude codes), 1 asymmetric INT4, 2 asymmetric INT2
enum QMode : int { QM_SYM4 = 0, QM_ASYM4 = 1, QM_ASYM2 = 2 };

DEVI float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
DEVI float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
DEVI uint32_t bf16_rn(float f) {  // round to nearest even (finite inputs)
  const uint32_t u = __float_as_uint(f);
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
// The value is pinned in a VGPR first: without that the compiler folds a preceding fp32 multiply into one
// v_fma_mixlo_f16, which rounds the exact product once to fp16 instead of fp32-then-fp16.
DEVI uint32_t f16_bits_rn(float f) {
  asm volatile("" : "+v"(f));
  const _Float16 h = static_cast<_Float16>(f);
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, h));
}
DEVI float f16_value(uint32_t bits) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits)));
}

// exchange inside a 32-lane half wave: lane ^ m.  For the distances the butterflies and trees use (1, 2, 4, 8, 16, known
// after unrolling) this is a DPP move (1, 2: quad permute; 8: rotation of the 16-lane row by 8) or a ds_swizzle (4, 16);
// any other distance goes through ds_bpermute.
DEVI float hx(float v, int m) {
  const int i = __float_as_int(v);
  if (__builtin_constant_p(m)) {
    if (m == 1) return __int_as_float(__builtin_amdgcn_update_dpp(0, i, 0xB1, 0xF, 0xF, true));
    if (m == 2) return __int_as_float(__builtin_amdgcn_update_dpp(0, i, 0x4E, 0xF, 0xF, true));
    if (m == 8) return __int_as_float(__builtin_amdgcn_update_dpp(0, i, 0x128, 0xF, 0xF, true));   // row_ror:8
    if (m == 4) return __int_as_float(__builtin_amdgcn_ds_swizzle(i, (4 << 10) | 0x1F));
    if (m == 16) return __int_as_float(__builtin_amdgcn_ds_swizzle(i, (16 << 10) | 0x1F));
  }
  return __shfl_xor(v, m, 32);
}
DEVI uint32_t hdown(uint32_t v, int n) { return __shfl_down(v, n, 32); }

// ---------------------------------------------------------------------------------------------- butterflies
// Sylvester stages with partner distance 1, 2 (inside the lane) then 4, 8, .. (across lanes), (a + b, a - b).
template <int N>  // N = 32: eight lanes per vector; N = 128: the whole half wave
DEVI void butterflies(float (&x)[4], int l32) {
  {
    const float a = x[0], b = x[1], c = x[2], d = x[3];
    x[0] = a + b; x[1] = a - b; x[2] = c + d; x[3] = c - d;
  }
  {
    const float a = x[0], b = x[1], c = x[2], d = x[3];
    x[0] = a + c; x[2] = a - c; x[1] = b + d; x[3] = b - d;
  }
#pragma unroll
  for (int lm = 1; lm < N / 4; lm <<= 1) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float o = hx(x[i], lm);
      x[i] = (l32 & lm) ? (o - x[i]) : (x[i] + o);
    }
  }
}
template <int N>
DEVI void fwht(float (&x)[4], int l32) {  // orthonormal: butterflies, then one multiply
  butterflies<N>(x, l32);
  constexpr float c = N == 32 ? kC32 : kC128;
#pragma unroll
  for (int i = 0; i < 4; ++i) x[i] = x[i] * c;
}
// orthonormal H_256 of a row that a half wave holds as two 128-d halves (lane l: dims 128 s + 4 l + i): the 128-d
// butterflies per half, the stage of distance 128 inside the lane, the exact factor 1/16 -- stages in the order of the
// smaller transforms (distance 1, 2, 4, ..), every operation rounded on its own
DEVI void h256(float (&y)[2][4], int l32) {
  butterflies<128>(y[0], l32);
  butterflies<128>(y[1], l32);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float a = y[0][i], b = y[1][i];
    y[0][i] = (a + b) * 0.0625f;
    y[1][i] = (a - b) * 0.0625f;
  }
}

// ---------------------------------------------------------------------------------------------- group statistics
DEVI float gmax8(float a) {  // over the 8 lanes of a 32-group
  a = fmaxf(a, hx(a, 1)); a = fmaxf(a, hx(a, 2)); a = fmaxf(a, hx(a, 4));
  return a;
}
DEVI float gmin8(float a) {
  a = fminf(a, hx(a, 1)); a = fminf(a, hx(a, 2)); a = fminf(a, hx(a, 4));
  return a;
}

// ---------------------------------------------------------------------------------------------- quantisers
// symmetric INT4: s = fp16(amax * fp32(1/7)), q = clamp(rne(y / s), -7, 7), 0 where s == 0
DEVI uint32_t quant_sym4(const float (&y)[4], float (&q)[4], float (&deq)[4]) {
  float am = fmaxf(fmaxf(fabsf(y[0]), fabsf(y[1])), fmaxf(fabsf(y[2]), fabsf(y[3])));
  am = gmax8(am);
  const uint32_t w = f16_bits_rn(am * (1.0f / 7.0f));
  const float s = f16_value(w);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float v = s != 0.f ? rintf(y[i] / s) : 0.f;
    v = fminf(fmaxf(v, -7.f), 7.f);
    q[i] = v;
    deq[i] = v * s;
  }
  return w;
}
template <int NB>
DEVI uint32_t scale_word(float s, uint32_t z) {  // FP16 pattern nearest to RN16(s) with the NB low bits = z
  constexpr int M = (1 << NB) - 1;
  const int h = static_cast<int>(f16_bits_rn(s));
  const int x = min(max(h - static_cast<int>(z) + (1 << (NB - 1)), 0) & ~M, 0x7C00 - (1 << NB));
  return static_cast<uint32_t>(x) + z;
}
template <int NB>
DEVI void asym_params(float mn, float mx, float& s, float& z) {
  constexpr float inv = 1.0f / static_cast<float>((1 << NB) - 1);
  s = fmaxf((mx - mn) * inv, 1e-12f);
  z = rintf(-mn / s);
}
template <int NB>
DEVI float asym_code(float y, float s, float z) {
  return fminf(fmaxf(rintf(y / s) + z, 0.f), static_cast<float>((1 << NB) - 1));
}
// asymmetric INT4 / INT2.  q, word: the stored form (range widened to include 0, zero point in the NB low bits of
// the word).  deq (optional): the error form (FP32 step, unbounded zero point) the selection errors are measured on.
template <int NB, bool WANT_DEQ>
DEVI uint32_t quant_asym(const float (&y)[4], float (&q)[4], float (&deq)[4]) {
  float mn = fminf(fminf(y[0], y[1]), fminf(y[2], y[3])), mx = fmaxf(fmaxf(y[0], y[1]), fmaxf(y[2], y[3]));
  mn = gmin8(mn);
  mx = gmax8(mx);
  float s, z;
  if (WANT_DEQ) {
    asym_params<NB>(mn, mx, s, z);
#pragma unroll
    for (int i = 0; i < 4; ++i) deq[i] = (asym_code<NB>(y[i], s, z) - z) * s;
  }
  asym_params<NB>(fminf(mn, 0.f), fmaxf(mx, 0.f), s, z);
#pragma unroll
  for (int i = 0; i < 4; ++i) q[i] = asym_code<NB>(y[i], s, z);
  return scale_word<NB>(s, static_cast<uint32_t>(z));
}
template <int QM, bool WANT_DEQ>
DEVI uint32_t quant_group(const float (&y)[4], float (&q)[4], float (&deq)[4]) {
  if constexpr (QM == QM_SYM4) return quant_sym4(y, q, deq);
  else return quant_asym<QM == QM_ASYM4 ? 4 : 2, WANT_DEQ>(y, q, deq);
}

// ---------------------------------------------------------------------------------------------- wave reductions
// xor 1 / 2 by DPP quad permutes, xor 4 / 8 / 16 by ds_swizzle, xor 32 by a wave shuffle
DEVI float dpp_xor1(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));
}
DEVI float dpp_xor2(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));
}
template <int X> DEVI float swz_xor(float v) {  // xor 4 / 8 / 16 inside a 32-lane half
  return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), (X << 10) | 0x1F));
}
DEVI float xor32(float v) { return __shfl_xor(v, 32, 64); }
DEVI float wave_max_over_tokens(float v) {  // lanes of a quad already agree
  v = fmaxf(v, swz_xor<4>(v)); v = fmaxf(v, swz_xor<8>(v)); v = fmaxf(v, swz_xor<16>(v));
  return fmaxf(v, xor32(v));
}
DEVI float wave_sum_over_tokens(float v) {
  v += swz_xor<4>(v); v += swz_xor<8>(v); v += swz_xor<16>(v);
  return v + xor32(v);
}
DEVI float wave_max64(float v) {
  v = fmaxf(v, dpp_xor1(v)); v = fmaxf(v, dpp_xor2(v));
  return wave_max_over_tokens(v);
}
DEVI float wave_sum64(float v) {
  v += dpp_xor1(v); v += dpp_xor2(v);
  return wave_sum_over_tokens(v);
}
DEVI void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------------------------------------- page layout
template <int QM, int P> struct Lay {
  static constexpr int CB = QM == QM_ASYM2 ? 32 : 64;  // code bytes per (token, K or V row)
  static constexpr int K_OFF = 0, V_OFF = CB * P, KS_OFF = 2 * CB * P, VS_OFF = 2 * CB * P + 8 * P;
  static constexpr int CHUNK = 2 * CB * P + 16 * P;
};
DEVI int vs_slot8(int pos) { const int r8 = pos & 7; return (r8 & 1) ? 4 + (r8 >> 1) : (r8 >> 1); }

// placement of one INT4 element (A or B of byte i) inside its 32-bit word
template <int QM>
DEVI void place4(uint32_t c, bool isB, int i, uint32_t& mask, uint32_t& bits) {
  if constexpr (QM == QM_ASYM4) {
    mask = (isB ? 0xF0u : 0x0Fu) << (8 * i);
    bits = c << (8 * i + (isB ? 4 : 0));
  } else {  // sign-magnitude: c = sign << 3 | magnitude
    const uint32_t s = (c >> 3) & 1u, mag = c & 7u;
    if (!isB) { mask = 0x87u << (8 * i); bits = ((s << 7) | mag) << (8 * i); }
    else {
      const int k = (i + 3) & 3;
      mask = (0x08u << (8 * i)) | (0x70u << (8 * k));
      bits = (s << (8 * i + 3)) | (mag << (8 * k + 4));
    }
  }
}

// V^T fields of one token by 32-bit atomics (tokens of a page may arrive from different waves): the lane's 4 codes
template <int QM, int P>
DEVI void store_v_codes(uint8_t* chunk, int pos, const uint32_t (&code)[4], int l32) {
  using L = Lay<QM, P>;
  const int c8 = pos >> 3, ii = (pos & 7) >> 1;
  const bool isB = pos & 1;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int dd = 4 * l32 + i;
    const int e = ((dd & 63) >> 4) * 8 + (dd & 7);
    if constexpr (QM == QM_ASYM2) {
      uint32_t* wp = reinterpret_cast<uint32_t*>(chunk + L::V_OFF + (e * (P / 8) + c8) * 8 + 4 * (dd >> 6));
      const int sh = 8 * ii + 4 * ((dd & 15) >> 3) + 2 * (isB ? 1 : 0);
      atomicAnd(wp, ~(3u << sh));
      atomicOr(wp, code[i] << sh);
    } else {
      const int sub = 2 * (dd >> 6) + ((dd & 15) >> 3);
      uint32_t* wp = reinterpret_cast<uint32_t*>(chunk + L::V_OFF + (e * (P / 8) + c8) * 16 + 4 * sub);
      uint32_t m, b;
      place4<QM>(code[i], isB, ii, m, b);
      atomicAnd(wp, ~m);
      atomicOr(wp, b);
    }
  }
}
// the V scale word of the lane's group (lanes 0, 8, 16, 24 of the half wave store)
template <int QM, int P>
DEVI void store_v_word(uint8_t* chunk, int pos, uint32_t word, int l32, bool keep_flag) {
  using L = Lay<QM, P>;
  const int g = l32 >> 3, c8 = pos >> 3;
  if ((l32 & 7) == 0) {
    const int off = L::VS_OFF + (g * P + 8 * c8 + vs_slot8(pos)) * 2;
    if (keep_flag && g == 0) {  // the low 15 bits only; bit 15 belongs to the key pass
      uint32_t* wp = reinterpret_cast<uint32_t*>(chunk + (off & ~3));
      const int sh = (off & 2) * 8;
      atomicAnd(wp, ~(0x7FFFu << sh));
      atomicOr(wp, (word & 0x7FFFu) << sh);
    } else {
      *reinterpret_cast<uint16_t*>(chunk + off) = static_cast<uint16_t>(word);
    }
  }
}
// One V^T word of an aligned run of 8 tokens (slots 8 c8 .. 8 c8 + 7 of one page), whole: word j of the run is
// (entry e = j >> 2, sub = j & 3) for the 4-bit formats, (entry e = j >> 1, half m = j & 1) for the 2-bit format;
// codes[token of the run][dim].
template <int QM, int P>
DEVI void store_v_run_word(uint8_t* chunk, int c8, int j, const uint8_t (*codes)[128]) {
  using L = Lay<QM, P>;
  if constexpr (QM == QM_ASYM2) {
    const int e = j >> 1, m = j & 1;
    uint32_t wd = 0;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int dd = 64 * m + 16 * (e >> 3) + 8 * r + (e & 7);
#pragma unroll
      for (int tk = 0; tk < 8; ++tk) wd |= static_cast<uint32_t>(codes[tk][dd]) << (8 * (tk >> 1) + 4 * r + 2 * (tk & 1));
    }
    *reinterpret_cast<uint32_t*>(chunk + L::V_OFF + (e * (P / 8) + c8) * 8 + 4 * m) = wd;
  } else {
    const int e = j >> 2, sub = j & 3;
    const int dd = 64 * (sub >> 1) + 16 * (e >> 3) + 8 * (sub & 1) + (e & 7);
    uint32_t wd = 0;
#pragma unroll
    for (int tk = 0; tk < 8; ++tk) {
      uint32_t m, b;
      place4<QM>(codes[tk][dd], (tk & 1) != 0, tk >> 1, m, b);
      wd |= b;
    }
    *reinterpret_cast<uint32_t*>(chunk + L::V_OFF + (e * (P / 8) + c8) * 16 + 4 * sub) = wd;
  }
}
// Writes one row (K or V) of one token: the lane's 4 codes (d = 4 * l32 + i) and its group's scale word.
// K rows are stored as whole words; V^T fields with 32-bit atomics (tokens of a page arrive from different waves).
// VW: 0 plain 16-bit store of the V scale word, 1 keep bit 15 of V word 0 (a concurrent key pass owns it).
template <int QM, int P>
DEVI void store_row(uint8_t* chunk, int pos, bool isv, const uint32_t (&code)[4], uint32_t word, int l32, bool keep_flag) {
  using L = Lay<QM, P>;
  const int g = l32 >> 3;
  if (!isv) {
    uint32_t cb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) cb[i] = hdown(code[i], 4);
    const int tg = l32 & 7;
    if constexpr (QM == QM_ASYM2) {
      uint32_t hw = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) hw |= (code[i] << (8 * i)) | (cb[i] << (8 * i + 2));
      const uint32_t hw1 = hdown(hw, 8);
      if (tg < 4 && !(g & 1))
        *reinterpret_cast<uint32_t*>(chunk + L::K_OFF + 32 * (pos ^ ((pos >> 1) & 2)) + 8 * tg + 4 * (g >> 1)) = hw | (hw1 << 4);
    } else {
      if (tg < 4) {
        uint32_t wd = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          uint32_t m, b;
          place4<QM>(code[i], false, i, m, b); wd |= b;
          place4<QM>(cb[i], true, i, m, b); wd |= b;
        }
        *reinterpret_cast<uint32_t*>(chunk + L::K_OFF + 64 * pos + 16 * tg + 4 * g) = wd;
      }
    }
    if ((l32 & 7) == 0) *reinterpret_cast<uint16_t*>(chunk + L::KS_OFF + 8 * pos + 2 * g) = static_cast<uint16_t>(word);
  } else {
    store_v_codes<QM, P>(chunk, pos, code, l32);
    store_v_word<QM, P>(chunk, pos, word, l32, keep_flag);
  }
}

DEVI uint32_t code_bits(float q, bool sym) {
  const int qi = static_cast<int>(q);
  return sym ? static_cast<uint32_t>(qi < 0 ? (8 | -qi) : qi) : static_cast<uint32_t>(qi);
}

}  // namespace fr
