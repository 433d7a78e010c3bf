// The per-row work of the KIVI-style value writers, shared by the 128-d kernel (kivi_write.hip, NH = 1) and the 256-d
// kernel (kivi_wide.hip, NH = 2): a half wave owns a row as NH halves of 128 channels, lane l owns channels
// 128 s + 4 l + i.  Three steps, each a function of its own:
//   trial_in_basis   quantise the row in one basis (as stored / H32 per 32-channel sub-vector / whole-head Hadamard),
//                    reconstruct, return to the original basis: levels, (step, floor) per sub-vector, the miss vector;
//   pick_*           which basis each sub-vector takes and whether the whole head takes the Hadamard: by the diagonal
//                    weights (sum miss^2 c_o) or by a full matrix per head (miss^T M miss);
//   chosen_*         the levels and the (step, floor) pair of the basis picked.
// Include from translation units compiled with -ffp-contract=off.  What is fixed by the byte contract is the quantiser
// (kivi_quant.hpp) and the decision rule (integrations/vllm_flagrot/csrc/kivi.cu:164-328: H32 where its weighted miss
// is strictly smaller, whole head where it is strictly smaller than the combination of the sub-vector picks).
#pragma once
#include "fr_common.hpp"
#include "kivi_quant.hpp"

namespace frkv {
namespace vrow {
using namespace fr;

enum Basis { AS_STORED = 0, BLOCK32 = 1, WHOLE = 2 };

template <int NH>
struct Trial {
  float step[NH], floor[NH];        // of this lane's sub-vector in each half (the 8 lanes of a sub-vector hold the same)
  int level[NH][4];
  float miss[NH][4];                // reconstruction - row, original basis
};

struct Picks {
  unsigned block32;                 // bit s: this lane's sub-vector of half s takes H32
  bool whole;                       // the row takes the whole-head Hadamard (then block32 does not matter)
};

// the bases are involutions: the same call goes there and comes back
template <int NH, int B> DEVI void rebase(float (&y)[NH][4], int l32) {
  if constexpr (B == BLOCK32) {
#pragma unroll
    for (int s = 0; s < NH; ++s) fwht<32>(y[s], l32);
  }
  if constexpr (B == WHOLE) {
    if constexpr (NH == 1) fwht<128>(y[0], l32);
    else h256(y, l32);
  }
}

DEVI float over8(float v) { v += hx(v, 1); v += hx(v, 2); v += hx(v, 4); return v; }       // a sub-vector's 8 lanes
DEVI float over32(float v) {                                                                // the half wave
#pragma unroll
  for (int m = 1; m < 32; m <<= 1) v += hx(v, m);
  return v;
}

template <int NH, int B, bool F8>
DEVI void trial_in_basis(const float (&x)[NH][4], int l32, Trial<NH>& t) {
  float y[NH][4];
#pragma unroll
  for (int s = 0; s < NH; ++s)
#pragma unroll
    for (int i = 0; i < 4; ++i) y[s][i] = x[s][i];
  rebase<NH, B>(y, l32);
#pragma unroll
  for (int s = 0; s < NH; ++s) {
    float lo = gmin8(fminf(fminf(y[s][0], y[s][1]), fminf(y[s][2], y[s][3])));
    const float hi = gmax8(fmaxf(fmaxf(y[s][0], y[s][1]), fmaxf(y[s][2], y[s][3])));
    float st = kv_scale(lo, hi);
    kv_params<F8>(lo, st);
    t.step[s] = st; t.floor[s] = lo;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      t.level[s][i] = kv_code(y[s][i], lo, st);
      y[s][i] = kv_rec(t.level[s][i], lo, st);
    }
  }
  rebase<NH, B>(y, l32);
#pragma unroll
  for (int s = 0; s < NH; ++s)
#pragma unroll
    for (int i = 0; i < 4; ++i) t.miss[s][i] = y[s][i] - x[s][i];
}

// ---- diagonal weights: a candidate costs sum miss^2 w over the channels it covers
template <int NH>
DEVI Picks pick_diagonal(const Trial<NH> (&t)[3], const float (&w)[NH][4], int l32) {
  float cost[3][NH];
#pragma unroll
  for (int b = 0; b < 3; ++b)
#pragma unroll
    for (int s = 0; s < NH; ++s) {
      float c = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) c += t[b].miss[s][i] * t[b].miss[s][i] * w[s][i];
      cost[b][s] = c;
    }
  Picks p{0u, false};
  float combined = 0.f, whole = 0.f;
#pragma unroll
  for (int s = 0; s < NH; ++s) {
    const float plain = over8(cost[AS_STORED][s]), rot = over8(cost[BLOCK32][s]);
    const bool take = rot < plain;                       // as stored on ties
    if (take) p.block32 |= 1u << s;
    combined += take ? rot : plain;                      // the same on the 8 lanes of the sub-vector
    whole += cost[WHOLE][s];
  }
  whole = over32(whole);
  combined = over32((l32 & 7) == 0 ? combined : 0.f);   // once per sub-vector
  p.whole = whole < combined;                            // the sub-vector picks on ties
  return p;
}

// ---- matrix weights: a candidate costs miss^T M miss; a sub-vector's choice sees only its diagonal 32-block of M, the
//      whole-head candidate and the combination of the sub-vector picks see all of M.  The miss vectors go through an
//      LDS strip per half wave (float [3][128 NH]); a lane forms the products of its own 4 NH rows of M.
template <int NH>
DEVI Picks pick_matrix(const Trial<NH> (&t)[3], const float* __restrict__ Mh, float* strip, int l32) {
  constexpr int W = 128 * NH;
  const int j = l32 >> 3;
  auto put = [&](int plane, int s, const float (&v)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) strip[plane * W + 128 * s + 4 * l32 + i] = v[i];
  };
  // sum over this lane's row (128 s + 4 l32 + i) of M against columns [k0, k1) of a strip plane
  auto against = [&](int s, int i, int plane, int k0, int k1) {
    const float* row = Mh + static_cast<long long>(128 * s + 4 * l32 + i) * W;
    const float* col = strip + plane * W;
    float a = 0.f;
#pragma unroll 8
    for (int k = k0; k < k1; ++k) a += row[k] * col[k];
    return a;
  };
#pragma unroll
  for (int b = 0; b < 3; ++b)
#pragma unroll
    for (int s = 0; s < NH; ++s) put(b, s, t[b].miss[s]);
  wave_lds_sync();
  Picks p{0u, false};
  float whole = 0.f;
  bool take[NH];
#pragma unroll
  for (int s = 0; s < NH; ++s) {
    float plain = 0.f, rot = 0.f;
    const int k0 = 128 * s + 32 * j;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      plain += t[AS_STORED].miss[s][i] * against(s, i, AS_STORED, k0, k0 + 32);
      rot += t[BLOCK32].miss[s][i] * against(s, i, BLOCK32, k0, k0 + 32);
      whole += t[WHOLE].miss[s][i] * against(s, i, WHOLE, 0, W);
    }
    take[s] = over8(rot) < over8(plain);                 // as stored on ties
    if (take[s]) p.block32 |= 1u << s;
  }
  whole = over32(whole);
  wave_lds_sync();                                       // every lane has read plane 0: it takes the combination now
#pragma unroll
  for (int s = 0; s < NH; ++s)
    if (take[s]) put(AS_STORED, s, t[BLOCK32].miss[s]);
  wave_lds_sync();
  float combined = 0.f;
#pragma unroll
  for (int s = 0; s < NH; ++s)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      combined += (take[s] ? t[BLOCK32].miss[s][i] : t[AS_STORED].miss[s][i]) * against(s, i, AS_STORED, 0, W);
  p.whole = whole < over32(combined);                    // the sub-vector picks on ties
  return p;
}

// ---- what the row stores for half s once the picks are made
template <int NH> DEVI int basis_of(const Picks& p, int s) { return p.whole ? WHOLE : ((p.block32 >> s) & 1u) ? BLOCK32 : AS_STORED; }

template <int NH> DEVI uint32_t chosen_byte(const Trial<NH> (&t)[3], int b, int s) {      // the lane's four 2-bit levels
  uint32_t byte = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int lv = b == AS_STORED ? t[0].level[s][i] : b == BLOCK32 ? t[1].level[s][i] : t[2].level[s][i];
    byte |= static_cast<uint32_t>(lv & 3) << (2 * i);
  }
  return byte;
}
// the stored (step, floor) word of a sub-vector: FP16 pair with the H32 flag in the step's sign bit, or the E4M3 byte
// pair with the flag in bit 7 of the step byte
template <int NH, bool F8> DEVI uint32_t chosen_meta(const Trial<NH> (&t)[3], int b, int s) {
  const float st = b == AS_STORED ? t[0].step[s] : b == BLOCK32 ? t[1].step[s] : t[2].step[s];
  const float lo = b == AS_STORED ? t[0].floor[s] : b == BLOCK32 ? t[1].floor[s] : t[2].floor[s];
  if (F8) return e4m3_bits(st) | (b == BLOCK32 ? 0x80u : 0u) | (e4m3_bits(lo) << 8);
  return (f16_bits_rn(st) & 0x7FFFu) | (b == BLOCK32 ? 0x8000u : 0u) | (f16_bits_rn(lo) << 16);
}

}  // namespace vrow
}  // namespace frkv
