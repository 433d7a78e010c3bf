// KIVI-style FlagRot INT2 pages at head dim 256 for gfx950: value writer, key group encoder, page dequantiser and the
// decode attention with its split merge (integrations/vllm_flagrot/csrc/kivi.cu:163-328 k_v_write<256>, :343-663
// k_k_encode<256>, :2067-2300 the dequantisers, :1997-2036 the 256-d attention launches).  Compiled with
// -ffp-contract=off like the 128-d writers: the quantiser rounds every operation on its own.
//
// Page chunk per (16-token page, KV head), D = 256, NV = 8 sub-vectors (kivi.cu:15-35):
//   FP16 meta, 3088 bytes: KC @0 [16][64] key codes (32-bit words of 16 channels, channel i at bit 2 (i >> 1) +
//     16 (i & 1)) | KM @1024 [16][8] (fp16 scale, fp16 min) of the token's GROUP: cell i = position % 32 holds channels
//     [8 i, 8 i + 8) | VC @1536 [16][64] value codes | VM @2560 [16][8] (fp16 scale with sign = H32, fp16 min) |
//     VF @3072 [16] u8 (value uses H_256).  Key flags: scale sign of channel j < 8 = sub-vector j is H32, of channel 8 =
//     whole head H_256.
//   FP8 meta, 2560 bytes: KC @0 | KM8 @1024 [16][8] byte pairs | VC @1280 | VM8 @2304 [16][8] byte pairs.  Key flags:
//     bit 7 of the scale byte of channel 8 j (slot 0 of cell j), of channel 64 (slot 0 of cell 8) = whole head; bit 7 of
//     the key scale byte in slot 7 of a cell = whole-head flag of the VALUE row stored in that cell.
//
// A half wave (32 lanes) owns a 256-d row as two 128-d halves: lane l holds channels 128 s + 4 l + i (s = 0, 1), so the
// 32-blocks and the 128-d butterflies are the helpers of fr_common.hpp on each half, and H_256 adds the stage of
// distance 128 between the two registers of a lane and the exact factor 1/16.  The staged butterflies meet their
// partners in the reference's order (distance 1, 2, 4, ..), so every transformed value is the reference's bit for bit.
//
// The attention kernel here is the plain fp32 form (no matrix cores): per 32-token group, scores by (token, sub-vector)
// threads against the three rotated queries, one softmax per head in a half wave, values by channel threads into one
// accumulator per (head, basis), the two inverse transforms once at the end.  It runs only when
// FLAGROT_KIVI_WIDE_PLAIN=1 asks for it: the launches go through the matrix-pipe kernel of kivi_decode_wide.hip.
// Same partials either way, one merge kernel.
#include <cstdlib>

#include "fr_common.hpp"
#include "kivi_launch.hpp"
#include "kivi_merge.hpp"
#include "kivi_quant.hpp"
#include "kivi_vrow.hpp"

namespace frkv {
using namespace fr;
namespace {

constexpr int D2 = 256, NV2 = 8;
template <bool F8> constexpr long long CHUNK2 = F8 ? 2560 : 3088;
constexpr int KM2 = 1024;
template <bool F8> constexpr int VC2 = F8 ? 1280 : 1536;
template <bool F8> constexpr int VM2 = F8 ? 2304 : 2560;
constexpr int VF2 = 3072;
template <bool F8> constexpr int CELL = F8 ? 16 : 32;                 // bytes of meta per cell (8 entries)

template <int C> DEVI void to_basis2(float (&y)[2][4], int l32) {     // candidate 0 identity, 1 H32, 2 H256 (involutions)
  if (C == 1) { fwht<32>(y[0], l32); fwht<32>(y[1], l32); }
  if (C == 2) h256(y, l32);
}
DEVI void load_row(const uint16_t* row, int l32, float (&x)[2][4]) {  // bf16 row of 256
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const uint2 raw = *reinterpret_cast<const uint2*>(row + 128 * s + 4 * l32);
    x[s][0] = bf16_lo(raw.x); x[s][1] = bf16_hi(raw.x); x[s][2] = bf16_lo(raw.y); x[s][3] = bf16_hi(raw.y);
  }
}
template <bool F8> DEVI void meta_read(const uint8_t* at, float& s, float& mn, bool& flag) {   // one (scale, min) entry
  if (F8) { flag = at[0] >> 7; s = e4m3_value(at[0] & 0x7Fu); mn = e4m3_value(at[1]); }
  else {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(at);
    flag = (w >> 15) & 1u; s = f16_value(w & 0x7FFFu); mn = f16_value(w >> 16);
  }
}
template <bool F8> DEVI bool value_whole(const uint8_t* chunk, int cell) {
  return F8 ? (chunk[KM2 + cell * 16 + 14] >> 7) != 0 : chunk[VF2 + cell] != 0;
}

// ------------------------------------------------------------------------------------------------ value writer
// Half wave per (token, KV head), the row as two halves of 128 channels: the three trials, the picks, the stores
// (kivi_vrow.hpp has the per-row work).  WMAT: picks by a full 256 x 256 matrix per head (kivi.cu:213-287) through an
// LDS strip per half wave; `vfix` bits 0..7: H32 per sub-vector, bit 16: whole head.
template <bool F8, bool WMAT>
__global__ void __launch_bounds__(256) k_v_write256(const uint16_t* __restrict__ kv, long long kv_rs, int n, int Hkv,
                                                    const long long* __restrict__ slots, const float* __restrict__ co,
                                                    const float* __restrict__ M, uint8_t* __restrict__ pool, int ident,
                                                    const int* __restrict__ vfix) {
  __shared__ float strips[WMAT ? 8 : 1][WMAT ? 3 * D2 : 1];
  const int l32 = threadIdx.x & 31;
  const long long item = static_cast<long long>(blockIdx.x) * 8 + (threadIdx.x >> 5);
  if (item >= static_cast<long long>(n) * Hkv) return;
  const int t = static_cast<int>(item / Hkv), h = static_cast<int>(item % Hkv);
  const long long slot = slots[t];
  if (slot < 0) return;
  float x[2][4];
  load_row(kv + static_cast<long long>(t) * kv_rs + static_cast<long long>(Hkv + h) * D2, l32, x);
  vrow::Trial<2> tr[3];
  vrow::trial_in_basis<2, vrow::AS_STORED, F8>(x, l32, tr[0]);
  vrow::trial_in_basis<2, vrow::BLOCK32, F8>(x, l32, tr[1]);
  vrow::trial_in_basis<2, vrow::WHOLE, F8>(x, l32, tr[2]);
  const int j = l32 >> 3;
  vrow::Picks pk{0u, false};
  if (ident) {
  } else if (vfix != nullptr) {
    pk.whole = (vfix[h] >> 16) & 1;
    pk.block32 = ((vfix[h] >> j) & 1u) | (((vfix[h] >> (4 + j)) & 1u) << 1);
  } else if constexpr (WMAT) {
    pk = vrow::pick_matrix<2>(tr, M + static_cast<long long>(h) * D2 * D2, strips[threadIdx.x >> 5], l32);
  } else {
    float w[2][4];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const float4 c4 = *reinterpret_cast<const float4*>(co + h * D2 + 128 * s + 4 * l32);
      w[s][0] = c4.x; w[s][1] = c4.y; w[s][2] = c4.z; w[s][3] = c4.w;
    }
    pk = vrow::pick_diagonal<2>(tr, w, l32);
  }
  uint8_t* chunk = pool + ((slot / 16) * Hkv + h) * CHUNK2<F8>;
  const int off = static_cast<int>(slot % 16);
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const int basis = vrow::basis_of<2>(pk, s);
    chunk[VC2<F8> + off * 64 + 32 * s + l32] = static_cast<uint8_t>(vrow::chosen_byte<2>(tr, basis, s));
    if ((l32 & 7) == 0) {
      const uint32_t meta = vrow::chosen_meta<2, F8>(tr, basis, s);
      const int jj = 4 * s + j;
      if (F8) *reinterpret_cast<uint16_t*>(chunk + VM2<true> + off * 16 + 2 * jj) = static_cast<uint16_t>(meta);
      else *reinterpret_cast<uint32_t*>(chunk + VM2<false> + off * 32 + 4 * jj) = meta;
    }
  }
  if (l32 == 0) {
    if (F8) {                                              // bit 7 of the key scale byte in slot 7 of this token's cell
      uint8_t* kb = chunk + KM2 + off * 16 + 14;
      *kb = static_cast<uint8_t>((*kb & 0x7Fu) | (pk.whole ? 0x80u : 0u));
    } else chunk[VF2 + off] = pk.whole ? 1 : 0;
  }
}

// ------------------------------------------------------------------------------------------------ key group encoder
constexpr int LD2 = 260;                                  // padded row of 256 floats
constexpr int QT2 = 8;                                    // calibration queries per tile
struct KEnc2 {
  float xs[32][LD2];
  float es[3][32][LD2];
  float qt[QT2][LD2];
  float lzt[QT2];
  float par[3][2][D2];                                    // per candidate (min, scale) per channel
  float red[4][20];
  int valid[32];
  int choice[9];                                          // sub-vectors 0..7: H32; [8]: whole head
  float ef;
};

DEVI void lds_row(const float* row, int l32, float (&x)[2][4]) {
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const float4 v = *reinterpret_cast<const float4*>(row + 128 * s + 4 * l32);
    x[s][0] = v.x; x[s][1] = v.y; x[s][2] = v.z; x[s][3] = v.w;
  }
}
DEVI void lds_put(float* row, int l32, const float (&x)[2][4]) {
#pragma unroll
  for (int s = 0; s < 2; ++s) *reinterpret_cast<float4*>(row + 128 * s + 4 * l32) = make_float4(x[s][0], x[s][1], x[s][2], x[s][3]);
}

template <bool F8>
__global__ void __launch_bounds__(256) k_k_encode256(const uint16_t* __restrict__ src, long long src_rs,
                                                     const uint16_t* __restrict__ src2, long long src2_rs,
                                                     const long long* __restrict__ sidx, const long long* __restrict__ dslot,
                                                     int Hkv, const float* __restrict__ qs, const float* __restrict__ lz,
                                                     int NQ, float qsc, uint8_t* __restrict__ pool, int ident,
                                                     const int* __restrict__ kfix) {
  extern __shared__ __align__(16) uint8_t lds[];
  KEnc2& S = *reinterpret_cast<KEnc2*>(lds);
  const int item = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, hw = tid >> 5, l32 = tid & 31;
  const long long* si = sidx + static_cast<long long>(item) * 32;
  const long long* ds = dslot + static_cast<long long>(item) * 32;
  if (ds[0] < 0) return;
  if (tid < 32) S.valid[tid] = si[tid] != -1;
  __syncthreads();
  for (int e = tid; e < 32 * D2; e += 256) {
    const int t = e >> 8, c = e & 255;
    const long long r = si[t];
    float v = 0.f;
    if (r >= 0) v = bf16_lo(src[r * src_rs + h * D2 + c]);
    else if (r <= -2) v = bf16_lo(src2[(-r - 2) * src2_rs + h * D2 + c]);
    S.xs[t][c] = v;
  }
  __syncthreads();
  // candidates in their bases: one half wave per token
  for (int t = hw; t < 32; t += 8) {
    float xv[2][4];
    lds_row(S.xs[t], l32, xv);
    lds_put(S.es[0][t], l32, xv);
    float y[2][4];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) y[s][i] = xv[s][i];
    to_basis2<1>(y, l32);
    lds_put(S.es[1][t], l32, y);
    to_basis2<2>(xv, l32);
    lds_put(S.es[2][t], l32, xv);
  }
  __syncthreads();
  // per (candidate, channel): range over the valid tokens, parameters, reconstruction in place
  for (int e = tid; e < 3 * D2; e += 256) {
    const int c = e >> 8, ch = e & 255;
    float mn = INFINITY, mx = -INFINITY;
    for (int t = 0; t < 32; ++t)
      if (S.valid[t]) { const float v = S.es[c][t][ch]; mn = fminf(mn, v); mx = fmaxf(mx, v); }
    float s = kv_scale(mn, mx);
    kv_params<F8>(mn, s);
    S.par[c][0][ch] = mn; S.par[c][1][ch] = s;
    for (int t = 0; t < 32; ++t)
      if (S.valid[t]) S.es[c][t][ch] = kv_rec(kv_code(S.es[c][t][ch], mn, s), mn, s);
  }
  __syncthreads();
  if (ident) {
    if (tid < 9) S.choice[tid] = 0;
  } else if (kfix != nullptr) {
    if (tid < 9) S.choice[tid] = tid < 8 ? (kfix[h] >> tid) & 1 : (kfix[h] >> 16) & 1;
  } else {
    // errors e = rec - x in the original basis (0 for tokens outside the group)
    for (int t = hw; t < 32; t += 8) {
      float xx[2][4];
      lds_row(S.xs[t], l32, xx);
      const bool v = S.valid[t];
#pragma unroll
      for (int c = 0; c < 3; ++c) {
        float y[2][4];
        lds_row(S.es[c][t], l32, y);
        if (c == 1) to_basis2<1>(y, l32);
        if (c == 2) to_basis2<2>(y, l32);
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int i = 0; i < 4; ++i) y[s][i] = v ? y[s][i] - xx[s][i] : 0.f;
        lds_put(S.es[c][t], l32, y);
      }
    }
    __syncthreads();
    // thread <-> (token t, query slot qi of the tile)
    const int t = tid & 31, qi = tid >> 5;
    const bool tv = S.valid[t];
    const float* qh = qs + static_cast<long long>(h) * NQ * D2;
    const float* lzh = lz + static_cast<long long>(h) * NQ;
    for (int pass = 0; pass < 2; ++pass) {
      float acc[18];                                      // [0..7] identity, [8..15] H32 per sub-vector, [16] whole, [17] base
#pragma unroll
      for (int k = 0; k < 18; ++k) acc[k] = 0.f;
      for (int q0 = 0; q0 < NQ; q0 += QT2) {
        __syncthreads();
        for (int e = tid; e < QT2 * D2; e += 256) {
          const int qq = e >> 8, c = e & 255;
          S.qt[qq][c] = q0 + qq < NQ ? qh[static_cast<long long>(q0 + qq) * D2 + c] : 0.f;
        }
        if (tid < QT2) S.lzt[tid] = q0 + tid < NQ ? lzh[q0 + tid] : 0.f;
        __syncthreads();
        float lg = 0.f;
        for (int c = 0; c < D2; ++c) lg += S.xs[t][c] * S.qt[qi][c];
        const float w = (tv && q0 + qi < NQ) ? fminf(expf(qsc * lg - S.lzt[qi]), 1.f) : 0.f;
        if (pass == 0) {
          float pf = 0.f;
#pragma unroll
          for (int j = 0; j < NV2; ++j) {
            float p0 = 0.f, p1 = 0.f;
            for (int c = 32 * j; c < 32 * j + 32; ++c) {
              const float qv = S.qt[qi][c];
              p0 += S.es[0][t][c] * qv; p1 += S.es[1][t][c] * qv; pf += S.es[2][t][c] * qv;
            }
            acc[j] += w * p0 * p0; acc[8 + j] += w * p1 * p1;
          }
          acc[16] += w * pf * pf;
        } else {
          float pb = 0.f;
          for (int c = 0; c < D2; ++c) pb += S.es[0][t][c] * S.qt[qi][c];
          acc[17] += w * pb * pb;
        }
      }
      // block reduction: half waves by exchange, then the four wavefronts in order
#pragma unroll
      for (int k = 0; k < 18; ++k) {
#pragma unroll
        for (int m = 1; m < 32; m <<= 1) acc[k] += hx(acc[k], m);
        acc[k] += __shfl_xor(acc[k], 32, 64);
      }
      __syncthreads();
      if ((tid & 63) == 0)
#pragma unroll
        for (int k = 0; k < 18; ++k) S.red[tid >> 6][k] = acc[k];
      __syncthreads();
      if (pass == 0) {
        if (tid < 8) {
          const float a = ((S.red[0][tid] + S.red[1][tid]) + S.red[2][tid]) + S.red[3][tid];
          const float b = ((S.red[0][8 + tid] + S.red[1][8 + tid]) + S.red[2][8 + tid]) + S.red[3][8 + tid];
          S.choice[tid] = b < a ? 1 : 0;                          // identity on ties
        }
        if (tid == 32) S.ef = ((S.red[0][16] + S.red[1][16]) + S.red[2][16]) + S.red[3][16];
        __syncthreads();
        for (int e = tid; e < 32 * D2; e += 256) {                // errors of the chosen sub-vector candidates
          const int tt = e >> 8, c = e & 255;
          if (S.choice[c >> 5]) S.es[0][tt][c] = S.es[1][tt][c];
        }
      } else if (tid == 0) {
        const float b = ((S.red[0][17] + S.red[1][17]) + S.red[2][17]) + S.red[3][17];
        S.choice[8] = S.ef < b ? 1 : 0;                           // base on ties
      }
    }
  }
  __syncthreads();
  const bool useF = S.choice[8] != 0;
  // codes of the valid tokens in the chosen bases
  for (int t = hw; t < 32; t += 8) {
    if (!S.valid[t]) continue;
    float yi[2][4], yh[2][4], yf[2][4];
    lds_row(S.xs[t], l32, yi);
    lds_row(S.xs[t], l32, yh);
    lds_row(S.xs[t], l32, yf);
    to_basis2<1>(yh, l32);
    to_basis2<2>(yf, l32);
    const long long slot = ds[t];
    uint8_t* chunk = pool + ((slot / 16) * Hkv + h) * CHUNK2<F8>;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int cand = useF ? 2 : S.choice[4 * s + (l32 >> 3)];
      uint32_t word = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = 128 * s + 4 * l32 + i;
        const float y = cand == 0 ? yi[s][i] : cand == 1 ? yh[s][i] : yf[s][i];
        const int ci = c & 15;
        word |= static_cast<uint32_t>(kv_code(y, S.par[cand][0][c], S.par[cand][1][c]) & 3) << (2 * (ci >> 1) + 16 * (ci & 1));
      }
      word |= __shfl_xor(word, 1, 32);
      word |= __shfl_xor(word, 2, 32);
      if ((l32 & 3) == 0) reinterpret_cast<uint32_t*>(chunk + (slot % 16) * 64)[8 * s + (l32 >> 2)] = word;
    }
  }
  // meta of all 32 cells: cell i holds channels [8 i, 8 i + 8)
  {
    const int c = tid;
    const int cand = useF ? 2 : S.choice[c >> 5];
    const long long slot = ds[c >> 3];
    if (slot >= 0) {
      uint8_t* chunk = pool + ((slot / 16) * Hkv + h) * CHUNK2<F8>;
      if (F8) {                                                     // flags at slot 0 of cells 0 .. 8
        const bool neg = (c & 7) == 0 && (c < 64 ? (!useF && S.choice[c >> 3] != 0) : (c == 64 ? useF : false));
        uint8_t* at = chunk + KM2 + (slot % 16) * 16 + 2 * (c & 7);
        uint32_t sb = e4m3_bits(S.par[cand][1][c]) | (neg ? 0x80u : 0u);
        if ((c & 7) == 7) sb |= at[0] & 0x80u;                      // the value row's whole-head flag lives here
        *reinterpret_cast<uint16_t*>(at) = static_cast<uint16_t>(sb | (e4m3_bits(S.par[cand][0][c]) << 8));
      } else {
        uint32_t sb = f16_bits_rn(S.par[cand][1][c]) & 0x7FFFu;
        const bool neg = c < 8 ? (!useF && S.choice[c] != 0) : (c == 8 ? useF : false);
        if (neg) sb |= 0x8000u;
        reinterpret_cast<uint32_t*>(chunk + KM2 + (slot % 16) * 32)[c & 7] = sb | (f16_bits_rn(S.par[cand][0][c]) << 16);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------ dequantiser
template <typename OT> DEVI OT cvt_out2(float v);
template <> DEVI float cvt_out2<float>(float v) { return v; }
template <> DEVI uint16_t cvt_out2<uint16_t>(float v) { return static_cast<uint16_t>(bf16_rn(v)); }

// key flags of a group from its first page: bits 0..7 = sub-vector j is H32, bit 8 = whole head
template <bool F8> DEVI uint32_t key_flags(const uint8_t* chA) {
  uint32_t f = 0;
  if (F8) {
    for (int j = 0; j < 9; ++j) f |= static_cast<uint32_t>(chA[KM2 + 16 * j] >> 7) << j;
  } else {
    const uint32_t* m0 = reinterpret_cast<const uint32_t*>(chA + KM2);           // cell 0 slots 0..7, cell 1 slot 0
    for (int j = 0; j < 9; ++j) f |= ((m0[j] >> 15) & 1u) << j;
  }
  return f;
}

template <typename OT, bool F8>
__global__ void __launch_bounds__(256) k_dequant256(const uint8_t* __restrict__ pool, const int* __restrict__ bt, int g0,
                                                    int Hkv, int nvalid, OT* __restrict__ ok, OT* __restrict__ ov) {
  const int gi = blockIdx.x, h = blockIdx.y, hw = threadIdx.x >> 5, l32 = threadIdx.x & 31;
  const int g = g0 + gi;
  const uint8_t* chA = pool + (static_cast<long long>(bt[2 * g]) * Hkv + h) * CHUNK2<F8>;
  const uint8_t* chB = pool + (static_cast<long long>(bt[2 * g + 1]) * Hkv + h) * CHUNK2<F8>;
  const uint32_t kfl = key_flags<F8>(chA);
  // this lane's key channels 128 s + 4 l32 + i: cell 16 s + (l32 >> 1) (page s), slots 4 (l32 & 1) + i
  float ks[2][4], kmn[2][4];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const uint8_t* km = (s ? chB : chA) + KM2 + (l32 >> 1) * CELL<F8> + 4 * (l32 & 1) * (F8 ? 2 : 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) { bool fl; meta_read<F8>(km + i * (F8 ? 2 : 4), ks[s][i], kmn[s][i], fl); }
  }
  const int j = l32 >> 3;
  for (int t = hw; t < 32; t += 8) {
    const long long o = static_cast<long long>(gi) * 32 + t;
    const uint8_t* ch = t < 16 ? chA : chB;
    const int cell = t & 15;
    {
      float x[2][4];
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const uint32_t w = reinterpret_cast<const uint32_t*>(ch + cell * 64)[8 * s + (l32 >> 2)];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int ci = (4 * l32 + i) & 15;
          x[s][i] = static_cast<float>((w >> (2 * (ci >> 1) + 16 * (ci & 1))) & 3u) * ks[s][i] + kmn[s][i];
        }
      }
      if ((kfl >> 8) & 1u) h256(x, l32);
      else if (kfl & 0xFFu) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          float y[4] = {x[s][0], x[s][1], x[s][2], x[s][3]};
          fwht<32>(y, l32);
          if ((kfl >> (4 * s + j)) & 1u) { x[s][0] = y[0]; x[s][1] = y[1]; x[s][2] = y[2]; x[s][3] = y[3]; }
        }
      }
      if (o < nvalid)
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int i = 0; i < 4; ++i) ok[(o * Hkv + h) * D2 + 128 * s + 4 * l32 + i] = cvt_out2<OT>(x[s][i]);
    }
    {
      const bool f = value_whole<F8>(ch, cell);
      float x[2][4];
      uint32_t l = 0;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        float vs, vmn;
        bool fl;
        meta_read<F8>(ch + VM2<F8> + cell * CELL<F8> + (4 * s + j) * (F8 ? 2 : 4), vs, vmn, fl);
        l |= (fl ? 1u : 0u) << s;
        const uint32_t byte = ch[VC2<F8> + cell * 64 + 32 * s + l32];
#pragma unroll
        for (int i = 0; i < 4; ++i) x[s][i] = static_cast<float>((byte >> (2 * i)) & 3u) * vs + vmn;
      }
      // (the butterflies exchange across the half wave: every lane runs them, the flag only selects the result)
      if (f) h256(x, l32);
      else {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          float y[4] = {x[s][0], x[s][1], x[s][2], x[s][3]};
          fwht<32>(y, l32);
          if ((l >> s) & 1u) { x[s][0] = y[0]; x[s][1] = y[1]; x[s][2] = y[2]; x[s][3] = y[3]; }
        }
      }
      if (o < nvalid)
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int i = 0; i < 4; ++i) ov[(o * Hkv + h) * D2 + 128 * s + 4 * l32 + i] = cvt_out2<OT>(x[s][i]);
    }
  }
}

// ------------------------------------------------------------------------------------------------ decode attention
constexpr int GW = 8;                                     // query heads per KV head, at most
struct WideAttn {
  float qv[3][GW][D2];                                    // query x qscale: as it is, H32 per sub-vector, H256
  float ks[D2], kmn[D2];                                  // channel (scale, min) of the current group
  float part[NV2][GW][32];                                // partial scores per sub-vector
  float pr[GW][32];                                       // probabilities of the group
  float alpha[GW];
  float vs[32][NV2], vmn[32][NV2];
  int vcls[32][NV2];                                      // basis of (token, sub-vector): 0 identity, 1 H32, 2 H256
  int kfl;
};

// One workgroup per (sequence, KV head, split).  Split sp < NS: page tokens [max(sp chunk, kv_start), min((sp + 1) chunk,
// cached)); split NS: the BF16 ring rows.  Partials: opart fp32 [G][256] unnormalised, ml fp32 [G][2] = (max, sum).
template <bool F8>
__global__ void __launch_bounds__(256) k_attn256(const uint16_t* __restrict__ q, long long q_rs,
                                                 const uint8_t* __restrict__ pool, const int* __restrict__ bt, long long bt_rs,
                                                 const int* __restrict__ cached, int kv_start, int Hkv, int G, int NS,
                                                 int chunk, float qscale, const uint16_t* __restrict__ ring,
                                                 const int* __restrict__ tail_len, const int* __restrict__ tail_idx, int T,
                                                 float* __restrict__ opart, float* __restrict__ ml) {
  extern __shared__ __align__(16) uint8_t lds[];
  WideAttn& S = *reinterpret_cast<WideAttn*>(lds);
  const int b = blockIdx.x, h = blockIdx.y, sp = blockIdx.z;
  const int tid = threadIdx.x, hw = tid >> 5, l32 = tid & 31;
  const long long pidx = (static_cast<long long>(b) * Hkv + h) * (NS + 1) + sp;
  float* op = opart + pidx * G * D2;
  float* mlp = ml + pidx * G * 2;
  const bool tail = sp == NS;
  int t0, t1;
  if (tail) { t0 = 0; t1 = tail_len != nullptr ? tail_len[b] : 0; }
  else { t0 = max(sp * chunk, kv_start); t1 = min((sp + 1) * chunk, cached[b]); }
  if (t1 <= t0) {
    if (tid < G) { mlp[2 * tid] = -INFINITY; mlp[2 * tid + 1] = 0.f; }
    return;
  }
  // rotated queries: half wave hw <-> head hw (zero rows past the group)
  {
    float x[2][4];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) x[s][i] = 0.f;
    if (hw < G) load_row(q + static_cast<long long>(b) * q_rs + (static_cast<long long>(h) * G + hw) * D2, l32, x);
    float y[2][4], z[2][4];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) { y[s][i] = x[s][i]; z[s][i] = x[s][i]; }
    to_basis2<1>(y, l32);
    to_basis2<2>(z, l32);
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) { x[s][i] *= qscale; y[s][i] *= qscale; z[s][i] *= qscale; }
    lds_put(S.qv[0][hw], l32, x);
    lds_put(S.qv[1][hw], l32, y);
    lds_put(S.qv[2][hw], l32, z);
  }
  const int* btb = bt + static_cast<long long>(b) * bt_rs;
  const uint16_t* rbase = tail ? ring + static_cast<long long>(tail_idx != nullptr ? tail_idx[b] : 0) * T * 2 * Hkv * D2 : nullptr;
  float m_run = -INFINITY, l_run = 0.f;                   // of head hw (the same in every lane of the half wave)
  float o[3][GW];                                         // channel tid, per basis and head
#pragma unroll
  for (int c = 0; c < 3; ++c)
#pragma unroll
    for (int g = 0; g < GW; ++g) o[c][g] = 0.f;
  const int g_first = t0 / 32, g_end = (t1 + 31) / 32;
  for (int grp = g_first; grp < g_end; ++grp) {
    __syncthreads();                                      // the previous group's values are done with the staged fields
    const uint8_t *chA = nullptr, *chB = nullptr;
    if (!tail) {
      chA = pool + (static_cast<long long>(btb[2 * grp]) * Hkv + h) * CHUNK2<F8>;
      chB = pool + (static_cast<long long>(btb[2 * grp + 1]) * Hkv + h) * CHUNK2<F8>;
      {                                                   // channel tid: cell tid >> 3 (page B from cell 16 on), slot tid & 7
        const int cell = tid >> 3;
        bool fl;
        meta_read<F8>((cell < 16 ? chA : chB) + KM2 + (cell & 15) * CELL<F8> + (tid & 7) * (F8 ? 2 : 4), S.ks[tid], S.kmn[tid], fl);
      }
      if (tid == 0) S.kfl = static_cast<int>(key_flags<F8>(chA));
      {                                                   // value meta of (token l32, sub-vector hw)
        const uint8_t* cht = l32 < 16 ? chA : chB;
        bool fl;
        meta_read<F8>(cht + VM2<F8> + (l32 & 15) * CELL<F8> + hw * (F8 ? 2 : 4), S.vs[l32][hw], S.vmn[l32][hw], fl);
        S.vcls[l32][hw] = value_whole<F8>(cht, l32 & 15) ? 2 : (fl ? 1 : 0);
      }
    }
    __syncthreads();
    // scores: thread (token l32, sub-vector hw)
    {
      const int pos = 32 * grp + l32;
      float acc[GW];
#pragma unroll
      for (int g = 0; g < GW; ++g) acc[g] = 0.f;
      if (tail) {
        if (pos < t1) {
          const uint16_t* row = rbase + static_cast<long long>(pos) * 2 * Hkv * D2 + static_cast<long long>(h) * D2 + 32 * hw;
          for (int c8 = 0; c8 < 4; ++c8) {
            const uint4 raw = *reinterpret_cast<const uint4*>(row + 8 * c8);
            const float kf[8] = {bf16_lo(raw.x), bf16_hi(raw.x), bf16_lo(raw.y), bf16_hi(raw.y),
                                 bf16_lo(raw.z), bf16_hi(raw.z), bf16_lo(raw.w), bf16_hi(raw.w)};
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
              for (int g = 0; g < GW; ++g) acc[g] += kf[i] * S.qv[0][g][32 * hw + 8 * c8 + i];
          }
        }
      } else {
        const int var = (S.kfl >> 8) & 1 ? 2 : (S.kfl >> hw) & 1;
        const uint8_t* cht = l32 < 16 ? chA : chB;
        const uint2 w2 = *reinterpret_cast<const uint2*>(cht + (l32 & 15) * 64 + 8 * hw);
        const float (*qr)[D2] = S.qv[var];
#pragma unroll
        for (int wi = 0; wi < 2; ++wi) {
          const uint32_t w = wi ? w2.y : w2.x;
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int c = 32 * hw + 16 * wi + i;
            const float k = static_cast<float>((w >> (2 * (i >> 1) + 16 * (i & 1))) & 3u) * S.ks[c] + S.kmn[c];
#pragma unroll
            for (int g = 0; g < GW; ++g) acc[g] += k * qr[g][c];
          }
        }
      }
#pragma unroll
      for (int g = 0; g < GW; ++g) S.part[hw][g][l32] = acc[g];
    }
    __syncthreads();
    // softmax: half wave hw <-> head hw, lane <-> token
    {
      const int pos = 32 * grp + l32;
      float sc = 0.f;
#pragma unroll
      for (int j = 0; j < NV2; ++j) sc += S.part[j][hw][l32];
      if (pos < t0 || pos >= t1) sc = -INFINITY;
      float mx = sc;
#pragma unroll
      for (int m = 1; m < 32; m <<= 1) mx = fmaxf(mx, hx(mx, m));
      const float m_new = fmaxf(m_run, mx);
      const float p = sc == -INFINITY ? 0.f : exp2f(sc - m_new);
      const float a = m_run == -INFINITY ? 0.f : exp2f(m_run - m_new);
      float ps = p;
#pragma unroll
      for (int m = 1; m < 32; m <<= 1) ps += hx(ps, m);
      l_run = l_run * a + ps;
      m_run = m_new;
      S.pr[hw][l32] = p;
      if (l32 == 0) S.alpha[hw] = m_new == -INFINITY ? 1.f : a;
    }
    __syncthreads();
    // values: thread <-> channel tid
    {
#pragma unroll
      for (int c = 0; c < 3; ++c)
#pragma unroll
        for (int g = 0; g < GW; ++g) o[c][g] *= S.alpha[g];
      const int j = tid >> 5, nrow = min(32, t1 - 32 * grp);
      for (int t = max(0, t0 - 32 * grp); t < nrow; ++t) {
        float v;
        int cls = 0;
        if (tail) v = bf16_lo(rbase[static_cast<long long>(32 * grp + t) * 2 * Hkv * D2 + static_cast<long long>(Hkv + h) * D2 + tid]);
        else {
          const uint8_t* cht = t < 16 ? chA : chB;
          const uint32_t byte = cht[VC2<F8> + (t & 15) * 64 + (tid >> 2)];
          v = static_cast<float>((byte >> (2 * (tid & 3))) & 3u) * S.vs[t][j] + S.vmn[t][j];
          cls = S.vcls[t][j];
        }
        const float v0 = cls == 0 ? v : 0.f, v1 = cls == 1 ? v : 0.f, v2 = cls == 2 ? v : 0.f;
#pragma unroll
        for (int g = 0; g < GW; ++g) {
          const float p = S.pr[g][t];
          o[0][g] += p * v0; o[1][g] += p * v1; o[2][g] += p * v2;
        }
      }
    }
  }
  // back to the original basis: the H32 and the H256 accumulators through LDS (the query rows are free now)
  __syncthreads();
#pragma unroll
  for (int c = 1; c < 3; ++c)
#pragma unroll
    for (int g = 0; g < GW; ++g) S.qv[c][g][tid] = o[c][g];
  __syncthreads();
  {
    float y[2][4], z[2][4];
    lds_row(S.qv[1][hw], l32, y);
    lds_row(S.qv[2][hw], l32, z);
    to_basis2<1>(y, l32);
    to_basis2<2>(z, l32);
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) y[s][i] += z[s][i];
    lds_put(S.qv[1][hw], l32, y);
  }
  __syncthreads();
  for (int g = 0; g < G; ++g) op[g * D2 + tid] = o[0][g] + S.qv[1][g][tid];
  if (l32 == 0 && hw < G) { mlp[2 * hw] = m_run; mlp[2 * hw + 1] = l_run; }
}

template <typename K> bool carve(K kern, size_t bytes) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                             static_cast<int>(bytes)) == hipSuccess;
}

}  // namespace

int v_write256_launch(const void* kv, long long kv_rs, int n, int Hkv, const long long* slots, const float* co, uint8_t* pool,
                      const float* M, int ident, const int* vfix, int f8, hipStream_t st) {
  const long long items = static_cast<long long>(n) * Hkv;
  const bool wmat = M != nullptr && !ident && vfix == nullptr;
  const auto kern = wmat ? (f8 ? k_v_write256<true, true> : k_v_write256<false, true>)
                         : (f8 ? k_v_write256<true, false> : k_v_write256<false, false>);
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>((items + 7) / 8)), dim3(256), 0, st, static_cast<const uint16_t*>(kv),
                     kv_rs, n, Hkv, slots, co, M, pool, ident, vfix);
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

int k_encode256_launch(const void* src, long long src_rs, const void* src2, long long src2_rs, const long long* sidx,
                       const long long* dslot, int N, int Hkv, const float* qs, const float* lz, int NQ, float qsc,
                       uint8_t* pool, int ident, const int* kfix, int f8, hipStream_t st) {
  static bool attr = false;
  if (!attr) {
    if (!carve(&k_k_encode256<false>, sizeof(KEnc2)) || !carve(&k_k_encode256<true>, sizeof(KEnc2))) return 1;
    attr = true;
  }
  const auto kern = f8 ? k_k_encode256<true> : k_k_encode256<false>;
  hipLaunchKernelGGL(kern, dim3(N, Hkv), dim3(256), sizeof(KEnc2), st, static_cast<const uint16_t*>(src), src_rs,
                     static_cast<const uint16_t*>(src2), src2_rs, sidx, dslot, Hkv, qs, lz, NQ, qsc, pool, ident, kfix);
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

int dequant256_launch(const uint8_t* pool, const int* bt, int g0, int g1, int nvalid, int Hkv, int fp32, void* ok, void* ov,
                      int f8, hipStream_t st) {
  dim3 grid(g1 - g0, Hkv);
  if (fp32) {
    const auto kern = f8 ? k_dequant256<float, true> : k_dequant256<float, false>;
    hipLaunchKernelGGL(kern, grid, dim3(256), 0, st, pool, bt, g0, Hkv, nvalid, static_cast<float*>(ok), static_cast<float*>(ov));
  } else {
    const auto kern = f8 ? k_dequant256<uint16_t, true> : k_dequant256<uint16_t, false>;
    hipLaunchKernelGGL(kern, grid, dim3(256), 0, st, pool, bt, g0, Hkv, nvalid, static_cast<uint16_t*>(ok), static_cast<uint16_t*>(ov));
  }
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

int attn256_launch(int G, const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs, const void* cached,
                   int kv_start, int B, int Hkv, int NS, int chunk, float qscale, const void* ring, const void* tail_len,
                   const void* tail_idx, int T, void* opart, void* ml, void* out, long long out_rs, int f8, hipStream_t st) {
  if (G < 1 || G > GW) return 2;
  static bool attr = false;
  if (!attr) {
    if (!carve(&k_attn256<false>, sizeof(WideAttn)) || !carve(&k_attn256<true>, sizeof(WideAttn))) return 1;
    attr = true;
  }
  // every split through the matrix-pipe kernel file (kivi_decode_wide.hip) unless FLAGROT_KIVI_WIDE_PLAIN=1 (read at
  // every call) asks for the plain kernel of this file
  const char* env = std::getenv("FLAGROT_KIVI_WIDE_PLAIN");
  if (env != nullptr && env[0] == '1') {
    const auto kern = f8 ? k_attn256<true> : k_attn256<false>;
    hipLaunchKernelGGL(kern, dim3(B, Hkv, NS + 1), dim3(256), sizeof(WideAttn), st, static_cast<const uint16_t*>(q), q_rs,
                       static_cast<const uint8_t*>(pool), static_cast<const int*>(bt), bt_rs, static_cast<const int*>(cached),
                       kv_start, Hkv, G, NS, chunk, qscale, static_cast<const uint16_t*>(ring), static_cast<const int*>(tail_len),
                       static_cast<const int*>(tail_idx), T, static_cast<float*>(opart), static_cast<float*>(ml));
    if (hipPeekAtLastError() != hipSuccess) return 1;
  } else {
    const int rc = attn_pages256_launch(G, q, q_rs, pool, bt, bt_rs, cached, kv_start, B, Hkv, NS, chunk, qscale, ring, tail_len,
                                        tail_idx, T, opart, ml, f8, st);
    if (rc) return rc;
  }
  hipLaunchKernelGGL(k_merge_parts<D2>, dim3(B, Hkv * G), dim3(256), 0, st, static_cast<const float*>(opart), static_cast<const float*>(ml),
                     Hkv, G, NS, static_cast<uint16_t*>(out), out_rs);
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

}  // namespace frkv
