// KIVI-style FlagRot INT2 pages for gfx950: per-token value writer, per-(32-token group, KV head) key encoder,
// page dequantiser and the bf16 LSE merge.  Compiled with -ffp-contract=off: the quantiser (scale, codes,
// reconstruction) rounds every operation on its own, as the reference's (integrations/vllm_flagrot/csrc/kivi.cu:94-125).
//
// Page chunk per (16-token page, KV head), D = 128: KC @0 [16][32] key codes (32-bit words of 16 channels, channel i at
// bit 2 (i >> 1) + 16 (i & 1)) | KM @512 [16][4] (fp16 scale, fp16 min) of the token's GROUP: cell i = position % 32
// holds channels [4 i, 4 i + 4) | VC @768 [16][32] value codes (byte c / 4, bits 2 (c % 4)) | VM @1280 [16][4]
// (fp16 scale with sign = H32, fp16 min) | VF @1536 [16] u8 (value uses H_128).  Key flags: scale sign of channel
// j < 4 = sub-vector j is H32; of channel 4 = whole head H_128.
//
// FP8-meta pages (F8; kivi.cu:28-35, 84-88, 123-128): scale and min are rounded to E4M3 (nearest even, saturating at
// +-448) BEFORE the codes are computed, so the codes belong to the stored values.  Chunk of 1280 bytes: KC @0 | KM8 @512
// [16][4] byte pairs (s8 | flag << 7, m8) | VC @640 | VM8 @1152 [16][4] byte pairs (bit 7 of s8 = H32).  Key flags: bit 7
// of the scale byte of channel 4 j (slot 0 of cell j) = sub-vector j is H32, of channel 16 (slot 0 of cell 4) = whole
// head.  Bit 7 of the KEY scale byte in slot 3 of a cell is the whole-head flag of the VALUE row stored in that cell: the
// value writer sets it with a byte read-modify-write, the key encoder keeps what it finds there.
//
// One half wave (32 lanes) owns a 128-d row, 4 channels per lane (the helpers of fr_common.hpp).
#include "fr_common.hpp"
#include "kivi_launch.hpp"
#include "kivi_quant.hpp"
#include "kivi_vrow.hpp"

namespace frkv {
using namespace fr;
namespace {

template <bool F8> constexpr long long CHUNK = F8 ? 1280 : 1552;
template <bool F8> constexpr int VC_AT = F8 ? 640 : 768;
template <bool F8> constexpr int VM_AT = F8 ? 1152 : 1280;

// ------------------------------------------------------------------------------------------------ value writer
// Half wave per (token, KV head): the three trials, the picks, the stores (kivi_vrow.hpp has the per-row work; the
// kernel loads the row and knows where the chunk keeps what).  WMAT: the picks weigh the miss vectors by a full matrix
// per head (kivi.cu:213-287) and need an LDS strip per half wave; `ident` stores the row as it is, `vfix` takes the
// picks from a word per head (bits 0..3: H32 per sub-vector, bit 16: whole head).
template <bool F8, bool WMAT>
__global__ void __launch_bounds__(256) k_v_write(const uint16_t* __restrict__ kv, long long kv_rs, int n, int Hkv,
                                                 const long long* __restrict__ slots, const float* __restrict__ co,
                                                 const float* __restrict__ M, uint8_t* __restrict__ pool, int ident,
                                                 const int* __restrict__ vfix) {
  __shared__ float strips[WMAT ? 8 : 1][WMAT ? 3 * 128 : 1];
  const int l32 = threadIdx.x & 31;
  const long long item = static_cast<long long>(blockIdx.x) * 8 + (threadIdx.x >> 5);
  if (item >= static_cast<long long>(n) * Hkv) return;
  const int t = static_cast<int>(item / Hkv), h = static_cast<int>(item % Hkv);
  const long long slot = slots[t];
  if (slot < 0) return;
  const uint2 raw = *reinterpret_cast<const uint2*>(kv + static_cast<long long>(t) * kv_rs + (Hkv + h) * 128 + 4 * l32);
  const float x[1][4] = {{bf16_lo(raw.x), bf16_hi(raw.x), bf16_lo(raw.y), bf16_hi(raw.y)}};
  vrow::Trial<1> tr[3];
  vrow::trial_in_basis<1, vrow::AS_STORED, F8>(x, l32, tr[0]);
  vrow::trial_in_basis<1, vrow::BLOCK32, F8>(x, l32, tr[1]);
  vrow::trial_in_basis<1, vrow::WHOLE, F8>(x, l32, tr[2]);
  const int j = l32 >> 3;
  vrow::Picks pk{0u, false};
  if (ident) {
  } else if (vfix != nullptr) {
    pk.whole = (vfix[h] >> 16) & 1;
    pk.block32 = (vfix[h] >> j) & 1u;
  } else if constexpr (WMAT) {
    pk = vrow::pick_matrix<1>(tr, M + static_cast<long long>(h) * 128 * 128, strips[threadIdx.x >> 5], l32);
  } else {
    const float4 c4 = *reinterpret_cast<const float4*>(co + h * 128 + 4 * l32);
    const float w[1][4] = {{c4.x, c4.y, c4.z, c4.w}};
    pk = vrow::pick_diagonal<1>(tr, w, l32);
  }
  const int basis = vrow::basis_of<1>(pk, 0);
  uint8_t* chunk = pool + ((slot / 16) * Hkv + h) * CHUNK<F8>;
  const int off = static_cast<int>(slot % 16);
  chunk[VC_AT<F8> + off * 32 + l32] = static_cast<uint8_t>(vrow::chosen_byte<1>(tr, basis, 0));
  if ((l32 & 7) == 0) {
    const uint32_t meta = vrow::chosen_meta<1, F8>(tr, basis, 0);
    if (F8) *reinterpret_cast<uint16_t*>(chunk + VM_AT<true> + off * 8 + 2 * j) = static_cast<uint16_t>(meta);
    else *reinterpret_cast<uint32_t*>(chunk + VM_AT<false> + off * 16 + 4 * j) = meta;
  }
  if (l32 == 0) {
    if (F8) {                                            // bit 7 of the key scale byte in slot 3 of this token's cell
      uint8_t* kb = chunk + 512 + off * 8 + 6;
      *kb = static_cast<uint8_t>((*kb & 0x7Fu) | (pk.whole ? 0x80u : 0u));
    } else chunk[1536 + off] = pk.whole ? 1 : 0;
  }
}

// ------------------------------------------------------------------------------------------------ key group encoder
constexpr int LD = 132;                                   // padded row of 128 floats
constexpr int QT = 8;                                     // calibration queries per tile
struct KEnc {
  float xs[32][LD];
  float es[3][32][LD];
  float qt[QT][LD];
  float lzt[QT];
  float par[3][2][128];                                   // per candidate (min, scale) per channel
  float red[4][12];
  int valid[32];
  int choice[5];
  float ef;
};

template <bool F8>
__global__ void __launch_bounds__(256) k_k_encode(const uint16_t* __restrict__ src, long long src_rs,
                                                  const uint16_t* __restrict__ src2, long long src2_rs,
                                                  const long long* __restrict__ sidx, const long long* __restrict__ dslot,
                                                  int Hkv, const float* __restrict__ qs, const float* __restrict__ lz,
                                                  int NQ, float qsc, uint8_t* __restrict__ pool, int ident,
                                                  const int* __restrict__ kfix) {
  extern __shared__ __align__(16) uint8_t lds[];
  KEnc& S = *reinterpret_cast<KEnc*>(lds);
  const int item = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, hw = tid >> 5, l32 = tid & 31;
  const long long* si = sidx + static_cast<long long>(item) * 32;
  const long long* ds = dslot + static_cast<long long>(item) * 32;
  if (ds[0] < 0) return;
  if (tid < 32) S.valid[tid] = si[tid] != -1;
  __syncthreads();
  for (int e = tid; e < 32 * 128; e += 256) {
    const int t = e >> 7, c = e & 127;
    const long long r = si[t];
    float v = 0.f;
    if (r >= 0) v = bf16_lo(src[r * src_rs + h * 128 + c]);
    else if (r <= -2) v = bf16_lo(src2[(-r - 2) * src2_rs + h * 128 + c]);
    S.xs[t][c] = v;
  }
  __syncthreads();
  // candidates in their bases: one half wave per token
  for (int t = hw; t < 32; t += 8) {
    const float4 xv = *reinterpret_cast<const float4*>(&S.xs[t][4 * l32]);
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      float y[4] = {xv.x, xv.y, xv.z, xv.w};
      if (c == 1) fwht<32>(y, l32);
      if (c == 2) fwht<128>(y, l32);
      *reinterpret_cast<float4*>(&S.es[c][t][4 * l32]) = make_float4(y[0], y[1], y[2], y[3]);
    }
  }
  __syncthreads();
  // per (candidate, channel): range over the valid tokens, parameters, reconstruction in place
  for (int e = tid; e < 3 * 128; e += 256) {
    const int c = e >> 7, ch = e & 127;
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
    if (tid < 5) S.choice[tid] = 0;
  } else if (kfix != nullptr) {
    if (tid < 5) S.choice[tid] = tid < 4 ? (kfix[h] >> tid) & 1 : (kfix[h] >> 16) & 1;
  } else {
    // errors e = rec - x in the original basis (0 for tokens outside the group)
    for (int t = hw; t < 32; t += 8) {
      const float4 xv = *reinterpret_cast<const float4*>(&S.xs[t][4 * l32]);
      const float xx[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
      for (int c = 0; c < 3; ++c) {
        const float4 yv = *reinterpret_cast<const float4*>(&S.es[c][t][4 * l32]);
        float y[4] = {yv.x, yv.y, yv.z, yv.w};
        if (c == 1) fwht<32>(y, l32);
        if (c == 2) fwht<128>(y, l32);
        const bool v = S.valid[t];
        *reinterpret_cast<float4*>(&S.es[c][t][4 * l32]) =
            make_float4(v ? y[0] - xx[0] : 0.f, v ? y[1] - xx[1] : 0.f, v ? y[2] - xx[2] : 0.f, v ? y[3] - xx[3] : 0.f);
      }
    }
    __syncthreads();
    // thread <-> (token t, query slot qi of the tile)
    const int t = tid & 31, qi = tid >> 5;
    const bool tv = S.valid[t];
    const float* qh = qs + static_cast<long long>(h) * NQ * 128;
    const float* lzh = lz + static_cast<long long>(h) * NQ;
    for (int pass = 0; pass < 2; ++pass) {
      float accI[4] = {0.f, 0.f, 0.f, 0.f}, accH[4] = {0.f, 0.f, 0.f, 0.f}, accF = 0.f, accB = 0.f;
      for (int q0 = 0; q0 < NQ; q0 += QT) {
        __syncthreads();
        for (int e = tid; e < QT * 128; e += 256) {
          const int qq = e >> 7, c = e & 127;
          S.qt[qq][c] = q0 + qq < NQ ? qh[static_cast<long long>(q0 + qq) * 128 + c] : 0.f;
        }
        if (tid < QT) S.lzt[tid] = q0 + tid < NQ ? lzh[q0 + tid] : 0.f;
        __syncthreads();
        float lg = 0.f;
        for (int c = 0; c < 128; ++c) lg += S.xs[t][c] * S.qt[qi][c];
        const float w = (tv && q0 + qi < NQ) ? fminf(expf(qsc * lg - S.lzt[qi]), 1.f) : 0.f;
        if (pass == 0) {
          float pf = 0.f;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            float p0 = 0.f, p1 = 0.f;
            for (int c = 32 * j; c < 32 * j + 32; ++c) {
              const float qv = S.qt[qi][c];
              p0 += S.es[0][t][c] * qv; p1 += S.es[1][t][c] * qv; pf += S.es[2][t][c] * qv;
            }
            accI[j] += w * p0 * p0; accH[j] += w * p1 * p1;
          }
          accF += w * pf * pf;
        } else {
          float pb = 0.f;
          for (int c = 0; c < 128; ++c) pb += S.es[0][t][c] * S.qt[qi][c];
          accB += w * pb * pb;
        }
      }
      // block reduction: half waves by exchange, then the four wavefronts in order
      float v[10] = {accI[0], accI[1], accI[2], accI[3], accH[0], accH[1], accH[2], accH[3], accF, accB};
#pragma unroll
      for (int k = 0; k < 10; ++k) {
#pragma unroll
        for (int m = 1; m < 32; m <<= 1) v[k] += hx(v[k], m);
        v[k] += __shfl_xor(v[k], 32, 64);
      }
      __syncthreads();
      if ((tid & 63) == 0)
        for (int k = 0; k < 10; ++k) S.red[tid >> 6][k] = v[k];
      __syncthreads();
      if (pass == 0) {
        if (tid < 4) {
          const float a = ((S.red[0][tid] + S.red[1][tid]) + S.red[2][tid]) + S.red[3][tid];
          const float b = ((S.red[0][4 + tid] + S.red[1][4 + tid]) + S.red[2][4 + tid]) + S.red[3][4 + tid];
          S.choice[tid] = b < a ? 1 : 0;                          // identity on ties
        }
        if (tid == 32) S.ef = ((S.red[0][8] + S.red[1][8]) + S.red[2][8]) + S.red[3][8];
        __syncthreads();
        for (int e = tid; e < 32 * 128; e += 256) {               // errors of the chosen sub-vector candidates
          const int tt = e >> 7, c = e & 127;
          if (S.choice[c >> 5]) S.es[0][tt][c] = S.es[1][tt][c];
        }
      } else if (tid == 0) {
        const float b = ((S.red[0][9] + S.red[1][9]) + S.red[2][9]) + S.red[3][9];
        S.choice[4] = S.ef < b ? 1 : 0;                           // base on ties
      }
    }
  }
  __syncthreads();
  const bool useF = S.choice[4] != 0;
  // codes of the valid tokens in the chosen bases
  for (int t = hw; t < 32; t += 8) {
    if (!S.valid[t]) continue;
    const float4 xv = *reinterpret_cast<const float4*>(&S.xs[t][4 * l32]);
    float yi[4] = {xv.x, xv.y, xv.z, xv.w}, yh[4] = {xv.x, xv.y, xv.z, xv.w}, yf[4] = {xv.x, xv.y, xv.z, xv.w};
    fwht<32>(yh, l32);
    fwht<128>(yf, l32);
    const int cand = useF ? 2 : S.choice[l32 >> 3];
    uint32_t word = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = 4 * l32 + i;
      const float y = cand == 0 ? yi[i] : cand == 1 ? yh[i] : yf[i];
      const int ci = c & 15;
      word |= static_cast<uint32_t>(kv_code(y, S.par[cand][0][c], S.par[cand][1][c]) & 3) << (2 * (ci >> 1) + 16 * (ci & 1));
    }
    word |= __shfl_xor(word, 1, 32);
    word |= __shfl_xor(word, 2, 32);
    const long long slot = ds[t];
    uint8_t* chunk = pool + ((slot / 16) * Hkv + h) * CHUNK<F8>;
    if ((l32 & 3) == 0) reinterpret_cast<uint32_t*>(chunk + (slot % 16) * 32)[l32 >> 2] = word;
  }
  // meta of all 32 cells: cell i holds channels [4 i, 4 i + 4)
  for (int c = tid; c < 128; c += 256) {
    const int cand = useF ? 2 : S.choice[c >> 5];
    const long long slot = ds[c >> 2];
    if (slot < 0) continue;
    uint8_t* chunk = pool + ((slot / 16) * Hkv + h) * CHUNK<F8>;
    if (F8) {                                                     // flags at slot 0 of cells 0 .. 4
      const bool neg = (c & 3) == 0 && (c < 16 ? (!useF && S.choice[c >> 2] != 0) : (c == 16 ? useF : false));
      uint8_t* at = chunk + 512 + (slot % 16) * 8 + 2 * (c & 3);
      uint32_t sb = e4m3_bits(S.par[cand][1][c]) | (neg ? 0x80u : 0u);
      if ((c & 3) == 3) sb |= at[0] & 0x80u;                      // the value row's whole-head flag lives here
      *reinterpret_cast<uint16_t*>(at) = static_cast<uint16_t>(sb | (e4m3_bits(S.par[cand][0][c]) << 8));
    } else {
      uint32_t sb = f16_bits_rn(S.par[cand][1][c]) & 0x7FFFu;
      const bool neg = c < 4 ? (!useF && S.choice[c] != 0) : (c == 4 ? useF : false);
      if (neg) sb |= 0x8000u;
      reinterpret_cast<uint32_t*>(chunk + 512 + (slot % 16) * 16)[c & 3] = sb | (f16_bits_rn(S.par[cand][0][c]) << 16);
    }
  }
}

// ------------------------------------------------------------------------------------------------ dequantiser
template <typename OT> DEVI OT cvt_out(float v);
template <> DEVI float cvt_out<float>(float v) { return v; }
template <> DEVI uint16_t cvt_out<uint16_t>(float v) { return static_cast<uint16_t>(bf16_rn(v)); }

template <typename OT, bool F8>
__global__ void __launch_bounds__(256) k_dequant(const uint8_t* __restrict__ pool, const int* __restrict__ bt, int g0,
                                                 int Hkv, int nvalid, OT* __restrict__ ok, OT* __restrict__ ov) {
  const int gi = blockIdx.x, h = blockIdx.y, hw = threadIdx.x >> 5, l32 = threadIdx.x & 31;
  const int g = g0 + gi;
  const uint8_t* chA = pool + (static_cast<long long>(bt[2 * g]) * Hkv + h) * CHUNK<F8>;
  const uint8_t* chB = pool + (static_cast<long long>(bt[2 * g + 1]) * Hkv + h) * CHUNK<F8>;
  uint32_t lm = 0;
  bool kF;
  float ks[4], kmn[4];
  // this lane's channels [4 l32, 4 l32 + 4) = key cell l32
  if (F8) {
    for (int j = 0; j < 4; ++j) lm |= static_cast<uint32_t>(chA[512 + 8 * j] >> 7) << j;
    kF = chA[512 + 8 * 4] >> 7;
    const uint8_t* km = (l32 < 16 ? chA : chB) + 512 + (l32 & 15) * 8;
#pragma unroll
    for (int i = 0; i < 4; ++i) { ks[i] = e4m3_value(km[2 * i] & 0x7Fu); kmn[i] = e4m3_value(km[2 * i + 1]); }
  } else {
    const uint32_t* m0 = reinterpret_cast<const uint32_t*>(chA + 512);
    for (int j = 0; j < 4; ++j) lm |= ((m0[j] >> 15) & 1u) << j;
    kF = (m0[4] >> 15) & 1u;                                    // cell 1, slot 0
    const uint32_t* km = reinterpret_cast<const uint32_t*>((l32 < 16 ? chA : chB) + 512 + (l32 & 15) * 16);
#pragma unroll
    for (int i = 0; i < 4; ++i) { ks[i] = f16_value(km[i] & 0x7FFFu); kmn[i] = f16_value(km[i] >> 16); }
  }
  const int j = l32 >> 3;
  for (int t = hw; t < 32; t += 8) {
    const long long o = static_cast<long long>(gi) * 32 + t;
    const uint8_t* ch = t < 16 ? chA : chB;
    const int cell = t & 15;
    // keys
    {
      const uint32_t w = reinterpret_cast<const uint32_t*>(ch + cell * 32)[l32 >> 2];
      float x[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int ci = (4 * l32 + i) & 15;
        x[i] = static_cast<float>((w >> (2 * (ci >> 1) + 16 * (ci & 1))) & 3u) * ks[i] + kmn[i];
      }
      if (kF) fwht<128>(x, l32);
      else if (lm) {
        float y[4] = {x[0], x[1], x[2], x[3]};
        fwht<32>(y, l32);
        if ((lm >> j) & 1u) { x[0] = y[0]; x[1] = y[1]; x[2] = y[2]; x[3] = y[3]; }
      }
      if (o < nvalid)
#pragma unroll
        for (int i = 0; i < 4; ++i) ok[(o * Hkv + h) * 128 + 4 * l32 + i] = cvt_out<OT>(x[i]);
    }
    // values
    {
      uint32_t l = 0;
      bool f;
      float vs, vmn;
      if (F8) {
        const uint8_t* vm = ch + VM_AT<true> + cell * 8;
        for (int jj = 0; jj < 4; ++jj) l |= static_cast<uint32_t>(vm[2 * jj] >> 7) << jj;
        f = ch[512 + cell * 8 + 6] >> 7;
        vs = e4m3_value(vm[2 * j] & 0x7Fu); vmn = e4m3_value(vm[2 * j + 1]);
      } else {
        const uint32_t* vm = reinterpret_cast<const uint32_t*>(ch + VM_AT<false> + cell * 16);
        for (int jj = 0; jj < 4; ++jj) l |= ((vm[jj] >> 15) & 1u) << jj;
        f = ch[1536 + cell] != 0;
        vs = f16_value(vm[j] & 0x7FFFu); vmn = f16_value(vm[j] >> 16);
      }
      const uint32_t byte = ch[VC_AT<F8> + cell * 32 + l32];
      float x[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = static_cast<float>((byte >> (2 * i)) & 3u) * vs + vmn;
      // The two tokens of a wavefront may differ in their flags: the stages H32 and H128 share (distance 1 .. 16 channels
      // first, in H128's own order) run once for both, H128 adds its two stages across the sub-vectors.
      if (f || l) {
        float y[4] = {x[0], x[1], x[2], x[3]};
        butterflies<32>(y, l32);
        if (f) {
#pragma unroll
          for (int lm = 8; lm <= 16; lm <<= 1) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float o2 = hx(y[i], lm);
              y[i] = (l32 & lm) ? (o2 - y[i]) : (y[i] + o2);
            }
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) x[i] = y[i] * kC128;
        } else if ((l >> j) & 1u) {
#pragma unroll
          for (int i = 0; i < 4; ++i) x[i] = y[i] * kC32;
        }
      }
      if (o < nvalid)
#pragma unroll
        for (int i = 0; i < 4; ++i) ov[(o * Hkv + h) * 128 + 4 * l32 + i] = cvt_out<OT>(x[i]);
    }
  }
}

// ------------------------------------------------------------------------------------------------ LSE merge
__global__ void k_lse_merge(const uint16_t* __restrict__ oa, const float* __restrict__ la, long long la_hs,
                            const uint16_t* __restrict__ ob, const float* __restrict__ lb, long long lb_hs,
                            uint16_t* __restrict__ out, long long out_rs, int na, int H, int D) {
  const long long e = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (e >= static_cast<long long>(na) * H * D) return;
  const int c = static_cast<int>(e % D);
  const long long rh = e / D;
  const int hh = static_cast<int>(rh % H);
  const long long r = rh / H;
  float a = la[hh * la_hs + r], b = lb[hh * lb_hs + r];
  if (a == INFINITY) a = -INFINITY;
  if (b == INFINITY) b = -INFINITY;
  const float m = (a != a || b != b) ? NAN : fmaxf(a, b);
  const float wa = expf(a - m), wb = expf(b - m);
  const float va = bf16_lo(oa[(r * H + hh) * D + c]), vb = bf16_lo(ob[(r * H + hh) * D + c]);
  const float num = va * wa + vb * wb;
  out[r * out_rs + static_cast<long long>(hh) * D + c] = static_cast<uint16_t>(bf16_rn(num / (wa + wb)));
}

}  // namespace

int v_write_launch(const void* kv, long long kv_rs, int n, int Hkv, const long long* slots, const float* co, uint8_t* pool,
                   const float* M, int ident, const int* vfix, int f8, hipStream_t st) {
  const long long items = static_cast<long long>(n) * Hkv;
  const bool wmat = M != nullptr && !ident && vfix == nullptr;
  const auto kern = wmat ? (f8 ? k_v_write<true, true> : k_v_write<false, true>) : (f8 ? k_v_write<true, false> : k_v_write<false, false>);
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>((items + 7) / 8)), dim3(256), 0, st,
                     static_cast<const uint16_t*>(kv), kv_rs, n, Hkv, slots, co, M, pool, ident, vfix);
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

int k_encode_launch(const void* src, long long src_rs, const void* src2, long long src2_rs, const long long* sidx,
                    const long long* dslot, int N, int Hkv, const float* qs, const float* lz, int NQ, float qsc,
                    uint8_t* pool, int ident, const int* kfix, int f8, hipStream_t st) {
  static bool attr = false;
  if (!attr) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_k_encode<false>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(sizeof(KEnc))) != hipSuccess) return 1;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_k_encode<true>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(sizeof(KEnc))) != hipSuccess) return 1;
    attr = true;
  }
  const auto kern = f8 ? k_k_encode<true> : k_k_encode<false>;
  hipLaunchKernelGGL(kern, dim3(N, Hkv), dim3(256), sizeof(KEnc), st, static_cast<const uint16_t*>(src), src_rs,
                     static_cast<const uint16_t*>(src2), src2_rs, sidx, dslot, Hkv, qs, lz, NQ, qsc, pool, ident, kfix);
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

int dequant_launch(const uint8_t* pool, const int* bt, int g0, int g1, int nvalid, int Hkv, int fp32, void* ok, void* ov,
                   int f8, hipStream_t st) {
  dim3 grid(g1 - g0, Hkv);
  if (fp32) {
    const auto kern = f8 ? k_dequant<float, true> : k_dequant<float, false>;
    hipLaunchKernelGGL(kern, grid, dim3(256), 0, st, pool, bt, g0, Hkv, nvalid, static_cast<float*>(ok), static_cast<float*>(ov));
  } else {
    const auto kern = f8 ? k_dequant<uint16_t, true> : k_dequant<uint16_t, false>;
    hipLaunchKernelGGL(kern, grid, dim3(256), 0, st, pool, bt, g0, Hkv, nvalid, static_cast<uint16_t*>(ok), static_cast<uint16_t*>(ov));
  }
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

int lse_merge_launch(const void* oa, const float* la, long long la_hs, const void* ob, const float* lb, long long lb_hs,
                     void* out, long long out_rs, int na, int H, int D, hipStream_t st) {
  const long long tot = static_cast<long long>(na) * H * D;
  hipLaunchKernelGGL(k_lse_merge, dim3(static_cast<unsigned>((tot + 255) / 256)), dim3(256), 0, st,
                     static_cast<const uint16_t*>(oa), la, la_hs, static_cast<const uint16_t*>(ob), lb, lb_hs,
                     static_cast<uint16_t*>(out), out_rs, na, H, D);
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

}  // namespace frkv
