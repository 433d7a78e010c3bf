// Paged split-K decode attention over KIVI-style FlagRot INT2 pages at head dim 256 for gfx950, both products on the
// matrix pipe: the page splits, and the BF16 ring rows as one more split (plain fp32, a wavefront per row).
//
// The design is the 128-d kernel's (kivi_decode.hip) worked through a head in halves, so that the per-wavefront LDS
// strips and the register sets keep the 128-d size and two workgroups of 4 wavefronts stay resident per CU:
//   keys     the 256 channels as two halves of 128 (half 0 = the first page's meta cells, half 1 = the second
//            page's): per half the q' * scale strips (value + remainder), the bias products and the score products
//            of the 128-d kernel, all into the same accumulators; the three query rotations (as is / H32 per
//            sub-vector / H256) are made once per workgroup per half.
//   softmax  once per group, as at 128.
//   values   the eight sub-vectors as two passes of four: per pass the class-masked scale strips, the transposed code
//            bytes and the products of the 128-d kernel into accumulators 4 pass .. 4 pass + 3 (128 accumulator
//            registers per lane: two wavefronts per SIMD).
//   end      o = accI + H32(accH) + H256(accF) per head over all 256 channels, once per workgroup.
// Page chunk (kivi.cu:15-35), FP16 meta 3088 bytes: KC @0 [16][64] | KM @1024 [16][8] cells of 8 channels | VC @1536
// [16][64] | VM @2560 [16][8] | VF @3072 [16]; FP8 meta 2560 bytes: KM8 @1024 | VC @1280 | VM8 @2304.  Key flags: FP16
// scale sign of channel j < 8 = sub-vector j is H32, of channel 8 = whole head; FP8 bit 7 of the scale byte of channel
// 8 j, of channel 64 = whole head; the value row's whole-head flag is VF (FP16) or bit 7 of the key scale byte in slot 7
// of the token's cell (FP8).  Semantics follow integrations/vllm_flagrot/csrc/kivi.cu:729-980 (k_attn, <256>).
#include "fr_common.hpp"
#include "kivi_launch.hpp"
#include "kivi_mma.hpp"

namespace frkv {
using namespace fr;
using namespace mma;
namespace {

constexpr int KMW = 1024, VFW = 3072;
template <bool F8> constexpr int CHUNKW = F8 ? 2560 : 3088;
template <bool F8> constexpr int VCW = F8 ? 1280 : 1536;
template <bool F8> constexpr int VMW = F8 ? 2304 : 2560;
constexpr int OROWW = 260;                      // floats per row of the merged accumulators: 256 + 4 pad

struct ScrW {                                   // per wavefront, rewritten for every half / pass of every 32-token group
  alignas(16) uint32_t qs[GT][QROW];            // fp16 pairs of q' * scale * 2^-shift per (head, channel pair of the half)
  alignas(16) uint32_t ql[GT][QROW];            // what the rounding of those products dropped
  alignas(16) uint32_t mn[64];                  // fp16 pair of the channel mins per channel pair of the half
  alignas(16) _Float16 pst[GT][PROW];           // p per (head, token)
  alignas(16) uint16_t vsm[3][4 * 32 + 8];      // value scale per (class, sub-vector of the pass * 32 + token), 0 off its class
  alignas(16) uint16_t vmm[3][4 * 32 + 8];      // value min likewise
  alignas(16) uint16_t vt[4][8 * PROW + 16];    // value code bytes (zero-extended) per (sub-vector of the pass, byte * PROW + token)
};
struct SmemW {
  alignas(16) uint32_t qh[3][GT][2][QROW];      // query rotations as fp16 pairs per (variant, head, half, channel pair)
  alignas(16) uint32_t qr[3][GT][2][QROW];      // their remainders
  union {
    ScrW w[4];
    float ob[3][GT][OROWW];                     // merged accumulators per class (after the page loop)
  };
  float ams[4][GT][24];                         // per wavefront: sum p * min per (head, pass, class, sub-vector of the pass)
  float mw[4][GT], lw[4][GT];
};

struct GroupRegsW {
  u32x2 ka[2], kb[2];  // per half: lane (token m = lane & 15 of page A / B, quarter kc = lane >> 4): code words 2 kc, 2 kc + 1 of the half
  u32x2 km[2];         // per half: lane = channel pair: (scale | min << 16) of channels 2 l, 2 l + 1; F8: .x = bytes (s, m, s, m)
  u32x4 vc[2];         // per pass: lane (token, hh): the token's code bytes of sub-vectors 4 pass + 2 hh, + 1
  u32x2 vm[2];         // per pass: (scale | min << 16) of those two sub-vectors; F8: .x = bytes (s, m, s, m)
  uint32_t vf;         // the token's whole-head flag: non-zero = H256
};

// The key words and the value words of a group are requested apart: each set as soon as the phase that read the
// previous group's set is over, into the same registers (one register set per wavefront instead of two).
template <bool F8>
DEVI void load_group_keys(GroupRegsW& r, const uint8_t* chA, const uint8_t* chB, int lane) {
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    r.ka[hf] = gload<u32x2>(chA + (lane & 15) * 64 + 32 * hf + 8 * (lane >> 4));
    r.kb[hf] = gload<u32x2>(chB + (lane & 15) * 64 + 32 * hf + 8 * (lane >> 4));
    // the half's 64 channel pairs are the 16 cells of one page: half 0 in the group's first page, half 1 in its second
    if (F8) r.km[hf] = u32x2{gload<uint32_t>((hf ? chB : chA) + KMW + lane * 4), 0u};
    else r.km[hf] = gload<u32x2>((hf ? chB : chA) + KMW + lane * 8);
  }
}
template <bool F8>
DEVI void load_group_values(GroupRegsW& r, const uint8_t* chA, const uint8_t* chB, int lane) {
  const int t = lane & 31, hh = lane >> 5;
  const uint8_t* cht = t < 16 ? chA : chB;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    r.vc[p] = gload<u32x4>(cht + VCW<F8> + (t & 15) * 64 + 32 * p + 16 * hh);
    if (F8) r.vm[p] = u32x2{gload<uint32_t>(cht + VMW<true> + (t & 15) * 16 + 8 * p + 4 * hh), 0u};
    else r.vm[p] = gload<u32x2>(cht + VMW<false> + (t & 15) * 32 + 16 * p + 8 * hh);
  }
  if (F8) r.vf = gload<uint8_t>(cht + KMW + (t & 15) * 16 + 14) & 0x80u;
  else r.vf = gload<uint8_t>(cht + VFW + (t & 15));
}


// The BF16 ring rows of one sequence (split index NS): rows [0, tail_len) of ring block tail_idx, K row h, V row Hkv + h,
// original basis.  A wavefront takes every fourth row, lanes own 4 dims; same partial format as the page splits.
template <int G>
DEVI void tail_split256(SmemW& S, const uint16_t* __restrict__ q, long long q_rs, const uint16_t* __restrict__ ring,
                        const int* __restrict__ tail_len, const int* __restrict__ tail_idx, int T, int Hkv, int Gq, int b, int h,
                        float qscale, float* __restrict__ op, float* __restrict__ mlp) {
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
  const int n = tail_len != nullptr ? tail_len[b] : 0;
  if (n <= 0) {
    if (tid < Gq) { mlp[2 * tid] = -INFINITY; mlp[2 * tid + 1] = 0.f; }
    return;
  }
  float qa[G][4], m[G], l[G], oa[G][4];
#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int i = 0; i < 4; ++i) qa[g][i] = oa[g][i] = 0.f;
    if (g < Gq) {
      const uint2 raw = *reinterpret_cast<const uint2*>(q + static_cast<long long>(b) * q_rs + (static_cast<long long>(h) * Gq + g) * 256 + 4 * lane);
      qa[g][0] = bf16_lo(raw.x) * qscale; qa[g][1] = bf16_hi(raw.x) * qscale;
      qa[g][2] = bf16_lo(raw.y) * qscale; qa[g][3] = bf16_hi(raw.y) * qscale;
    }
    m[g] = -INFINITY; l[g] = 0.f;
  }
  const uint16_t* rbase = ring + static_cast<long long>(tail_idx != nullptr ? tail_idx[b] : 0) * T * 2 * Hkv * 256;
  // eight rows of the wavefront in flight at a time (past the end: the last row again, skipped): a row's work is
  // short against the latency of its loads
  for (int tb = wv; tb < n; tb += 32) {
    uint2 kr[8], vr[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint16_t* row = rbase + static_cast<long long>(min(tb + 4 * i, n - 1)) * 2 * Hkv * 256;
      kr[i] = *reinterpret_cast<const uint2*>(row + h * 256 + 4 * lane);
      vr[i] = *reinterpret_cast<const uint2*>(row + (Hkv + h) * 256 + 4 * lane);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (tb + 4 * i >= n) break;
      const float k[4] = {bf16_lo(kr[i].x), bf16_hi(kr[i].x), bf16_lo(kr[i].y), bf16_hi(kr[i].y)};
      const float v[4] = {bf16_lo(vr[i].x), bf16_hi(vr[i].x), bf16_lo(vr[i].y), bf16_hi(vr[i].y)};
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float sc = wave_sum64(qa[g][0] * k[0] + qa[g][1] * k[1] + qa[g][2] * k[2] + qa[g][3] * k[3]);
        const float mn = fmaxf(m[g], sc);
        const float alpha = m[g] == -INFINITY ? 0.f : fexp2(m[g] - mn), p = fexp2(sc - mn);
        l[g] = l[g] * alpha + p;
#pragma unroll
        for (int c = 0; c < 4; ++c) oa[g][c] = oa[g][c] * alpha + p * v[c];
        m[g] = mn;
      }
    }
  }
  if (lane == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g) { S.mw[wv][g] = m[g]; S.lw[wv][g] = l[g]; }
  }
  __syncthreads();
  for (int r = 0; r < 4; ++r) {
    if (wv == r) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float M = fmaxf(fmaxf(S.mw[0][g], S.mw[1][g]), fmaxf(S.mw[2][g], S.mw[3][g]));
        const float f = m[g] == -INFINITY ? 0.f : fexp2(m[g] - M);
        float4* dst = reinterpret_cast<float4*>(&S.ob[0][g][4 * lane]);
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        if (r) acc = *dst;
        *dst = make_float4(acc.x + f * oa[g][0], acc.y + f * oa[g][1], acc.z + f * oa[g][2], acc.w + f * oa[g][3]);
      }
    }
    __syncthreads();
  }
  for (int g = wv; g < G && g < Gq; g += 4) {
    *reinterpret_cast<float4*>(op + g * 256 + 4 * lane) = *reinterpret_cast<const float4*>(&S.ob[0][g][4 * lane]);
    if (lane == 0) {
      const float M = fmaxf(fmaxf(S.mw[0][g], S.mw[1][g]), fmaxf(S.mw[2][g], S.mw[3][g]));
      float L = 0.f;
      for (int w = 0; w < 4; ++w) L += S.mw[w][g] == -INFINITY ? 0.f : fexp2(S.mw[w][g] - M) * S.lw[w][g];
      mlp[2 * g] = M; mlp[2 * g + 1] = L;
    }
  }
}

template <bool F8>
__global__ void __launch_bounds__(256, 2) k_attn_pages256(const uint16_t* __restrict__ q, long long q_rs,
                                                       const uint8_t* __restrict__ pool, const int* __restrict__ bt,
                                                       long long bt_rs, const int* __restrict__ cached, int kv_start,
                                                       int Hkv, int NS, int chunk, float qscale,
                                                       float* __restrict__ opart, float* __restrict__ ml, int Gq,
                                                       const uint16_t* __restrict__ ring, const int* __restrict__ tail_len,
                                                       const int* __restrict__ tail_idx, int T) {
  constexpr int G = GT;
  extern __shared__ __align__(16) uint8_t lds[];
  SmemW& S = *reinterpret_cast<SmemW*>(lds);
  const int b = blockIdx.x, h = blockIdx.y, sp = blockIdx.z;
  const int tid = threadIdx.x, wv = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
  const long long pidx = (static_cast<long long>(b) * Hkv + h) * (NS + 1) + sp;
  float* op = opart + pidx * Gq * 256;
  float* mlp = ml + pidx * Gq * 2;
  if (sp == NS) {
    tail_split256<G>(S, q, q_rs, ring, tail_len, tail_idx, T, Hkv, Gq, b, h, qscale, op, mlp);
    return;
  }
  const int t0 = max(sp * chunk, kv_start), t1 = min((sp + 1) * chunk, cached[b]);
  if (t1 <= t0) {
    if (tid < Gq) { mlp[2 * tid] = -INFINITY; mlp[2 * tid + 1] = 0.f; }
    return;
  }
  // query rotations: half wave per (variant, head), the row as two 128-d halves; heads past the group are zero
  for (int r = tid >> 5; r < 3 * G; r += 8) {
    const int var = r / G, g = r % G, lq = tid & 31;
    float x[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    if (g < Gq) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const uint2 raw = *reinterpret_cast<const uint2*>(q + static_cast<long long>(b) * q_rs + (static_cast<long long>(h) * Gq + g) * 256 + 128 * s + 4 * lq);
        x[s][0] = bf16_lo(raw.x); x[s][1] = bf16_hi(raw.x); x[s][2] = bf16_lo(raw.y); x[s][3] = bf16_hi(raw.y);
      }
    }
    if (var == 1) { fwht<32>(x[0], lq); fwht<32>(x[1], lq); }
    if (var == 2) h256(x, lq);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const uint32_t h01 = pack_rn(x[s][0], x[s][1]), h23 = pack_rn(x[s][2], x[s][3]);
      const uint32_t l01 = pack_rn(x[s][0] - f16_value(h01 & 0xFFFFu), x[s][1] - f16_value(h01 >> 16));
      const uint32_t l23 = pack_rn(x[s][2] - f16_value(h23 & 0xFFFFu), x[s][3] - f16_value(h23 >> 16));
      *reinterpret_cast<u32x2*>(&S.qh[var][g][s][2 * lq]) = u32x2{h01, h23};
      *reinterpret_cast<u32x2*>(&S.qr[var][g][s][2 * lq]) = u32x2{l01, l23};
    }
  }
  __syncthreads();

  ScrW& W = S.w[wv];
  // Score layout: lane = (head sn = lane & 15 (heads 8..15 repeat 0..7 and are ignored), token quarter kc = lane >> 4);
  // value layout: lane = (column vn = lane & 31 = (class vn >> 3, head vn & 7; columns 24..31 ignored), token half lane >> 5).
  const int sn = lane & 15, kc = lane >> 4, sh = sn & 7;
  const int vcl = min(l32 >> 3, 2), vh = l32 & 7;
  float m_run = -INFINITY, l_run = 0.f;
  f32x16 accv[8];                                // [sub-vector]: rows = its 32 channels, this lane's column
  f32x4 amd[2];                                  // per pass: sum p * min, rows = heads 4 kc + r, column sn = (class sn >> 2, sub-vector sn & 3)
#pragma unroll
  for (int j = 0; j < 8; ++j) {
#pragma unroll
    for (int i = 0; i < 16; ++i) accv[j][i] = 0.f;
  }
  amd[0] = f32x4{0.f, 0.f, 0.f, 0.f}; amd[1] = amd[0];
  const int* btb = bt + static_cast<long long>(b) * bt_rs;
  const int g_first = t0 / 32, g_end = (t1 + 31) / 32;
  // power of two folded into the query operand of this lane's channel pair (pair k = lane & 7 of its word):
  // fields 0..4 are masked in place (code * 2^(2k - 24)), fields 5..7 after a shift by 10 (code * 2^(2(k-5) - 24))
  const int kq = lane & 7;
  const float qfold = __uint_as_float((127u - 2u * static_cast<uint32_t>(kq < 5 ? kq : kq - 5)) << 23);
  const uint32_t vmask = 0x00030003u << (2 * (l32 & 3));      // value layout row = channel l32: field l32 & 3 of byte l32 >> 2
  const uint32_t qfold8 = pack_rn(256.f * qfold, 256.f * qfold);

  GroupRegsW cur;
  int gi = g_first + wv;
  if (gi < g_end) {
    const uint8_t* chA = pool + (static_cast<long long>(btb[2 * gi]) * Hkv + h) * CHUNKW<F8>;
    const uint8_t* chB = pool + (static_cast<long long>(btb[2 * gi + 1]) * Hkv + h) * CHUNKW<F8>;
    load_group_keys<F8>(cur, chA, chB, lane);
    load_group_values<F8>(cur, chA, chB, lane);
  }
  for (; gi < g_end; gi += 4) {
    const bool full = gi * 32 >= t0 && gi * 32 + 32 <= t1;     // every token of the group is inside the range (wave uniform)
    // the next group's pages (past the range: the range's last group again, a cache hit nobody uses)
    const int gn = min(gi + 4, g_end - 1);
    const uint8_t* const chAn = pool + (static_cast<long long>(btb[2 * gn]) * Hkv + h) * CHUNKW<F8>;
    const uint8_t* const chBn = pool + (static_cast<long long>(btb[2 * gn + 1]) * Hkv + h) * CHUNKW<F8>;
    // ---- group flags, all in the meta of half 0: sub-vector j = channel j (FP8: channel 8 j), whole head = channel 8 (FP8: 64)
    bool useF;
    uint32_t lmask = 0;
    {
      constexpr int FB = F8 ? 7 : 15;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t sj = F8 ? __builtin_amdgcn_readlane(cur.km[0].x, 4 * j)
                               : ((j & 1) ? __builtin_amdgcn_readlane(cur.km[0].y, j >> 1) : __builtin_amdgcn_readlane(cur.km[0].x, j >> 1));
        lmask |= ((sj >> FB) & 1u) << j;
      }
      const uint32_t sw = __builtin_amdgcn_readlane(cur.km[0].x, F8 ? 32 : 4);
      useF = (sw >> FB) & 1u;
    }
    f32x4 bacc = {0.f, 0.f, 0.f, 0.f}, sa0 = bacc, sa1 = bacc;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      // ---- q' * scale strips and the channel mins of this half: lane = channel pair
      {
        const u32x2 kmv = cur.km[hf];
        const int which = useF ? 2 : static_cast<int>((lmask >> (4 * hf + (lane >> 4))) & 1u);
        uint32_t spair, mpair;
        if (F8) {
          const uint32_t mb = (kmv.x >> 8) & 0x00FF00FFu;
          spair = pk_mul((kmv.x & 0x007F007Fu) << 7, qfold8);
          mpair = pk_mul(((mb & 0x007F007Fu) << 7) | ((mb & 0x00800080u) << 8), X256);
        } else {
          spair = pack_rn(f16_value(kmv.x & 0x7FFFu) * qfold, f16_value(kmv.y & 0x7FFFu) * qfold);
          mpair = (kmv.x >> 16) | (kmv.y & 0xFFFF0000u);
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const uint32_t qv = S.qh[which][g][hf][lane], qrem = S.qr[which][g][hf][lane];
          const uint32_t b1 = pk_mul(qv, spair);
          const uint32_t rem = pk_fma(qv, spair, b1 ^ 0x80008000u);        // exact: what the rounding of b1 dropped
          W.qs[g][lane] = b1;
          W.ql[g][lane] = pk_fma(qrem, spair, rem);
        }
        W.mn[lane] = mpair;
      }
      wave_lds_sync();
      const int wkc = useF ? 2 : static_cast<int>((lmask >> (4 * hf + kc)) & 1u);   // sub-vector 4 hf + kc = pairs 16 kc .. 16 kc + 15 of the half
      // ---- bias: sum q' * min of head sh over the half (every row of the product is that sum)
      // Columns 0..7 of a product take the values (of the rotation / of q' * scale), columns 8..15 the remainders: one
      // product where there would be two; the halves of a row of 16 lanes are added at the end.  Every product starts
      // from zero and the partial sums are added by the vector unit (round to nearest): the matrix pipe cuts addends
      // far below the largest one of an instruction short, and with a token in the group that is hundreds of times
      // larger than its neighbours a chain of 32 instructions through one accumulator left the scores of the whole
      // group ~5e-3 (log2 units) low.
      const uint32_t* qsel = sn < 8 ? &S.qh[wkc][sh][hf][0] : &S.qr[wkc][sh][hf][0];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const u32x4 m4 = *reinterpret_cast<const u32x4*>(&W.mn[16 * kc + 4 * s]);
        const u32x4 q0 = *reinterpret_cast<const u32x4*>(qsel + 16 * kc + 4 * s);
        const f32x4 z4 = {0.f, 0.f, 0.f, 0.f};
        const f32x4 t0_ = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, m4), __builtin_bit_cast(half8, q0), z4, 0, 0, 0);
        bacc[0] += t0_[0];
      }
      // ---- scores: rows = the 16 tokens of a page, columns = heads, the half's 128 channels in four steps of 32
      const uint32_t* bsel = sn < 8 ? &W.qs[sh][0] : &W.ql[sh][0];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const uint32_t wa = (s >> 1) ? cur.ka[hf].y : cur.ka[hf].x, wb = (s >> 1) ? cur.kb[hf].y : cur.kb[hf].x;
        u32x4 xa, xb;
        if (s & 1) {
          const uint32_t wa10 = wa >> 10, wb10 = wb >> 10;
          xa = u32x4{wa & 0x03000300u, wa10 & 0x00030003u, wa10 & 0x000C000Cu, wa10 & 0x00300030u};
          xb = u32x4{wb & 0x03000300u, wb10 & 0x00030003u, wb10 & 0x000C000Cu, wb10 & 0x00300030u};
        } else {
          xa = u32x4{wa & 0x00030003u, wa & 0x000C000Cu, wa & 0x00300030u, wa & 0x00C000C0u};
          xb = u32x4{wb & 0x00030003u, wb & 0x000C000Cu, wb & 0x00300030u, wb & 0x00C000C0u};
        }
        const u32x4 b0 = *reinterpret_cast<const u32x4*>(bsel + 16 * kc + 4 * s);
        const f32x4 z4 = {0.f, 0.f, 0.f, 0.f};
        sa0 += __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, xa), __builtin_bit_cast(half8, b0), z4, 0, 0, 0);
        sa1 += __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, xb), __builtin_bit_cast(half8, b0), z4, 0, 0, 0);
      }
      wave_lds_sync();                            // the strips are free for the other half / the next group
    }
    // the key words are read: the next group's take their registers (in flight over the softmax and the value phase)
    __builtin_amdgcn_sched_barrier(0);
    load_group_keys<F8>(cur, chAn, chBn, lane);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 4; ++i) { sa0[i] += ror8(sa0[i]); sa1[i] += ror8(sa1[i]); }      // value part + remainder part
    const float bq = (bacc[0] + ror8(bacc[0])) * qscale;
    // ---- softmax: lane = (head sh, tokens 4 kc + r of page A (columns 0..7) or of page B (columns 8..15))
    {
      // after the halves were added both column halves hold the totals: the lanes of columns 0..7 go on with page A's
      // four tokens, those of columns 8..15 with page B's
      const int pgb = sn >> 3;
      float sc[4];                       // raw accumulators: score = sc * 2^24 * qscale (a positive factor)
      const float up = 16777216.f * qscale;
#pragma unroll
      for (int i = 0; i < 4; ++i) sc[i] = pgb ? sa1[i] : sa0[i];
      if (!full) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int pos = gi * 32 + 16 * pgb + 4 * kc + i;
          sc[i] = (pos >= t0 && pos < t1) ? sc[i] : -INFINITY;
        }
      }
      float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])) * up + bq;
      if (__any(mx > m_run)) {
        mx = fmaxf(mx, ror8(mx));
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mn = fmaxf(m_run, mx);
        const float alpha = m_run == -INFINITY ? 0.f : fexp2(m_run - mn);
        m_run = mn;
        l_run *= alpha;
        const float av = __shfl(alpha, vh, 64);          // the factor of this lane's value column (head vh)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
#pragma unroll
          for (int i = 0; i < 16; ++i) accv[j][i] *= av;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float ar = __shfl(alpha, 4 * kc + r, 64);                          // rows = heads 4 kc + r (8..15 repeat 0..7)
          amd[0][r] *= ar; amd[1][r] *= ar;
        }
      }
      float p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p[i] = fexp2(__builtin_fmaf(sc[i], up, bq - m_run));
        l_run += p[i];
      }
      *reinterpret_cast<u32x2*>(&W.pst[sh][16 * pgb + 4 * kc]) = u32x2{pack_rn(p[0], p[1]), pack_rn(p[2], p[3])};
    }
    // ---- values: two passes of four sub-vectors
#pragma unroll
    for (int ps = 0; ps < 2; ++ps) {
      // value strips: lane = (token l32, half hh) serves sub-vectors 2 hh, 2 hh + 1 of the pass.  Scale and min go to the
      // strip of the token's class (0 in the other two; tokens outside the range have no class), the code bytes to byte rows.
      // Passes that hold a value scale above WIDE_SCALE (wave uniform) keep their scales times 2^-8 in the strips and
      // run a second set of value products (below, where the reason is given).
      bool wide_scales;
      {
        const int pos = gi * 32 + l32;
        const bool vF = cur.vf != 0;
        uint32_t w2[2];                                  // fp16 scale (bit 15 = H32) | fp16 min << 16 of sub-vectors 2 hh, 2 hh + 1 of the pass
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          if (F8) {
            const uint32_t b2 = jj ? cur.vm[ps].x >> 16 : cur.vm[ps].x;                // s8 | m8 << 8
            w2[jj] = pk_mul(((b2 & 0x7Fu) << 7) | ((b2 & 0x7F00u) << 15) | ((b2 & 0x8000u) << 16), X256) | ((b2 & 0x80u) << 8);
          } else w2[jj] = jj ? cur.vm[ps].y : cur.vm[ps].x;
        }
        wide_scales = __any(max(w2[0] & 0x7FFFu, w2[1] & 0x7FFFu) > WIDE_SCALE);
        const uint32_t sfold = wide_scales ? 0x1C00u : 0x3C00u;                          // fp16 2^-8 or 1
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const uint32_t w = w2[jj];
          const int j = 2 * hh + jj;
          int cls = vF ? 2 : static_cast<int>((w >> 15) & 1u);
          if (!full) cls = (pos >= t0 && pos < t1) ? cls : 3;
          const uint16_t sc16 = static_cast<uint16_t>(pk_mul(w & 0x7FFFu, sfold));
#pragma unroll
          for (int c = 0; c < 3; ++c) {
            W.vsm[c][32 * j + l32] = cls == c ? sc16 : static_cast<uint16_t>(0);
            W.vmm[c][32 * j + l32] = cls == c ? static_cast<uint16_t>(w >> 16) : static_cast<uint16_t>(0);
          }
          const uint32_t c0 = jj ? cur.vc[ps].z : cur.vc[ps].x, c1 = jj ? cur.vc[ps].w : cur.vc[ps].y;
          const uint32_t c01 = __builtin_amdgcn_perm(0u, c0, 0x0C010C00u), c23 = __builtin_amdgcn_perm(0u, c0, 0x0C030C02u);
          const uint32_t c45 = __builtin_amdgcn_perm(0u, c1, 0x0C010C00u), c67 = __builtin_amdgcn_perm(0u, c1, 0x0C030C02u);
          uint16_t* vt = &W.vt[j][l32];
          vt[0 * PROW] = static_cast<uint16_t>(c01); vt[1 * PROW] = static_cast<uint16_t>(c01 >> 16);
          vt[2 * PROW] = static_cast<uint16_t>(c23); vt[3 * PROW] = static_cast<uint16_t>(c23 >> 16);
          vt[4 * PROW] = static_cast<uint16_t>(c45); vt[5 * PROW] = static_cast<uint16_t>(c45 >> 16);
          vt[6 * PROW] = static_cast<uint16_t>(c67); vt[7 * PROW] = static_cast<uint16_t>(c67 >> 16);
        }
      }
      wave_lds_sync();
      {   // sum p * min: rows = heads, columns = (class, sub-vector of the pass), the 32 tokens in one step
        const u32x4 pa = *reinterpret_cast<const u32x4*>(&W.pst[sh][8 * kc]);
        const u32x4 mb = *reinterpret_cast<const u32x4*>(&W.vmm[min(sn >> 2, 2)][32 * (sn & 3) + 8 * kc]);
        amd[ps] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, pa), __builtin_bit_cast(half8, mb), amd[ps], 0, 0, 0);
      }
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int tk = 16 * s + 8 * hh;
        const u32x4 pr = *reinterpret_cast<const u32x4*>(&W.pst[vh][tk]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const u32x4 sv = *reinterpret_cast<const u32x4*>(&W.vsm[vcl][32 * j + tk]);
          const u32x4 by = *reinterpret_cast<const u32x4*>(&W.vt[j][(l32 >> 2) * PROW + tk]);     // (token 2 i | token 2 i + 1 << 16) per word
          const u32x4 bo = u32x4{pk_mul(pr.x, sv.x), pk_mul(pr.y, sv.y), pk_mul(pr.z, sv.z), pk_mul(pr.w, sv.w)};
          const u32x4 ao = u32x4{by.x & vmask, by.y & vmask, by.z & vmask, by.w & vmask};
          accv[4 * ps + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, ao), __builtin_bit_cast(half8, bo), accv[4 * ps + j], 0, 0, 0);
        }
      }
      // The matrix pipe aligns the addends of an instruction to the largest NOMINAL exponent (a denormal code operand
      // counts as 2^-14) and keeps 24 bits from there; a token whose p * scale is hundreds of times its neighbours'
      // lifts that window for all of them and for the accumulator.  In such passes the strips hold scale * 2^-8: the
      // products above came to 1/256 of their value, the other 255/256 follow here with the code operands times 255
      // (exact), and what the fp16 rounding of p * scale dropped with the code operands times 256.
      if (__builtin_expect(wide_scales, 0)) {
        // (read again through an offset the compiler cannot see through: recognised as the reads of the products
        // above, they would keep every operand of those in registers until here)
        int again = 0;
        asm volatile("" : "+s"(again));
        constexpr uint32_t X255 = 0x5BF85BF8u;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const int tk = 16 * s + 8 * hh + again;
          const u32x4 pr = *reinterpret_cast<const u32x4*>(&W.pst[vh][tk]);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const u32x4 sv = *reinterpret_cast<const u32x4*>(&W.vsm[vcl][32 * j + tk]);
            const u32x4 by = *reinterpret_cast<const u32x4*>(&W.vt[j][(l32 >> 2) * PROW + tk]);
            const u32x4 bo = u32x4{pk_mul(pr.x, sv.x), pk_mul(pr.y, sv.y), pk_mul(pr.z, sv.z), pk_mul(pr.w, sv.w)};
            const u32x4 br = u32x4{pk_fma(pr.x, sv.x, bo.x ^ 0x80008000u), pk_fma(pr.y, sv.y, bo.y ^ 0x80008000u),
                                   pk_fma(pr.z, sv.z, bo.z ^ 0x80008000u), pk_fma(pr.w, sv.w, bo.w ^ 0x80008000u)};
            const u32x4 ao = u32x4{by.x & vmask, by.y & vmask, by.z & vmask, by.w & vmask};
            const u32x4 a255 = u32x4{pk_mul(ao.x, X255), pk_mul(ao.y, X255), pk_mul(ao.z, X255), pk_mul(ao.w, X255)};
            const u32x4 a256 = u32x4{pk_mul(ao.x, X256), pk_mul(ao.y, X256), pk_mul(ao.z, X256), pk_mul(ao.w, X256)};
            accv[4 * ps + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a255), __builtin_bit_cast(half8, bo), accv[4 * ps + j], 0, 0, 0);
            accv[4 * ps + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a256), __builtin_bit_cast(half8, br), accv[4 * ps + j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);      // one step's operands at a time: this path is rare and must not claim registers
          }
        }
      }
      wave_lds_sync();
    }
    // ... and the value words likewise (in flight over the next group's key phase)
    __builtin_amdgcn_sched_barrier(0);
    load_group_values<F8>(cur, chAn, chBn, lane);
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- merge of the wavefronts: maxima, sums, accumulators per class (in wavefront order), inverse transforms
  {
    float lt = l_run + ror8(l_run);
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    if (lane < G) { S.mw[wv][lane] = m_run; S.lw[wv][lane] = lt; }
    if (sn < 12 && kc < 2) {
#pragma unroll
      for (int ps = 0; ps < 2; ++ps)
#pragma unroll
        for (int r = 0; r < 4; ++r) S.ams[wv][4 * kc + r][12 * ps + sn] = amd[ps][r];
    }
  }
  __syncthreads();          // every wavefront is done with its strips: the merged accumulators take their place
  float fac;
  {
    const float M = fmaxf(fmaxf(S.mw[0][vh], S.mw[1][vh]), fmaxf(S.mw[2][vh], S.mw[3][vh]));
    const float mine = S.mw[wv][vh];
    fac = mine == -INFINITY ? 0.f : fexp2(mine - M);
  }
  for (int r = 0; r < 4; ++r) {
    if (wv == r && l32 < 24) {
      float* orow = &S.ob[l32 >> 3][vh][0];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float mj = S.ams[wv][vh][12 * (j >> 2) + 4 * (l32 >> 3) + (j & 3)];
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          float4* dst = reinterpret_cast<float4*>(orow + 32 * j + 8 * i4 + 4 * hh);      // row = 8 (i >> 2) + 4 hh + (i & 3)
          float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
          if (r) acc = *dst;
          // field f = i & 3 of its byte: code * 2^(2 f - 24) was accumulated
          acc.x += fac * (accv[j][4 * i4 + 0] * 16777216.f + mj);
          acc.y += fac * (accv[j][4 * i4 + 1] * 4194304.f + mj);
          acc.z += fac * (accv[j][4 * i4 + 2] * 1048576.f + mj);
          acc.w += fac * (accv[j][4 * i4 + 3] * 262144.f + mj);
          *dst = acc;
        }
      }
    }
    __syncthreads();
  }
  for (int g = tid >> 5; g < Gq; g += 8) {
    const int lq = tid & 31;
    float yh[2][4], yf[2][4], ya[2][4];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const float4 a4 = *reinterpret_cast<const float4*>(&S.ob[0][g][128 * s + 4 * lq]);
      const float4 b4 = *reinterpret_cast<const float4*>(&S.ob[1][g][128 * s + 4 * lq]);
      const float4 c4 = *reinterpret_cast<const float4*>(&S.ob[2][g][128 * s + 4 * lq]);
      ya[s][0] = a4.x; ya[s][1] = a4.y; ya[s][2] = a4.z; ya[s][3] = a4.w;
      yh[s][0] = b4.x; yh[s][1] = b4.y; yh[s][2] = b4.z; yh[s][3] = b4.w;
      yf[s][0] = c4.x; yf[s][1] = c4.y; yf[s][2] = c4.z; yf[s][3] = c4.w;
      fwht<32>(yh[s], lq);
    }
    h256(yf, lq);
#pragma unroll
    for (int s = 0; s < 2; ++s)
      *reinterpret_cast<float4*>(op + g * 256 + 128 * s + 4 * lq) =
          make_float4(ya[s][0] + yh[s][0] + yf[s][0], ya[s][1] + yh[s][1] + yf[s][1], ya[s][2] + yh[s][2] + yf[s][2], ya[s][3] + yh[s][3] + yf[s][3]);
    if (lq == 0) {
      const float M = fmaxf(fmaxf(S.mw[0][g], S.mw[1][g]), fmaxf(S.mw[2][g], S.mw[3][g]));
      float L = 0.f;
      for (int w = 0; w < 4; ++w) L += S.mw[w][g] == -INFINITY ? 0.f : fexp2(S.mw[w][g] - M) * S.lw[w][g];
      mlp[2 * g] = M; mlp[2 * g + 1] = L;
    }
  }
}

}  // namespace

int attn_pages256_launch(int Gq, const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs,
                         const void* cached, int kv_start, int B, int Hkv, int NS, int chunk, float qscale, const void* ring,
                         const void* tail_len, const void* tail_idx, int T, void* opart, void* ml, int f8, hipStream_t st) {
  if (Gq < 1 || Gq > GT) return 2;
  static bool attr = false;
  if (!attr) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_attn_pages256<false>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(sizeof(SmemW))) != hipSuccess) return 1;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_attn_pages256<true>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(sizeof(SmemW))) != hipSuccess) return 1;
    attr = true;
  }
  const auto kern = f8 ? k_attn_pages256<true> : k_attn_pages256<false>;
  hipLaunchKernelGGL(kern, dim3(B, Hkv, NS + 1), dim3(256), sizeof(SmemW), st, static_cast<const uint16_t*>(q), q_rs,
                     static_cast<const uint8_t*>(pool), static_cast<const int*>(bt), bt_rs, static_cast<const int*>(cached),
                     kv_start, Hkv, NS, chunk, qscale, static_cast<float*>(opart), static_cast<float*>(ml), Gq,
                     static_cast<const uint16_t*>(ring), static_cast<const int*>(tail_len), static_cast<const int*>(tail_idx), T);
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

}  // namespace frkv
