// Paged KV-cache writers for gfx950: static FlagRot writer (fixed per-head flags), the selecting key-only 2x2 writer
// (per token: identity / H32 per 32-group / whole-head H128 by the C_q-weighted reconstruction error) and the
// whole-head +-1 Hadamard of flagged heads.
//
// Bit-exact contract: every fp32 product, sum and quotient is rounded on its own, in the order of the reference's
// PyTorch encoders (kernels/ref.py:22-33,151-182; kernels/codebook_ref.py:119-236; blockflag/formats.py:135-174);
// this file is compiled with -ffp-contract=off and IEEE division.
//
// Mapping: one half wave (32 lanes) owns one 128-d row, 4 consecutive dims per lane.  The selecting writer keeps the
// head's 64 KB C_q^T in LDS for the whole workgroup and walks its tokens eight rows at a time; the error vectors of
// the candidates live in a small per-half-wave LDS strip so that the fixed-order matvec reads them as broadcasts.
#include <cstdlib>

#include "fr_common.hpp"
#include "fr_launch.hpp"

namespace fr {
namespace {

DEVI void wave_lds_sync() {  // LDS hand-over between lanes of one wavefront
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

DEVI void load_row(const void* kv, long long off, float (&x)[4]) {
  const uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(kv) + off);
  x[0] = bf16_lo(raw.x); x[1] = bf16_hi(raw.x); x[2] = bf16_lo(raw.y); x[3] = bf16_hi(raw.y);
}

// ------------------------------------------------------------------------------------------------ static writer
template <int QM, int P>
__global__ void __launch_bounds__(256) k_static_write(const StaticWriteParams p) {
  using L = Lay<QM, P>;
  // workgroup = eight consecutive tokens of one head row (K or V), one per half wave
  __shared__ long long vslot[8];
  __shared__ __align__(16) uint8_t vcodes[8][128];
  const int l32 = threadIdx.x & 31, hw = threadIdx.x >> 5;
  const int H2 = 2 * p.Hkv;
  const int hr = static_cast<int>(blockIdx.x % H2);
  const int t = static_cast<int>(blockIdx.x / H2) * 8 + hw;
  long long slot = -1;
  if (t < p.T) slot = p.slots[t];
  const bool live = slot >= 0;
  const bool isv = hr >= p.Hkv;
  const int head = isv ? hr - p.Hkv : hr;
  if (!isv && !live) return;             // key rows need no hand-over between the half waves
  uint8_t* chunk = p.pool + ((live ? slot / P : 0) * p.Hkv + head) * L::CHUNK;
  const int pos = live ? static_cast<int>(slot % P) : 0;

  float x[4] = {0.f, 0.f, 0.f, 0.f};
  if (live) load_row(p.kv, static_cast<long long>(t) * p.kv_ts + hr * 128 + 4 * l32, x);
  if (p.hfull != nullptr && p.hfull[hr]) {  // whole-head +-1 Hadamard / 16, rounded to bf16 (the stored basis)
    butterflies<128>(x, l32);
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = __uint_as_float(bf16_rn(x[i] * 0.0625f) << 16);
  }
  if (p.kmu != nullptr && !isv) {
    const float4 m = *reinterpret_cast<const float4*>(p.kmu + hr * 128 + 4 * l32);
    x[0] = x[0] - m.x; x[1] = x[1] - m.y; x[2] = x[2] - m.z; x[3] = x[3] - m.w;
  }
  if (p.mask != nullptr) {
    const bool f = p.mask[hr * 4 + (l32 >> 3)] != 0;
    float y[4] = {x[0], x[1], x[2], x[3]};
    fwht<32>(y, l32);
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = f ? y[i] : x[i];
  }
  float q[4], deq[4];
  const uint32_t word = quant_group<QM, false>(x, q, deq);
  uint32_t code[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) code[i] = code_bits(q[i], QM == QM_SYM4);
  if (!isv) {
    store_row<QM, P>(chunk, pos, false, code, word, l32, false);
    return;
  }
  // value rows: an aligned run of 8 slots of one page gets its V^T words assembled in LDS and stored whole
  if (live) store_v_word<QM, P>(chunk, pos, word, l32, false);
  if (l32 == 0) vslot[hw] = slot;
  *reinterpret_cast<uint32_t*>(&vcodes[hw][4 * l32]) = code[0] | (code[1] << 8) | (code[2] << 16) | (code[3] << 24);
  __syncthreads();
  const long long s0 = vslot[0];
  bool run = s0 >= 0 && (s0 & 7) == 0;
#pragma unroll
  for (int i = 1; i < 8; ++i) run = run && vslot[i] == s0 + i;
  if (run) {
    constexpr int NWORD = QM == QM_ASYM2 ? 64 : 128;
    if (threadIdx.x < NWORD)
      store_v_run_word<QM, P>(p.pool + ((s0 / P) * p.Hkv + head) * L::CHUNK, static_cast<int>(s0 % P) >> 3, threadIdx.x, vcodes);
  } else if (live) {
    store_v_codes<QM, P>(chunk, pos, code, l32);
  }
}

// ------------------------------------------------------------------------------------------------ head Hadamard
template <int D>
__global__ void __launch_bounds__(256) k_head_fwht(const uint16_t* __restrict__ x, long long x_ts, uint16_t* out,
                                                   long long o_ts, int T, int H, const uint8_t* __restrict__ flags,
                                                   float scale) {
  const int l32 = threadIdx.x & 31;
  const long long row = static_cast<long long>(blockIdx.x) * 8 + (threadIdx.x >> 5);
  if (row >= static_cast<long long>(T) * H) return;
  const int t = static_cast<int>(row / H), h = static_cast<int>(row % H);
  const uint16_t* xr = x + static_cast<long long>(t) * x_ts + h * D;
  uint16_t* orow = out + static_cast<long long>(t) * o_ts + h * D;
  constexpr int NS = D / 128;
  uint2 raw[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) raw[s] = *reinterpret_cast<const uint2*>(xr + 128 * s + 4 * l32);
  if (!flags[h]) {
#pragma unroll
    for (int s = 0; s < NS; ++s) *reinterpret_cast<uint2*>(orow + 128 * s + 4 * l32) = raw[s];
    return;
  }
  float v[NS][4];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    v[s][0] = bf16_lo(raw[s].x); v[s][1] = bf16_hi(raw[s].x); v[s][2] = bf16_lo(raw[s].y); v[s][3] = bf16_hi(raw[s].y);
    butterflies<128>(v[s], l32);
  }
  if constexpr (NS == 2) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = v[0][i], b = v[1][i];
      v[0][i] = a + b;
      v[1][i] = a - b;
    }
  }
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    uint2 r;
    r.x = bf16_rn(v[s][0] * scale) | (bf16_rn(v[s][1] * scale) << 16);
    r.y = bf16_rn(v[s][2] * scale) | (bf16_rn(v[s][3] * scale) << 16);
    *reinterpret_cast<uint2*>(orow + 128 * s + 4 * l32) = r;
  }
}

// ------------------------------------------------------------------------------------------------ selecting writer
constexpr int K2_ROWS = 8;                                   // half waves per workgroup
constexpr int K2_LDS_C = 128 * 128 * 4;                       // C_q^T of the head
constexpr int K2_LDS = K2_LDS_C + K2_ROWS * 2 * 128 * 4;      // + error strips [row][candidate][128]

DEVI float tree128(const float (&p)[4]) {  // halving tree of a 128-vector, 4 consecutive elements per lane
  float v[4] = {p[0], p[1], p[2], p[3]};
#pragma unroll
  for (int o = 16; o > 0; o >>= 1)
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = v[i] + hx(v[i], o);
  return (v[0] + v[2]) + (v[1] + v[3]);
}
DEVI float tree32(const float (&p)[4]) {  // the same over the 32 elements held by 8 lanes
  float v[4] = {p[0], p[1], p[2], p[3]};
#pragma unroll
  for (int o = 4; o > 0; o >>= 1)
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = v[i] + hx(v[i], o);
  return (v[0] + v[2]) + (v[1] + v[3]);
}

template <int QM, int P>
__global__ void __launch_bounds__(256) k_k2_write(const K2WriteParams p, int tokens_per_wg) {
  using L = Lay<QM, P>;
  extern __shared__ __align__(16) uint8_t lds[];
  float* Cs = reinterpret_cast<float*>(lds);                   // [k][i] = C_q[i][k]
  const int hw = threadIdx.x >> 5, l32 = threadIdx.x & 31;
  float* es = reinterpret_cast<float*>(lds + K2_LDS_C) + hw * 256;  // [2][128]: base / local-I, F / local-H
  const int h = blockIdx.x;
  const int t_lo = blockIdx.y * tokens_per_wg;
  const int t_hi = min(p.T, t_lo + tokens_per_wg);
  const bool do_k = p.passes & 1, do_v = p.passes & 2;
  if (do_k) {
    const float4* src = reinterpret_cast<const float4*>(p.CT + static_cast<size_t>(h) * 128 * 128);
    float4* dst = reinterpret_cast<float4*>(Cs);
    for (int i = threadIdx.x; i < 128 * 128 / 4; i += 256) dst[i] = src[i];
  }
  __syncthreads();
  const int g = l32 >> 3;
  __shared__ long long vslot[K2_ROWS];
  __shared__ __align__(16) uint8_t vcodes[K2_ROWS][128];
  for (int tb = t_lo; tb < t_hi; tb += K2_ROWS) {      // one token per half wave; the trip count is the workgroup's
    const int t = tb + hw;
    long long slot = -1;
    if (t < t_hi) slot = p.slots[static_cast<long long>(t) * (p.slot_ph ? p.Hkv : 1) + (p.slot_ph ? h : 0)];
    const bool live = slot >= 0;
    uint8_t* chunk = p.pool + ((live ? slot / P : 0) * p.Hkv + h) * L::CHUNK;
    const int pos = live ? static_cast<int>(slot % P) : 0;
    bool key_full = false;
    if (do_k && live) {
      float x[4];
      load_row(p.kv, static_cast<long long>(t) * p.kv_ts + h * 128 + 4 * l32, x);
      if (p.kmu != nullptr) {
        const float4 m = *reinterpret_cast<const float4*>(p.kmu + h * 128 + 4 * l32);
        x[0] = x[0] - m.x; x[1] = x[1] - m.y; x[2] = x[2] - m.z; x[3] = x[3] - m.w;
      }
      // ---- local candidates: identity and H32 of every 32-group
      float qi[4], ei[4], qh[4], eh[4], y[4];
      const uint32_t wi = quant_group<QM, true>(x, qi, ei);
#pragma unroll
      for (int i = 0; i < 4; ++i) { ei[i] = ei[i] - x[i]; y[i] = x[i]; }
      fwht<32>(y, l32);
      const uint32_t wh = quant_group<QM, true>(y, qh, eh);
      fwht<32>(eh, l32);
#pragma unroll
      for (int i = 0; i < 4; ++i) eh[i] = eh[i] - x[i];
      wave_lds_sync();  // the strip may still be read by the previous token's head pass
      *reinterpret_cast<float4*>(es + 4 * l32) = make_float4(ei[0], ei[1], ei[2], ei[3]);
      *reinterpret_cast<float4*>(es + 128 + 4 * l32) = make_float4(eh[0], eh[1], eh[2], eh[3]);
      wave_lds_sync();
      float ui[4], uh[4];
      {
        const float* crow = Cs + (32 * g) * 128 + 4 * l32;   // C[4 l + i][32 g + k] at crow[k * 128 + i]
        const float* e0 = es + 32 * g;
#pragma unroll 4
        for (int k = 0; k < 32; ++k) {
          const float4 cv = *reinterpret_cast<const float4*>(crow + k * 128);
          const float a = e0[k], b = e0[128 + k];
          const float c[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float pa = c[i] * a, pb = c[i] * b;
            ui[i] = k == 0 ? pa : ui[i] + pa;
            uh[i] = k == 0 ? pb : uh[i] + pb;
          }
        }
      }
      float pi[4], ph[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { pi[i] = ei[i] * ui[i]; ph[i] = eh[i] * uh[i]; }
      const bool use_h = tree32(ph) < tree32(pi);   // strict: ties keep the identity
      float qb[4], eb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { qb[i] = use_h ? qh[i] : qi[i]; eb[i] = use_h ? eh[i] : ei[i]; }
      const uint32_t wb = use_h ? wh : wi;
      // ---- whole-head candidate
      float qf[4], ef[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = x[i];
      fwht<128>(y, l32);
      const uint32_t wf = quant_group<QM, true>(y, qf, ef);
      fwht<128>(ef, l32);
#pragma unroll
      for (int i = 0; i < 4; ++i) ef[i] = ef[i] - x[i];
      wave_lds_sync();
      *reinterpret_cast<float4*>(es + 4 * l32) = make_float4(eb[0], eb[1], eb[2], eb[3]);
      *reinterpret_cast<float4*>(es + 128 + 4 * l32) = make_float4(ef[0], ef[1], ef[2], ef[3]);
      wave_lds_sync();
      float tb[4], tf[4];
#pragma unroll 1
      for (int b = 0; b < 4; ++b) {
        float ub[4], uf[4];
        const float* crow = Cs + (32 * b) * 128 + 4 * l32;
        const float* e0 = es + 32 * b;
#pragma unroll 4
        for (int k = 0; k < 32; ++k) {
          const float4 cv = *reinterpret_cast<const float4*>(crow + k * 128);
          const float a = e0[k], f = e0[128 + k];
          const float c[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float pa = c[i] * a, pf = c[i] * f;
            ub[i] = k == 0 ? pa : ub[i] + pa;
            uf[i] = k == 0 ? pf : uf[i] + pf;
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          tb[i] = b == 0 ? ub[i] : tb[i] + ub[i];
          tf[i] = b == 0 ? uf[i] : tf[i] + uf[i];
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) { tb[i] = eb[i] * tb[i]; tf[i] = ef[i] * tf[i]; }
      key_full = tree128(tf) < tree128(tb);
      uint32_t code[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) code[i] = code_bits(key_full ? qf[i] : qb[i], QM == QM_SYM4);
      uint32_t word = key_full ? wf : wb;
      if (!key_full && use_h) word |= 0x8000u;
      store_row<QM, P>(chunk, pos, false, code, word, l32, false);
      if (!do_v && l32 == 0) {  // key-only pass: own bit 15 of the token's group-0 V scale word
        const int off = L::VS_OFF + (8 * (pos >> 3) + vs_slot8(pos)) * 2;
        uint32_t* wp = reinterpret_cast<uint32_t*>(chunk + (off & ~3));
        const uint32_t bit = 0x8000u << ((off & 2) * 8);
        if (key_full) atomicOr(wp, bit); else atomicAnd(wp, ~bit);
      }
    }
    if (do_v) {
      // Value rows.  The eight tokens of the step usually fill one aligned run of 8 slots of a page: their V^T words
      // are then assembled in LDS and stored whole; otherwise field by field with atomics.
      uint32_t code[4] = {0u, 0u, 0u, 0u};
      if (live) {
        float x[4], q[4], deq[4];
        load_row(p.kv, static_cast<long long>(t) * p.kv_ts + (p.Hkv + h) * 128 + 4 * l32, x);
        uint32_t word = quant_group<QM, false>(x, q, deq);
        if (do_k && g == 0 && key_full) word |= 0x8000u;
#pragma unroll
        for (int i = 0; i < 4; ++i) code[i] = code_bits(q[i], QM == QM_SYM4);
        store_v_word<QM, P>(chunk, pos, word, l32, !do_k);
      }
      if (l32 == 0) vslot[hw] = slot;
      *reinterpret_cast<uint32_t*>(&vcodes[hw][4 * l32]) = code[0] | (code[1] << 8) | (code[2] << 16) | (code[3] << 24);
      __syncthreads();
      const long long s0 = vslot[0];
      bool run = s0 >= 0 && (s0 & 7) == 0;
#pragma unroll
      for (int i = 1; i < K2_ROWS; ++i) run = run && vslot[i] == s0 + i;
      if (run) {
        constexpr int NWORD = QM == QM_ASYM2 ? 64 : 128;
        uint8_t* c0 = p.pool + ((s0 / P) * p.Hkv + h) * L::CHUNK;
        if (threadIdx.x < NWORD) store_v_run_word<QM, P>(c0, static_cast<int>(s0 % P) >> 3, threadIdx.x, vcodes);
      } else if (live) {
        store_v_codes<QM, P>(chunk, pos, code, l32);
      }
      __syncthreads();
    }
  }
}


// ------------------------------------------------------------------------------------------------ head dim 256
// Selecting writer of the key-only kinds for 256-d heads (attn_codebook.cu:384-392, 432; codebook_ref.encode with
// Dq = 256).  A half wave owns a (token, head): lane l holds dims 4 l + i of BOTH 128-d halves, so the transforms of a
// half are the 128-d ones and H256 adds one stage between the two registers of a lane (distance 128) and the exact
// factor 1/16.  The eight key 32-groups choose I / H32 by their diagonal block of C_q, the head chooses between that
// combination and H256 by all of C_q (the eight column blocks folded left to right, every product and sum rounded on
// its own: the order of codebook_ref.key_head_err).  C_q^T (256 KB per head) does not fit in LDS: its rows come from
// L2; the error vectors sit in an LDS strip per half wave.  The page chunk is two 128-d half chunks, half s = dims
// [128 s, 128 s + 128), each in the 128-d layout; H32 flag of group g = sign bit of its K scale word, H256 flag = sign
// bit of the token's group-0 V scale word of half 0.  Values are quantised as they are.

template <int QM, int P>
__global__ void __launch_bounds__(256) k_k2_write256(const K2WriteParams p) {
  using L = Lay<QM, P>;
  __shared__ __align__(16) float strips[8][2][256];
  const int hw = threadIdx.x >> 5, l32 = threadIdx.x & 31, g = l32 >> 3;
  const int h = blockIdx.x;
  const long long t = static_cast<long long>(blockIdx.y) * 8 + hw;
  if (t >= p.T) return;                                          // (no workgroup barrier below)
  const long long slot = p.slots[t * (p.slot_ph ? p.Hkv : 1) + (p.slot_ph ? h : 0)];
  if (slot < 0) return;
  float (*es)[256] = strips[hw];
  const float* CT = p.CT + static_cast<size_t>(h) * 256 * 256;   // CT[k][i] = C_q[i][k]
  float x[2][4];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    load_row(p.kv, t * p.kv_ts + h * 256 + 128 * s + 4 * l32, x[s]);
    if (p.kmu != nullptr) {
      const float4 m = *reinterpret_cast<const float4*>(p.kmu + h * 256 + 128 * s + 4 * l32);
      x[s][0] = x[s][0] - m.x; x[s][1] = x[s][1] - m.y; x[s][2] = x[s][2] - m.z; x[s][3] = x[s][3] - m.w;
    }
  }
  // ---- local candidates of the eight groups: identity and H32
  float qb[2][4], eb[2][4];
  uint32_t wb[2];
  bool use_h[2];
  {
    float qi[2][4], ei[2][4], qh[2][4], eh[2][4];
    uint32_t wi[2], wh[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      float y[4];
      wi[s] = quant_group<QM, true>(x[s], qi[s], ei[s]);
#pragma unroll
      for (int i = 0; i < 4; ++i) { ei[s][i] = ei[s][i] - x[s][i]; y[i] = x[s][i]; }
      fwht<32>(y, l32);
      wh[s] = quant_group<QM, true>(y, qh[s], eh[s]);
      fwht<32>(eh[s], l32);
#pragma unroll
      for (int i = 0; i < 4; ++i) eh[s][i] = eh[s][i] - x[s][i];
      *reinterpret_cast<float4*>(&es[0][128 * s + 4 * l32]) = make_float4(ei[s][0], ei[s][1], ei[s][2], ei[s][3]);
      *reinterpret_cast<float4*>(&es[1][128 * s + 4 * l32]) = make_float4(eh[s][0], eh[s][1], eh[s][2], eh[s][3]);
    }
    wave_lds_sync();
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int c0 = 128 * s + 32 * g;                           // first channel of this lane's group
      const float* crow = CT + static_cast<size_t>(c0) * 256 + 128 * s + 4 * l32;
      float ui[4], uh[4];
#pragma unroll 4
      for (int k = 0; k < 32; ++k) {
        const float4 cv = *reinterpret_cast<const float4*>(crow + static_cast<size_t>(k) * 256);
        const float a = es[0][c0 + k], b = es[1][c0 + k];
        const float c[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float pa = c[i] * a, pb = c[i] * b;
          ui[i] = k == 0 ? pa : ui[i] + pa;
          uh[i] = k == 0 ? pb : uh[i] + pb;
        }
      }
      float pi[4], ph[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { pi[i] = ei[s][i] * ui[i]; ph[i] = eh[s][i] * uh[i]; }
      use_h[s] = tree32(ph) < tree32(pi);                        // strict: ties keep the identity
#pragma unroll
      for (int i = 0; i < 4; ++i) { qb[s][i] = use_h[s] ? qh[s][i] : qi[s][i]; eb[s][i] = use_h[s] ? eh[s][i] : ei[s][i]; }
      wb[s] = use_h[s] ? wh[s] : wi[s];
    }
  }
  // ---- whole-head candidate: H256
  float qf[2][4], ef[2][4];
  uint32_t wf[2];
  {
    float y[2][4];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) y[s][i] = x[s][i];
    h256(y, l32);
    wf[0] = quant_group<QM, true>(y[0], qf[0], ef[0]);
    wf[1] = quant_group<QM, true>(y[1], qf[1], ef[1]);
    h256(ef, l32);
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) ef[s][i] = ef[s][i] - x[s][i];
  }
  wave_lds_sync();                                               // the local pass has read its strips
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    *reinterpret_cast<float4*>(&es[0][128 * s + 4 * l32]) = make_float4(eb[s][0], eb[s][1], eb[s][2], eb[s][3]);
    *reinterpret_cast<float4*>(&es[1][128 * s + 4 * l32]) = make_float4(ef[s][0], ef[s][1], ef[s][2], ef[s][3]);
  }
  wave_lds_sync();
  float tb[2][4], tf[2][4];
#pragma unroll 1
  for (int b = 0; b < 8; ++b) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      float ub[4], uf[4];
      const float* crow = CT + static_cast<size_t>(32 * b) * 256 + 128 * s + 4 * l32;
#pragma unroll 4
      for (int k = 0; k < 32; ++k) {
        const float4 cv = *reinterpret_cast<const float4*>(crow + static_cast<size_t>(k) * 256);
        const float a = es[0][32 * b + k], f = es[1][32 * b + k];
        const float c[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float pa = c[i] * a, pf = c[i] * f;
          ub[i] = k == 0 ? pa : ub[i] + pa;
          uf[i] = k == 0 ? pf : uf[i] + pf;
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        tb[s][i] = b == 0 ? ub[i] : tb[s][i] + ub[i];
        tf[s][i] = b == 0 ? uf[i] : tf[s][i] + uf[i];
      }
    }
  }
  bool key_full;
  {
    // halving tree of 256 products: dims d and d + 128 first (the two registers of a lane), then the 128-tree
    float pb[4], pf[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pb[i] = eb[0][i] * tb[0][i] + eb[1][i] * tb[1][i];
      pf[i] = ef[0][i] * tf[0][i] + ef[1][i] * tf[1][i];
    }
    key_full = tree128(pf) < tree128(pb);
  }
  const int pos = static_cast<int>(slot % P);
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    uint8_t* chunk = p.pool + ((slot / P) * (2 * p.Hkv) + 2 * h + s) * L::CHUNK;
    uint32_t code[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) code[i] = code_bits(key_full ? qf[s][i] : qb[s][i], QM == QM_SYM4);
    uint32_t word = key_full ? wf[s] : wb[s];
    if (!key_full && use_h[s]) word |= 0x8000u;
    store_row<QM, P>(chunk, pos, false, code, word, l32, false);
    // the value half row, as it is
    float v[4], q[4], deq[4];
    load_row(p.kv, t * p.kv_ts + (p.Hkv + h) * 256 + 128 * s + 4 * l32, v);
    uint32_t vword = quant_group<QM, false>(v, q, deq);
    if (s == 0 && g == 0 && key_full) vword |= 0x8000u;
#pragma unroll
    for (int i = 0; i < 4; ++i) code[i] = code_bits(q[i], QM == QM_SYM4);
    store_v_word<QM, P>(chunk, pos, vword, l32, false);
    store_v_codes<QM, P>(chunk, pos, code, l32);
  }
}


// Low-latency form of k_k2_write for a handful of tokens (a decode step): four half waves per (token, head) instead of
// one, two tokens per workgroup.  Every half wave repeats the cheap part (quantised candidates, transforms); the
// weighted error sums are shared out without touching the order of any sum: in the local pass half wave r carries the
// chains of output 4 l + r, in the whole-head pass half wave b carries the block sums of block b, and the block sums are
// added in block order as in k_k2_write.  Results are bit-identical to k_k2_write.
constexpr int K2LL_LDS = K2_LDS_C + 2 * (2 * 128 + 4 * 2 * 32 + 4 * 8 * 32) * 4;
template <int QM, int P>
__global__ void __launch_bounds__(256) k_k2_write_ll(const K2WriteParams p) {
  using L = Lay<QM, P>;
  extern __shared__ __align__(16) uint8_t lds[];
  float* Cs = reinterpret_cast<float*>(lds);                   // [k][i] = C_q[i][k]
  const int hw = threadIdx.x >> 5, l32 = threadIdx.x & 31, role = hw & 3, ts = hw >> 2;
  float* es = reinterpret_cast<float*>(lds + K2_LDS_C) + ts * (2 * 128 + 4 * 2 * 32 + 4 * 8 * 32);  // [2][128]
  float* xs = es + 2 * 128;                                    // [role][candidate][lane]: local sums of output 4 l + role
  float* ys = xs + 4 * 2 * 32;                                 // [block][8][lane]: block sums ub[4], uf[4]
  const int h = blockIdx.x;
  const int t = blockIdx.y * 2 + ts;
  const bool do_k = p.passes & 1, do_v = p.passes & 2;
  if (do_k) {
    const float4* src = reinterpret_cast<const float4*>(p.CT + static_cast<size_t>(h) * 128 * 128);
    float4* dst = reinterpret_cast<float4*>(Cs);
    for (int i = threadIdx.x; i < 128 * 128 / 4; i += 256) dst[i] = src[i];
  }
  __syncthreads();
  const int g = l32 >> 3;
  long long slot = -1;
  if (t < p.T) slot = p.slots[static_cast<long long>(t) * (p.slot_ph ? p.Hkv : 1) + (p.slot_ph ? h : 0)];
  const bool live = slot >= 0;                                 // the barriers below are passed by every thread
  uint8_t* chunk = p.pool + ((live ? slot / P : 0) * p.Hkv + h) * L::CHUNK;
  const int pos = live ? static_cast<int>(slot % P) : 0;
  bool key_full = false;
  if (do_k) {
    float x[4] = {0.f, 0.f, 0.f, 0.f};
    if (live) {
      load_row(p.kv, static_cast<long long>(t) * p.kv_ts + h * 128 + 4 * l32, x);
      if (p.kmu != nullptr) {
        const float4 m = *reinterpret_cast<const float4*>(p.kmu + h * 128 + 4 * l32);
        x[0] = x[0] - m.x; x[1] = x[1] - m.y; x[2] = x[2] - m.z; x[3] = x[3] - m.w;
      }
    }
    // ---- local candidates: identity and H32 of every 32-group
    float qi[4], ei[4], qh[4], eh[4], y[4];
    const uint32_t wi = quant_group<QM, true>(x, qi, ei);
#pragma unroll
    for (int i = 0; i < 4; ++i) { ei[i] = ei[i] - x[i]; y[i] = x[i]; }
    fwht<32>(y, l32);
    const uint32_t wh = quant_group<QM, true>(y, qh, eh);
    fwht<32>(eh, l32);
#pragma unroll
    for (int i = 0; i < 4; ++i) eh[i] = eh[i] - x[i];
    if (role == 0) {
      *reinterpret_cast<float4*>(es + 4 * l32) = make_float4(ei[0], ei[1], ei[2], ei[3]);
      *reinterpret_cast<float4*>(es + 128 + 4 * l32) = make_float4(eh[0], eh[1], eh[2], eh[3]);
    }
    __syncthreads();
    {
      float ui = 0.f, uh = 0.f;
      const float* crow = Cs + (32 * g) * 128 + 4 * l32 + role;   // C[4 l + role][32 g + k] at crow[k * 128]
      const float* e0 = es + 32 * g;
#pragma unroll 8
      for (int k = 0; k < 32; ++k) {
        const float c = crow[k * 128];
        const float pa = c * e0[k], pb = c * e0[128 + k];
        ui = k == 0 ? pa : ui + pa;
        uh = k == 0 ? pb : uh + pb;
      }
      xs[(role * 2 + 0) * 32 + l32] = ui;
      xs[(role * 2 + 1) * 32 + l32] = uh;
    }
    __syncthreads();
    float pi[4], ph[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { pi[i] = ei[i] * xs[(i * 2 + 0) * 32 + l32]; ph[i] = eh[i] * xs[(i * 2 + 1) * 32 + l32]; }
    const bool use_h = tree32(ph) < tree32(pi);   // strict: ties keep the identity
    float qb[4], eb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { qb[i] = use_h ? qh[i] : qi[i]; eb[i] = use_h ? eh[i] : ei[i]; }
    const uint32_t wb = use_h ? wh : wi;
    // ---- whole-head candidate
    float qf[4], ef[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) y[i] = x[i];
    fwht<128>(y, l32);
    const uint32_t wf = quant_group<QM, true>(y, qf, ef);
    fwht<128>(ef, l32);
#pragma unroll
    for (int i = 0; i < 4; ++i) ef[i] = ef[i] - x[i];
    if (role == 0) {      // every half wave has read the local strips (second barrier above)
      *reinterpret_cast<float4*>(es + 4 * l32) = make_float4(eb[0], eb[1], eb[2], eb[3]);
      *reinterpret_cast<float4*>(es + 128 + 4 * l32) = make_float4(ef[0], ef[1], ef[2], ef[3]);
    }
    __syncthreads();
    {
      float ub[4], uf[4];
      const int b = role;
      const float* crow = Cs + (32 * b) * 128 + 4 * l32;
      const float* e0 = es + 32 * b;
#pragma unroll 4
      for (int k = 0; k < 32; ++k) {
        const float4 cv = *reinterpret_cast<const float4*>(crow + k * 128);
        const float a = e0[k], f = e0[128 + k];
        const float c[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float pa = c[i] * a, pf = c[i] * f;
          ub[i] = k == 0 ? pa : ub[i] + pa;
          uf[i] = k == 0 ? pf : uf[i] + pf;
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) { ys[(b * 8 + i) * 32 + l32] = ub[i]; ys[(b * 8 + 4 + i) * 32 + l32] = uf[i]; }
    }
    __syncthreads();
    float tb[4], tf[4];
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float ub = ys[(b * 8 + i) * 32 + l32], uf = ys[(b * 8 + 4 + i) * 32 + l32];
        tb[i] = b == 0 ? ub : tb[i] + ub;
        tf[i] = b == 0 ? uf : tf[i] + uf;
      }
#pragma unroll
    for (int i = 0; i < 4; ++i) { tb[i] = eb[i] * tb[i]; tf[i] = ef[i] * tf[i]; }
    key_full = tree128(tf) < tree128(tb);
    if (live && role == 0) {
      uint32_t code[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) code[i] = code_bits(key_full ? qf[i] : qb[i], QM == QM_SYM4);
      uint32_t word = key_full ? wf : wb;
      if (!key_full && use_h) word |= 0x8000u;
      store_row<QM, P>(chunk, pos, false, code, word, l32, false);
      if (!do_v && l32 == 0) {  // key-only pass: own bit 15 of the token's group-0 V scale word
        const int off = L::VS_OFF + (8 * (pos >> 3) + vs_slot8(pos)) * 2;
        uint32_t* wp = reinterpret_cast<uint32_t*>(chunk + (off & ~3));
        const uint32_t bit = 0x8000u << ((off & 2) * 8);
        if (key_full) atomicOr(wp, bit); else atomicAnd(wp, ~bit);
      }
    }
  }
  if (do_v && live && role == 1) {
    float x[4], q[4], deq[4];
    load_row(p.kv, static_cast<long long>(t) * p.kv_ts + (p.Hkv + h) * 128 + 4 * l32, x);
    uint32_t word = quant_group<QM, false>(x, q, deq);
    if (do_k && g == 0 && key_full) word |= 0x8000u;
    uint32_t code[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) code[i] = code_bits(q[i], QM == QM_SYM4);
    store_row<QM, P>(chunk, pos, true, code, word, l32, !do_k);
  }
}

// ------------------------------------------------------------------------------------------------ screened selecting writer
// Same bytes as k_k2_write at a fraction of its vector instructions: the quadratic forms d^T C d of the candidates'
// error vectors are ESTIMATED on the matrix pipe (v_mfma_f32_32x32x2f32, fp32 operands) and a choice is taken from the
// estimates only where it cannot differ from the choice of the exactly ordered fp32 evaluation; every other token is
// evaluated exactly, in the reference's order, at the end of the workgroup.
//   Bound: with S = |d|^T |C| |d|, the reference's value (sums of <= 35 terms, one product, a tree of depth 7) lies
//   within 44 u S of the true form (u = 2^-24), the estimate (at most 128 products and sums inside the matrix pipe,
//   each taken as accurate to 2 u whatever its order and rounding mode, a 16-term dot, 6 more sums) within 300 u S;
//   S <= rho |d|^2 with rho = max(largest row sum, largest column sum of |C|), computed by the workgroup itself.  The
//   screen uses b = 2^-15 rho |d|^2 (1.5 x the sum of the two) + 2^-100: candidate a beats candidate b for certain when
//   e~_a + b_a < e~_b - b_b.
// Workgroup = (KV head, tile of tokens), four wavefronts; wavefront w keeps rows 32 w .. 32 w + 31 of C in registers as
// matrix A operands (the whole row for the whole-head forms, its diagonal 32-block for the local forms).  A step takes
// 16 tokens, two per half wave: candidates in registers exactly as in k_k2_write, error vectors as the 32 columns of a
// matrix in LDS, forms by MFMA, choices back through LDS.
constexpr int W3_TOK = 16;                   // tokens per step
constexpr int W3_DROW = 132;                 // floats per column of the error matrix in LDS: 128 + 4 pad
constexpr int W3_MAXTILE = 128;              // tokens per workgroup at most (fallback list)
constexpr float W3_KAPPA = 3.0517578125e-05f;   // 2^-15

struct W3Smem {
  float dm[2 * W3_TOK][W3_DROW];             // column 2 t + c: error vector of candidate c of token t of the step
  float part[2][4][2 * W3_TOK];              // [form | squared norm][row tile = wavefront][column]
  float colsum[128];
  float rinf[4];                             // largest row sum of |C| per row tile
  float es[8][256];                          // strips of the exact evaluation (per half wave)
  int fb[W3_MAXTILE];                        // tokens left to the exact evaluation
  int nfb;
  uint8_t choice[W3_TOK][4];                 // per (token, 32-group): 0 identity, 1 H32, 2 undecided
  long long vslot[W3_TOK];
  alignas(16) uint8_t vcodes[W3_TOK][128];   // value codes of the step's tokens
};

// the exact choice of one token, half wave: k_k2_write's evaluation with C^T read through `C` (LDS or memory)
template <int QM>
DEVI void k2_exact_choice(const float (&x)[4], const float* C, float* es, int l32, float (&qsel)[4], uint32_t& word, bool& key_full) {
  const int g = l32 >> 3;
  float qi[4], ei[4], qh[4], eh[4], y[4];
  const uint32_t wi = quant_group<QM, true>(x, qi, ei);
#pragma unroll
  for (int i = 0; i < 4; ++i) { ei[i] = ei[i] - x[i]; y[i] = x[i]; }
  fwht<32>(y, l32);
  const uint32_t wh = quant_group<QM, true>(y, qh, eh);
  fwht<32>(eh, l32);
#pragma unroll
  for (int i = 0; i < 4; ++i) eh[i] = eh[i] - x[i];
  wave_lds_sync();
  *reinterpret_cast<float4*>(es + 4 * l32) = make_float4(ei[0], ei[1], ei[2], ei[3]);
  *reinterpret_cast<float4*>(es + 128 + 4 * l32) = make_float4(eh[0], eh[1], eh[2], eh[3]);
  wave_lds_sync();
  float ui[4], uh[4];
  {
    const float* crow = C + (32 * g) * 128 + 4 * l32;
    const float* e0 = es + 32 * g;
#pragma unroll 4
    for (int k = 0; k < 32; ++k) {
      const float4 cv = *reinterpret_cast<const float4*>(crow + k * 128);
      const float a = e0[k], b = e0[128 + k];
      const float c[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pa = c[i] * a, pb = c[i] * b;
        ui[i] = k == 0 ? pa : ui[i] + pa;
        uh[i] = k == 0 ? pb : uh[i] + pb;
      }
    }
  }
  float pi[4], ph[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) { pi[i] = ei[i] * ui[i]; ph[i] = eh[i] * uh[i]; }
  const bool use_h = tree32(ph) < tree32(pi);
  float qb[4], eb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) { qb[i] = use_h ? qh[i] : qi[i]; eb[i] = use_h ? eh[i] : ei[i]; }
  const uint32_t wb = use_h ? wh : wi;
  float qf[4], ef[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) y[i] = x[i];
  fwht<128>(y, l32);
  const uint32_t wf = quant_group<QM, true>(y, qf, ef);
  fwht<128>(ef, l32);
#pragma unroll
  for (int i = 0; i < 4; ++i) ef[i] = ef[i] - x[i];
  wave_lds_sync();
  *reinterpret_cast<float4*>(es + 4 * l32) = make_float4(eb[0], eb[1], eb[2], eb[3]);
  *reinterpret_cast<float4*>(es + 128 + 4 * l32) = make_float4(ef[0], ef[1], ef[2], ef[3]);
  wave_lds_sync();
  float tb[4], tf[4];
#pragma unroll 1
  for (int b = 0; b < 4; ++b) {
    float ub[4], uf[4];
    const float* crow = C + (32 * b) * 128 + 4 * l32;
    const float* e0 = es + 32 * b;
#pragma unroll 4
    for (int k = 0; k < 32; ++k) {
      const float4 cv = *reinterpret_cast<const float4*>(crow + k * 128);
      const float a = e0[k], f = e0[128 + k];
      const float c[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pa = c[i] * a, pf = c[i] * f;
        ub[i] = k == 0 ? pa : ub[i] + pa;
        uf[i] = k == 0 ? pf : uf[i] + pf;
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      tb[i] = b == 0 ? ub[i] : tb[i] + ub[i];
      tf[i] = b == 0 ? uf[i] : tf[i] + uf[i];
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) { tb[i] = eb[i] * tb[i]; tf[i] = ef[i] * tf[i]; }
  key_full = tree128(tf) < tree128(tb);
#pragma unroll
  for (int i = 0; i < 4; ++i) qsel[i] = key_full ? qf[i] : qb[i];
  word = key_full ? wf : wb;
  if (!key_full && use_h) word |= 0x8000u;
}

// the key row of one token with its choice; in a key-only pass also the flag bit it owns in the value scale word
template <int QM, int P>
DEVI void k2_store_key(const K2WriteParams& p, int h, long long slot, bool flag_bit, const float (&qsel)[4], uint32_t word,
                       bool key_full, int l32) {
  using L = Lay<QM, P>;
  uint8_t* chunk = p.pool + ((slot / P) * p.Hkv + h) * L::CHUNK;
  const int pos = static_cast<int>(slot % P);
  uint32_t code[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) code[i] = code_bits(qsel[i], QM == QM_SYM4);
  store_row<QM, P>(chunk, pos, false, code, word, l32, false);
  if (flag_bit && l32 == 0) {
    const int off = L::VS_OFF + (8 * (pos >> 3) + vs_slot8(pos)) * 2;
    uint32_t* wp = reinterpret_cast<uint32_t*>(chunk + (off & ~3));
    const uint32_t bit = 0x8000u << ((off & 2) * 8);
    if (key_full) atomicOr(wp, bit); else atomicAnd(wp, ~bit);
  }
}
// the value scale words of one token (its codes are in the page already), with the key's whole-head flag
template <int QM, int P>
DEVI void k2_store_value_words(const K2WriteParams& p, int t, int h, long long slot, bool key_full, int l32) {
  using L = Lay<QM, P>;
  float x[4], q[4], deq[4];
  load_row(p.kv, static_cast<long long>(t) * p.kv_ts + (p.Hkv + h) * 128 + 4 * l32, x);
  uint32_t vword = quant_group<QM, false>(x, q, deq);
  if ((l32 >> 3) == 0 && key_full) vword |= 0x8000u;
  store_v_word<QM, P>(p.pool + ((slot / P) * p.Hkv + h) * L::CHUNK, static_cast<int>(slot % P), vword, l32, false);
}

DEVI float max32(float v) {   // over the 32 lanes of a half wave
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) v = fmaxf(v, hx(v, o));
  return v;
}
DEVI float sum32(float v) {
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) v = v + hx(v, o);
  return v;
}

typedef float w3_f32x16 __attribute__((ext_vector_type(16)));

typedef __attribute__((address_space(1))) float gfloat;      // a float in global memory: loads through it are global_load, not flat_load
template <int QM, int P>
__global__ void __launch_bounds__(256) k_k2_screen(const K2WriteParams p, int tile, float kappa) {
  __shared__ W3Smem S;
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, hw = tid >> 5, l32 = tid & 31, kq = lane >> 5;
  const int h = blockIdx.x;
  const int t_lo = blockIdx.y * tile, t_hi = min(p.T, t_lo + tile);
  const bool do_v = p.passes & 2;
  const float* CT = p.CT + static_cast<size_t>(h) * 128 * 128;       // CT[k * 128 + i] = C[i][k]
  // ---- A operands: lane (row m = l32 of tile wv, half kq): C[32 wv + m][64 kq + s] and C[32 wv + m][32 wv + 16 kq + s]
  // (read from memory at every use: C^T stays in L2, and the registers it would take cost three quarters of the occupancy)
  const float* ahp = CT + (64 * kq) * 128 + 32 * wv + l32;                 // + s * 128
  const float* alp = CT + (32 * wv + 16 * kq) * 128 + 32 * wv + l32;       // + s * 128
  if (tid < 128) S.colsum[tid] = 0.f;
  if (tid == 0) S.nfb = 0;
  __syncthreads();
  float rho_loc, rho_full;
  {
    float rs = 0.f, rl = 0.f, cl = 0.f;
#pragma unroll 8
    for (int s2 = 0; s2 < 64; ++s2) {
      const float a = fabsf(ahp[s2 * 128]);
      rs += a;
      const float cs = sum32(a);                                 // column 64 kq + s2 over the rows of this tile
      if (l32 == 0) atomicAdd(&S.colsum[64 * kq + s2], cs);
    }
#pragma unroll 8
    for (int s2 = 0; s2 < 16; ++s2) {
      const float a = fabsf(alp[s2 * 128]);
      rl += a;
      cl = fmaxf(cl, sum32(a));
    }
    rs += __shfl_xor(rs, 32, 64); rl += __shfl_xor(rl, 32, 64);
    cl = fmaxf(cl, __shfl_xor(cl, 32, 64));
    rho_loc = fmaxf(max32(rl), cl);
    const float ri = max32(rs);
    if (lane == 0) S.rinf[wv] = ri;
    __syncthreads();
    float c1 = fmaxf(S.colsum[lane], S.colsum[64 + lane]);
    c1 = max32(c1); c1 = fmaxf(c1, __shfl_xor(c1, 32, 64));
    rho_full = fmaxf(fmaxf(fmaxf(S.rinf[0], S.rinf[1]), fmaxf(S.rinf[2], S.rinf[3])), c1);
  }
  const float beta_loc = kappa * rho_loc, beta_full = kappa * rho_full;
  const int g = l32 >> 3;

  for (int tb0 = t_lo; tb0 < t_hi; tb0 += W3_TOK) {
    // ---- P1: candidates of the half wave's two tokens (exactly as in k_k2_write); error vectors to the matrix
    uint32_t cq[2][3], cw[2][3];        // per token: packed codes (one byte per element) and scale words of I, H, F
    float ef[2][4];
    long long slot[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int tk = 2 * hw + u, t = tb0 + tk;
      slot[u] = -1;
      if (t < t_hi) slot[u] = p.slots[static_cast<long long>(t) * (p.slot_ph ? p.Hkv : 1) + (p.slot_ph ? h : 0)];
      float x[4] = {0.f, 0.f, 0.f, 0.f};
      if (slot[u] >= 0) {
        load_row(p.kv, static_cast<long long>(t) * p.kv_ts + h * 128 + 4 * l32, x);
        if (p.kmu != nullptr) {
          const float4 m = *reinterpret_cast<const float4*>(p.kmu + h * 128 + 4 * l32);
          x[0] = x[0] - m.x; x[1] = x[1] - m.y; x[2] = x[2] - m.z; x[3] = x[3] - m.w;
        }
      }
      float qi[4], ei[4], qh[4], eh[4], qf[4], y[4];
      cw[u][0] = quant_group<QM, true>(x, qi, ei);
#pragma unroll
      for (int i = 0; i < 4; ++i) { ei[i] = ei[i] - x[i]; y[i] = x[i]; }
      fwht<32>(y, l32);
      cw[u][1] = quant_group<QM, true>(y, qh, eh);
      fwht<32>(eh, l32);
#pragma unroll
      for (int i = 0; i < 4; ++i) { eh[i] = eh[i] - x[i]; y[i] = x[i]; }
      fwht<128>(y, l32);
      cw[u][2] = quant_group<QM, true>(y, qf, ef[u]);
      fwht<128>(ef[u], l32);
#pragma unroll
      for (int i = 0; i < 4; ++i) ef[u][i] = ef[u][i] - x[i];
      cq[u][0] = cq[u][1] = cq[u][2] = 0u;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        cq[u][0] |= code_bits(qi[i], QM == QM_SYM4) << (8 * i);
        cq[u][1] |= code_bits(qh[i], QM == QM_SYM4) << (8 * i);
        cq[u][2] |= code_bits(qf[i], QM == QM_SYM4) << (8 * i);
      }
      *reinterpret_cast<float4*>(&S.dm[2 * tk][4 * l32]) = make_float4(ei[0], ei[1], ei[2], ei[3]);
      *reinterpret_cast<float4*>(&S.dm[2 * tk + 1][4 * l32]) = make_float4(eh[0], eh[1], eh[2], eh[3]);
    }
    __syncthreads();
    // ---- P2: local forms of block wv for the 32 columns; lane = (column l32, half kq)
    {
      w3_f32x16 acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
      const float* dcol = &S.dm[l32][32 * wv];
      const float* alq_ = alp;
      asm volatile("" : "+v"(alq_));            // keeps these loads inside the step (not hoisted into 80 registers)
      const gfloat* alq = reinterpret_cast<const gfloat*>(reinterpret_cast<uintptr_t>(alq_));   // (a global, not a flat, access)
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) {
        const float4 d4 = *reinterpret_cast<const float4*>(dcol + 16 * kq + 4 * s4);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(alq[(4 * s4 + 0) * 128], d4.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(alq[(4 * s4 + 1) * 128], d4.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(alq[(4 * s4 + 2) * 128], d4.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(alq[(4 * s4 + 3) * 128], d4.w, acc, 0, 0, 0);
      }
      float f = 0.f, n2 = 0.f;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {          // rows 8 q4 + 4 kq + r of the block
        const float4 d4 = *reinterpret_cast<const float4*>(dcol + 8 * q4 + 4 * kq);
        f = __builtin_fmaf(d4.x, acc[4 * q4 + 0], f); f = __builtin_fmaf(d4.y, acc[4 * q4 + 1], f);
        f = __builtin_fmaf(d4.z, acc[4 * q4 + 2], f); f = __builtin_fmaf(d4.w, acc[4 * q4 + 3], f);
        n2 = __builtin_fmaf(d4.x, d4.x, n2); n2 = __builtin_fmaf(d4.y, d4.y, n2);
        n2 = __builtin_fmaf(d4.z, d4.z, n2); n2 = __builtin_fmaf(d4.w, d4.w, n2);
      }
      f += __shfl_xor(f, 32, 64); n2 += __shfl_xor(n2, 32, 64);
      const float bnd = beta_loc * n2 + 7.888609052210118e-31f;
      // columns 2 t (identity) and 2 t + 1 (H32): the reference takes H32 iff its value is strictly smaller
      const float fo = hx(f, 1), bo = hx(bnd, 1);
      if ((l32 & 1) == 0 && kq == 0) {
        const float eI = f, bI = bnd, eH = fo, bH = bo;
        S.choice[l32 >> 1][wv] = (eH + bH < eI - bI) ? 1 : (eH - bH > eI + bI) ? 0 : 2;
      }
    }
    __syncthreads();
    // ---- P3: the half wave's tokens: base candidate from the local choices, or the exact list
    bool pend[2], kfull[2] = {false, false};
    uint32_t useh[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int tk = 2 * hw + u;
      const uint32_t ch = *reinterpret_cast<const uint32_t*>(&S.choice[tk][0]);
      const bool und = (ch & 0x02020202u) != 0;      // some group undecided
      pend[u] = slot[u] >= 0 && !und;
      if (slot[u] >= 0 && und && l32 == 0) S.fb[atomicAdd(&S.nfb, 1)] = tb0 + tk;
      useh[u] = (ch >> (8 * g)) & 1u;
      const float4 eI = *reinterpret_cast<const float4*>(&S.dm[2 * tk][4 * l32]);
      const float4 eH = *reinterpret_cast<const float4*>(&S.dm[2 * tk + 1][4 * l32]);
      const float4 eb = useh[u] ? eH : eI;
      wave_lds_sync();
      *reinterpret_cast<float4*>(&S.dm[2 * tk][4 * l32]) = eb;
      *reinterpret_cast<float4*>(&S.dm[2 * tk + 1][4 * l32]) = make_float4(ef[u][0], ef[u][1], ef[u][2], ef[u][3]);
    }
    __syncthreads();
    // ---- P4: whole-head forms: rows of tile wv, all 128 columns of C
    {
      w3_f32x16 acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
      const float* dcol = &S.dm[l32][0];
      const float* ahq_ = ahp;
      asm volatile("" : "+v"(ahq_));
      const gfloat* ahq = reinterpret_cast<const gfloat*>(reinterpret_cast<uintptr_t>(ahq_));
#pragma unroll 4
      for (int s4 = 0; s4 < 16; ++s4) {
        const float4 d4 = *reinterpret_cast<const float4*>(dcol + 64 * kq + 4 * s4);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ahq[(4 * s4 + 0) * 128], d4.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ahq[(4 * s4 + 1) * 128], d4.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ahq[(4 * s4 + 2) * 128], d4.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ahq[(4 * s4 + 3) * 128], d4.w, acc, 0, 0, 0);
      }
      float f = 0.f, n2 = 0.f;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const float4 d4 = *reinterpret_cast<const float4*>(dcol + 32 * wv + 8 * q4 + 4 * kq);
        f = __builtin_fmaf(d4.x, acc[4 * q4 + 0], f); f = __builtin_fmaf(d4.y, acc[4 * q4 + 1], f);
        f = __builtin_fmaf(d4.z, acc[4 * q4 + 2], f); f = __builtin_fmaf(d4.w, acc[4 * q4 + 3], f);
        n2 = __builtin_fmaf(d4.x, d4.x, n2); n2 = __builtin_fmaf(d4.y, d4.y, n2);
        n2 = __builtin_fmaf(d4.z, d4.z, n2); n2 = __builtin_fmaf(d4.w, d4.w, n2);
      }
      f += __shfl_xor(f, 32, 64); n2 += __shfl_xor(n2, 32, 64);
      if (kq == 0) { S.part[0][wv][l32] = f; S.part[1][wv][l32] = n2; }
    }
    __syncthreads();
    // ---- P5: base against whole head; rows of the decided tokens into their pages
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int tk = 2 * hw + u;
      float e[2], b[2];
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        e[c] = (S.part[0][0][2 * tk + c] + S.part[0][1][2 * tk + c]) + (S.part[0][2][2 * tk + c] + S.part[0][3][2 * tk + c]);
        const float n2 = (S.part[1][0][2 * tk + c] + S.part[1][1][2 * tk + c]) + (S.part[1][2][2 * tk + c] + S.part[1][3][2 * tk + c]);
        b[c] = beta_full * n2 + 7.888609052210118e-31f;
      }
      const int dec = (e[1] + b[1] < e[0] - b[0]) ? 1 : (e[1] - b[1] > e[0] + b[0]) ? 0 : 2;
      if (pend[u] && dec == 2) {
        if (l32 == 0) S.fb[atomicAdd(&S.nfb, 1)] = tb0 + tk;
        pend[u] = false;
      } else if (pend[u]) {
        const bool key_full = dec == 1;
        kfull[u] = key_full;
        const uint32_t cpk = key_full ? cq[u][2] : (useh[u] ? cq[u][1] : cq[u][0]);
        uint32_t word = key_full ? cw[u][2] : (useh[u] ? cw[u][1] : cw[u][0]);
        if (!key_full && useh[u]) word |= 0x8000u;
        float qsel[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t cb = (cpk >> (8 * i)) & 0xFFu;
          qsel[i] = QM == QM_SYM4 ? ((cb & 8u) ? -static_cast<float>(cb & 7u) : static_cast<float>(cb)) : static_cast<float>(cb);
        }
        k2_store_key<QM, P>(p, h, slot[u], !do_v, qsel, word, key_full, l32);
      }
    }
    // ---- value rows of the step: codes of all live tokens (whole words for aligned runs of 8 slots, else atomics),
    //      scale words of the decided tokens (the others' carry the key's flag and follow the exact evaluation)
    if (do_v) {
      uint32_t vcode[2][4];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int tk = 2 * hw + u;
#pragma unroll
        for (int i = 0; i < 4; ++i) vcode[u][i] = 0u;
        if (slot[u] >= 0) {
          float x[4], q[4], deq[4];
          load_row(p.kv, static_cast<long long>(tb0 + tk) * p.kv_ts + (p.Hkv + h) * 128 + 4 * l32, x);
          uint32_t vword = quant_group<QM, false>(x, q, deq);
          if (g == 0 && kfull[u]) vword |= 0x8000u;
#pragma unroll
          for (int i = 0; i < 4; ++i) vcode[u][i] = code_bits(q[i], QM == QM_SYM4);
          if (pend[u]) {
            using L = Lay<QM, P>;
            store_v_word<QM, P>(p.pool + ((slot[u] / P) * p.Hkv + h) * L::CHUNK, static_cast<int>(slot[u] % P), vword, l32, false);
          }
        }
        if (l32 == 0) S.vslot[tk] = slot[u];
        *reinterpret_cast<uint32_t*>(&S.vcodes[tk][4 * l32]) = vcode[u][0] | (vcode[u][1] << 8) | (vcode[u][2] << 16) | (vcode[u][3] << 24);
      }
      __syncthreads();
      using L = Lay<QM, P>;
      constexpr int NWORD = QM == QM_ASYM2 ? 64 : 128;
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const long long s0 = S.vslot[8 * r];
        bool run = s0 >= 0 && (s0 & 7) == 0;
#pragma unroll
        for (int i = 1; i < 8; ++i) run = run && S.vslot[8 * r + i] == s0 + i;
        if (run) {
          const int j = tid - r * 128;
          if (j >= 0 && j < NWORD)
            store_v_run_word<QM, P>(p.pool + ((s0 / P) * p.Hkv + h) * L::CHUNK, static_cast<int>(s0 % P) >> 3, j, &S.vcodes[8 * r]);
        } else if ((hw >> 2) == r) {
#pragma unroll
          for (int u = 0; u < 2; ++u)
            if (slot[u] >= 0)
              store_v_codes<QM, P>(p.pool + ((slot[u] / P) * p.Hkv + h) * L::CHUNK, static_cast<int>(slot[u] % P), vcode[u], l32);
        }
      }
    }
    // (the next step's P1 writes the matrix after every wavefront has passed the barrier behind P4; the value strips are
    //  rewritten after three more barriers)
  }
  // ---- the tokens the screen could not decide: exact evaluation, C^T from memory
  __syncthreads();
  const int nfb = S.nfb;
  for (int i = hw; i < nfb; i += 8) {
    const int t = S.fb[i];
    const long long slot = p.slots[static_cast<long long>(t) * (p.slot_ph ? p.Hkv : 1) + (p.slot_ph ? h : 0)];
    float x[4];
    load_row(p.kv, static_cast<long long>(t) * p.kv_ts + h * 128 + 4 * l32, x);
    if (p.kmu != nullptr) {
      const float4 m = *reinterpret_cast<const float4*>(p.kmu + h * 128 + 4 * l32);
      x[0] = x[0] - m.x; x[1] = x[1] - m.y; x[2] = x[2] - m.z; x[3] = x[3] - m.w;
    }
    float qsel[4];
    uint32_t word;
    bool key_full;
    k2_exact_choice<QM>(x, CT, &S.es[hw][0], l32, qsel, word, key_full);
    k2_store_key<QM, P>(p, h, slot, !do_v, qsel, word, key_full, l32);
    if (do_v) k2_store_value_words<QM, P>(p, t, h, slot, key_full, l32);
  }
}

template <int QM>
int static_write_qm(const StaticWriteParams& p, hipStream_t st) {
  const unsigned grid = static_cast<unsigned>(static_cast<long long>((p.T + 7) / 8) * 2 * p.Hkv);
  if (grid == 0) return 0;
  if (p.page == 16) hipLaunchKernelGGL((k_static_write<QM, 16>), dim3(grid), dim3(256), 0, st, p);
  else if (p.page == 32) hipLaunchKernelGGL((k_static_write<QM, 32>), dim3(grid), dim3(256), 0, st, p);
  else return -5;
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

template <int QM, int P>
int k2_write_p(const K2WriteParams& p, hipStream_t st) {
  auto k = k_k2_write<QM, P>;
  auto kll = k_k2_write_ll<QM, P>;
  static bool attr = false;
  if (!attr) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, K2_LDS) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(kll), hipFuncAttributeMaxDynamicSharedMemorySize, K2LL_LDS) != hipSuccess) {
      set_error("selecting writer: cannot reserve 76 KB of LDS");
      return -2;
    }
    attr = true;
  }
  // prefill-sized key passes: the screened kernel (same bytes)
  static const int w3mode = getenv("FLAGROT_W3") != nullptr ? atoi(getenv("FLAGROT_W3")) : 1;     // 0 off, 2 every token exact
  static const float w3kappa = getenv("FLAGROT_W3_KAPPA") != nullptr ? static_cast<float>(atof(getenv("FLAGROT_W3_KAPPA"))) : W3_KAPPA;
  if (w3mode != 0 && p.screen && (p.passes & 1) && static_cast<long long>(p.T) * p.Hkv > 1024) {
    int tile = W3_TOK;
    while (tile < W3_MAXTILE && static_cast<long long>(p.Hkv) * ((p.T + tile - 1) / tile) > 512) tile *= 2;
    hipLaunchKernelGGL((k_k2_screen<QM, P>), dim3(p.Hkv, (p.T + tile - 1) / tile), dim3(256), 0, st, p, tile,
                       w3mode == 2 ? 1e30f : w3kappa);
    return hipPeekAtLastError() == hipSuccess ? 0 : -1;
  }
  // a decode step's worth of tokens: four half waves per (token, head), at most two workgroups per CU in one round
  static const bool no_ll = getenv("FLAGROT_WRITER_LL") != nullptr && getenv("FLAGROT_WRITER_LL")[0] == '0';
  if (!no_ll && static_cast<long long>(p.T) * p.Hkv <= 1024) {
    hipLaunchKernelGGL(kll, dim3(p.Hkv, (p.T + 1) / 2), dim3(256), K2LL_LDS, st, p);
    return hipPeekAtLastError() == hipSuccess ? 0 : -1;
  }
  // tokens per workgroup: enough workgroups to fill 256 CUs twice, at least one round of 8 rows each
  int tpw = K2_ROWS;
  while (tpw < 128 && static_cast<long long>(p.Hkv) * ((p.T + 2 * tpw - 1) / (2 * tpw)) >= 1024) tpw *= 2;
  dim3 grid(p.Hkv, (p.T + tpw - 1) / tpw);
  hipLaunchKernelGGL(k, grid, dim3(256), K2_LDS, st, p, tpw);
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}
template <int QM>
int k2_write_qm(const K2WriteParams& p, hipStream_t st) {
  if (p.hd == 256) {
    if (p.passes != 3) return -8;                          // the two-pass forms exist for 128-d heads only
    const dim3 grid(p.Hkv, (p.T + 7) / 8);
    if (p.page == 16) hipLaunchKernelGGL((k_k2_write256<QM, 16>), grid, dim3(256), 0, st, p);
    else if (p.page == 32) hipLaunchKernelGGL((k_k2_write256<QM, 32>), grid, dim3(256), 0, st, p);
    else return -5;
    return hipPeekAtLastError() == hipSuccess ? 0 : -1;
  }
  if (p.page == 16) return k2_write_p<QM, 16>(p, st);
  if (p.page == 32) return k2_write_p<QM, 32>(p, st);
  return -5;
}

}  // namespace

int static_write_launch(int fmt, const StaticWriteParams& p, hipStream_t st) {
  switch (fmt) {
    case FMT_INT4: return static_write_qm<QM_SYM4>(p, st);
    case FMT_INT4A: return static_write_qm<QM_ASYM4>(p, st);
    case FMT_INT2A: return static_write_qm<QM_ASYM2>(p, st);
  }
  return -4;
}

int k2_write_launch(int kind, const K2WriteParams& p, hipStream_t st) {
  switch (kind) {
    case KIND_KONLY: return k2_write_qm<QM_SYM4>(p, st);
    case KIND_KONLYA: return k2_write_qm<QM_ASYM4>(p, st);
    case KIND_KONLYA2: return k2_write_qm<QM_ASYM2>(p, st);
  }
  return -4;
}
int k2_write_lds_bytes(int hd) {      // LDS a selecting-writer workgroup holds (the 256-d kernel: its error strips; C_q^T stays in L2)
  return hd == 256 ? static_cast<int>(8 * 2 * 256 * sizeof(float)) : K2_LDS;
}

int head_fwht_launch(const void* x, long long x_ts, void* out, long long o_ts, int T, int H, const uint8_t* flags,
                     float scale, hipStream_t st, int D) {
  const long long rows = static_cast<long long>(T) * H;
  const unsigned grid = static_cast<unsigned>((rows + 7) / 8);
  if (D == 128)
    hipLaunchKernelGGL((k_head_fwht<128>), dim3(grid), dim3(256), 0, st, static_cast<const uint16_t*>(x), x_ts,
                       static_cast<uint16_t*>(out), o_ts, T, H, flags, scale);
  else if (D == 256)
    hipLaunchKernelGGL((k_head_fwht<256>), dim3(grid), dim3(256), 0, st, static_cast<const uint16_t*>(x), x_ts,
                       static_cast<uint16_t*>(out), o_ts, T, H, flags, scale);
  else
    return -8;
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

}  // namespace fr
