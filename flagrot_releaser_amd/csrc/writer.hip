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
  const int l32 = threadIdx.x & 31;
  const long long row = static_cast<long long>(blockIdx.x) * 8 + (threadIdx.x >> 5);
  const int H2 = 2 * p.Hkv;
  if (row >= static_cast<long long>(p.T) * H2) return;
  const int t = static_cast<int>(row / H2), hr = static_cast<int>(row % H2);
  const long long slot = p.slots[t];
  if (slot < 0) return;
  const bool isv = hr >= p.Hkv;
  const int head = isv ? hr - p.Hkv : hr;
  uint8_t* chunk = p.pool + ((slot / P) * p.Hkv + head) * L::CHUNK;
  const int pos = static_cast<int>(slot % P);

  float x[4];
  load_row(p.kv, static_cast<long long>(t) * p.kv_ts + hr * 128 + 4 * l32, x);
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
  store_row<QM, P>(chunk, pos, isv, code, word, l32, false);
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
  for (int t = t_lo + hw; t < t_hi; t += K2_ROWS) {
    const long long slot = p.slots[static_cast<long long>(t) * (p.slot_ph ? p.Hkv : 1) + (p.slot_ph ? h : 0)];
    if (slot < 0) continue;
    uint8_t* chunk = p.pool + ((slot / P) * p.Hkv + h) * L::CHUNK;
    const int pos = static_cast<int>(slot % P);
    bool key_full = false;
    if (do_k) {
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

template <int QM>
int static_write_qm(const StaticWriteParams& p, hipStream_t st) {
  const long long rows = static_cast<long long>(p.T) * 2 * p.Hkv;
  const unsigned grid = static_cast<unsigned>((rows + 7) / 8);
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
int k2_write_lds_bytes() { return K2_LDS; }

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
