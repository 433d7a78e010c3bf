// Paged split-K decode attention over KIVI-style FlagRot INT2 pages for gfx950 (wave64, no matrix cores): the page
// splits and the BF16 ring rows (one more split).  (The split merge and the C ABI live in kivi_attn.hip.)
//
// Workgroup = 4 wavefronts per (sequence, KV head x tile of up to 4 query heads, split); a wavefront owns whole
// 32-token groups (two pages) and keeps its own running maximum, sum and accumulators; the wavefronts are merged
// through LDS at the end.  (Tiles of 4 heads keep the three accumulator classes in registers at 3 waves per SIMD; a
// GQA group of 8 reads its pages twice, which the path can afford: it is instruction bound, not bandwidth bound.)
// Per group:
//   q' * scale   lane = channel pair: the group's channel scales are folded into the query rotation the group's flags
//                select (identity / H32 per sub-vector / H128; the three rotations are made once per workgroup), stored
//                as fp16 pairs; q' . min becomes a per-head bias.
//   scores       lane = (token, 64-channel half): a 2-bit code field masked in place is an fp16 DENORMAL whose value is
//                code * 2^(shift - 24); the power of two is folded into the fp16 query operand, so a pair of codes costs
//                one v_and and feeds v_dot2_f32_f16 directly (exact products, fp32 accumulation).
//   softmax      exp2-domain, the running maximum is re-reduced only when some token beats it.
//   values       tokens of a (group, sub-vector) are ordered by class (stored as is / H32 / H128) with ballots; p * scale,
//                p * min (fp16) and the token's 8 code bytes are written in that order, so that lane = 4 channels walks
//                PAIRS of tokens of one class: the two code bytes are merged and masked into four denormal pairs,
//                contracted with v_dot2 into the accumulators of that class.  o = accI + H32(accH) + H128(accF) once per workgroup.
// Semantics follow integrations/vllm_flagrot/csrc/kivi.cu:729-980 (k_attn).
#include "fr_common.hpp"
#include "kivi_launch.hpp"

namespace frkv {
using namespace fr;
namespace {

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
DEVI uint32_t pack_rn(float a, float b) {
  half2_t v = {static_cast<_Float16>(a), static_cast<_Float16>(b)};
  return __builtin_bit_cast(uint32_t, v);
}
template <class T> DEVI T gload(const uint8_t* p) {
  typedef const __attribute__((address_space(1))) T* gp;
  return *(gp)(p);
}
constexpr int CHUNK = 1552, KM_OFF = 512, VC_OFF = 768, VM_OFF = 1280, VF_OFF = 1536;
constexpr int NPAIR = 18;                       // token pairs per (group, sub-vector): 32 tokens + two odd-class pads

template <int G> struct Scr {                   // per wavefront; G = heads of the tile (<= 4)
  uint32_t qs[G][64];                           // fp16 pairs of q' * scale * 2^-shift, per (head, channel pair)
  alignas(16) uint32_t pp[4][NPAIR][4];         // (p * scale) of the pair's two tokens, per (sub-vector, pair, head)
  alignas(16) uint32_t pm[4][NPAIR][4];         // (p * min)
  alignas(8) uint8_t vord[4][2 * NPAIR][8];     // the 8 code bytes of (sub-vector, slot)
  int cnt[4][2];                                // tokens of class 0 / 1 per sub-vector
};
template <int G> struct Smem {
  float qv[3][G][128];                          // query rotations (fp32)
  Scr<G> w[4];
  float ob[3][G][128];                          // merged accumulators per class
  float mw[4][G], lw[4][G];
};

struct GroupRegs {
  u32x4 kc;      // lane (token, half): the token's 4 code words of its 64 channels
  u32x2 km;      // lane = channel pair: (scale | min << 16) of channels 2 l, 2 l + 1
  u32x4 vc;      // lane (token, half): the token's code bytes of sub-vectors 2 half, 2 half + 1
  u32x2 vm;      // lane (token, half): (scale | min << 16) of sub-vectors 2 half, 2 half + 1
  uint32_t vf;   // the token's whole-head flag byte
};

DEVI void load_group(GroupRegs& r, const uint8_t* chA, const uint8_t* chB, int lane) {
  const int t = lane & 31, hh = lane >> 5;
  const uint8_t* cht = t < 16 ? chA : chB;
  r.kc = gload<u32x4>(cht + (t & 15) * 32 + 16 * hh);
  r.km = gload<u32x2>((lane < 32 ? chA : chB) + KM_OFF + (lane & 31) * 8);
  r.vc = gload<u32x4>(cht + VC_OFF + (t & 15) * 32 + 16 * hh);
  r.vm = gload<u32x2>(cht + VM_OFF + (t & 15) * 16 + 8 * hh);
  r.vf = gload<uint8_t>(cht + VF_OFF + (t & 15));
}

// The BF16 ring rows of one sequence (split index NS): rows [0, tail_len) of ring block tail_idx, K row h, V row Hkv + h,
// original basis.  A wavefront takes every fourth row, lanes own 2 dims; same partial format as the page splits.
template <int G>
DEVI void tail_split(Smem<G>& S, const uint16_t* __restrict__ q, long long q_rs, const uint16_t* __restrict__ ring,
                     const int* __restrict__ tail_len, const int* __restrict__ tail_idx, int T, int Hkv, int Gq, int b, int h,
                     int g0, float qscale, float* __restrict__ op, float* __restrict__ mlp) {
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
  const int n = tail_len != nullptr ? tail_len[b] : 0;
  if (n <= 0) {
    if (tid < G && g0 + tid < Gq) { mlp[2 * tid] = -INFINITY; mlp[2 * tid + 1] = 0.f; }
    return;
  }
  float qa[G], qb[G], m[G], l[G], oa[G], ob[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    qa[g] = qb[g] = 0.f;
    if (g0 + g < Gq) {
      const uint32_t raw = *reinterpret_cast<const uint32_t*>(q + static_cast<long long>(b) * q_rs + (static_cast<long long>(h) * Gq + g0 + g) * 128 + 2 * lane);
      qa[g] = bf16_lo(raw) * qscale; qb[g] = bf16_hi(raw) * qscale;
    }
    m[g] = -INFINITY; l[g] = 0.f; oa[g] = ob[g] = 0.f;
  }
  const uint16_t* rbase = ring + static_cast<long long>(tail_idx != nullptr ? tail_idx[b] : 0) * T * 2 * Hkv * 128;
  for (int t = wv; t < n; t += 4) {
    const uint16_t* row = rbase + static_cast<long long>(t) * 2 * Hkv * 128;
    const uint32_t kr = *reinterpret_cast<const uint32_t*>(row + h * 128 + 2 * lane);
    const uint32_t vr = *reinterpret_cast<const uint32_t*>(row + (Hkv + h) * 128 + 2 * lane);
    const float k0 = bf16_lo(kr), k1 = bf16_hi(kr), v0 = bf16_lo(vr), v1 = bf16_hi(vr);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float sc = wave_sum64(qa[g] * k0 + qb[g] * k1);
      const float mn = fmaxf(m[g], sc);
      const float alpha = m[g] == -INFINITY ? 0.f : fexp2(m[g] - mn), p = fexp2(sc - mn);
      l[g] = l[g] * alpha + p;
      oa[g] = oa[g] * alpha + p * v0;
      ob[g] = ob[g] * alpha + p * v1;
      m[g] = mn;
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
        float2* dst = reinterpret_cast<float2*>(&S.ob[0][g][2 * lane]);
        float2 acc = make_float2(0.f, 0.f);
        if (r) acc = *dst;
        *dst = make_float2(acc.x + f * oa[g], acc.y + f * ob[g]);
      }
    }
    __syncthreads();
  }
  for (int g = wv; g < G && g0 + g < Gq; g += 4) {
    *reinterpret_cast<float2*>(op + g * 128 + 2 * lane) = *reinterpret_cast<const float2*>(&S.ob[0][g][2 * lane]);
    if (lane == 0) {
      const float M = fmaxf(fmaxf(S.mw[0][g], S.mw[1][g]), fmaxf(S.mw[2][g], S.mw[3][g]));
      float L = 0.f;
      for (int w = 0; w < 4; ++w) L += S.mw[w][g] == -INFINITY ? 0.f : fexp2(S.mw[w][g] - M) * S.lw[w][g];
      mlp[2 * g] = M; mlp[2 * g + 1] = L;
    }
  }
}

template <int G>
__global__ void __launch_bounds__(256, 3) k_attn_pages(const uint16_t* __restrict__ q, long long q_rs,
                                                    const uint8_t* __restrict__ pool, const int* __restrict__ bt,
                                                    long long bt_rs, const int* __restrict__ cached, int kv_start, int Hkv,
                                                    int NS, int chunk, float qscale, float* __restrict__ opart,
                                                    float* __restrict__ ml, int Gq, int ntile,
                                                    const uint16_t* __restrict__ ring, const int* __restrict__ tail_len,
                                                    const int* __restrict__ tail_idx, int T) {
  constexpr int GP = 4;
  extern __shared__ __align__(16) uint8_t lds[];
  Smem<G>& S = *reinterpret_cast<Smem<G>*>(lds);
  const int b = blockIdx.x, h = blockIdx.y / ntile, g0 = (blockIdx.y % ntile) * G, sp = blockIdx.z;   // heads g0 .. g0 + G - 1
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
  const long long pidx = (static_cast<long long>(b) * Hkv + h) * (NS + 1) + sp;
  float* op = opart + (pidx * Gq + g0) * 128;
  float* mlp = ml + (pidx * Gq + g0) * 2;
  if (sp == NS) {
    tail_split<G>(S, q, q_rs, ring, tail_len, tail_idx, T, Hkv, Gq, b, h, g0, qscale, op, mlp);
    return;
  }
  const int t0 = max(sp * chunk, kv_start), t1 = min((sp + 1) * chunk, cached[b]);
  if (t1 <= t0) {
    if (tid < G && g0 + tid < Gq) { mlp[2 * tid] = -INFINITY; mlp[2 * tid + 1] = 0.f; }
    return;
  }
  // query rotations: half wave per (variant, head)
  for (int r = tid >> 5; r < 3 * G; r += 8) {
    const int var = r / G, g = r % G, lq = tid & 31;
    float x[4] = {0.f, 0.f, 0.f, 0.f};
    if (g0 + g < Gq) {
      const uint2 raw = *reinterpret_cast<const uint2*>(q + static_cast<long long>(b) * q_rs + (static_cast<long long>(h) * Gq + g0 + g) * 128 + 4 * lq);
      x[0] = bf16_lo(raw.x); x[1] = bf16_hi(raw.x); x[2] = bf16_lo(raw.y); x[3] = bf16_hi(raw.y);
    }
    if (var == 1) fwht<32>(x, lq);
    if (var == 2) fwht<128>(x, lq);
    *reinterpret_cast<float4*>(&S.qv[var][g][4 * lq]) = make_float4(x[0], x[1], x[2], x[3]);
  }
  __syncthreads();

  Scr<G>& W = S.w[wv];
  float m_run[G], l_run[G];
  float accI[G][4], accH[G][4], accF[G][4], mI[G], mH[G], mF[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m_run[g] = -INFINITY; l_run[g] = 0.f; mI[g] = mH[g] = mF[g] = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) accI[g][k] = accH[g][k] = accF[g][k] = 0.f;
  }
  const int* btb = bt + static_cast<long long>(b) * bt_rs;
  const int g_first = t0 / 32, g_end = (t1 + 31) / 32;
  // power of two folded into the query operand of this lane's channel pair (pair k = lane & 7 of its word):
  // fields 0..4 are masked in place (code * 2^(2k - 24)), fields 5..7 after a shift by 10 (code * 2^(2(k-5) - 24))
  const int kq = lane & 7;
  const float qfold = __uint_as_float((127u - 2u * static_cast<uint32_t>(kq < 5 ? kq : kq - 5)) << 23);
  const int jv = l32 >> 3;                                  // sub-vector of this lane's 4 value channels

  GroupRegs cur;
  int gi = g_first + wv;
  if (gi < g_end) load_group(cur, pool + (static_cast<long long>(btb[2 * gi]) * Hkv + h) * CHUNK,
                             pool + (static_cast<long long>(btb[2 * gi + 1]) * Hkv + h) * CHUNK, lane);
  for (; gi < g_end; gi += 4) {
    GroupRegs nxt;
    if (gi + 4 < g_end) load_group(nxt, pool + (static_cast<long long>(btb[2 * (gi + 4)]) * Hkv + h) * CHUNK,
                                   pool + (static_cast<long long>(btb[2 * (gi + 4) + 1]) * Hkv + h) * CHUNK, lane);
    // ---- group flags, q' * scale, bias
    const uint32_t s0 = __builtin_amdgcn_readlane(cur.km.x, 0), s1 = __builtin_amdgcn_readlane(cur.km.y, 0),
                   s2 = __builtin_amdgcn_readlane(cur.km.x, 1), s3 = __builtin_amdgcn_readlane(cur.km.y, 1),
                   s4 = __builtin_amdgcn_readlane(cur.km.x, 2);
    const bool useF = (s4 >> 15) & 1u;
    const uint32_t lmask = ((s0 >> 15) & 1u) | (((s1 >> 15) & 1u) << 1) | (((s2 >> 15) & 1u) << 2) | (((s3 >> 15) & 1u) << 3);
    const int which = useF ? 2 : static_cast<int>((lmask >> (lane >> 4)) & 1u);
    const float sa = f16_value(cur.km.x & 0x7FFFu), ma = f16_value(cur.km.x >> 16);
    const float sb = f16_value(cur.km.y & 0x7FFFu), mb = f16_value(cur.km.y >> 16);
    float bias[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float2 qq = *reinterpret_cast<const float2*>(&S.qv[which][g][2 * lane]);
      W.qs[g][lane] = pack_rn(qq.x * sa * qfold, qq.y * sb * qfold);
      bias[g] = wave_sum64(qq.x * ma + qq.y * mb);
    }
    // reset of the ordered strips (the pad slots of odd classes must weigh nothing)
    for (int i = lane; i < 2 * 4 * NPAIR * GP / 4; i += 64) reinterpret_cast<u32x4*>(&W.pp[0][0][0])[i] = u32x4{0u, 0u, 0u, 0u};
    wave_lds_sync();
    // ---- scores: lane = (token l32, channel half hh)
    float a[G];
#pragma unroll
    for (int g = 0; g < G; ++g) a[g] = 0.f;
#pragma unroll
    for (int wi = 0; wi < 4; ++wi) {
      const uint32_t w = cur.kc[wi], w10 = w >> 10;
      const uint32_t x[8] = {w & 0x00030003u, w & 0x000C000Cu, w & 0x00300030u, w & 0x00C000C0u, w & 0x03000300u,
                             w10 & 0x00030003u, w10 & 0x000C000Cu, w10 & 0x00300030u};
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const u32x4 qa = *reinterpret_cast<const u32x4*>(&W.qs[g][8 * (4 * hh + wi)]);
        const u32x4 qb = *reinterpret_cast<const u32x4*>(&W.qs[g][8 * (4 * hh + wi) + 4]);
        float v = a[g];
        v = dot2(x[0], qa.x, v); v = dot2(x[1], qa.y, v); v = dot2(x[2], qa.z, v); v = dot2(x[3], qa.w, v);
        v = dot2(x[4], qb.x, v); v = dot2(x[5], qb.y, v); v = dot2(x[6], qb.z, v); v = dot2(x[7], qb.w, v);
        a[g] = v;
      }
    }
    const int pos = gi * 32 + l32;
    const bool valid = pos >= t0 && pos < t1;
    float sc[G];
    bool beat = false;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float tot = (a[g] + __shfl_xor(a[g], 32, 64)) * 16777216.f + bias[g];
      sc[g] = valid ? tot * qscale : -INFINITY;
      beat |= sc[g] > m_run[g];
    }
    if (__any(beat)) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float mn = fmaxf(m_run[g], wave_max64(sc[g]));
        const float alpha = m_run[g] == -INFINITY ? 0.f : fexp2(m_run[g] - mn);
        m_run[g] = mn;
        l_run[g] *= alpha;
        mI[g] *= alpha; mH[g] *= alpha; mF[g] *= alpha;
#pragma unroll
        for (int k = 0; k < 4; ++k) { accI[g][k] *= alpha; accH[g][k] *= alpha; accF[g][k] *= alpha; }
      }
    }
    // ---- p, class order, ordered strips: lane (token, half) serves sub-vectors 2 hh, 2 hh + 1
    uint32_t ph[GP / 2];                                    // p as fp16 pairs of heads
    {
      float p[GP];
#pragma unroll
      for (int g = 0; g < GP; ++g) p[g] = 0.f;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        p[g] = valid ? fexp2(sc[g] - m_run[g]) : 0.f;
        if (hh == 0) l_run[g] += p[g];
      }
#pragma unroll
      for (int g2 = 0; g2 < GP / 2; ++g2) ph[g2] = pack_rn(p[2 * g2], p[2 * g2 + 1]);
    }
    const bool vF = cur.vf != 0;
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const uint32_t w = jj ? cur.vm.y : cur.vm.x;
      const int j = 2 * hh + jj;
      const int cls = vF ? 2 : static_cast<int>((w >> 15) & 1u);
      const unsigned long long b0 = __ballot(cls == 0), b1 = __ballot(cls == 1), b2 = __ballot(cls == 2);
      const uint32_t m0 = static_cast<uint32_t>(hh ? (b0 >> 32) : b0), m1 = static_cast<uint32_t>(hh ? (b1 >> 32) : b1),
                     m2 = static_cast<uint32_t>(hh ? (b2 >> 32) : b2);
      const uint32_t below = (1u << l32) - 1u;
      const int n0 = __popc(m0), n1 = __popc(m1);
      const int base1 = (n0 + 1) & ~1, base2 = base1 + ((n1 + 1) & ~1);
      const int slot = cls == 0 ? __popc(m0 & below) : cls == 1 ? base1 + __popc(m1 & below) : base2 + __popc(m2 & below);
      *reinterpret_cast<u32x2*>(&W.vord[j][slot][0]) = jj ? u32x2{cur.vc.z, cur.vc.w} : u32x2{cur.vc.x, cur.vc.y};
      if (l32 == 0) { W.cnt[j][0] = n0; W.cnt[j][1] = n1; }
      const uint32_t s2x = (w & 0x7FFFu) * 0x10001u, m2x = (w >> 16) * 0x10001u;
      _Float16* dp = reinterpret_cast<_Float16*>(&W.pp[j][slot >> 1][0]) + (slot & 1);
      _Float16* dm = reinterpret_cast<_Float16*>(&W.pm[j][slot >> 1][0]) + (slot & 1);
#pragma unroll
      for (int g2 = 0; g2 < GP / 2; ++g2) {
        const half2_t ps = __builtin_bit_cast(half2_t, pk_mul(ph[g2], s2x));
        const half2_t pn = __builtin_bit_cast(half2_t, pk_mul(ph[g2], m2x));
        dp[4 * g2] = ps.x; dp[4 * g2 + 2] = ps.y;
        dm[4 * g2] = pn.x; dm[4 * g2 + 2] = pn.y;
      }
    }
    wave_lds_sync();
    // ---- values: lane = (4 channels of byte l32, pair parity hh)
    {
      const int n0 = W.cnt[jv][0], n1 = W.cnt[jv][1];
      const int e0 = (n0 + 1) >> 1, e1 = e0 + ((n1 + 1) >> 1), e2 = e1 + ((32 - n0 - n1 + 1) >> 1);
      // every lane walks its own pair range in lockstep; lanes past their range contribute zero operands (no
      // divergent control flow: the accumulators stay in place)
      auto run = [&](int kb, int ke, float (&acc)[G][4], float (&am)[G]) {
        int kp = kb + ((kb ^ hh) & 1);
        int nit = max(0, (ke - kp + 1) >> 1);
        nit = max(nit, __builtin_amdgcn_ds_swizzle(nit, (8 << 10) | 0x1F));      // other sub-vectors
        nit = max(nit, __builtin_amdgcn_ds_swizzle(nit, (16 << 10) | 0x1F));
        nit = max(nit, __shfl_xor(nit, 32, 64));                                   // other pair parity
        nit = __builtin_amdgcn_readfirstlane(nit);
        for (int it = 0; it < nit; ++it, kp += 2) {
          const bool live = kp < ke;
          const int kr = live ? kp : 0;
          uint32_t comb = static_cast<uint32_t>(W.vord[jv][2 * kr][l32 & 7]) |
                          (static_cast<uint32_t>(W.vord[jv][2 * kr + 1][l32 & 7]) << 16);
          comb = live ? comb : 0u;
          const uint32_t ones = live ? 0x3C003C00u : 0u;
          const uint32_t x0 = comb & 0x00030003u, x1 = comb & 0x000C000Cu, x2 = comb & 0x00300030u, x3 = comb & 0x00C000C0u;
          const u32x4 pq = *reinterpret_cast<const u32x4*>(&W.pp[jv][kr][0]);
          const u32x4 mq = *reinterpret_cast<const u32x4*>(&W.pm[jv][kr][0]);
#pragma unroll
          for (int g = 0; g < G; ++g) {
            const uint32_t pv = pq[g];
            acc[g][0] = dot2(x0, pv, acc[g][0]);
            acc[g][1] = dot2(x1, pv, acc[g][1]);
            acc[g][2] = dot2(x2, pv, acc[g][2]);
            acc[g][3] = dot2(x3, pv, acc[g][3]);
            am[g] = dot2(ones, mq[g], am[g]);
          }
        }
      };
      run(0, e0, accI, mI);
      run(e0, e1, accH, mH);
      run(e1, e2, accF, mF);
    }
    wave_lds_sync();
    cur = nxt;
  }

  // ---- merge of the wavefronts: maxima, sums, accumulators per class (in wavefront order), inverse transforms
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const float lt = wave_sum64(l_run[g]);
    if (lane == 0) { S.mw[wv][g] = m_run[g]; S.lw[wv][g] = lt; }
  }
  __syncthreads();
  float fac[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const float M = fmaxf(fmaxf(S.mw[0][g], S.mw[1][g]), fmaxf(S.mw[2][g], S.mw[3][g]));
    fac[g] = m_run[g] == -INFINITY ? 0.f : fexp2(m_run[g] - M);
  }
  for (int r = 0; r < 4; ++r) {
    if (wv == r) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float vi[4], vh[4], vf[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float up = __uint_as_float((127u + 24u - 2u * k) << 23);          // 2^(24 - 2k)
          vi[k] = accI[g][k] * up + mI[g]; vh[k] = accH[g][k] * up + mH[g]; vf[k] = accF[g][k] * up + mF[g];
          vi[k] += __shfl_xor(vi[k], 32, 64); vh[k] += __shfl_xor(vh[k], 32, 64); vf[k] += __shfl_xor(vf[k], 32, 64);
          vi[k] *= fac[g]; vh[k] *= fac[g]; vf[k] *= fac[g];
        }
        if (hh == 0) {
          float4* pI = reinterpret_cast<float4*>(&S.ob[0][g][4 * l32]);
          float4* pH = reinterpret_cast<float4*>(&S.ob[1][g][4 * l32]);
          float4* pF = reinterpret_cast<float4*>(&S.ob[2][g][4 * l32]);
          float4 a4 = make_float4(0.f, 0.f, 0.f, 0.f), b4 = a4, c4 = a4;
          if (r) { a4 = *pI; b4 = *pH; c4 = *pF; }
          *pI = make_float4(a4.x + vi[0], a4.y + vi[1], a4.z + vi[2], a4.w + vi[3]);
          *pH = make_float4(b4.x + vh[0], b4.y + vh[1], b4.z + vh[2], b4.w + vh[3]);
          *pF = make_float4(c4.x + vf[0], c4.y + vf[1], c4.z + vf[2], c4.w + vf[3]);
        }
      }
    }
    __syncthreads();
  }
  for (int g = tid >> 5; g < G && g0 + g < Gq; g += 8) {
    const int lq = tid & 31;
    const float4 a4 = *reinterpret_cast<const float4*>(&S.ob[0][g][4 * lq]);
    const float4 b4 = *reinterpret_cast<const float4*>(&S.ob[1][g][4 * lq]);
    const float4 c4 = *reinterpret_cast<const float4*>(&S.ob[2][g][4 * lq]);
    float yh[4] = {b4.x, b4.y, b4.z, b4.w}, yf[4] = {c4.x, c4.y, c4.z, c4.w};
    fwht<32>(yh, lq);
    fwht<128>(yf, lq);
    *reinterpret_cast<float4*>(op + g * 128 + 4 * lq) = make_float4(a4.x + yh[0] + yf[0], a4.y + yh[1] + yf[1], a4.z + yh[2] + yf[2], a4.w + yh[3] + yf[3]);
    if (lq == 0) {
      const float M = fmaxf(fmaxf(S.mw[0][g], S.mw[1][g]), fmaxf(S.mw[2][g], S.mw[3][g]));
      float L = 0.f;
      for (int w = 0; w < 4; ++w) L += S.mw[w][g] == -INFINITY ? 0.f : fexp2(S.mw[w][g] - M) * S.lw[w][g];
      mlp[2 * g] = M; mlp[2 * g + 1] = L;
    }
  }
}

template <int G>
int launch_pages(int Gq, const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs, const void* cached,
                 int kv_start, int B, int Hkv, int NS, int chunk, float qscale, const void* ring, const void* tail_len,
                 const void* tail_idx, int T, void* opart, void* ml, hipStream_t st) {
  static bool attr = false;
  if (!attr) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_attn_pages<G>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(sizeof(Smem<G>))) != hipSuccess) return 1;
    attr = true;
  }
  const int ntile = (Gq + G - 1) / G;
  hipLaunchKernelGGL(k_attn_pages<G>, dim3(B, Hkv * ntile, NS + 1), dim3(256), sizeof(Smem<G>), st, static_cast<const uint16_t*>(q), q_rs,
                     static_cast<const uint8_t*>(pool), static_cast<const int*>(bt), bt_rs, static_cast<const int*>(cached),
                     kv_start, Hkv, NS, chunk, qscale, static_cast<float*>(opart), static_cast<float*>(ml), Gq, ntile,
                     static_cast<const uint16_t*>(ring), static_cast<const int*>(tail_len), static_cast<const int*>(tail_idx), T);
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

}  // namespace

int attn_splits_launch(int G, const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs,
                       const void* cached, int kv_start, int B, int Hkv, int NS, int chunk, float qscale, const void* ring,
                       const void* tail_len, const void* tail_idx, int T, void* opart, void* ml, hipStream_t st) {
  // heads per tile: a GQA group of up to 4 in one tile, of 5 .. 8 in two
  const int gt = G <= 4 ? G : (G + 1) / 2;
#define FRKV_P(GG) case GG: return launch_pages<GG>(G, q, q_rs, pool, bt, bt_rs, cached, kv_start, B, Hkv, NS, chunk, qscale, ring, tail_len, tail_idx, T, opart, ml, st);
  switch (gt) {
    FRKV_P(1) FRKV_P(2) FRKV_P(3) FRKV_P(4)
    default: return 2;
  }
#undef FRKV_P
}

}  // namespace frkv
