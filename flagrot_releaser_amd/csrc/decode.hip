// Paged split-K GQA decode attention over FlagRot INT4 / INT2 pages for gfx950 (wave64, no matrix cores).
//
// One workgroup (4 wavefronts) per (KV head x q tile of 4 heads, split, sequence).  A wavefront streams whole pages
// (16 tokens x one KV head = one contiguous 2304 / 1280 byte chunk) with 128-bit loads:
//   key phase    lane = (token, quarter): 16 B of the token's code row = 8 elements of each 32-group.  The codes are
//                turned into fp16 pairs by mask-and-or with an exponent pattern (value = offset + code, exact) and
//                contracted with the query by v_dot2_f32_f16.  The query is rotated three ways once per workgroup
//                (identity, H32 per group, H128) and kept in LDS in the code words' element order; every lane fetches
//                the variant its token / group flags ask for, so selection costs no arithmetic.  The exponent offsets
//                and the zero points are removed with per-(variant, head, group) query sums.
//   softmax      exp2-domain online softmax per wavefront; p * V-scale is written to LDS as fp16 in V^T token order.
//   value phase  lane = one 16-byte V^T entry (4 dims x 8 tokens): the same unpacking, contracted with p * scale over
//                the tokens; offsets / zero points are removed once per workgroup from running per-group sums.
// The four wavefronts are merged through LDS; splits through the caller's workspace with a ticket counter (the last
// arriving workgroup of a (sequence, KV head) merges, normalises, optionally rotates back, and stores bf16).
// The BF16 sink / window rows are one more split handled by an extra workgroup of the same grid.
//
// Semantics follow the reference's decode entry points: integrations/vllm_flagrot/csrc/flagrot_capi.cu:19-64,131-149,
// kernels/csrc/attn_codebook_attn.cuh:2093-2126 (per-(token, group) variant selection), attn_merge.cuh:23-84.
#include "fr_common.hpp"
#include "fr_launch.hpp"

namespace fr {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

DEVI half2_t as_h2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
DEVI float dot2(uint32_t a, uint32_t b, float c) { return __builtin_amdgcn_fdot2(as_h2(a), as_h2(b), c, false); }
DEVI float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }

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
DEVI void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------------------------------------- code unpacking
// A 32-bit word of eight 4-bit fields f0..f7 (or, INT2, the 2-bit fields at bit 4 n of a pre-shifted word) becomes
// four fp16 pairs (f0,f4) (f1,f5) (f2,f6) (f3,f7): the field is or-ed into the mantissa of 1024.0 (exact), then
// -(1024 + zero point) is added with one packed fp16 add, which is exact too: the pairs hold code - zero point.
DEVI uint32_t pk_add(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, as_h2(a) + as_h2(b));
}
template <int QM> struct Unpack;
template <> struct Unpack<QM_ASYM4> {
  static DEVI void run(uint32_t w, const uint32_t (&nz)[4], uint32_t (&x)[4]) {
    x[0] = pk_add((w & 0x000F000Fu) | 0x64006400u, nz[0]);
    x[1] = pk_add(((w >> 4) & 0x000F000Fu) | 0x64006400u, nz[1]);
    x[2] = pk_add(((w >> 8) & 0x000F000Fu) | 0x64006400u, nz[2]);
    x[3] = pk_add(((w >> 12) & 0x000F000Fu) | 0x64006400u, nz[3]);
  }
};
template <> struct Unpack<QM_ASYM2> {
  static DEVI void run(uint32_t w, const uint32_t (&nz)[4], uint32_t (&x)[4]) {  // fields at bits 0, 2, 8, 10 (+16)
    x[0] = pk_add((w & 0x00030003u) | 0x64006400u, nz[0]);
    x[1] = pk_add(((w >> 2) & 0x00030003u) | 0x64006400u, nz[1]);
    x[2] = pk_add(((w >> 8) & 0x00030003u) | 0x64006400u, nz[2]);
    x[3] = pk_add(((w >> 10) & 0x00030003u) | 0x64006400u, nz[3]);
  }
};
template <> struct Unpack<QM_SYM4> {  // sign-magnitude bytes s0000mmm -> exact signed fp16
  static DEVI uint32_t pair(uint32_t bytes02) {  // bytes at bits 0..7 and 16..23
    const uint32_t m = pk_add((bytes02 & 0x00070007u) | 0x64006400u, 0xE400E400u);
    return m ^ ((bytes02 & 0x00800080u) << 8);
  }
  static DEVI void run(uint32_t w, const uint32_t (&)[4], uint32_t (&x)[4]) {
    const uint32_t a = w & 0x87878787u;                                   // A_i in byte i
    const uint32_t b = ((w << 4) | (w >> 28)) & 0x87878787u;              // B_i in byte i
    x[0] = pair(a); x[1] = pair(b); x[2] = pair(a >> 8); x[3] = pair(b >> 8);
  }
};
// fp16 pattern of -(1024 + z)
DEVI uint32_t negz16(uint32_t z) { return 0xE400u | z; }

constexpr int NWAVE = 4;
constexpr int QV_BYTES = 3 * 4 * 16 * 16;          // [variant][head][tg][j][8 fp16]
constexpr int PB_BYTES = 2 * 4 * 4 * 16;           // per wave: [c8][group][head][8 fp16]
constexpr int ZB_BYTES = 2 * 4 * 16;               // per wave: [c8][group][8 fp16] = -(1024 + zero point) per token

struct Smem {
  alignas(16) uint8_t qv[QV_BYTES];
  alignas(16) uint8_t pb[NWAVE][PB_BYTES];
  alignas(16) uint8_t zb[NWAVE][ZB_BYTES];
  alignas(16) float o[NWAVE][4][128];
  float m[NWAVE][4], l[NWAVE][4];
  int last;
};

// slot of element (isB, i) of a K word / of token r8 of a V word inside the 8-fp16 operand vector
DEVI int kslot(int isB, int i) { return 2 * (2 * (i & 1) + isB) + (i >> 1); }
DEVI int vslot(int r8) { return 2 * (r8 & 3) + (r8 >> 2); }

// Rotates the q tile three ways and stores it as fp16 in code-word order (the identity variant of a bf16 query is
// exact in fp16; qscale is applied to the fp32 score).
template <int QM, bool K2>
DEVI void q_prologue(Smem& S, const DecodeParams& p, int b, int kvh, int tile) {
  const int w = threadIdx.x >> 6, half = (threadIdx.x >> 5) & 1, l32 = threadIdx.x & 31;
  const int hq = tile * 4 + w;                       // head inside the GQA group
  float x[4] = {0.f, 0.f, 0.f, 0.f};
  if (hq < p.gqa) {
    const uint16_t* qr = static_cast<const uint16_t*>(p.q) + static_cast<long long>(b) * p.q_bs +
                         (static_cast<long long>(kvh) * p.gqa + hq) * 128 + 4 * l32;
    const uint2 raw = *reinterpret_cast<const uint2*>(qr);
    x[0] = bf16_lo(raw.x); x[1] = bf16_hi(raw.x); x[2] = bf16_lo(raw.y); x[3] = bf16_hi(raw.y);
  }
  const int g = l32 >> 3;
  // half 0: variants 0 (identity, or the static kmask rotation) and 1 (H32); half 1: variant 2 (H128)
  const int nvar = K2 ? (half == 0 ? 2 : 1) : (half == 0 ? 1 : 0);
  float y[4] = {x[0], x[1], x[2], x[3]};
  if (half == 0) fwht<32>(y, l32); else fwht<128>(y, l32);
  for (int vi = 0; vi < nvar; ++vi) {
    int var;
    float v[4];
    if (K2) {
      var = half == 0 ? vi : 2;
      const bool rot = var != 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = rot ? y[i] : x[i];
    } else {
      var = 0;
      const bool rot = p.kmask != nullptr && p.kmask[kvh * 4 + g] != 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = rot ? y[i] : x[i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = 4 * l32 + i, r = d & 31;
      const int isB = r >> 4, tg = (r & 15) >> 2, ii = r & 3;
      reinterpret_cast<_Float16*>(S.qv)[(((var * 4 + w) * 4 + tg) * 4 + g) * 8 + kslot(isB, ii)] = static_cast<_Float16>(v[i]);
    }
  }
}

template <int QM> struct PageRegs {
  uint32_t kc[QM == QM_ASYM2 ? 2 : 4];
  uint32_t vc[QM == QM_ASYM2 ? 2 : 4];
  uint2 ks;                 // the token's 4 K scale words
  uint32_t vs, vs0;         // V scale word of (token, group = quarter), of (token, group 0)
};

template <int QM, int P>
DEVI void load_page(PageRegs<QM>& r, const uint8_t* chunk, int lane) {
  using L = Lay<QM, P>;
  const int t = lane >> 2, tg = lane & 3;
  if constexpr (QM == QM_ASYM2) {
    const uint2 k = *reinterpret_cast<const uint2*>(chunk + L::K_OFF + 32 * (t ^ ((t >> 1) & 2)) + 8 * tg);
    r.kc[0] = k.x; r.kc[1] = k.y;
    const uint2 v = *reinterpret_cast<const uint2*>(chunk + L::V_OFF + 8 * lane);
    r.vc[0] = v.x; r.vc[1] = v.y;
  } else {
    const uint4 k = *reinterpret_cast<const uint4*>(chunk + L::K_OFF + 64 * t + 16 * tg);
    r.kc[0] = k.x; r.kc[1] = k.y; r.kc[2] = k.z; r.kc[3] = k.w;
    const uint4 v = *reinterpret_cast<const uint4*>(chunk + L::V_OFF + 16 * lane);
    r.vc[0] = v.x; r.vc[1] = v.y; r.vc[2] = v.z; r.vc[3] = v.w;
  }
  r.ks = *reinterpret_cast<const uint2*>(chunk + L::KS_OFF + 8 * t);
  const int vo = L::VS_OFF + (8 * (t >> 3) + vs_slot8(t)) * 2;
  r.vs = *reinterpret_cast<const uint16_t*>(chunk + vo + tg * P * 2);
  r.vs0 = *reinterpret_cast<const uint16_t*>(chunk + vo);
}

struct WaveState {
  float m[4], l[4];
  float acc[4][4];   // [head][entry word] of the lane's V^T entry
};

template <int QM, bool K2, int P>
DEVI void process_page(Smem& S, WaveState& st, const PageRegs<QM>& r, int lane, int wave, int tok0, int lo, int hi,
                       float qscale) {
  constexpr int ZM = QM == QM_ASYM4 ? 15 : QM == QM_ASYM2 ? 3 : 0;
  const int t = lane >> 2, tg = lane & 3;
  const uint32_t kw[4] = {r.ks.x & 0xFFFFu, r.ks.x >> 16, r.ks.y & 0xFFFFu, r.ks.y >> 16};
  const bool full = K2 && (r.vs0 & 0x8000u);
  float part[4] = {0.f, 0.f, 0.f, 0.f};
  // ---- key phase
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t x[4];
    const uint32_t nz1 = negz16(kw[j] & ZM) * 0x00010001u;
    const uint32_t nz[4] = {nz1, nz1, nz1, nz1};
    if constexpr (QM == QM_ASYM2) Unpack<QM>::run((j & 1) ? (r.kc[j >> 1] >> 4) : r.kc[j >> 1], nz, x);
    else Unpack<QM>::run(r.kc[j], nz, x);
    const int var = K2 ? (full ? 2 : static_cast<int>(kw[j] >> 15)) : 0;
    const float s = f16_value(kw[j] & 0x7FFFu);
    const uint4* qp = reinterpret_cast<const uint4*>(S.qv) + (var * 16 + tg) * 4 + j;   // + head * 16
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const uint4 qq = qp[h * 16];
      float a = dot2(x[0], qq.x, 0.f);
      a = dot2(x[1], qq.y, a);
      a = dot2(x[2], qq.z, a);
      a = dot2(x[3], qq.w, a);
      part[h] += s * a;
    }
  }
  const int tok = tok0 + t;
  const bool valid = tok >= lo && tok < hi;
  float p[4];
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    float sc = part[h];
    sc += dpp_xor1(sc);
    sc += dpp_xor2(sc);
    sc = valid ? sc * qscale : -INFINITY;
    const float mx = wave_max_over_tokens(sc);
    const float mn = fmaxf(st.m[h], mx);
    const float alpha = mn == -INFINITY ? 1.f : fexp2(st.m[h] - mn);
    p[h] = valid ? fexp2(sc - mn) : 0.f;
    st.m[h] = mn;
    st.l[h] = st.l[h] * alpha + wave_sum_over_tokens(p[h]);   // one lane per token: the exchange keeps the quarter
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) st.acc[h][s4] *= alpha;
  }
  // ---- p' = p * V scale of (token, group tg) as fp16, and -(1024 + zero point), into the wave's LDS strips in
  //      V^T token order
  {
    const float sv = f16_value(r.vs & 0x7FFFu);
    const int so = ((t >> 3) * 4 + tg) * 8 + vslot(t & 7);
    _Float16* pb = reinterpret_cast<_Float16*>(S.pb[wave]) + 4 * (so & ~7) + (so & 7);
#pragma unroll
    for (int h = 0; h < 4; ++h) pb[h * 8] = valid ? static_cast<_Float16>(p[h] * sv) : static_cast<_Float16>(0.f);
    if constexpr (QM != QM_SYM4) reinterpret_cast<uint16_t*>(S.zb[wave])[so] = static_cast<uint16_t>(negz16(r.vs & ZM));
  }
  wave_lds_sync();
  // ---- value phase: lane = V^T entry (w = lane >> 4, gid, c8 = lane & 1)
  {
    const int c8 = lane & 1, g0 = lane >> 5;
    const uint4* pp = reinterpret_cast<const uint4*>(S.pb[wave]) + (c8 * 4) * 4;   // + group * 4 + head
    uint4 pa[4], pc[4];
#pragma unroll
    for (int h = 0; h < 4; ++h) { pa[h] = pp[g0 * 4 + h]; pc[h] = pp[(2 + g0) * 4 + h]; }
    uint4 za = make_uint4(0, 0, 0, 0), zc = za;
    if constexpr (QM != QM_SYM4) {
      const uint4* zp = reinterpret_cast<const uint4*>(S.zb[wave]) + c8 * 4;
      za = zp[g0]; zc = zp[2 + g0];
    }
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) {
      uint32_t x[4];
      const uint4 zz = sub < 2 ? za : zc;
      const uint32_t nz[4] = {zz.x, zz.y, zz.z, zz.w};
      if constexpr (QM == QM_ASYM2) Unpack<QM>::run((sub & 1) ? (r.vc[sub >> 1] >> 4) : r.vc[sub >> 1], nz, x);
      else Unpack<QM>::run(r.vc[sub], nz, x);
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        const uint4 pq = sub < 2 ? pa[h] : pc[h];
        float a = st.acc[h][sub];
        a = dot2(x[0], pq.x, a);
        a = dot2(x[1], pq.y, a);
        a = dot2(x[2], pq.z, a);
        a = dot2(x[3], pq.w, a);
        st.acc[h][sub] = a;
      }
    }
  }
  wave_lds_sync();
}

// BF16 sink / window rows of one sequence: partial softmax over tail_len rows, lanes own 2 dims.
DEVI void tail_partial(const DecodeParams& p, int b, int kvh, int tile, float (&m)[4], float (&l)[4], float (&o)[4][2]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = p.tail_len[b];
  const int row = p.tail_idx != nullptr ? p.tail_idx[b] : b;
  const uint16_t* base = static_cast<const uint16_t*>(p.tail) + static_cast<long long>(row) * p.tail_bs;
  float q[4][2];
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    const int hq = tile * 4 + h;
    q[h][0] = q[h][1] = 0.f;
    if (hq < p.gqa) {
      const uint32_t raw = *reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(p.q) + static_cast<long long>(b) * p.q_bs +
                                                              (static_cast<long long>(kvh) * p.gqa + hq) * 128 + 2 * lane);
      q[h][0] = bf16_lo(raw) * p.qscale;
      q[h][1] = bf16_hi(raw) * p.qscale;
    }
    m[h] = -INFINITY; l[h] = 0.f; o[h][0] = o[h][1] = 0.f;
  }
  for (int t = wave; t < n; t += NWAVE) {
    const uint16_t* tr = base + static_cast<long long>(t) * p.tail_ts;
    const uint32_t kr = *reinterpret_cast<const uint32_t*>(tr + kvh * 128 + 2 * lane);
    const uint32_t vr = *reinterpret_cast<const uint32_t*>(tr + (p.Hkv + kvh) * 128 + 2 * lane);
    const float k0 = bf16_lo(kr), k1 = bf16_hi(kr), v0 = bf16_lo(vr), v1 = bf16_hi(vr);
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      float s = q[h][0] * k0 + q[h][1] * k1;
      s += dpp_xor1(s); s += dpp_xor2(s);
      s = wave_sum_over_tokens(s);
      const float mn = fmaxf(m[h], s);
      const float alpha = fexp2(m[h] - mn), pe = fexp2(s - mn);
      m[h] = mn;
      l[h] = l[h] * alpha + pe;
      o[h][0] = o[h][0] * alpha + pe * v0;
      o[h][1] = o[h][1] * alpha + pe * v1;
    }
  }
}

template <int QM, bool K2, int P>
__global__ void __launch_bounds__(256) k_decode(const DecodeParams p, int ntile, int nparts) {
  using L = Lay<QM, P>;
  __shared__ Smem S;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kvh = blockIdx.x / ntile, tile = blockIdx.x % ntile;
  const int split = blockIdx.y, b = blockIdx.z;
  const bool is_tail = p.tail != nullptr && split == p.nsplit;
  const int len = p.seq_lens[b];
  const long long part_id = ((static_cast<long long>(b) * p.Hkv + kvh) * ntile + tile) * nparts + split;

  if (!is_tail) {
    const int lo = max(split * p.chunk, min(p.kv_start, len));
    const int hi = min(len, (split + 1) * p.chunk);
    WaveState st;
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      st.m[h] = -INFINITY; st.l[h] = 0.f;
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) st.acc[h][s4] = 0.f;
    }
    if (lo < hi) {   // uniform over the workgroup
      q_prologue<QM, K2>(S, p, b, kvh, tile);
      __syncthreads();
      const int pg0 = lo / P, pg1 = (hi + P - 1) / P;
      const int* bt = p.block_table + static_cast<long long>(b) * p.bt_stride;
      PageRegs<QM> cur, nxt;
      int pg = pg0 + wave;
      if (pg < pg1) load_page<QM, P>(cur, p.pool + (static_cast<long long>(bt[pg]) * p.Hkv + kvh) * L::CHUNK, lane);
      for (; pg < pg1; pg += NWAVE) {
        const int pn = pg + NWAVE;
        if (pn < pg1) load_page<QM, P>(nxt, p.pool + (static_cast<long long>(bt[pn]) * p.Hkv + kvh) * L::CHUNK, lane);
        process_page<QM, K2, P>(S, st, cur, lane, wave, pg * P, lo, hi, p.qscale);
        cur = nxt;
      }
    }
    // ---- fold the wave: entry pairs (c8 = 0 / 1), offset sums per (head, group)
#pragma unroll
    for (int h = 0; h < 4; ++h) {
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) st.acc[h][s4] += dpp_xor1(st.acc[h][s4]);
      if (lane == 0) { S.m[wave][h] = st.m[h]; S.l[wave][h] = st.l[h]; }
    }
    __syncthreads();
    {
      const int wq = lane >> 4, gid = (lane >> 1) & 7;
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        float M = fmaxf(fmaxf(S.m[0][h], S.m[1][h]), fmaxf(S.m[2][h], S.m[3][h]));
        const float f = st.m[h] == -INFINITY ? 0.f : fexp2(st.m[h] - M);
        if ((lane & 1) == 0) {
#pragma unroll
          for (int sub = 0; sub < 4; ++sub) {
            const int d = 64 * (sub >> 1) + 16 * wq + gid + 8 * (sub & 1);
            S.o[wave][h][d] = f * st.acc[h][sub];
          }
        }
      }
    }
    __syncthreads();
  } else {
    float m[4], l[4], o[4][2];
    tail_partial(p, b, kvh, tile, m, l, o);
#pragma unroll
    for (int h = 0; h < 4; ++h)
      if (lane == 0) { S.m[wave][h] = m[h]; S.l[wave][h] = l[h]; }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const float M = fmaxf(fmaxf(S.m[0][h], S.m[1][h]), fmaxf(S.m[2][h], S.m[3][h]));
      const float f = m[h] == -INFINITY ? 0.f : fexp2(m[h] - M);
      S.o[wave][h][2 * lane] = f * o[h][0];
      S.o[wave][h][2 * lane + 1] = f * o[h][1];
    }
    __syncthreads();
  }
  // ---- workgroup partial: (o[4][128] relative to M, M, L)
  float po[2], pm, pl;
  const int oh = threadIdx.x >> 6;   // head of this thread's two outputs
  {
    const float M = fmaxf(fmaxf(S.m[0][oh], S.m[1][oh]), fmaxf(S.m[2][oh], S.m[3][oh]));
    float Lsum = 0.f;
#pragma unroll
    for (int w = 0; w < NWAVE; ++w) Lsum += S.m[w][oh] == -INFINITY ? 0.f : fexp2(S.m[w][oh] - M) * S.l[w][oh];
    pm = M; pl = Lsum;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int d = 2 * lane + e;
      po[e] = (S.o[0][oh][d] + S.o[1][oh][d]) + (S.o[2][oh][d] + S.o[3][oh][d]);
    }
    if (is_tail && p.vmask != nullptr) {  // the merged sum is rotated back once: bring the tail into the stored basis
      __syncthreads();
      S.o[0][oh][2 * lane] = po[0]; S.o[0][oh][2 * lane + 1] = po[1];
      __syncthreads();
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int d = 2 * lane + e, g = d >> 5;
        if (p.vmask[kvh * 4 + g]) {
          float a = 0.f;
          for (int k = 0; k < 32; ++k) {
            const float v = S.o[0][oh][32 * g + k];
            a += (__builtin_popcount(d & k & 31) & 1) ? -v : v;
          }
          po[e] = a * kC32;
        }
      }
    }
  }
  if (nparts > 1) {
    float* op = p.opart + part_id * 512 + oh * 128 + 2 * lane;
    *reinterpret_cast<float2*>(op) = make_float2(po[0], po[1]);
    if (lane == 0) *reinterpret_cast<float2*>(p.mlpart + part_id * 8 + 2 * oh) = make_float2(pm, pl);
    __threadfence();
    __syncthreads();
    const int tpc = p.counter_div;                               // q tiles that share one counter slot
    int* ctr = p.counter + (static_cast<long long>(b) * p.Hkv + kvh) * (ntile / tpc) + tile / tpc;
    if (threadIdx.x == 0) {
      const int prev = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
      S.last = prev == tpc * nparts - 1;
      if (S.last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!S.last) return;
    __threadfence();
  }
  // ---- final merge (last arriving workgroup, or the only one): all tiles of this counter slot
  const int tpc = nparts > 1 ? p.counter_div : 1;
  const int tile0 = nparts > 1 ? (tile / tpc) * tpc : tile;
  for (int tt = tile0; tt < tile0 + tpc; ++tt) {
    float M = pm, Lsum = pl, o0 = po[0], o1 = po[1];
    if (nparts > 1) {
      const long long base = ((static_cast<long long>(b) * p.Hkv + kvh) * ntile + tt) * nparts;
      M = -INFINITY;
      for (int s = 0; s < nparts; ++s) M = fmaxf(M, p.mlpart[(base + s) * 8 + 2 * oh]);
      Lsum = 0.f; o0 = 0.f; o1 = 0.f;
      for (int s = 0; s < nparts; ++s) {
        const float ms = p.mlpart[(base + s) * 8 + 2 * oh];
        const float ls = p.mlpart[(base + s) * 8 + 2 * oh + 1];
        const float f = ms == -INFINITY ? 0.f : fexp2(ms - M);
        Lsum += f * ls;
        o0 += f * p.opart[(base + s) * 512 + oh * 128 + 2 * lane];
        o1 += f * p.opart[(base + s) * 512 + oh * 128 + 2 * lane + 1];
      }
    }
    const float inv = Lsum > 0.f ? 1.f / Lsum : 0.f;
    o0 *= inv; o1 *= inv;
    if (p.vmask != nullptr) {
      __syncthreads();
      S.o[0][oh][2 * lane] = o0; S.o[0][oh][2 * lane + 1] = o1;
      __syncthreads();
      float r[2] = {o0, o1};
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int d = 2 * lane + e, g = d >> 5;
        if (p.vmask[kvh * 4 + g]) {
          float a = 0.f;
          for (int k = 0; k < 32; ++k) {
            const float v = S.o[0][oh][32 * g + k];
            a += (__builtin_popcount(d & k & 31) & 1) ? -v : v;
          }
          r[e] = a * kC32;
        }
      }
      o0 = r[0]; o1 = r[1];
    }
    const int hq = tt * 4 + oh;
    if (hq < p.gqa) {
      uint16_t* orow = static_cast<uint16_t*>(p.out) + static_cast<long long>(b) * p.o_bs +
                       (static_cast<long long>(kvh) * p.gqa + hq) * 128 + 2 * lane;
      *reinterpret_cast<uint32_t*>(orow) = bf16_rn(o0) | (bf16_rn(o1) << 16);
    }
  }
}

template <int QM, bool K2>
int launch_qm(const DecodeParams& p, hipStream_t st) {
  if (p.page != 16) return -5;
  const int ntile = (p.gqa + 3) / 4;
  const int nparts = p.nsplit + (p.tail != nullptr ? 1 : 0);
  if (nparts <= 0 || p.B <= 0) return 0;
  dim3 grid(p.Hkv * ntile, nparts, p.B);
  hipLaunchKernelGGL((k_decode<QM, K2, 16>), grid, dim3(256), 0, st, p, ntile, nparts);
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

int decode_launch(int fmt, const DecodeParams& p, hipStream_t st) {
  switch (fmt) {
    case FMT_INT4: return launch_qm<QM_SYM4, false>(p, st);
    case FMT_INT4A: return launch_qm<QM_ASYM4, false>(p, st);
    case FMT_INT2A: return launch_qm<QM_ASYM2, false>(p, st);
    case FMT_KONLY: return launch_qm<QM_SYM4, true>(p, st);
    case FMT_KONLYA: return launch_qm<QM_ASYM4, true>(p, st);
    case FMT_KONLYA2: return launch_qm<QM_ASYM2, true>(p, st);
  }
  return -4;
}

int decode_occupancy(int fmt) {
  (void)fmt;
  return 2;   // resident workgroups per CU the split planner may count on
}

}  // namespace fr
