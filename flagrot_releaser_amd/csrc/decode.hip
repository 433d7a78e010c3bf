// Paged split-K GQA decode attention over FlagRot INT4 / INT2 pages for gfx950 (wave64; scores on the vector
// pipe, the value product on the matrix pipe).
//
// One workgroup (16 or 12 wavefronts = a whole CU's register file, or 4 for short chunks) per (KV head x q tile of 4 heads,
// split, sequence).  Its wavefronts draw quads of 4 pages from a counter in LDS, so they finish together whatever
// share of the issue slots each one got.  A wavefront streams whole pages (16 tokens x one KV head = one contiguous
// 2304 / 1280 byte chunk) with 128-bit loads:
//   key phase    lane = token: its code row, 8 elements of each 32-group per 16-byte quarter.  A code field masked in
//                place is an fp16 denormal (value code * 2^(position - 24), exact) and is contracted with the query by
//                v_dot2_f32_f16; the powers of two ride on the query operand and the scale.  The query is rotated three ways once per workgroup
//                (identity, H32 per group, H128) and kept in LDS in the code words' element order; every lane fetches
//                the variant its token / group flags ask for, so selection costs no arithmetic.  The exponent offsets
//                and the zero points are removed with per-(variant, head, group) query sums.
//   softmax      exp2-domain online softmax per wavefront; p * V-scale is written to LDS as fp16 in V^T token order.
//   value phase  lane = one 16-byte V^T entry (4 dims x 8 tokens) of a run of 8 tokens: its words masked in place (fp16
//                denormals, value code * 2^(position - 24), exact) are the A operands of v_mfma_f32_16x16x32_f16, the
//                p * scale strip rows the B operands (columns = (group, head)); the powers of two ride on the
//                p * scale operand and one final multiply, the zero points leave through sum p * scale * zero point,
//                contracted by v_dot2 once per (page half, group, head) from the same LDS strips.
// The wavefronts are merged through LDS; splits through the caller's workspace with a ticket counter (the last
// arriving workgroup of a (sequence, KV head) merges, normalises, optionally rotates back, and stores bf16).
// The BF16 sink / window rows are one more split handled by an extra workgroup of the same grid.
//
// Semantics follow the reference's decode entry points: integrations/vllm_flagrot/csrc/flagrot_capi.cu:19-64,131-149,
// kernels/csrc/attn_codebook_attn.cuh:2093-2126 (per-(token, group) variant selection), attn_merge.cuh:23-84.
#include <cstdlib>
#include "fr_common.hpp"
#include "fr_launch.hpp"
#include "fr_unpack.hpp"

namespace fr {
namespace {

DEVI float dot2(uint32_t a, uint32_t b, float c) { return __builtin_amdgcn_fdot2(as_h2(a), as_h2(b), c, false); }
DEVI float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }


// LDS strips are padded so that the few distinct 16-byte rows the lanes of one instruction touch (one per variant /
// per row group) start in different banks.
constexpr int QV_VSTRIDE = 65;                     // uint4 per variant: 64 + 1 pad
constexpr int QV_BYTES = 3 * QV_VSTRIDE * 16;      // [variant][head][tg][j][8 fp16]
constexpr int PB_RSTRIDE = 17;                     // uint4 per row group (page, c8): 16 + 1 pad
constexpr int PB_BYTES = 8 * PB_RSTRIDE * 16;      // per wave: [page][c8][group][head][8 fp16]
constexpr int ZB_RSTRIDE = 5;                      // uint4 per row group: 4 + 1 pad
constexpr int ZB_BYTES = 8 * ZB_RSTRIDE * 16;      // per wave: [page][c8][group][8 fp16] = zero point (x 2^SH for odd tokens)
constexpr int STRIP_BYTES = PB_BYTES + ZB_BYTES;   // per wave
constexpr int DRAW_BATCH = 2;                      // quads per draw from the shared (device-scope) counter
constexpr int DRAW_BITS = 21, DRAW_MASK = (1 << DRAW_BITS) - 1;   // counter slot: quad draws below, merge tickets above
constexpr int BT_CACHE = 1024;                     // block-table entries of the workgroup's page range kept in LDS

template <int NW>
struct Smem {
  alignas(16) uint8_t qv[QV_BYTES];
  // per-wave strips during the page loop; the waves' partial outputs o[NW][4][128] (fp32) afterwards
  alignas(16) uint8_t work[NW * STRIP_BYTES > NW * 2048 ? NW * STRIP_BYTES : NW * 2048];
  alignas(16) uint32_t zero[4 * (4 * PB_RSTRIDE + 1)];   // zeros where the matrix value phase reads the strip rows of foreign groups
  alignas(16) float qsum[3][4][4];                   // [variant][group][head]: sum of the group's (fp16) query elements
  float m[NW][4], l[NW][4];
  int btc[BT_CACHE];
  int next;                                          // next quad of 4 pages nobody has taken yet
  int last;
  DEVI uint8_t* pb(int w) { return work + w * STRIP_BYTES; }
  DEVI const uint8_t* pb(int w) const { return work + w * STRIP_BYTES; }
  DEVI uint8_t* zb(int w) { return work + w * STRIP_BYTES + PB_BYTES; }
  DEVI const uint8_t* zb(int w) const { return work + w * STRIP_BYTES + PB_BYTES; }
  DEVI float* o(int w, int h) { return reinterpret_cast<float*>(work) + (w * 4 + h) * 128; }
};

// slot of element (isB, i) of a K word / of token r8 of a V word inside the 8-fp16 operand vector
DEVI int kslot(int isB, int i) { return 2 * (2 * (i & 1) + isB) + (i >> 1); }
DEVI int vslot(int r8) { return 2 * (r8 & 3) + (r8 >> 2); }

// Rotates the q tile three ways and stores it as fp16 in code-word order (the identity variant of a bf16 query is
// exact in fp16; qscale is applied to the fp32 score), with the sums per 32-group that remove the key zero points.
template <int QM, bool K2, class SM>
DEVI void q_prologue(SM& S, const DecodeParams& p, int b, int kvh, int tile) {   // wavefronts 0..3: one head each
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
    // the B elements of a code word are unpacked with the factor 2^SH (UnpackD): their query slots carry 2^-SH
    const float fold = ((l32 >> 2) & 1) ? 1.f / static_cast<float>(1 << UnpackD<QM>::SH) : 1.f;
    float qs = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = 4 * l32 + i, r = d & 31;
      const int isB = r >> 4, tg = (r & 15) >> 2, ii = r & 3;
      qs += static_cast<float>(static_cast<_Float16>(v[i]));
      reinterpret_cast<_Float16*>(S.qv)[(var * QV_VSTRIDE + (w * 4 + tg) * 4 + g) * 8 + kslot(isB, ii)] = static_cast<_Float16>(v[i] * fold);
    }
    qs += hx(qs, 1); qs += hx(qs, 2); qs += hx(qs, 4);
    if ((l32 & 7) == 0) S.qsum[var][g][w] = qs;
  }
}

// Page loads are forced into the global address space: a generic (flat) load also counts on the LDS counter, so
// every wait for an LDS read would wait for the page data in flight as well.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <class T> DEVI T gload(const uint8_t* p) {
  typedef const __attribute__((address_space(1))) T* gp;
  return *(gp)(p);
}

// One wave iteration covers 4 consecutive pages = 64 tokens.  Key phase: lane = token (page lane >> 4, position
// lane & 15).  Value phase: lane = V^T entry `lane` of each of the 4 pages in turn.
template <int QM> struct KRegs {
  static constexpr int NW = QM == QM_ASYM2 ? 2 : 4;   // code words per 16-byte / 8-byte quarter row
  uint32_t kc[4][NW];       // [quarter tg][word]
  uint2 ks;                 // the token's 4 K scale words
  uint16_t vs[4];           // the token's 4 V scale words (one per group); 16 bits wide so that their widening belongs to the use
                            // (a widening at the load would be scheduled right behind it and wait for the keys in flight)
};
// The value product P' V runs on the matrix pipe: sixteen v_mfma_f32_16x16x32_f16 per quad of pages, rows = 16 V^T
// entries, columns = (group, head), 32 tokens deep.  An entry word masked in place (eight tokens as fp16 denormal
// pairs; the matrix pipe keeps denormal inputs) is the A operand of its lane, one 16-byte strip row (p' of a run's eight
// tokens for a (group, head)) the B operand.  The scores stay on the vector pipe (v_dot2_f32_f16).
template <int QM> struct VRegs {
  static constexpr int NW = QM == QM_ASYM2 ? 2 : 4;
  uint32_t vc[4][NW];       // [2 (page pair s) + entry half][entry word] of lane (entry m = lane & 15, run kc = lane >> 4)
};

template <int QM, int P>
DEVI void load_k(KRegs<QM>& r, const uint8_t* chunk, int pos) {
  using L = Lay<QM, P>;
  if constexpr (QM == QM_ASYM2) {
    const uint8_t* row = chunk + L::K_OFF + 32 * (pos ^ ((pos >> 1) & 2));
#pragma unroll
    for (int tg = 0; tg < 4; ++tg) {
      const u32x2 k = gload<u32x2>(row + 8 * tg);
      r.kc[tg][0] = k.x; r.kc[tg][1] = k.y;
    }
  } else {
    const uint8_t* row = chunk + L::K_OFF + 64 * pos;
#pragma unroll
    for (int tg = 0; tg < 4; ++tg) {
      const u32x4 k = gload<u32x4>(row + 16 * tg);
      r.kc[tg][0] = k.x; r.kc[tg][1] = k.y; r.kc[tg][2] = k.z; r.kc[tg][3] = k.w;
    }
  }
  { const u32x2 t2 = gload<u32x2>(chunk + L::KS_OFF + 8 * pos); r.ks = make_uint2(t2.x, t2.y); }
  const uint8_t* vo = chunk + L::VS_OFF + (8 * (pos >> 3) + vs_slot8(pos)) * 2;
#pragma unroll
  for (int g = 0; g < 4; ++g) r.vs[g] = gload<uint16_t>(vo + g * P * 2);
}

template <int QM, int P>
DEVI void load_v(VRegs<QM>& r, const uint8_t* const (&chunk)[4], int lane) {
  using L = Lay<QM, P>;
  // lane = (entry m = lane & 15 (+ 16 for the second half), run kc = lane >> 4 of the 32 tokens of half s of the quad:
  // 16-token pages 2 s, 2 s + 1 with two runs each, or the 32-token page s with four)
  constexpr int R = P / 8;                       // runs of 8 tokens (entries per dim group) per page
  const int m = lane & 15, kc = lane >> 4;
#pragma unroll
  for (int s2 = 0; s2 < 2; ++s2) {
    const uint8_t* ch = P == 16 ? ((kc >> 1) ? chunk[2 * s2 + 1] : chunk[2 * s2]) : chunk[s2];
    const int c8 = P == 16 ? (kc & 1) : kc;
#pragma unroll
    for (int eh = 0; eh < 2; ++eh) {
      if constexpr (QM == QM_ASYM2) {
        const u32x2 v = gload<u32x2>(ch + L::V_OFF + 8 * (R * (16 * eh + m) + c8));
        r.vc[2 * s2 + eh][0] = v.x; r.vc[2 * s2 + eh][1] = v.y;
      } else {
        const u32x4 v = gload<u32x4>(ch + L::V_OFF + 16 * (R * (16 * eh + m) + c8));
        r.vc[2 * s2 + eh][0] = v.x; r.vc[2 * s2 + eh][1] = v.y; r.vc[2 * s2 + eh][2] = v.z; r.vc[2 * s2 + eh][3] = v.w;
      }
    }
  }
}

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
struct WaveState {
  float m[4];        // running maximum per head (wave uniform)
  float l[4];        // this lane's share of the running sum per head
  // 2^-24 sum p' code (zero points not yet removed), [entry word parity]: column lane & 15 = (group g, head), rows =
  // entries 16 (g & 1) + 4 (lane >> 4) + r, entry word 2 (g >> 1) + parity
  f32x4 ot[2];
  float z[2];        // lane = (page, half, group, head pair): its share of sum p' zero point, heads 2 hp and 2 hp + 1
};

// scores of the lane's token against the 4 q heads (log2 domain, unmasked)
template <int QM, bool K2, class SM>
DEVI void key_phase(const SM& S, const KRegs<QM>& r, float qscale, float (&sc)[4]) {
  constexpr int ZM = QM == QM_ASYM4 ? 15 : QM == QM_ASYM2 ? 3 : 0;
  const uint32_t kw[4] = {r.ks.x & 0xFFFFu, r.ks.x >> 16, r.ks.y & 0xFFFFu, r.ks.y >> 16};
  const bool full = K2 && (r.vs[0] & 0x8000u);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int var = K2 ? (full ? 2 : static_cast<int>(kw[j] >> 15)) : 0;
    const uint4* qp = reinterpret_cast<const uint4*>(S.qv) + var * QV_VSTRIDE + j;   // + head * 16 + tg * 4
    float a[4];
#pragma unroll
    for (int tg = 0; tg < 4; ++tg) {
      uint32_t x[4];
      if constexpr (QM == QM_ASYM2) {     // two groups per word: the odd one 4 bits higher, 2^4 folded into its scale
        if (j & 1) UnpackD<QM>::run_hi(r.kc[tg][j >> 1], x); else UnpackD<QM>::run(r.kc[tg][j >> 1], x);
      }
      else UnpackD<QM>::run(r.kc[tg][j], x);
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        const uint4 qq = qp[h * 16 + tg * 4];
        float v;
        if (tg == 0) asm("v_dot2_f32_f16 %0, %1, %2, 0" : "=v"(v) : "v"(x[0]), "v"(qq.x));   // no register clear
        else v = dot2(x[0], qq.x, a[h]);
        v = dot2(x[1], qq.y, v);
        v = dot2(x[2], qq.z, v);
        v = dot2(x[3], qq.w, v);
        a[h] = v;
      }
    }
    // a = 2^-24 sum code q: score += scale (2^24 a - zero point * sum q)
    const float sj = f16_value(kw[j] & 0x7FFFu) * qscale;
    const float sj24 = sj * ((QM == QM_ASYM2 && (j & 1)) ? 1048576.f : 16777216.f);
    if constexpr (ZM != 0) {
      const float4 qs = *reinterpret_cast<const float4*>(&S.qsum[var][j][0]);
      const float sz = -sj * static_cast<float>(kw[j] & ZM);
      sc[0] += sz * qs.x; sc[1] += sz * qs.y; sc[2] += sz * qs.z; sc[3] += sz * qs.w;
    }
#pragma unroll
    for (int h = 0; h < 4; ++h) sc[h] += sj24 * a[h];
  }
}

// online softmax step for 64 tokens: the running maximum is only re-reduced over the wave when some lane beats it
template <int QM, class SM>
DEVI void softmax_phase(SM& S, WaveState& st, const KRegs<QM>& r, float (&sc)[4], bool valid, int lane, int wave) {
  constexpr int ZM = QM == QM_ASYM4 ? 15 : QM == QM_ASYM2 ? 3 : 0;
  bool beat = false;
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    sc[h] = valid ? sc[h] : -INFINITY;
    beat |= sc[h] > st.m[h];
  }
  // The state is multiplied every time (by 1 unless the maxima moved): modifying it only inside the rare branch makes
  // the compiler keep two copies of all its registers and move them on the common path.
  float alpha[4] = {1.f, 1.f, 1.f, 1.f};
  if (__builtin_expect(__any(beat), 0)) {   // rare after the first quads
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const float mn = fmaxf(st.m[h], wave_max64(sc[h]));
      alpha[h] = mn == -INFINITY ? 1.f : fexp2(st.m[h] - mn);
      st.m[h] = mn;
    }
  }
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    st.l[h] *= alpha[h];
  }
  {   // the lane's accumulator column belongs to head lane & 3
    const float al = (lane & 2) ? ((lane & 1) ? alpha[3] : alpha[2]) : ((lane & 1) ? alpha[1] : alpha[0]);
    st.ot[0] *= al; st.ot[1] *= al;
  }
  st.z[0] *= (lane & 1) ? alpha[2] : alpha[0];
  st.z[1] *= (lane & 1) ? alpha[3] : alpha[1];
  float p[4];
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    p[h] = fexp2(sc[h] - st.m[h]);       // masked tokens: 2^-inf = 0 (the maximum is finite once a quad has been seen)
    st.l[h] += p[h];
  }
  // p' = p * V scale per group as fp16 (packed fp16 products of head pairs) and the zero points, in V^T token order
  // of the token's page.  Odd tokens are unpacked with the factor 2^SH (UnpackD): their scores were lowered by SH
  // (p carries 2^-SH), their zero point is raised by 2^SH; zero points are fp16 denormals like the codes.
  const int rg = lane >> 3, sl = vslot(lane & 7);         // run of 8 tokens (page, page eighth) and the slot inside it
  uint16_t* pb = reinterpret_cast<uint16_t*>(S.pb(wave)) + rg * PB_RSTRIDE * 8 + sl;     // + (group * 4 + head) * 8
  uint16_t* zb = reinterpret_cast<uint16_t*>(S.zb(wave)) + rg * ZB_RSTRIDE * 8 + sl;     // + group * 8
  const uint32_t p01 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(p[0], p[1]));
  const uint32_t p23 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(p[2], p[3]));
  const uint32_t keep = valid ? 0x7FFF7FFFu : 0u;        // unwritten slots may hold any pattern
  const int zsh = (lane & 1) ? UnpackD<QM>::SH : 0;      // odd position inside the page
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const uint32_t sv2 = (r.vs[g] * 0x10001u) & keep;
    const uint32_t x01 = pk_mul(p01, sv2), x23 = pk_mul(p23, sv2);
    pb[(g * 4 + 0) * 8] = static_cast<uint16_t>(x01);
    pb[(g * 4 + 1) * 8] = static_cast<uint16_t>(x01 >> 16);
    pb[(g * 4 + 2) * 8] = static_cast<uint16_t>(x23);
    pb[(g * 4 + 3) * 8] = static_cast<uint16_t>(x23 >> 16);
    if constexpr (QM != QM_SYM4) zb[g * 8] = static_cast<uint16_t>((r.vs[g] & ZM) << zsh);
  }
}

template <int QM, class SM>
DEVI void value_phase(const SM& S, WaveState& st, const VRegs<QM>& r, int lane, int wave) {
  // An entry word (entry half eh, word sub) holds channels of group 2 (sub >> 1) + eh only.  The products of all
  // four groups share one accumulator per word parity: the B operand of a group is the strip row with the columns of
  // the other groups zero (those lanes read a row of zeros instead), so each column collects its own group's rows.
  const int n = lane & 15, kc = lane >> 4;
  const uint4* own = reinterpret_cast<const uint4*>(S.pb(wave)) + kc * PB_RSTRIDE + n;
#pragma unroll
  for (int s2 = 0; s2 < 2; ++s2) {            // 32 tokens: the runs (page 2 s + (kc >> 1), c8 = kc & 1) = strip row group 4 s + kc
    half8 b[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint4* src = (n >> 2) == g ? own : reinterpret_cast<const uint4*>(S.zero);
      b[g] = __builtin_bit_cast(half8, src[4 * s2 * PB_RSTRIDE]);
    }
#pragma unroll
    for (int eh = 0; eh < 2; ++eh)
#pragma unroll
      for (int sub = 0; sub < 4; ++sub) {
        uint32_t x[4];
        if constexpr (QM == QM_ASYM2) {   // two sub-vectors per word: the odd one's sums carry 2^4 until the fold
          if (sub & 1) UnpackD<QM>::run_hi(r.vc[2 * s2 + eh][sub >> 1], x); else UnpackD<QM>::run(r.vc[2 * s2 + eh][sub >> 1], x);
        }
        else UnpackD<QM>::run(r.vc[2 * s2 + eh][sub], x);
        const uint4 aq = make_uint4(x[0], x[1], x[2], x[3]);
        st.ot[sub & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, aq), b[2 * (sub >> 1) + eh], st.ot[sub & 1], 0, 0, 0);
      }
  }
  if constexpr (QM != QM_SYM4) {   // sum p' zero point: lane = (page, page half, group, head pair)
    const int rg = lane >> 3, g = (lane >> 1) & 3, hp = lane & 1;
    const uint4 zq = (reinterpret_cast<const uint4*>(S.zb(wave)) + rg * ZB_RSTRIDE)[g];
    const uint4* pp = reinterpret_cast<const uint4*>(S.pb(wave)) + rg * PB_RSTRIDE + g * 4 + 2 * hp;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const uint4 pq = pp[e];
      float a = st.z[e];
      a = dot2(zq.x, pq.x, a); a = dot2(zq.y, pq.y, a); a = dot2(zq.z, pq.z, a); a = dot2(zq.w, pq.w, a);
      st.z[e] = a;
    }
  }
}

// BF16 sink / window rows of one sequence: partial softmax over tail_len rows, lanes own 2 dims.
template <int NW>
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
  for (int t = wave; t < n; t += NW) {
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

template <int QM, bool K2, int P, int NW>
__global__ void __launch_bounds__(64 * NW, NW == 16 ? 4 : NW == 12 ? 3 : (K2 ? 4 : 1)) k_decode(const DecodeParams p, int ntile, int nparts) {
  using L = Lay<QM, P>;
  __shared__ Smem<NW> S;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kvh = blockIdx.x / ntile, tile = blockIdx.x % ntile;
  // Workgroups are dispatched in linear order and the CU's arbiter favours the older wavefronts: the splits of one
  // sequence are spread over the whole dispatch order (split slowest) so that every sequence gets the same mix.
  const int lin = blockIdx.z * gridDim.y + blockIdx.y;
  const int split = lin / p.B, b = lin % p.B;
  const bool is_tail = p.tail != nullptr && split == p.nsplit;
  const int len = p.seq_lens[b];
  const long long part_id = ((static_cast<long long>(b) * p.Hkv + kvh) * ntile + tile) * nparts + split;
  const bool act = wave < 4;      // the 256 threads that own the workgroup's 4 x 128 outputs

  // the (sequence, KV head, q tile)'s counter slot: merge ticket, and in the dynamic mode the quad draw counter
  const int tpc = p.counter_div;                                 // q tiles that share one counter slot
  int* const ctr = p.counter + (static_cast<long long>(b) * p.Hkv + kvh) * (ntile / tpc) + tile / tpc;
  const bool dyn = p.dyn != 0;    // the body workgroups of a (sequence, KV head, q tile) draw quads from one counter
  if (!is_tail) {
    const int lo = dyn ? min(p.kv_start, len) : max(split * p.chunk, min(p.kv_start, len));
    const int hi = dyn ? len : min(len, (split + 1) * p.chunk);
    WaveState st;
#pragma unroll
    for (int h = 0; h < 4; ++h) { st.m[h] = -INFINITY; st.l[h] = 0.f; }
    st.z[0] = st.z[1] = 0.f;
    st.ot[0] = st.ot[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (lo < hi) {   // uniform over the workgroup
      const int pg0 = lo / P, pg1 = (hi + P - 1) / P;
      const int* bt = p.block_table + static_cast<long long>(b) * p.bt_stride;
      // quads beyond a wave's first one are drawn: from S.next (the workgroup owns a range) or from the slot's draw
      // counter (all body wavefronts of the slot share the range); a draw is made a whole iteration before its use
      auto draw = [&]() {
        int t = 0;
        if (lane == 0)
          // (shared counter: one increment = DRAW_BATCH quads.  An increment and not an addition: the compiler rewrites
          // additions into a wave-wide reduction whose broadcast waits for the counter's round trip on the spot)
          // what comes back is unpacked where it is used (undraw): any arithmetic on it here would wait for it here
          t = dyn ? static_cast<int>(__builtin_amdgcn_atomic_inc32(reinterpret_cast<unsigned*>(ctr), 0xFFFFFFFFu, __ATOMIC_RELAXED, "agent"))
                  : atomicAdd(&S.next, 1);
        return t;
      };
      int take = 0;
      if (dyn) take = draw();        // the first round trip to the device-scope counter hides behind the prologue
      for (int i = threadIdx.x; i < min(pg1 - pg0, BT_CACHE); i += 64 * NW) S.btc[i] = bt[pg0 + i];
      if (threadIdx.x == 0) S.next = NW;
      for (int i = threadIdx.x; i < 4 * (4 * PB_RSTRIDE + 1); i += 64 * NW) S.zero[i] = 0u;
      if (act) q_prologue<QM, K2>(S, p, b, kvh, tile);
      __syncthreads();
      constexpr int PPQ = 64 / P;                 // pages per quad of 64 tokens (the name stays: 4 pages of 16, 2 of 32)
      const int nquad = (pg1 - pg0 + PPQ - 1) / PPQ;
      const int pi = lane / P, pos = lane % P;
      // odd tokens: the B fields of a V^T word come out of the unpacking with the factor 2^SH, so their scores are
      // lowered by SH (log2 domain) and their share of the softmax sum is raised again at the end
      const float sc0 = (pos & 1) ? -static_cast<float>(UnpackD<QM>::SH) : 0.f;
      typedef const __attribute__((address_space(1))) uint8_t* gptr;
      const gptr pool = (gptr)p.pool;
      auto chunk_of = [&](int quad) {   // pages past the range read the last page of the range; their tokens are masked
        const int i = min(PPQ * quad + pi, pg1 - pg0 - 1);
        // The entry comes from LDS.  Past the cached window it is read from memory inside a branch and consumed there:
        // a select between the two addresses would be one generic load, which waits for every page load in flight.
        int page = S.btc[min(i, BT_CACHE - 1)];
        if (__builtin_expect(i >= BT_CACHE, 0)) {
          const int far = gload<int>(reinterpret_cast<const uint8_t*>(bt + pg0 + i));
          asm volatile("v_mov_b32 %0, %1" : "=v"(page) : "v"(far));
        }
        return (const uint8_t*)(pool + (static_cast<long long>(page) * p.Hkv + kvh) * L::CHUNK);
      };
      __builtin_amdgcn_s_setprio(1);
      KRegs<QM> cur;
      // this wave's current quad of 4 pages: the first one by position
      const int nworker = dyn ? p.nsplit * NW : 0;
      int qi = dyn ? split * NW + wave : wave;
      const uint8_t* mine = chunk_of(qi);
      if (qi < nquad) load_k<QM, P>(cur, mine, pos);
      if (!dyn) take = draw();
      int more = 0, nextq = 0;       // quads left of the batch drawn last (the shared counter hands out DRAW_BATCH at a time)
      while (qi < nquad) {
        // the next quad: read where the keys of this one are awaited anyway (every older memory operation is then
        // complete), the following draw goes out ahead of this iteration's loads
        int qn;
        if (more > 0) { qn = nextq++; --more; }
        else {
          // (the draw made an iteration ago is read here and not before: without the opaque copy its broadcast is
          // moved up to the draw itself, which then waits for the counter's round trip on the spot)
          int drawn = take;
          asm volatile("" : "+v"(drawn));
          drawn = __builtin_amdgcn_readfirstlane(drawn);
          qn = (dyn ? (drawn & DRAW_MASK) * DRAW_BATCH : drawn) + nworker;
          take = draw();
          if (dyn) { nextq = qn + 1; more = DRAW_BATCH - 1; }
        }
        VRegs<QM> vr;                // this quad's V^T entries: in flight during the key phase
        const uint8_t* ch[4];
        {
          const unsigned long long mp = reinterpret_cast<unsigned long long>(mine);
#pragma unroll
          for (int k = 0; k < 4; ++k) {             // (32-token pages: entries 2, 3 repeat page 1 and are not read)
            const uint32_t lo32 = __builtin_amdgcn_readlane(static_cast<uint32_t>(mp), (P * k) & 63);
            const uint32_t hi32 = __builtin_amdgcn_readlane(static_cast<uint32_t>(mp >> 32), (P * k) & 63);
            ch[k] = reinterpret_cast<const uint8_t*>((static_cast<unsigned long long>(hi32) << 32) | lo32);
          }
        }
        const int tok = (pg0 + PPQ * qi + pi) * P + pos;
        const bool valid = tok >= lo && tok < hi;
        // (The scheduler moves the requests for the value entries below the key phase, where the code words' registers
        // are free.  Pinning them, or half of them, above or inside it costs registers the loop does not have at four
        // wavefronts per SIMD, and gains nothing at three: measured.)
        float sc[4] = {sc0, sc0, sc0, sc0};
        load_v<QM, P>(vr, ch, lane);
        key_phase<QM, K2>(S, cur, p.qscale, sc);
        softmax_phase<QM>(S, st, cur, sc, valid, lane, wave);
        // The key registers are free: the next quad's keys fly during the value phase.  The loads are issued on every
        // path (past the range chunk_of names the range's last page again, a cache hit nobody uses): were they inside
        // the branch, the wait counts after the join would be those of the path without them, and the value phase
        // would wait for these loads as well.
        mine = chunk_of(qn);
        load_k<QM, P>(cur, mine, pos);
        if (qn < nquad) {
          // once the counter has run dry, the wavefronts that still hold a quad go first: they all end together
          if (qn + NW >= nquad) __builtin_amdgcn_s_setprio(3);
        } else {
          __builtin_amdgcn_s_setprio(0);
        }
        wave_lds_sync();
        value_phase<QM>(S, st, vr, lane, wave);
        wave_lds_sync();
        qi = qn;
      }
      // the last draw is never used: it must have reached the counter before this workgroup takes its ticket (the
      // last arriver clears the word)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    // ---- fold the wave: zero-point sums per (head, group) through the wave's strip, codes -> values:
    //      2^24 (acc - sum p' zero point)
    if constexpr (QM != QM_SYM4) {
      float z0 = st.z[0], z1 = st.z[1];
      z0 += swz_xor<8>(z0); z1 += swz_xor<8>(z1);
      z0 += swz_xor<16>(z0); z1 += swz_xor<16>(z1);
      z0 += xor32(z0); z1 += xor32(z1);
      float* zs = reinterpret_cast<float*>(S.pb(wave));          // [head][group]; the strips are dead by now
      if (lane < 8) { zs[(2 * (lane & 1)) * 4 + (lane >> 1)] = z0; zs[(2 * (lane & 1) + 1) * 4 + (lane >> 1)] = z1; }
      wave_lds_sync();
    }
    const float unfold = (lane & 1) ? static_cast<float>(1 << UnpackD<QM>::SH) : 1.f;   // lane & 1 = token parity
    const int hl = lane & 3, gl = (lane >> 2) & 3;      // the lane's accumulator column: head hl, group gl
    {
      float zg = 0.f;
      if constexpr (QM != QM_SYM4) zg = reinterpret_cast<const float*>(S.pb(wave))[hl * 4 + gl];
      if constexpr (QM == QM_ASYM2) st.ot[1] *= 0.0625f;            // fields unpacked 4 bits up
#pragma unroll
      for (int y = 0; y < 2; ++y)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) st.ot[y][r4] = (st.ot[y][r4] - zg) * 16777216.f;
    }
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const float lsum = wave_sum64(st.l[h] * unfold);
      if (lane == 0) { S.m[wave][h] = st.m[h]; S.l[wave][h] = lsum; }
    }
    __syncthreads();     // every wave is done with its strip: the partial outputs may overwrite them
    {
      const int kc = lane >> 4;      // the lane's four entry rows: 4 kc + r
      float M = S.m[0][hl];
#pragma unroll
      for (int w = 1; w < NW; ++w) M = fmaxf(M, S.m[w][hl]);
      const float mh = (hl & 2) ? ((hl & 1) ? st.m[3] : st.m[2]) : ((hl & 1) ? st.m[1] : st.m[0]);
      const float f = mh == -INFINITY ? 0.f : fexp2(mh - M);
      float* o = S.o(wave, hl);
#pragma unroll
      for (int y = 0; y < 2; ++y) {
        // entry e = 16 (gl & 1) + 4 kc + r, word sub = 2 (gl >> 1) + y: dim 64 (sub >> 1) + 16 (e >> 3) + 8 (sub & 1) + (e & 7)
        const int d = 32 * gl + 16 * (kc >> 1) + 8 * y + 4 * (kc & 1);
        *reinterpret_cast<float4*>(o + d) = make_float4(f * st.ot[y][0], f * st.ot[y][1], f * st.ot[y][2], f * st.ot[y][3]);
      }
    }
    __syncthreads();
  } else {
    float m[4], l[4], o[4][2];
    tail_partial<NW>(p, b, kvh, tile, m, l, o);
#pragma unroll
    for (int h = 0; h < 4; ++h)
      if (lane == 0) { S.m[wave][h] = m[h]; S.l[wave][h] = l[h]; }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      float M = S.m[0][h];
#pragma unroll
      for (int w = 1; w < NW; ++w) M = fmaxf(M, S.m[w][h]);
      const float f = m[h] == -INFINITY ? 0.f : fexp2(m[h] - M);
      float* so = S.o(wave, h);
      so[2 * lane] = f * o[h][0];
      so[2 * lane + 1] = f * o[h][1];
    }
    __syncthreads();
  }
  // ---- workgroup partial: (o[4][128] relative to M, M, L); thread = (head, 2 dims) for the first 4 wavefronts
  float po[2] = {0.f, 0.f}, pm = -INFINITY, pl = 0.f;
  const int oh = wave & 3;           // head of this thread's two outputs
  if (act) {
    float M = S.m[0][oh];
#pragma unroll
    for (int w = 1; w < NW; ++w) M = fmaxf(M, S.m[w][oh]);
    float Lsum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) Lsum += S.m[w][oh] == -INFINITY ? 0.f : fexp2(S.m[w][oh] - M) * S.l[w][oh];
    pm = M; pl = Lsum;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float2 v = *reinterpret_cast<const float2*>(S.o(w, oh) + 2 * lane);
      po[0] += v.x; po[1] += v.y;
    }
  }
  if (is_tail && p.vmask != nullptr) {  // the merged sum is rotated back once: bring the tail into the stored basis
    __syncthreads();
    if (act) { S.o(0, oh)[2 * lane] = po[0]; S.o(0, oh)[2 * lane + 1] = po[1]; }
    __syncthreads();
    if (act) {
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int d = 2 * lane + e, g = d >> 5;
        if (p.vmask[kvh * 4 + g]) {
          float a = 0.f;
          for (int k = 0; k < 32; ++k) {
            const float v = S.o(0, oh)[32 * g + k];
            a += (__builtin_popcount(d & k & 31) & 1) ? -v : v;
          }
          po[e] = a * kC32;
        }
      }
    }
  }
  if (nparts > 1) {
    // Partials cross workgroups (and XCDs, each with its own L2) through device-scope relaxed atomic stores / loads,
    // which are write-through / read-through; a device-scope fence here would write back and invalidate the whole
    // L2 once per workgroup.  Order: every storing wavefront waits until its stores are acknowledged (an explicit
    // wait on the vector memory counter, which counts stores on this target: a workgroup-scope fence emits no such
    // wait), barrier, ticket; the last arriver reads (device-scope loads) after its ticket has returned.
    if (act) {
      float* op = p.opart + part_id * 512 + oh * 128 + 2 * lane;
      __hip_atomic_store(op, po[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(op + 1, po[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (lane == 0) {
        __hip_atomic_store(p.mlpart + part_id * 8 + 2 * oh, pm, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(p.mlpart + part_id * 8 + 2 * oh + 1, pl, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // this wavefront's partial stores have been acknowledged
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) {    // every draw of this workgroup precedes its ticket: the last arriver may clear the slot
      const int prev = __hip_atomic_fetch_add(ctr, dyn ? DRAW_MASK + 1 : 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      S.last = (dyn ? static_cast<int>(static_cast<unsigned>(prev) >> DRAW_BITS) : prev) == tpc * nparts - 1;
      if (S.last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!S.last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  } else if (dyn && threadIdx.x == 0) {
    __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // the only workgroup of the slot
  }
  // ---- final merge (last arriving workgroup, or the only one): all tiles of this counter slot
  const int ntt = nparts > 1 ? tpc : 1;
  const int tile0 = nparts > 1 ? (tile / tpc) * tpc : tile;
  for (int tt = tile0; tt < tile0 + ntt; ++tt) {
    float M = pm, Lsum = pl, o0 = po[0], o1 = po[1];
    if (nparts > 1 && act) {
      const long long base = ((static_cast<long long>(b) * p.Hkv + kvh) * ntile + tt) * nparts;
      M = -INFINITY;
      for (int s = 0; s < nparts; ++s) M = fmaxf(M, __hip_atomic_load(p.mlpart + (base + s) * 8 + 2 * oh, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
      Lsum = 0.f; o0 = 0.f; o1 = 0.f;
      for (int s = 0; s < nparts; ++s) {
        const float ms = __hip_atomic_load(p.mlpart + (base + s) * 8 + 2 * oh, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const float ls = __hip_atomic_load(p.mlpart + (base + s) * 8 + 2 * oh + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const float f = ms == -INFINITY ? 0.f : fexp2(ms - M);
        Lsum += f * ls;
        o0 += f * __hip_atomic_load(p.opart + (base + s) * 512 + oh * 128 + 2 * lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        o1 += f * __hip_atomic_load(p.opart + (base + s) * 512 + oh * 128 + 2 * lane + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    const float inv = Lsum > 0.f ? 1.f / Lsum : 0.f;
    o0 *= inv; o1 *= inv;
    if (p.vmask != nullptr) {
      __syncthreads();
      if (act) { S.o(0, oh)[2 * lane] = o0; S.o(0, oh)[2 * lane + 1] = o1; }
      __syncthreads();
      float r[2] = {o0, o1};
      if (act) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const int d = 2 * lane + e, g = d >> 5;
          if (p.vmask[kvh * 4 + g]) {
            float a = 0.f;
            for (int k = 0; k < 32; ++k) {
              const float v = S.o(0, oh)[32 * g + k];
              a += (__builtin_popcount(d & k & 31) & 1) ? -v : v;
            }
            r[e] = a * kC32;
          }
        }
      }
      o0 = r[0]; o1 = r[1];
    }
    const int hq = tt * 4 + oh;
    if (act && hq < p.gqa) {
      uint16_t* orow = static_cast<uint16_t*>(p.out) + static_cast<long long>(b) * p.o_bs +
                       (static_cast<long long>(kvh) * p.gqa + hq) * 128 + 2 * lane;
      *reinterpret_cast<uint32_t*>(orow) = bf16_rn(o0) | (bf16_rn(o1) << 16);
    }
  }
}

// Wavefronts per workgroup: 4, or from 1024 tokens per split one large workgroup that fills a CU.  The codebook
// kernels fit 128 registers per lane: 16 wavefronts (4 per SIMD); the static-mask kernels need more: 12 (168 registers).
template <bool K2> constexpr int BIGW = K2 ? 16 : 12;
constexpr int BIG_CHUNK = 1024;   // tokens per split from which the large workgroup pays (measured: batch 1-16, 2-32 k tokens)
inline int waves_for(int chunk_tokens) { return chunk_tokens >= BIG_CHUNK ? 16 : 4; }   // > 4 selects the large workgroup

template <int QM, bool K2>
int launch_qm(const DecodeParams& p, hipStream_t st) {
  if (p.page != 16 && p.page != 32) return -5;
  const int ntile = (p.gqa + 3) / 4;
  const int nparts = p.nsplit + (p.tail != nullptr ? 1 : 0);
  if (nparts <= 0 || p.B <= 0) return 0;
  dim3 grid(p.Hkv * ntile, nparts, p.B);
  if (p.page == 32) {
    if (p.wg_waves > 4) hipLaunchKernelGGL((k_decode<QM, K2, 32, BIGW<K2>>), grid, dim3(64 * BIGW<K2>), 0, st, p, ntile, nparts);
    else hipLaunchKernelGGL((k_decode<QM, K2, 32, 4>), grid, dim3(256), 0, st, p, ntile, nparts);
  } else if (p.wg_waves > 4) hipLaunchKernelGGL((k_decode<QM, K2, 16, BIGW<K2>>), grid, dim3(64 * BIGW<K2>), 0, st, p, ntile, nparts);
  else hipLaunchKernelGGL((k_decode<QM, K2, 16, 4>), grid, dim3(256), 0, st, p, ntile, nparts);
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

int decode_dispatch(int fmt, const DecodeParams& p, hipStream_t st) {
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

template <int QM, bool K2>
int occupancy_qm(int waves) {
  int n = 0;
  const void* f = waves > 4 ? reinterpret_cast<const void*>(&k_decode<QM, K2, 16, BIGW<K2>>) : reinterpret_cast<const void*>(&k_decode<QM, K2, 16, 4>);
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, f, 64 * (waves > 4 ? BIGW<K2> : 4), 0) != hipSuccess || n < 1) {
    (void)hipGetLastError();
    return waves > 4 ? 1 : 2;
  }
  return n;
}

}  // namespace

int decode_launch(int fmt, const DecodeParams& p, hipStream_t st) { return decode_dispatch(fmt, p, st); }
int decode_waves(int chunk_tokens) { return waves_for(chunk_tokens); }
int decode_big_chunk() {      // FLAGROT_BIG_CHUNK overrides (experiments)
  static const int v = getenv("FLAGROT_BIG_CHUNK") != nullptr ? atoi(getenv("FLAGROT_BIG_CHUNK")) : BIG_CHUNK;
  return v;
}

// resident workgroups per CU the host split planner may count on (queried once per format and workgroup size)
int decode_occupancy(int fmt, int waves) {
  static int cache[16][2] = {{0}};
  if (fmt < 0 || fmt >= 16) return 0;
  const int wi = waves > 4 ? 1 : 0;
  if (cache[fmt][wi] == 0) {
    switch (fmt) {
      case FMT_INT4: cache[fmt][wi] = occupancy_qm<QM_SYM4, false>(waves); break;
      case FMT_INT4A: cache[fmt][wi] = occupancy_qm<QM_ASYM4, false>(waves); break;
      case FMT_INT2A: cache[fmt][wi] = occupancy_qm<QM_ASYM2, false>(waves); break;
      case FMT_KONLY: cache[fmt][wi] = occupancy_qm<QM_SYM4, true>(waves); break;
      case FMT_KONLYA: cache[fmt][wi] = occupancy_qm<QM_ASYM4, true>(waves); break;
      case FMT_KONLYA2: cache[fmt][wi] = occupancy_qm<QM_ASYM2, true>(waves); break;
      default: return 0;
    }
  }
  return cache[fmt][wi];
}

}  // namespace fr
