// Paged split-K GQA decode attention over FlagRot INT4 / INT2 pages for gfx950 (wave64).  The kernel is priced
// against HBM only: every page byte is read once; both contractions use the matrix pipe as a wide dot product on
// operands that already sit in the right shape (nothing is reshaped into a GEMM).
//
// One workgroup (16 or 12 wavefronts = a whole CU's register file, or 4 for short chunks) per (KV head x q tile of 4 heads,
// split, sequence).  Its wavefronts draw quads of 4 pages from a counter in LDS, so they finish together whatever
// share of the issue slots each one got.  A wavefront streams whole pages (16 tokens x one KV head = one contiguous
// 2304 / 1280 byte chunk) with 128-bit loads:
//   key phase    lane = (token t of a page, quarter x of its code row): one 16-byte load is the four code words (one
//                per 32-group) of that quarter.  A code field masked in place is an fp16 denormal (value
//                code * 2^(position - 24), exact); the eight fields of a word are the lane's share of the B operand of
//                v_mfma_f32_16x16x32_f16 (columns = the page's 16 tokens, 32 deep = the group's 32 dims).  The A
//                operand rows are (head, query variant): the query tile is rotated three ways once per workgroup
//                (identity, H32 per group, H128), split into an fp16 pair (value + remainder: two products) and kept
//                in LDS in the code words' element order.  The zero point leaves through one more small product
//                (zero point x sum of the group's query elements).  A lane then holds, for its (token, head), the
//                score parts of all variants: the one its (token, group) flag bits ask for is picked and scaled by the
//                group's scale word.
//   softmax      exp2-domain online softmax, lane = (token, head); p * V-scale is written to LDS as fp16 in V^T token
//                order (the four lanes of a token exchange their V scale words).
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


// LDS strips are padded so that the few distinct 16-byte rows the lanes of one instruction touch (one per
// row group) start in different banks.
// A wave iteration covers QB blocks of 16 tokens: 4 (64 tokens) for every format.  (Measured for the 2-bit formats:
// 8 blocks per iteration -- the bytes in flight of a 4-bit iteration -- need 155 registers, i.e. three wavefronts per
// SIMD instead of four, and are 4 % slower on configs[2]: that loop is bound by instruction issue, not by latency.)
template <int QM> constexpr int QBLK = 4;
constexpr int PB_RSTRIDE = 17;                     // uint4 per row group (block, c8): 16 + 1 pad (the pad stays zero: below)
constexpr int ZB_RSTRIDE = 5;                      // uint4 per row group: 4 + 1 pad
template <int QM> struct Strip {
  static constexpr int ROWS = 2 * QBLK<QM>;                    // row groups = runs of 8 tokens
  static constexpr int PB_BYTES = ROWS * PB_RSTRIDE * 16;      // per wave: [block][c8][group][head][8 fp16]
  static constexpr int ZB_BYTES = ROWS * ZB_RSTRIDE * 16;      // per wave: [block][c8][group][8 fp16] = zero point (x 2^SH for odd tokens)
  static constexpr int BYTES = PB_BYTES + ZB_BYTES;            // per wave
};
constexpr int DRAW_BATCH = 2;                      // quads per draw from the shared (device-scope) counter
constexpr int DRAW_BITS = 21, DRAW_MASK = (1 << DRAW_BITS) - 1;   // counter slot: quad draws below, merge tickets above
constexpr int BT_CACHE = 1024;                     // block-table entries of the workgroup's page range kept in LDS
constexpr float QPRE = 16.f;                       // the query operands carry 2^4 (fp16 range: |q| up to 127 in any rotation)

template <int QM, int NW>
struct Smem {
  static constexpr int STRIP_BYTES = Strip<QM>::BYTES, PB_BYTES = Strip<QM>::PB_BYTES;
  // A operands of the score products: [group j][lane of the matrix instruction = row (head, variant) + 16 x k block]
  alignas(16) uint4 qhi[4][64];                      // fp16(q * 2^4 / element factor)
  alignas(16) uint4 qlo[4][64];                      // fp16 of what that rounding left
  alignas(16) uint4 qz[4][64];                       // -(sum of the group's query elements), fp16 pair in k blocks 0 / 1 (first word)
  // per-wave strips during the page loop; the waves' partial outputs o[NW][4][128] (fp32) afterwards
  alignas(16) uint8_t work[NW * STRIP_BYTES > NW * 2048 ? NW * STRIP_BYTES : NW * 2048];
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

// Rotates the q tile three ways and stores it as the A operands of the score products: rows = (head, variant), per
// 32-group j and k block (= quarter tg of a code row) the eight elements in the order the masked code words give
// them.  An element is held as an fp16 pair (value + what its rounding left), both times 2^4 and divided by the
// factor its code field comes out of the unpacking with (2^SH for the B elements of a word, 2^4 more for the odd
// groups of the 2-bit words).  The third operand removes the zero points: -(sum of the group's elements as held).
// Wavefronts 0..3: one head each; half 0 writes the rows of variants 0 (identity, or the static kmask rotation) and
// 1 (H32), half 1 those of variant 2 (H128) and the idle row 3; rows of variants a format does not use are zero.
template <int QM, bool K2, class SM>
DEVI void q_prologue(SM& S, const DecodeParams& p, int b, int kvh, int tile) {
  const int w = threadIdx.x >> 6, half = (threadIdx.x >> 5) & 1, l32 = threadIdx.x & 31;
  const int hq = tile * 4 + w;                       // head inside the GQA group
  float x[4] = {0.f, 0.f, 0.f, 0.f};
  if (hq < p.gqa) {
    const uint16_t* qr = static_cast<const uint16_t*>(p.q) + static_cast<long long>(b) * p.q_bs +
                         (static_cast<long long>(kvh) * p.gqa + hq) * 128 + 4 * l32;
    const uint2 raw = *reinterpret_cast<const uint2*>(qr);
    x[0] = bf16_lo(raw.x); x[1] = bf16_hi(raw.x); x[2] = bf16_lo(raw.y); x[3] = bf16_hi(raw.y);
  }
  const int g = l32 >> 3, isB = (l32 >> 2) & 1, tg = l32 & 3;   // the lane's dims 4 l32 + i: group, word half, quarter
  float y[4] = {x[0], x[1], x[2], x[3]};
  if (half == 0) fwht<32>(y, l32); else fwht<128>(y, l32);
  // factor of the lane's code fields after the unpacking (the operand is divided by it)
  const float beta = (isB ? static_cast<float>(1 << UnpackD<QM>::SH) : 1.f) * ((QM == QM_ASYM2 && (g & 1)) ? 16.f : 1.f);
  const float fold = QPRE / beta;
#pragma unroll
  for (int vi = 0; vi < 2; ++vi) {
    const int var = 2 * half + vi;
    float v[4];
    bool live;
    if (K2) {
      live = var < 3;
      const bool rot = var != 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = rot ? y[i] : x[i];
    } else {
      live = var == 0;
      // (a bit mask and not `rot ? y[i] : x[i]`: the compiler turns that into a choice between the two arrays'
      // addresses, which puts both into scratch memory)
      const uint32_t rot = (p.kmask != nullptr && p.kmask[kvh * 4 + g] != 0) ? 0xFFFFFFFFu : 0u;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = __uint_as_float((__float_as_uint(y[i]) & rot) | (__float_as_uint(x[i]) & ~rot));
    }
    uint32_t hb[4], lb[4];
    float qs = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = live ? v[i] * fold : 0.f;
      const _Float16 hi = static_cast<_Float16>(a);
      const _Float16 lo = static_cast<_Float16>(a - static_cast<float>(hi));
      hb[i] = __builtin_bit_cast(uint16_t, hi);
      lb[i] = __builtin_bit_cast(uint16_t, lo);
      qs += (static_cast<float>(hi) + static_cast<float>(lo)) * beta;
    }
    // elements i = 0, 2 are halves 2 isB, 2 isB + 1 of the operand (word isB), i = 1, 3 halves 4 + 2 isB, 5 + 2 isB
    const int m = 4 * w + var, ln = m + 16 * tg;
    uint32_t* dh = reinterpret_cast<uint32_t*>(&S.qhi[g][ln]);
    uint32_t* dl = reinterpret_cast<uint32_t*>(&S.qlo[g][ln]);
    dh[isB] = hb[0] | (hb[2] << 16); dh[2 + isB] = hb[1] | (hb[3] << 16);
    dl[isB] = lb[0] | (lb[2] << 16); dl[2 + isB] = lb[1] | (lb[3] << 16);
    if constexpr (QM != QM_SYM4) {
      qs += hx(qs, 1); qs += hx(qs, 2); qs += hx(qs, 4);
      if ((l32 & 7) == 0) {   // k blocks 0 / 1 carry the pair, in the half the zero point of group g is masked into
        const _Float16 zh = static_cast<_Float16>(-qs);
        const _Float16 zl = static_cast<_Float16>(-qs - static_cast<float>(zh));
        const int sh = 16 * (g & 1);
        S.qz[g][m] = make_uint4(static_cast<uint32_t>(__builtin_bit_cast(uint16_t, zh)) << sh, 0u, 0u, 0u);
        S.qz[g][m + 16] = make_uint4(static_cast<uint32_t>(__builtin_bit_cast(uint16_t, zl)) << sh, 0u, 0u, 0u);
        S.qz[g][m + 32] = make_uint4(0u, 0u, 0u, 0u);
        S.qz[g][m + 48] = make_uint4(0u, 0u, 0u, 0u);
      }
    }
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

// One wave iteration covers a quad = 64 consecutive tokens (four 16-token pages or two 32-token pages), as four
// blocks of 16 tokens.  Key phase: lane = (token t = lane & 15 of a block, quarter x = lane >> 4 of its code row).
// Value phase: lane = V^T entry `lane` of each of the 4 blocks in turn.
template <int QM> struct KRegs {
  static constexpr int NW = QM == QM_ASYM2 ? 2 : 4;   // code words per 16-byte / 8-byte quarter row
  static constexpr int QB = QBLK<QM>;
  uint32_t kc[QB][NW];      // [block][word]: quarter x of token t's code row (word j = group j; 2-bit: groups 2 j, 2 j + 1)
  uint2 ks[QB];             // [block]: the token's 4 K scale words
  uint16_t vs[QB];          // [block]: the token's V scale word of group x; 16 bits wide so that the widening belongs to the use
                            // (a widening at the load would be scheduled right behind it and wait for the keys in flight)
};
// The value product P' V runs on the matrix pipe: sixteen v_mfma_f32_16x16x32_f16 per quad of pages, rows = 16 V^T
// entries, columns = (group, head), 32 tokens deep.  An entry word masked in place (eight tokens as fp16 denormal
// pairs; the matrix pipe keeps denormal inputs) is the A operand of its lane, one 16-byte strip row (p' of a run's eight
// tokens for a (group, head)) the B operand.  The scores stay on the vector pipe (v_dot2_f32_f16).
template <int QM> struct VRegs {
  static constexpr int NW = QM == QM_ASYM2 ? 2 : 4;
  uint32_t vc[QBLK<QM>][NW];   // [2 (block pair s) + entry half][entry word] of lane (entry m = lane & 15, run kc = lane >> 4)
};

// lane offsets of the key-side loads inside a chunk (block 0 of a page; a 32-token page's second block adds constants)
template <int QM, int P> struct KOffs { int k, ks, vs; };
template <int QM, int P>
DEVI KOffs<QM, P> key_offsets(int lane) {
  using L = Lay<QM, P>;
  const int t = lane & 15, x = lane >> 4;
  KOffs<QM, P> o;
  o.k = QM == QM_ASYM2 ? L::K_OFF + 32 * (t ^ ((t >> 1) & 2)) + 8 * x : L::K_OFF + 64 * t + 16 * x;
  o.ks = L::KS_OFF + 8 * t;
  o.vs = L::VS_OFF + (x * P + 8 * (t >> 3) + vs_slot8(t)) * 2;
  return o;
}
// chunk[b]: the chunk of block b's page (wave uniform); 32-token pages: blocks 2 s, 2 s + 1 are the halves of page s
template <int QM, int P>
DEVI void load_k(KRegs<QM>& r, const uint8_t* const (&chunk)[QBLK<QM>], const KOffs<QM, P>& o) {
#pragma unroll
  for (int b = 0; b < QBLK<QM>; ++b) {
    const int hp = P == 32 ? (b & 1) : 0;            // second half of a 32-token page: 16 tokens further
    const uint8_t* ch = chunk[b];
    if constexpr (QM == QM_ASYM2) {
      const u32x2 k = gload<u32x2>(ch + o.k + hp * 16 * 32);
      r.kc[b][0] = k.x; r.kc[b][1] = k.y;
    } else {
      const u32x4 k = gload<u32x4>(ch + o.k + hp * 16 * 64);
      r.kc[b][0] = k.x; r.kc[b][1] = k.y; r.kc[b][2] = k.z; r.kc[b][3] = k.w;
    }
    { const u32x2 t2 = gload<u32x2>(ch + o.ks + hp * 16 * 8); r.ks[b] = make_uint2(t2.x, t2.y); }
    r.vs[b] = gload<uint16_t>(ch + o.vs + hp * 16 * 2);
  }
}

template <int QM, int P>
DEVI void load_v(VRegs<QM>& r, const uint8_t* const (&chunk)[QBLK<QM>], int lane) {
  using L = Lay<QM, P>;
  // lane = (entry m = lane & 15 (+ 16 for the second half), run kc = lane >> 4 of the 32 tokens of half s of the quad:
  // 16-token pages 2 s, 2 s + 1 with two runs each, or the 32-token page s with four)
  constexpr int R = P / 8;                       // runs of 8 tokens (entries per dim group) per page
  const int m = lane & 15, kc = lane >> 4;
#pragma unroll
  for (int s2 = 0; s2 < QBLK<QM> / 2; ++s2) {
    const uint8_t* ch = P == 16 ? ((kc >> 1) ? chunk[2 * s2 + 1] : chunk[2 * s2]) : chunk[2 * s2];
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
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
struct WaveState {
  float m;           // running maximum of head x = lane >> 4 (log2 domain; uniform over the head's 16 lanes)
  float l;           // this lane's share of the running sum of head x
  // 2^-24 sum p' code (zero points not yet removed), [entry word parity]: column lane & 15 = (group g, head), rows =
  // entries 16 (g & 1) + 4 (lane >> 4) + r, entry word 2 (g >> 1) + parity
  f32x4 ot[2];
  float z[2];        // lane = (page, half, group, head pair): its share of sum p' zero point, heads 2 hp and 2 hp + 1
};

// exchange among the four lanes of a token (lane ^ 16, ^ 32, ^ 48): one crossbar instruction each, no vector ALU work
// (a v_permlane32_swap costs two copies, a wait state and a select around it).  byte address of the source lane: 4 x lane
DEVI uint32_t lane_from(uint32_t v, int src_lane4) {
  return static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(src_lane4, static_cast<int>(v)));
}
// all-reduce over the 16 lanes of a row (DPP: quad permutes, then the mirrors of 8 and of 16 lanes)
DEVI float row_max16(float v) {
  v = fmaxf(v, dpp_xor1(v)); v = fmaxf(v, dpp_xor2(v));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true)));   // row_half_mirror
  return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true))); // row_mirror
}
DEVI float row_sum16(float v) {
  v += dpp_xor1(v); v += dpp_xor2(v);
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));
  return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));
}
// the 16-bit scale word `j` of a packed pair as fp32; its sign bit is a flag, which the caller drops with fabsf (a
// source modifier of the multiply-add that uses the value).  Plain code on purpose: instructions written as inline
// assembly are invisible to the compiler's hazard handling, and a register that a matrix instruction is still
// writing (an unused row of its result) may be handed to them as their output.
DEVI float word_value(uint32_t pair, int j) {
  const uint16_t w = static_cast<uint16_t>((j & 1) ? (pair >> 16) : pair);
  return static_cast<float>(__builtin_bit_cast(_Float16, w));
}

// Scores of the lane's (token, head) for the four blocks of the quad: raw sums 2^-20 sum_j scale_j sum (c - z) q'
// (the factor and qscale are applied with the softmax).
template <int QM, bool K2, class SM>
DEVI void key_phase(const SM& S, const KRegs<QM>& r, int lane, float (&sc)[QBLK<QM>]) {
  constexpr int QB = QBLK<QM>;
  constexpr int ZM = QM == QM_ASYM4 ? 15 : QM == QM_ASYM2 ? 3 : 0;
  // the zero point of group j, masked in place (an fp16 denormal z 2^-24 in the low half of the pair word for even j,
  // in the high half for odd j): lanes of k blocks 0 and 1 feed it (first element pair of their eight) against the pair
  // -(sum q) of the third operand
  const uint32_t zlane = (lane < 32) ? static_cast<uint32_t>(ZM) : 0u;
  bool full[QB];
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    // the whole-head flag is bit 15 of the token's group-0 V scale word (lane x = 0 of the token's four lanes holds it);
    // the words of the other value groups never carry that bit (scale words are non-negative fp16 patterns), so the
    // union over the four lanes names it
    full[b] = false;
    if constexpr (K2) {
      uint32_t f = r.vs[b] & 0x8000u;
      f |= lane_from(f, 4 * (lane ^ 16));
      f |= lane_from(f, 4 * (lane ^ 32));
      full[b] = f != 0u;
    }
    sc[b] = 0.f;
  }
  // group by group (one set of A operands live at a time), the four blocks of a group back to back
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const half8 qh = __builtin_bit_cast(half8, S.qhi[j][lane]), ql = __builtin_bit_cast(half8, S.qlo[j][lane]);
    half8 qz;
    if constexpr (ZM != 0) qz = __builtin_bit_cast(half8, S.qz[j][lane]);
#pragma unroll
    for (int b0 = 0; b0 < QB; b0 += 4) {
    f32x4 acc[4];
#pragma unroll
    for (int bb = 0; bb < 4; ++bb) {
      const int b = b0 + bb;
      uint32_t x[4];
      if constexpr (QM == QM_ASYM2) {     // two groups per word: the odd one 4 bits higher (2^4 is in its query operand)
        if (j & 1) UnpackD<QM>::run_hi(r.kc[b][j >> 1], x); else UnpackD<QM>::run(r.kc[b][j >> 1], x);
      }
      else UnpackD<QM>::run(r.kc[b][j], x);
      const half8 kb = __builtin_bit_cast(half8, make_uint4(x[0], x[1], x[2], x[3]));
      f32x4 a = __builtin_amdgcn_mfma_f32_16x16x32_f16(qh, kb, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
      a = __builtin_amdgcn_mfma_f32_16x16x32_f16(ql, kb, a, 0, 0, 0);
      if constexpr (ZM != 0) {
        const uint32_t kwz = (j & 2) ? r.ks[b].y : r.ks[b].x;
        const uint32_t zz = kwz & (zlane << (16 * (j & 1)));
        // (the same instruction as the two products before it: a chain of one kind on one accumulator)
        a = __builtin_amdgcn_mfma_f32_16x16x32_f16(qz, __builtin_bit_cast(half8, make_uint4(zz, 0u, 0u, 0u)), a, 0, 0, 0);
      }
      acc[bb] = a;
    }
#pragma unroll
    for (int bb = 0; bb < 4; ++bb) {     // rows 4 x + variant of the product: the lane's head, every variant
      const int b = b0 + bb;
      const uint32_t kw = (j & 2) ? r.ks[b].y : r.ks[b].x;
      float pick = acc[bb][0];
      if constexpr (K2) {
        const bool h32 = (kw >> (16 * (j & 1) + 15)) & 1u;
        pick = full[b] ? acc[bb][2] : (h32 ? acc[bb][1] : acc[bb][0]);
      }
      sc[b] += pick * fabsf(word_value(kw, j));
    }
    }
  }
}

// online softmax step for the quad, lane = (token, head x): the running maximum is only re-reduced when some lane
// beats it; then p' = p * V scale per group as fp16 and the zero points go to the wave's strips in V^T token order.
// qs20 = qscale * 2^20 (the factor the raw score sums lack); sc0 lowers the scores of odd tokens by SH (below).
template <int QM, class SM>
DEVI void softmax_phase(SM& S, WaveState& st, const KRegs<QM>& r, float (&sc)[QBLK<QM>], const bool (&valid)[QBLK<QM>],
                        float qs20, float sc0, int lane, int wave) {
  constexpr int ZM = QM == QM_ASYM4 ? 15 : QM == QM_ASYM2 ? 3 : 0;
  constexpr int QB = QBLK<QM>;
  bool beat = false;
  float mx = -INFINITY;
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    sc[b] = valid[b] ? sc[b] * qs20 + sc0 : -INFINITY;
    mx = fmaxf(mx, sc[b]);
  }
  beat = mx > st.m;
  // The state is multiplied every time (by 1 unless the maxima moved): modifying it only inside the rare branch makes
  // the compiler keep two copies of all its registers and move them on the common path.
  float al = 1.f, az0 = 1.f, az1 = 1.f, am = 1.f;
  if (__builtin_expect(__any(beat), 0)) {   // rare after the first quads
    const float mn = fmaxf(st.m, row_max16(mx));
    am = mn == -INFINITY ? 1.f : fexp2(st.m - mn);
    st.m = mn;
    // the factors of the four heads (rows of 16 lanes) for the lanes whose accumulator columns belong to them
    const float a0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am), 0));
    const float a1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am), 16));
    const float a2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am), 32));
    const float a3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am), 48));
    al = (lane & 2) ? ((lane & 1) ? a3 : a2) : ((lane & 1) ? a1 : a0);     // accumulator column: head lane & 3
    az0 = (lane & 1) ? a2 : a0;
    az1 = (lane & 1) ? a3 : a1;
  }
  st.l *= am;
  st.ot[0] *= al; st.ot[1] *= al;
  st.z[0] *= az0; st.z[1] *= az1;
  // Odd tokens are unpacked from the V^T words with the factor 2^SH (UnpackD): their scores were lowered by SH (p
  // carries 2^-SH), their zero point is raised by 2^SH; zero points are fp16 denormals like the codes.
  const int t = lane & 15, x = lane >> 4;
  const int sl = vslot(t & 7);
  uint16_t* pb = reinterpret_cast<uint16_t*>(S.pb(wave)) + (t >> 3) * PB_RSTRIDE * 8 + sl;   // + block * 2 rows; + (group * 4 + head) * 8
  uint16_t* zb = reinterpret_cast<uint16_t*>(S.zb(wave)) + (t >> 3) * ZB_RSTRIDE * 8 + x * 8 + sl;
  const int zsh = (lane & 1) ? UnpackD<QM>::SH : 0;      // odd position inside the page
  const int c0 = ((x) * 4 + x) * 8, c1 = ((x ^ 1) * 4 + x) * 8, c2 = ((x ^ 2) * 4 + x) * 8, c3 = ((x ^ 3) * 4 + x) * 8;
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    const float pe = fexp2(sc[b] - st.m);       // masked tokens: 2^-inf = 0 (the maximum is finite once a quad has been seen)
    st.l += pe;
    const uint32_t pp = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(pe, pe));
    // the token's four V scale words, sign bits stripped: own group x, then the lanes 16, 32, 48 further (groups
    // x ^ 1, x ^ 2, x ^ 3); unwritten slots may hold any pattern: masked
    const uint32_t v0 = valid[b] ? (r.vs[b] & 0x7FFFu) : 0u;
    const uint32_t v1 = lane_from(v0, 4 * (lane ^ 16)), v2 = lane_from(v0, 4 * (lane ^ 32)), v3 = lane_from(v0, 4 * (lane ^ 48));
    const uint32_t xa = pk_mul(pp, (v1 << 16) | v0), xb = pk_mul(pp, (v3 << 16) | v2);
    uint16_t* row = pb + b * 2 * PB_RSTRIDE * 8;
    row[c0] = static_cast<uint16_t>(xa);
    row[c1] = static_cast<uint16_t>(xa >> 16);
    row[c2] = static_cast<uint16_t>(xb);
    row[c3] = static_cast<uint16_t>(xb >> 16);
    if constexpr (QM != QM_SYM4) zb[b * 2 * ZB_RSTRIDE * 8] = static_cast<uint16_t>((r.vs[b] & ZM) << zsh);
  }
}

template <int QM, class SM>
DEVI void value_phase(const SM& S, WaveState& st, const VRegs<QM>& r, int lane, int wave) {
  // An entry word (entry half eh, word sub) holds channels of group 2 (sub >> 1) + eh only.  The products of all
  // four groups share one accumulator per word parity: the B operand of a group is the strip row with the columns of
  // the other groups zero (those lanes read the row group's pad entry, which nobody writes and which is zeroed once),
  // so each column collects its own group's rows.
  const int n = lane & 15, kc = lane >> 4;
  const uint4* rowg = reinterpret_cast<const uint4*>(S.pb(wave)) + kc * PB_RSTRIDE;
#pragma unroll
  for (int s2 = 0; s2 < QBLK<QM> / 2; ++s2) {   // 32 tokens: the runs (block 2 s + (kc >> 1), c8 = kc & 1) = strip row group 4 s + kc
    half8 b[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint4* src = rowg + ((n >> 2) == g ? n : 16);
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
  if constexpr (QM != QM_SYM4) {   // sum p' zero point: lane = (block, block half, group, head pair), 8 row groups at a time
#pragma unroll
    for (int r8 = 0; r8 < Strip<QM>::ROWS; r8 += 8) {
    const int rg = r8 + (lane >> 3), g = (lane >> 1) & 3, hp = lane & 1;
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

// The workgroup's running maxima per head after every wavefront has put its four into S.m: lane w < NW fetches
// wavefront w's four at once, one row reduction, one broadcast -- a single LDS round trip (a loop over the
// wavefronts is NW dependent ones).
template <int NW, class SM>
DEVI void workgroup_max(const SM& S, int lane, float (&M)[4]) {
  float4 v = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
  if (lane < NW) v = *reinterpret_cast<const float4*>(&S.m[lane][0]);
  M[0] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, row_max16(v.x))));
  M[1] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, row_max16(v.y))));
  M[2] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, row_max16(v.z))));
  M[3] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, row_max16(v.w))));
}
// element i of four values held in registers (selects on values: an index into an array of locals would put the
// array into scratch memory, and a kernel that uses scratch starts its workgroups late)
DEVI float pick4(float v0, float v1, float v2, float v3, int i) {
  const float lo = (i & 1) ? v1 : v0, hi = (i & 1) ? v3 : v2;
  return (i & 2) ? hi : lo;
}

template <int QM, bool K2, int P, int NW>
__global__ void __launch_bounds__(64 * NW, 4) k_decode(const DecodeParams p, int ntile, int nparts) {
  using L = Lay<QM, P>;
  __shared__ Smem<QM, NW> S;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kvh = blockIdx.x / ntile, tile = blockIdx.x % ntile;
  // Workgroups are dispatched in linear order and the CU's arbiter favours the older wavefronts: the splits of one
  // sequence are spread over the whole dispatch order (split slowest) so that every sequence gets the same mix.
  const int lin = blockIdx.z * gridDim.y + blockIdx.y;
  const int split = lin / p.B, b = lin % p.B;
  const bool is_tail = p.tail != nullptr && split == p.nsplit;
  // The block-table entries of the workgroup's page range are requested before the sequence length is known (the
  // length load and these loads are then in flight together: one memory latency less before the first page arrives).
  // If the range is not empty it starts at this token; entries are bounded by the row's length, and whatever lies
  // past the sequence's last page is never used (page indices are clamped to the range).  Shared rows (stride 0)
  // have no known length: they are fetched once the length is there.
  const bool dyn = p.dyn != 0;    // the body workgroups of a (sequence, KV head, q tile) draw quads from one counter
  const int* const btrow = p.block_table + static_cast<long long>(b) * p.bt_stride;
  const int pg0s = (dyn ? p.kv_start : max(split * p.chunk, p.kv_start)) / P;
  constexpr int SPEC = BT_CACHE / (64 * NW);      // entries per thread
  int spec[SPEC];
  int nspec = 0;
  if (!is_tail && p.bt_stride > 0)
    nspec = min(min(BT_CACHE, p.bt_stride - pg0s), ((dyn ? p.nsplit : 1) * p.chunk + P - 1) / P + 1);
#pragma unroll
  for (int k = 0; k < SPEC; ++k) {
    const int i = threadIdx.x + k * 64 * NW;
    spec[k] = i < nspec ? btrow[pg0s + i] : 0;
  }
  // ... and each wavefront asks for the entries of its own first quad itself (lanes 0..3), so that the quad's keys can
  // be requested as soon as the length has confirmed that the quad lies inside the range: before the query prologue
  // and its barrier, not after them
  constexpr int QB = QBLK<QM>;                // blocks of 16 tokens per wave iteration ("quad": the name stays)
  constexpr int PPQ = 16 * QB / P;            // pages per wave iteration
  const int qi0 = dyn ? split * NW + wave : wave;
  int mine4 = 0;
  if (nspec > 0 && lane < PPQ && PPQ * qi0 + lane < p.bt_stride - pg0s) mine4 = btrow[pg0s + PPQ * qi0 + lane];   // (PPQ <= 8)
  const int len = p.seq_lens[b];
  const long long part_id = ((static_cast<long long>(b) * p.Hkv + kvh) * ntile + tile) * nparts + split;
  const bool act = wave < 4;      // the 256 threads that own the workgroup's 4 x 128 outputs

  // the (sequence, KV head, q tile)'s counter slot: merge ticket, and in the dynamic mode the quad draw counter
  const int tpc = p.counter_div;                                 // q tiles that share one counter slot
  int* const ctr = p.counter + (static_cast<long long>(b) * p.Hkv + kvh) * (ntile / tpc) + tile / tpc;
  float Mwg[4];                   // the workgroup's maxima per head (uniform)
  if (!is_tail) {
    const int lo = dyn ? min(p.kv_start, len) : max(split * p.chunk, min(p.kv_start, len));
    const int hi = dyn ? len : min(len, (split + 1) * p.chunk);
    WaveState st;
    st.m = -INFINITY; st.l = 0.f;
    st.z[0] = st.z[1] = 0.f;
    st.ot[0] = st.ot[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (lo < hi) {   // uniform over the workgroup
      const int pg0 = lo / P, pg1 = (hi + P - 1) / P;
      const int* bt = p.block_table + static_cast<long long>(b) * p.bt_stride;
      // quads beyond a wave's first one are drawn: from S.next (the workgroup owns a range) or from the slot's draw
      // counter (all body wavefronts of the slot share the range)
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
      // this wavefront's first quad, requested now if it lies wholly inside the range (its entries came with mine4)
      typedef const __attribute__((address_space(1))) uint8_t* gptr;
      const gptr pool = (gptr)p.pool;
      const KOffs<QM, P> koff = key_offsets<QM, P>(lane);
      KRegs<QM> cur;
      const uint8_t* ch[QB];
      const bool early = nspec > 0 && PPQ * (qi0 + 1) <= pg1 - pg0;      // uniform over the wavefront
      if (early) {
#pragma unroll
        for (int k = 0; k < PPQ; ++k) {
          const int page = __builtin_amdgcn_readlane(mine4, k);
          const uint8_t* c = (const uint8_t*)(pool + (static_cast<long long>(page) * p.Hkv + kvh) * L::CHUNK);
          if constexpr (P == 16) ch[k] = c;
          else { ch[2 * k] = c; ch[2 * k + 1] = c; }
        }
        load_k<QM, P>(cur, ch, koff);
      }
      if (nspec > 0) {      // (pg0 == pg0s whenever the range is not empty)
#pragma unroll
        for (int k = 0; k < SPEC; ++k) {
          const int i = threadIdx.x + k * 64 * NW;
          if (i < nspec) S.btc[i] = spec[k];
        }
      } else {
        for (int i = threadIdx.x; i < min(pg1 - pg0, BT_CACHE); i += 64 * NW) S.btc[i] = bt[pg0 + i];
      }
      if (threadIdx.x == 0) S.next = NW;
      // the pad entry of every strip row group: what the value phase reads for the columns of foreign groups
      for (int i = threadIdx.x; i < NW * Strip<QM>::ROWS; i += 64 * NW)
        (reinterpret_cast<uint4*>(S.pb(i / Strip<QM>::ROWS)) + (i % Strip<QM>::ROWS) * PB_RSTRIDE)[16] = make_uint4(0u, 0u, 0u, 0u);
      if (act) q_prologue<QM, K2>(S, p, b, kvh, tile);
      __syncthreads();
      const int npg = pg1 - pg0;
      const int nquad = (npg + PPQ - 1) / PPQ;
      // odd tokens: the B fields of a V^T word come out of the unpacking with the factor 2^SH, so their scores are
      // lowered by SH (log2 domain) and their share of the softmax sum is raised again at the end
      const float sc0 = (lane & 1) ? -static_cast<float>(UnpackD<QM>::SH) : 0.f;
      const float qs20 = p.qscale * (16777216.f / QPRE);         // raw score sums carry 2^-24 from the codes and QPRE from the query
      // chunk addresses of a quad's four blocks (wave uniform).  Pages past the range name the range's last page again
      // (their tokens are masked).  The entry comes from LDS; past the cached window it is read from memory.
      auto chunks_of = [&](int quad, const uint8_t* (&ch)[QB]) {
#pragma unroll
        for (int k = 0; k < PPQ; ++k) {
          const int i = min(PPQ * quad + k, npg - 1);
          int page = S.btc[min(i, BT_CACHE - 1)];
          if (__builtin_expect(i >= BT_CACHE, 0)) page = bt[pg0 + i];
          page = __builtin_amdgcn_readfirstlane(page);
          const uint8_t* c = (const uint8_t*)(pool + (static_cast<long long>(page) * p.Hkv + kvh) * L::CHUNK);
          if constexpr (P == 16) ch[k] = c;
          else { ch[2 * k] = c; ch[2 * k + 1] = c; }
        }
      };
      __builtin_amdgcn_s_setprio(1);
      // this wave's current quad: the first one by position
      const int nworker = dyn ? p.nsplit * NW : 0;
      int qi = qi0;
      if (!early) {
        chunks_of(qi, ch);
        if (qi < nquad) load_k<QM, P>(cur, ch, koff);
      }
      int more = 0, nextq = 0;       // quads left of the batch drawn last (the shared counter hands out DRAW_BATCH at a time)
      while (qi < nquad) {
        // The next quad.  Shared (device-scope) counter: the draw made an iteration ago is read where the keys of this
        // quad are awaited anyway, and the following draw goes out ahead of this iteration's loads.  Counter in LDS:
        // the draw goes out here and is read after the softmax, in this same iteration -- a wavefront that held its
        // next quad for a whole iteration would start the range's last quad a whole iteration after the others ran dry.
        int qn = 0;
        if (dyn) {
          if (more > 0) { qn = nextq++; --more; }
          else {
            // (read here and not before: without the opaque copy its broadcast is moved up to the draw itself, which
            // then waits for the counter's round trip on the spot)
            int drawn = take;
            asm volatile("" : "+v"(drawn));
            drawn = __builtin_amdgcn_readfirstlane(drawn);
            qn = (drawn & DRAW_MASK) * DRAW_BATCH + nworker;
            take = draw();
            nextq = qn + 1; more = DRAW_BATCH - 1;
          }
        } else {
          take = draw();
        }
        VRegs<QM> vr;                // this quad's V^T entries: in flight during the key phase
        load_v<QM, P>(vr, ch, lane);
        bool valid[QB];
        {
          const int tok0 = (pg0 + PPQ * qi) * P + (lane & 15);
#pragma unroll
          for (int k = 0; k < QB; ++k) valid[k] = tok0 + 16 * k >= lo && tok0 + 16 * k < hi;
        }
        float sc[QB];
        key_phase<QM, K2>(S, cur, lane, sc);
        softmax_phase<QM>(S, st, cur, sc, valid, qs20, sc0, lane, wave);
        // The key registers are free: the next quad's keys fly during the value phase.  The loads are issued on every
        // path (past the range chunks_of names the range's last page again, a cache hit nobody uses): were they inside
        // a branch, the wait counts after the join would be those of the path without them, and the value phase
        // would wait for these loads as well.
        if (!dyn) {
          int drawn = take;
          asm volatile("" : "+v"(drawn));
          qn = __builtin_amdgcn_readfirstlane(drawn);
        }
        chunks_of(qn, ch);
        load_k<QM, P>(cur, ch, koff);
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
    // head x = lane >> 4 lives in a row of 16 lanes
    const float lsum = row_sum16(st.l * unfold);
    if ((lane & 15) == 0) S.m[wave][lane >> 4] = st.m;
    __syncthreads();     // every wave is done with its strip: the partial outputs may overwrite them
    {
      workgroup_max<NW>(S, lane, Mwg);
      // this wavefront's factors 2^(m - M) per head (uniform): its own maxima sit in lanes 0, 16, 32, 48
      float f[4];
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        const float mh = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, st.m), 16 * h));
        f[h] = mh == -INFINITY ? 0.f : fexp2(mh - Mwg[h]);
      }
      if ((lane & 15) == 0) S.l[wave][lane >> 4] = pick4(f[0], f[1], f[2], f[3], lane >> 4) * lsum;
      const float fl = pick4(f[0], f[1], f[2], f[3], hl);
      const int kc = lane >> 4;      // the lane's four entry rows: 4 kc + r
      float* o = S.o(wave, hl);
#pragma unroll
      for (int y = 0; y < 2; ++y) {
        // entry e = 16 (gl & 1) + 4 kc + r, word sub = 2 (gl >> 1) + y: dim 64 (sub >> 1) + 16 (e >> 3) + 8 (sub & 1) + (e & 7)
        const int d = 32 * gl + 16 * (kc >> 1) + 8 * y + 4 * (kc & 1);
        *reinterpret_cast<float4*>(o + d) = make_float4(fl * st.ot[y][0], fl * st.ot[y][1], fl * st.ot[y][2], fl * st.ot[y][3]);
      }
    }
    __syncthreads();
  } else {
    float m[4], l[4], o[4][2];
    tail_partial<NW>(p, b, kvh, tile, m, l, o);
    if (lane < 4) S.m[wave][lane] = pick4(m[0], m[1], m[2], m[3], lane);
    __syncthreads();
    workgroup_max<NW>(S, lane, Mwg);
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const float f = m[h] == -INFINITY ? 0.f : fexp2(m[h] - Mwg[h]);
      if (lane == 0) S.l[wave][h] = f * l[h];
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
    // the sums were scaled by their wavefront's factor when they were stored: lane w fetches wavefront w's
    const float lw = lane < NW ? S.l[lane][oh] : 0.f;
    pm = pick4(Mwg[0], Mwg[1], Mwg[2], Mwg[3], oh);
    pl = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, row_sum16(lw))));
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

// Wavefronts per workgroup: 4, or from 1024 tokens per split one large workgroup that fills a CU: 16 wavefronts
// (4 per SIMD; every format's loop fits 128 registers per lane).
template <int QM> constexpr int BIGW = 16;
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
    if (p.wg_waves > 4) hipLaunchKernelGGL((k_decode<QM, K2, 32, BIGW<QM>>), grid, dim3(64 * BIGW<QM>), 0, st, p, ntile, nparts);
    else hipLaunchKernelGGL((k_decode<QM, K2, 32, 4>), grid, dim3(256), 0, st, p, ntile, nparts);
  } else if (p.wg_waves > 4) hipLaunchKernelGGL((k_decode<QM, K2, 16, BIGW<QM>>), grid, dim3(64 * BIGW<QM>), 0, st, p, ntile, nparts);
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
  const void* f = waves > 4 ? reinterpret_cast<const void*>(&k_decode<QM, K2, 16, BIGW<QM>>) : reinterpret_cast<const void*>(&k_decode<QM, K2, 16, 4>);
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, f, 64 * (waves > 4 ? BIGW<QM> : 4), 0) != hipSuccess || n < 1) {
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
