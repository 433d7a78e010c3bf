// Building blocks of the matrix-pipe decode kernels over FlagRot INT4 / INT2 pages (decode.hip: head dim 128;
// decode_wide_mma.hip: head dim 256 as two 128-d half chunks): LDS strip geometry, the query prologue, the page loaders,
// and the three phases of a wave iteration over a quad of 64 tokens -- key phase (scores on the matrix pipe), online
// softmax with the p * V-scale strips, value phase.  The phases take the LDS block as a template parameter: anything
// with qhi / qlo / qz [group][lane] operand tables and pb(wave) / zb(wave) strips serves.
#pragma once
#include "fr_common.hpp"
#include "fr_launch.hpp"
#include "fr_unpack.hpp"

namespace fr {
namespace dec {

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
constexpr uint32_t WIDE_VSCALE = 0x4800u;          // fp16 pattern of the V scale (8.0) above which a quad's value products are rescaled (value_phase)
// ... by 2^-8, or by 2^-4 where the odd tokens' p already carries 2^-4 (the 4-bit fields with zero points): p * scale
// must stay a NORMAL fp16 number for ordinary scales, or the strips themselves lose what the rescaling is there to keep
// (measured with 2^-8 on those pages: 3e-3 on sums of 25 with equal weights).  fold: fp16 pattern of the factor; up: its
// inverse as an fp16 pair; rest: inverse - 1, what the zero-point sums (plain vector sums) still lack.
template <int QM> struct WideFold {
  static constexpr uint32_t fold = QM == QM_ASYM4 ? 0x2C00u : 0x1C00u;
  static constexpr uint32_t up = QM == QM_ASYM4 ? 0x4C004C00u : 0x5C005C00u;
  static constexpr float rest = QM == QM_ASYM4 ? 15.f : 255.f;
};
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
  alignas(16) float tailw[NW][64];                   // tail_partial: a wavefront's weights of 16 BF16 rows x 4 heads
  int btc[BT_CACHE];
  int next;                                          // next quad of 4 pages nobody has taken yet
  int last;
  static_assert(STRIP_BYTES >= 2048 && STRIP_BYTES % 16 == 0, "a wavefront's strips must hold its partial outputs");
  DEVI uint8_t* pb(int w) { return work + w * STRIP_BYTES; }
  DEVI const uint8_t* pb(int w) const { return work + w * STRIP_BYTES; }
  DEVI uint8_t* zb(int w) { return work + w * STRIP_BYTES + PB_BYTES; }
  DEVI const uint8_t* zb(int w) const { return work + w * STRIP_BYTES + PB_BYTES; }
  // a wavefront's partial outputs [4][128] take the place of its OWN strips (2 KB of them): no other wavefront's strip is touched
  DEVI float* o(int w, int h) { return reinterpret_cast<float*>(work + w * (STRIP_BYTES > 2048 ? STRIP_BYTES : 2048)) + h * 128; }
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
      const float a = live ? v[i] * (QPRE / key_field_factor<QM>(isB, g, i)) : 0.f;
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
// page words: read once per launch (twice where two q tiles share a KV head), never written by it -- the non-temporal
// hint keeps them from displacing each other in the caches; a kernel that only reads the pages of a launch is 11 %
// faster with it (46.9 vs 52.6 us for 302 MB)
template <class T, bool STREAM = true> DEVI T gload_stream(const uint8_t* p) {
  typedef const __attribute__((address_space(1))) T* gp;
  if constexpr (STREAM) return __builtin_nontemporal_load((gp)(p));
  else return *(gp)(p);
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
// (unsigned 32-bit lane offsets on a wave-uniform chunk address: the loads then take the chunk address from scalar
// registers and the offset from one vector register -- no 64-bit vector additions per load)
template <int QM, int P> struct KOffs { uint32_t k, ks, vs; };
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
// STREAM = false: ordinary loads, for the kernels whose q tiles of one KV head count on finding each other's lines in L2
template <int QM, int P, bool STREAM = true>
DEVI void load_k(KRegs<QM>& r, const uint8_t* const (&chunk)[QBLK<QM>], const KOffs<QM, P>& o0) {
  // (the offsets are made opaque at the point of use: hoisted out of the page loop as 64-bit values they would be added
  // to the chunk address by vector instructions, one 64-bit addition per load)
  KOffs<QM, P> o = o0;
  asm volatile("" : "+v"(o.k), "+v"(o.ks), "+v"(o.vs));
#pragma unroll
  for (int b = 0; b < QBLK<QM>; ++b) {
    const int hp = P == 32 ? (b & 1) : 0;            // second half of a 32-token page: 16 tokens further
    const uint8_t* ch = chunk[b];
    if constexpr (QM == QM_ASYM2) {
      const u32x2 k = gload_stream<u32x2, STREAM>(ch + static_cast<size_t>(o.k + hp * 16 * 32));
      r.kc[b][0] = k.x; r.kc[b][1] = k.y;
    } else {
      const u32x4 k = gload_stream<u32x4, STREAM>(ch + static_cast<size_t>(o.k + hp * 16 * 64));
      r.kc[b][0] = k.x; r.kc[b][1] = k.y; r.kc[b][2] = k.z; r.kc[b][3] = k.w;
    }
    { const u32x2 t2 = gload_stream<u32x2, STREAM>(ch + static_cast<size_t>(o.ks + hp * 16 * 8)); r.ks[b] = make_uint2(t2.x, t2.y); }
    r.vs[b] = gload_stream<uint16_t, STREAM>(ch + static_cast<size_t>(o.vs + hp * 16 * 2));
  }
}

template <int QM, int P, bool STREAM = true>
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
        const u32x2 v = gload_stream<u32x2, STREAM>(ch + L::V_OFF + 8 * (R * (16 * eh + m) + c8));
        r.vc[2 * s2 + eh][0] = v.x; r.vc[2 * s2 + eh][1] = v.y;
      } else {
        const u32x4 v = gload_stream<u32x4, STREAM>(ch + L::V_OFF + 16 * (R * (16 * eh + m) + c8));
        r.vc[2 * s2 + eh][0] = v.x; r.vc[2 * s2 + eh][1] = v.y; r.vc[2 * s2 + eh][2] = v.z; r.vc[2 * s2 + eh][3] = v.w;
      }
    }
  }
}

// The split merge of one output thread (head oh, channels 2 lane and 2 lane + 1) over the nparts partials of its
// (sequence, KV head, q tile), in their order.  Eight partials at a time, every load of a batch -- maxima, sums and
// channels alike -- in flight before the first is used and none under a condition (the batch's last partial is read
// again in place of those past the end, with weight 0); the running maximum moves from batch to batch and what was
// summed so far is rescaled with it.  One partial per turn of a loop waits a memory latency per turn (32 splits then
// took 20 of the 28 us of a single-sequence launch), and a pass for the maxima ahead of the sums is one latency more.
DEVI void merge_parts(const float* mlpart, const float* opart, long long base, int nparts, int oh, int lane,
                      float& M, float& Lsum, float& o0, float& o1) {
  constexpr int NB = 8;
  auto ld = [](const float* q) { return __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
  M = -INFINITY; Lsum = 0.f; o0 = 0.f; o1 = 0.f;
  for (int s0 = 0; s0 < nparts; s0 += NB) {
    float m[NB], l[NB], a[NB], c[NB];
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      const long long part = base + min(s0 + k, nparts - 1);
      m[k] = ld(mlpart + part * 8 + 2 * oh);
      l[k] = ld(mlpart + part * 8 + 2 * oh + 1);
      a[k] = ld(opart + part * 512 + oh * 128 + 2 * lane);
      c[k] = ld(opart + part * 512 + oh * 128 + 2 * lane + 1);
    }
    float top = M;
#pragma unroll
    for (int k = 0; k < NB; ++k) top = fmaxf(top, m[k]);          // (a partial read twice changes no maximum)
    const float keep = M == -INFINITY ? 0.f : fexp2(M - top);      // nothing summed yet, or top is finite
    M = top;
    Lsum *= keep; o0 *= keep; o1 *= keep;
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      const float f = (s0 + k < nparts && m[k] != -INFINITY) ? fexp2(m[k] - M) : 0.f;
      Lsum += f * l[k];
      o0 += f * a[k];
      o1 += f * c[k];
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
// the tokens' whole-head flags (key-only kinds; false otherwise)
template <int QM, bool K2>
DEVI void whole_head_flags(const KRegs<QM>& r, int lane, bool (&full)[QBLK<QM>]) {
#pragma unroll
  for (int b = 0; b < QBLK<QM>; ++b) {
    // the whole-head flag is bit 15 of the token's group-0 V scale word (lane x = 0 of the token's four lanes holds it);
    // the words of the other value groups never carry that bit (scale words are non-negative fp16 patterns), so the
    // union over the four lanes names it
    full[b] = false;
    if constexpr (K2) {
      // as a lane mask in scalar registers: the four lanes of token t are bits t, t + 16, t + 32, t + 48 -- folded onto
      // 16 bits and spread again by scalar instructions, no lane exchange and no vector work beyond the bit test
      unsigned long long m = __builtin_amdgcn_ballot_w64((r.vs[b] & 0x8000u) != 0u);
      m |= m >> 32; m |= m >> 16; m &= 0xFFFFull; m |= m << 16; m |= m << 32;
      full[b] = __builtin_amdgcn_inverse_ballot_w64(m);
    }
  }
}

// sc += the score parts of the lane's (token, head) for the four blocks, given the tokens' whole-head flags
template <int QM, bool K2, class SM>
DEVI void key_scores(const SM& S, const KRegs<QM>& r, int lane, const bool (&full)[QBLK<QM>], float (&sc)[QBLK<QM>]) {
  constexpr int QB = QBLK<QM>;
  constexpr int ZM = QM == QM_ASYM4 ? 15 : QM == QM_ASYM2 ? 3 : 0;
  // the zero point of group j, masked in place (an fp16 denormal z 2^-24 in the low half of the pair word for even j,
  // in the high half for odd j): lanes of k blocks 0 and 1 feed it (first element pair of their eight) against the pair
  // -(sum q) of the third operand
  const uint32_t zlane = (lane < 32) ? static_cast<uint32_t>(ZM) : 0u;
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
      else unpack_key<QM>(r.kc[b][j], x);
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

template <int QM, bool K2, class SM>
DEVI void key_phase(const SM& S, const KRegs<QM>& r, int lane, float (&sc)[QBLK<QM>]) {
  bool full[QBLK<QM>];
  whole_head_flags<QM, K2>(r, lane, full);
#pragma unroll
  for (int b = 0; b < QBLK<QM>; ++b) sc[b] = 0.f;
  key_scores<QM, K2>(S, r, lane, full, sc);
}

// p' = p * V scale per group as fp16 and the zero points go to the wave's strips in V^T token order (vs: the lane's
// V scale words of its group x per block).
// Whether the quad holds a V scale above WIDE_VSCALE (wave uniform; slots outside the range count too, which at worst
// sends a quad through the second set of products for nothing): the strips then hold p * scale * 2^-8 and the value
// phase runs a second set of products (value_phase, where the reason is given).
template <int QM>
DEVI bool quad_is_wide(const uint16_t (&vs)[QBLK<QM>]) {
  uint32_t top = 0u;
#pragma unroll
  for (int b = 0; b < QBLK<QM>; ++b) top = max(top, static_cast<uint32_t>(vs[b]) & 0x7FFFu);
  return __any(top > WIDE_VSCALE);
}

template <int QM, class SM>
DEVI void write_strips(SM& S, const uint16_t (&vs)[QBLK<QM>], const float (&pe)[QBLK<QM>], const bool (&valid)[QBLK<QM>],
                       int lane, int wave, bool wide) {
  constexpr int ZM = QM == QM_ASYM4 ? 15 : QM == QM_ASYM2 ? 3 : 0;
  constexpr int QB = QBLK<QM>;
  // Odd tokens are unpacked from the V^T words with the factor 2^SH (UnpackD): their scores were lowered by SH (p
  // carries 2^-SH), their zero point is raised by 2^SH; zero points are fp16 denormals like the codes.
  const int t = lane & 15, x = lane >> 4;
  const int sl = vslot(t & 7);
  uint16_t* pb = reinterpret_cast<uint16_t*>(S.pb(wave)) + (t >> 3) * PB_RSTRIDE * 8 + sl;   // + block * 2 rows; + (group * 4 + head) * 8
  uint16_t* zb = reinterpret_cast<uint16_t*>(S.zb(wave)) + (t >> 3) * ZB_RSTRIDE * 8 + x * 8 + sl;
  const int zsh = (lane & 1) ? UnpackD<QM>::SH : 0;      // odd position inside the page
  const int c0 = ((x) * 4 + x) * 8, c1 = ((x ^ 1) * 4 + x) * 8, c2 = ((x ^ 2) * 4 + x) * 8, c3 = ((x ^ 3) * 4 + x) * 8;
  const uint32_t sfold = wide ? WideFold<QM>::fold : 0x3C00u;      // fp16 2^-8 (2^-4) or 1
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    const uint32_t pp = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(pe[b], pe[b]));
    // the token's four V scale words, sign bits stripped: own group x, then the lanes 16, 32, 48 further (groups
    // x ^ 1, x ^ 2, x ^ 3); unwritten slots may hold any pattern: masked
    const uint32_t v0 = pk_mul(valid[b] ? (vs[b] & 0x7FFFu) : 0u, sfold);
    const uint32_t v1 = lane_from(v0, 4 * (lane ^ 16)), v2 = lane_from(v0, 4 * (lane ^ 32)), v3 = lane_from(v0, 4 * (lane ^ 48));
    const uint32_t xa = pk_mul(pp, (v1 << 16) | v0), xb = pk_mul(pp, (v3 << 16) | v2);
    uint16_t* row = pb + b * 2 * PB_RSTRIDE * 8;
    row[c0] = static_cast<uint16_t>(xa);
    row[c1] = static_cast<uint16_t>(xa >> 16);
    row[c2] = static_cast<uint16_t>(xb);
    row[c3] = static_cast<uint16_t>(xb >> 16);
    if constexpr (QM != QM_SYM4) zb[b * 2 * ZB_RSTRIDE * 8] = static_cast<uint16_t>((vs[b] & ZM) << zsh);
  }
}

// The raw score sums of key_scores keep about 14.6 bits below the largest query x code product of an instruction (the
// code fields are fp16 denormals with up to 10 leading zeros, and the matrix pipe keeps 24 bits below the largest NOMINAL
// exponent; value_phase has the mechanism), and the key scale multiplies what is lost: nothing on ordinary scores, but
// 0.03-0.1 log2 units on a score of a thousand, which moves per cent of the weight where two such tokens compete.  A quad
// that holds a score above FINE_SCORE (softmax_phase: one compare on the maximum it forms anyway) is scored again with
// the code operands times 2^8, which the scale multiplication takes back: the fields sit 8 bits higher in their fp16
// words, the window 8 bits lower.  Block by block, one group at a time, codes and scale words fetched again and the
// query operands read again, all behind a value the compiler cannot see through: nothing of the ordinary pass stays in
// registers for this one, and this pass needs fewer registers than the ordinary one.
// chunk_of(b): the chunk address of block b's page (wave uniform), formed when block b's turn comes: four addresses
// at once are eight scalar registers, and those are as short as the vector ones in these kernels.
constexpr float FINE_SCORE = 64.f;       // log2 units
// NT: q tiles of 4 heads that share the unpacked words (k_decode: 1, raw[block]; k_decode8: 2, raw[tile][block])
template <int QM, bool K2, int P, int NT, class SM, class ChunkOf>
DEVI void rescore_fine(const SM& S, const uint16_t (&vs)[QBLK<QM>], int lane, float (&raw)[NT * QBLK<QM>], ChunkOf&& chunk_of) {
  constexpr int ZM = QM == QM_ASYM4 ? 15 : QM == QM_ASYM2 ? 3 : 0;
  int again = 0;
  asm volatile("" : "+s"(again));
  const int lane2 = lane + again;
  const KOffs<QM, P> o0 = key_offsets<QM, P>(lane2);
  uint32_t ok = o0.k, oks = o0.ks;
  asm volatile("" : "+v"(ok), "+v"(oks));
  const uint32_t zlane = (lane2 < 32) ? static_cast<uint32_t>(ZM) : 0u;
#pragma unroll
  for (int b = 0; b < QBLK<QM>; ++b) {
    const int hp = P == 32 ? (b & 1) : 0;
    uint32_t kc[KRegs<QM>::NW];
    const uint8_t* chunk = chunk_of(b);
    if constexpr (QM == QM_ASYM2) {
      const u32x2 k = gload<u32x2>(chunk + static_cast<size_t>(ok + hp * 16 * 32));
      kc[0] = k.x; kc[1] = k.y;
    } else {
      const u32x4 k = gload<u32x4>(chunk + static_cast<size_t>(ok + hp * 16 * 64));
      kc[0] = k.x; kc[1] = k.y; kc[2] = k.z; kc[3] = k.w;
    }
    const u32x2 ks = gload<u32x2>(chunk + static_cast<size_t>(oks + hp * 16 * 8));
    bool full = false;
    if constexpr (K2) {      // whole_head_flags
      unsigned long long m = __builtin_amdgcn_ballot_w64((vs[b] & 0x8000u) != 0u);
      m |= m >> 32; m |= m >> 16; m &= 0xFFFFull; m |= m << 16; m |= m << 32;
      full = __builtin_amdgcn_inverse_ballot_w64(m);
    }
    float sum[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) sum[t] = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t x[4];
      if constexpr (QM == QM_ASYM2) {
        if (j & 1) UnpackD<QM>::run_hi(kc[j >> 1], x); else UnpackD<QM>::run(kc[j >> 1], x);
      }
      else UnpackD<QM>::run(kc[j], x);
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = pk_mul(x[i], 0x5C005C00u);       // times 2^8: exact, the fields have at most 10 bits
      const half8 kb = __builtin_bit_cast(half8, make_uint4(x[0], x[1], x[2], x[3]));
      const uint32_t kw = (j & 2) ? ks.y : ks.x;
      const uint32_t zz = pk_mul(kw & (zlane << (16 * (j & 1))), 0x5C005C00u);
      const float scale = fabsf(word_value(kw, j)) * 0.00390625f;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        half8 qh, ql, qz;
        if constexpr (NT == 1) {
          qh = __builtin_bit_cast(half8, S.qhi[j][lane2]); ql = __builtin_bit_cast(half8, S.qlo[j][lane2]);
          if constexpr (ZM != 0) qz = __builtin_bit_cast(half8, S.qz[j][lane2]);
        } else {
          qh = __builtin_bit_cast(half8, S.qhi[t][j][lane2]); ql = __builtin_bit_cast(half8, S.qlo[t][j][lane2]);
          if constexpr (ZM != 0) qz = __builtin_bit_cast(half8, S.qz[t][j][lane2]);
        }
        f32x4 a = __builtin_amdgcn_mfma_f32_16x16x32_f16(qh, kb, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
        a = __builtin_amdgcn_mfma_f32_16x16x32_f16(ql, kb, a, 0, 0, 0);
        if constexpr (ZM != 0)
          a = __builtin_amdgcn_mfma_f32_16x16x32_f16(qz, __builtin_bit_cast(half8, make_uint4(zz, 0u, 0u, 0u)), a, 0, 0, 0);
        float pick = a[0];
        if constexpr (K2) {
          const bool h32 = (kw >> (16 * (j & 1) + 15)) & 1u;
          pick = full ? a[2] : (h32 ? a[1] : a[0]);
        }
        sum[t] += pick * scale;
        __builtin_amdgcn_sched_barrier(0);     // in program order: scheduled freely, several steps' operands are formed ahead
      }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) raw[t * QBLK<QM> + b] = sum[t];
  }
}

// online softmax step for the quad, lane = (token, head x): the running maximum is only re-reduced when some lane
// beats it; then p' = p * V scale per group as fp16 and the zero points go to the wave's strips in V^T token order.
// qs20 = qscale * 2^20 (the factor the raw score sums lack); sc0 lowers the scores of odd tokens by SH (below).
// rescore(raw): the quad's raw score sums again through rescore_fine (the caller knows the quad's chunk addresses)
template <int QM, class SM, class Rescore>
DEVI bool softmax_phase(SM& S, WaveState& st, const KRegs<QM>& r, float (&sc)[QBLK<QM>], const bool (&valid)[QBLK<QM>],
                        float qs20, float sc0, int lane, int wave, Rescore&& rescore) {
  constexpr int QB = QBLK<QM>;
  bool beat = false;
  float mx = -INFINITY;
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    sc[b] = valid[b] ? sc[b] * qs20 + sc0 : -INFINITY;
    mx = fmaxf(mx, sc[b]);
  }
  if constexpr (QM == QM_ASYM2) {      // rescore_fine has the reason, and why the 2-bit pages only
    if (__builtin_expect(__any(mx > FINE_SCORE), 0)) {
      float raw[QB];
      rescore(raw);
      mx = -INFINITY;
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        sc[b] = valid[b] ? raw[b] * qs20 + sc0 : -INFINITY;
        mx = fmaxf(mx, sc[b]);
      }
    }
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
  float pe[QB];
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    pe[b] = fexp2(sc[b] - st.m);       // masked tokens: 2^-inf = 0 (the maximum is finite once a quad has been seen)
    st.l += pe[b];
  }
  const bool wide = quad_is_wide<QM>(r.vs);
  write_strips<QM>(S, r.vs, pe, valid, lane, wave, wide);
  return wide;
}

template <int QM, class SM>
DEVI void value_phase(const SM& S, WaveState& st, const VRegs<QM>& r, int lane, int wave, bool wide) {
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
  // The code fields enter the matrix pipe as fp16 denormals, and the pipe aligns the addends of an instruction --
  // products and accumulator -- to the largest NOMINAL exponent (a denormal counts as 2^-14 whatever its leading zeros)
  // and keeps 24 bits from there.  A token whose p * V-scale is hundreds of times its neighbours' lifts that window for
  // its whole instruction: neighbours and accumulator lose up to 2^-13 of ITS p * scale each, which shows where the exact
  // output is near zero (measured with equal weights: 0.05 on sums of 500 beside a group scaled x300, nothing without
  // it).  In a quad that holds such a scale the strips carry p * scale * 2^-8 (write_strips): the products above came to
  // 1/256 of their value with the window 8 bits lower, and here the other 255/256 follow: the code operands times 256
  // (exact) against the strips, minus the plain product once more.  The zero-point sums are vector sums: times 255.
  if (__builtin_expect(wide, 0)) {
    // (strips and entry words go through values the compiler cannot see through: recognised as the operands of the
    // products above, those would all stay in registers until here)
    // (... and the lane's own indices likewise: as loop invariants their derived addresses are computed ahead of the
    // page loop and, used here only, parked in scratch memory -- a kernel that uses scratch starts its workgroups late)
    int again = 0;
    asm volatile("" : "+s"(again));
    const int n2 = (lane + again) & 15, kc2 = (lane + again) >> 4;
    const uint4* rowg2 = reinterpret_cast<const uint4*>(S.pb(wave)) + kc2 * PB_RSTRIDE;
#pragma unroll
    for (int s2 = 0; s2 < QBLK<QM> / 2; ++s2) {
#pragma unroll
      for (int eh = 0; eh < 2; ++eh)
#pragma unroll
        for (int sub = 0; sub < 4; ++sub) {
          const int g = 2 * (sub >> 1) + eh;
          const uint4 bq = (rowg2 + ((n2 >> 2) == g ? n2 : 16))[4 * s2 * PB_RSTRIDE];
          uint32_t w = QM == QM_ASYM2 ? r.vc[2 * s2 + eh][sub >> 1] : r.vc[2 * s2 + eh][sub];
          asm volatile("" : "+v"(w));
          uint32_t x[4];
          if constexpr (QM == QM_ASYM2) {
            if (sub & 1) UnpackD<QM>::run_hi(w, x); else UnpackD<QM>::run(w, x);
          }
          else UnpackD<QM>::run(w, x);
          const uint4 aq = make_uint4(x[0], x[1], x[2], x[3]);
          const uint4 a256 = make_uint4(pk_mul(x[0], WideFold<QM>::up), pk_mul(x[1], WideFold<QM>::up), pk_mul(x[2], WideFold<QM>::up), pk_mul(x[3], WideFold<QM>::up));
          const uint4 nb = make_uint4(bq.x ^ 0x80008000u, bq.y ^ 0x80008000u, bq.z ^ 0x80008000u, bq.w ^ 0x80008000u);
          st.ot[sub & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a256), __builtin_bit_cast(half8, bq), st.ot[sub & 1], 0, 0, 0);
          st.ot[sub & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, aq), __builtin_bit_cast(half8, nb), st.ot[sub & 1], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);      // one step's operands at a time: this path is rare and must not claim registers
        }
    }
    if constexpr (QM != QM_SYM4) {
#pragma unroll
      for (int r8 = 0; r8 < Strip<QM>::ROWS; r8 += 8) {
        const int l2 = lane + again;
        const int rg = r8 + (l2 >> 3), g = (l2 >> 1) & 3, hp = l2 & 1;
        const uint4 zq = (reinterpret_cast<const uint4*>(S.zb(wave)) + rg * ZB_RSTRIDE)[g];
        const uint4* pp = reinterpret_cast<const uint4*>(S.pb(wave)) + rg * PB_RSTRIDE + g * 4 + 2 * hp;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const uint4 pq = pp[e];
          float a = dot2(zq.x, pq.x, 0.f);
          a = dot2(zq.y, pq.y, a); a = dot2(zq.z, pq.z, a); a = dot2(zq.w, pq.w, a);
          st.z[e] += WideFold<QM>::rest * a;
        }
      }
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

// ---------------------------------------------------------------------------------------------------------------
// Tiles of 8 query heads (GQA groups of 5 .. 8 heads at head dim 128; the reference's GT = 8 kernels,
// kernels/csrc/attn_decode_v2g.cuh:5-10): one workgroup serves both 4-head halves of the tile on ONE unpacking of a quad
// -- the pages are read once.  The key phase runs the score products of both halves against the same masked code
// words (two sets of query operands), the softmax keeps two (token, head) states per lane, the strips hold p * V-scale
// for 8 heads per group, and the value phase multiplies the same masked V^T entries with two sets of strip rows into
// two sets of accumulators.  Everything that depends only on the tokens (unpacking, flags, scale words and their
// exchange among a token's four lanes, zero points) is done once.
constexpr int PB8_RSTRIDE = 33;                    // uint4 per row group: 32 (group, head of 8) entries + 1 pad (stays zero)
template <int QM> struct Strip8 {
  static constexpr int ROWS = 2 * QBLK<QM>;
  static constexpr int PB_BYTES = ROWS * PB8_RSTRIDE * 16;     // per wave: [block][c8][group][head of 8][8 fp16]
  static constexpr int ZB_BYTES = ROWS * ZB_RSTRIDE * 16;
  static constexpr int BYTES = PB_BYTES + ZB_BYTES;
};
template <int QM, int NW>
struct Smem8 {
  static constexpr int STRIP_BYTES = Strip8<QM>::BYTES, PB_BYTES = Strip8<QM>::PB_BYTES;
  static_assert(STRIP_BYTES >= 8 * 128 * 4 && STRIP_BYTES % 16 == 0, "a wavefront's strips must hold its partial outputs");
  alignas(16) uint4 qhi[2][4][64];                   // [half of the tile][group][lane of the matrix instruction]: as Smem::qhi
  alignas(16) uint4 qlo[2][4][64];
  alignas(16) uint4 qz[2][4][64];
  alignas(16) uint8_t work[NW * STRIP_BYTES];
  float m[NW][8], l[NW][8];
  alignas(16) float tailw[NW][64];                   // tail_partial: a wavefront's weights of 16 BF16 rows x 4 heads
  int btc[BT_CACHE];
  int next;
  int last;
  DEVI uint8_t* pb(int w) { return work + w * STRIP_BYTES; }
  DEVI const uint8_t* pb(int w) const { return work + w * STRIP_BYTES; }
  DEVI uint8_t* zb(int w) { return work + w * STRIP_BYTES + PB_BYTES; }
  DEVI const uint8_t* zb(int w) const { return work + w * STRIP_BYTES + PB_BYTES; }
  DEVI float* o(int w, int h) { return reinterpret_cast<float*>(work + w * STRIP_BYTES) + h * 128; }   // h: head of 8
};
struct WaveState8 {          // WaveState for the two halves of the tile
  float m[2], l[2];
  f32x4 ot[2][2];
  float z[2][2];
};

// q_prologue for a tile of 8 heads: head hh (0..7) is prepared by wavefront hh (workgroups of fewer wavefronts take
// several heads in turn) into the operand tables of half hh >> 2, rows of head hh & 3.
template <int QM, bool K2, int NW, class SM>
DEVI void q_prologue8(SM& S, const DecodeParams& p, int b, int kvh, int tile) {
  const int wv = threadIdx.x >> 6, half = (threadIdx.x >> 5) & 1, l32 = threadIdx.x & 31;
  for (int hh = wv; hh < 8; hh += NW) {
  const int th = hh >> 2, w = hh & 3;
  const int hq = tile * 8 + hh;                      // head inside the GQA group
  float x[4] = {0.f, 0.f, 0.f, 0.f};
  if (hq < p.gqa) {
    const uint16_t* qr = static_cast<const uint16_t*>(p.q) + static_cast<long long>(b) * p.q_bs +
                         (static_cast<long long>(kvh) * p.gqa + hq) * 128 + 4 * l32;
    const uint2 raw = *reinterpret_cast<const uint2*>(qr);
    x[0] = bf16_lo(raw.x); x[1] = bf16_hi(raw.x); x[2] = bf16_lo(raw.y); x[3] = bf16_hi(raw.y);
  }
  const int g = l32 >> 3, isB = (l32 >> 2) & 1, tg = l32 & 3;
  float y[4] = {x[0], x[1], x[2], x[3]};
  if (half == 0) fwht<32>(y, l32); else fwht<128>(y, l32);
  const float beta = (isB ? static_cast<float>(1 << UnpackD<QM>::SH) : 1.f) * ((QM == QM_ASYM2 && (g & 1)) ? 16.f : 1.f);
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
      const uint32_t rot = (p.kmask != nullptr && p.kmask[kvh * 4 + g] != 0) ? 0xFFFFFFFFu : 0u;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = __uint_as_float((__float_as_uint(y[i]) & rot) | (__float_as_uint(x[i]) & ~rot));
    }
    uint32_t hb[4], lb[4];
    float qs = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = live ? v[i] * (QPRE / key_field_factor<QM>(isB, g, i)) : 0.f;
      const _Float16 hi = static_cast<_Float16>(a);
      const _Float16 lo = static_cast<_Float16>(a - static_cast<float>(hi));
      hb[i] = __builtin_bit_cast(uint16_t, hi);
      lb[i] = __builtin_bit_cast(uint16_t, lo);
      qs += (static_cast<float>(hi) + static_cast<float>(lo)) * beta;
    }
    const int m = 4 * w + var, ln = m + 16 * tg;
    uint32_t* dh = reinterpret_cast<uint32_t*>(&S.qhi[th][g][ln]);
    uint32_t* dl = reinterpret_cast<uint32_t*>(&S.qlo[th][g][ln]);
    dh[isB] = hb[0] | (hb[2] << 16); dh[2 + isB] = hb[1] | (hb[3] << 16);
    dl[isB] = lb[0] | (lb[2] << 16); dl[2 + isB] = lb[1] | (lb[3] << 16);
    if constexpr (QM != QM_SYM4) {
      qs += hx(qs, 1); qs += hx(qs, 2); qs += hx(qs, 4);
      if ((l32 & 7) == 0) {
        const _Float16 zh = static_cast<_Float16>(-qs);
        const _Float16 zl = static_cast<_Float16>(-qs - static_cast<float>(zh));
        const int sh = 16 * (g & 1);
        S.qz[th][g][m] = make_uint4(static_cast<uint32_t>(__builtin_bit_cast(uint16_t, zh)) << sh, 0u, 0u, 0u);
        S.qz[th][g][m + 16] = make_uint4(static_cast<uint32_t>(__builtin_bit_cast(uint16_t, zl)) << sh, 0u, 0u, 0u);
        S.qz[th][g][m + 32] = make_uint4(0u, 0u, 0u, 0u);
        S.qz[th][g][m + 48] = make_uint4(0u, 0u, 0u, 0u);
      }
    }
  }
  }
}

// scores of the lane's token for heads x and 4 + x (x = lane >> 4), four blocks: the group's masked words are made once
// and multiplied with the query operands of both halves of the tile
template <int QM, bool K2, class SM>
DEVI void key_phase8(const SM& S, const KRegs<QM>& r, int lane, float (&sc)[2][QBLK<QM>]) {
  constexpr int QB = QBLK<QM>;
  static_assert(QB == 4, "four blocks per wave iteration");
  constexpr int ZM = QM == QM_ASYM4 ? 15 : QM == QM_ASYM2 ? 3 : 0;
  bool full[QB];
  whole_head_flags<QM, K2>(r, lane, full);
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int b = 0; b < QB; ++b) sc[t][b] = 0.f;
  const uint32_t zlane = (lane < 32) ? static_cast<uint32_t>(ZM) : 0u;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    half8 kb[QB], kz[QB];
    float sv[QB];
    bool h32[QB];
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      uint32_t x[4];
      if constexpr (QM == QM_ASYM2) {
        if (j & 1) UnpackD<QM>::run_hi(r.kc[b][j >> 1], x); else UnpackD<QM>::run(r.kc[b][j >> 1], x);
      }
      else unpack_key<QM>(r.kc[b][j], x);
      kb[b] = __builtin_bit_cast(half8, make_uint4(x[0], x[1], x[2], x[3]));
      const uint32_t kw = (j & 2) ? r.ks[b].y : r.ks[b].x;
      kz[b] = __builtin_bit_cast(half8, make_uint4(kw & (zlane << (16 * (j & 1))), 0u, 0u, 0u));
      sv[b] = fabsf(word_value(kw, j));
      h32[b] = (kw >> (16 * (j & 1) + 15)) & 1u;
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const half8 qh = __builtin_bit_cast(half8, S.qhi[t][j][lane]), ql = __builtin_bit_cast(half8, S.qlo[t][j][lane]);
      half8 qz;
      if constexpr (ZM != 0) qz = __builtin_bit_cast(half8, S.qz[t][j][lane]);
      f32x4 acc[QB];
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        f32x4 a = __builtin_amdgcn_mfma_f32_16x16x32_f16(qh, kb[b], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
        a = __builtin_amdgcn_mfma_f32_16x16x32_f16(ql, kb[b], a, 0, 0, 0);
        if constexpr (ZM != 0) a = __builtin_amdgcn_mfma_f32_16x16x32_f16(qz, kz[b], a, 0, 0, 0);
        acc[b] = a;
      }
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        float pick = acc[b][0];
        if constexpr (K2) pick = full[b] ? acc[b][2] : (h32[b] ? acc[b][1] : acc[b][0]);
        sc[t][b] += pick * sv[b];
      }
    }
  }
}

// softmax step of both halves; the strips take p * V-scale of heads x and 4 + x for all four groups
template <int QM, class SM, class Rescore>
DEVI bool softmax_phase8(SM& S, WaveState8& st, const KRegs<QM>& r, float (&sc)[2][QBLK<QM>], const bool (&valid)[QBLK<QM>],
                         float qs20, float sc0, int lane, int wave, Rescore&& rescore) {
  constexpr int QB = QBLK<QM>;
  constexpr int ZM = QM == QM_ASYM4 ? 15 : QM == QM_ASYM2 ? 3 : 0;
  float mx[2];
  bool beat = false;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    mx[t] = -INFINITY;
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      sc[t][b] = valid[b] ? sc[t][b] * qs20 + sc0 : -INFINITY;
      mx[t] = fmaxf(mx[t], sc[t][b]);
    }
  }
  if constexpr (QM == QM_ASYM2) {      // as in softmax_phase
    if (__builtin_expect(__any(fmaxf(mx[0], mx[1]) > FINE_SCORE), 0)) {
      float raw[2 * QB];
      rescore(raw);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        mx[t] = -INFINITY;
#pragma unroll
        for (int b = 0; b < QB; ++b) {
          sc[t][b] = valid[b] ? raw[t * QB + b] * qs20 + sc0 : -INFINITY;
          mx[t] = fmaxf(mx[t], sc[t][b]);
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < 2; ++t) beat = beat || mx[t] > st.m[t];
  float al[2] = {1.f, 1.f}, az0[2] = {1.f, 1.f}, az1[2] = {1.f, 1.f}, am[2] = {1.f, 1.f};
  if (__builtin_expect(__any(beat), 0)) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const float mn = fmaxf(st.m[t], row_max16(mx[t]));
      am[t] = mn == -INFINITY ? 1.f : fexp2(st.m[t] - mn);
      st.m[t] = mn;
      const float a0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am[t]), 0));
      const float a1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am[t]), 16));
      const float a2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am[t]), 32));
      const float a3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am[t]), 48));
      al[t] = (lane & 2) ? ((lane & 1) ? a3 : a2) : ((lane & 1) ? a1 : a0);
      az0[t] = (lane & 1) ? a2 : a0;
      az1[t] = (lane & 1) ? a3 : a1;
    }
  }
  float pe[2][QB];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    st.l[t] *= am[t];
    st.ot[t][0] *= al[t]; st.ot[t][1] *= al[t];
    st.z[t][0] *= az0[t]; st.z[t][1] *= az1[t];
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      pe[t][b] = fexp2(sc[t][b] - st.m[t]);
      st.l[t] += pe[t][b];
    }
  }
  // strips: row entry (group g, head of 8) of the token's run; the token's four V scale words are exchanged once
  const int tk = lane & 15, x = lane >> 4;
  const int sl = vslot(tk & 7);
  uint16_t* pb = reinterpret_cast<uint16_t*>(S.pb(wave)) + (tk >> 3) * PB8_RSTRIDE * 8 + sl;
  uint16_t* zb = reinterpret_cast<uint16_t*>(S.zb(wave)) + (tk >> 3) * ZB_RSTRIDE * 8 + x * 8 + sl;
  const int zsh = (lane & 1) ? UnpackD<QM>::SH : 0;
  const int c0 = ((x) * 8 + x) * 8, c1 = ((x ^ 1) * 8 + x) * 8, c2 = ((x ^ 2) * 8 + x) * 8, c3 = ((x ^ 3) * 8 + x) * 8;
  const bool wide = quad_is_wide<QM>(r.vs);      // its strips then keep p * scale * 2^-8 (value_phase has the reason)
  const uint32_t sfold = wide ? WideFold<QM>::fold : 0x3C00u;      // fp16 2^-8 (2^-4) or 1
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    const uint32_t v0 = pk_mul(valid[b] ? (r.vs[b] & 0x7FFFu) : 0u, sfold);
    const uint32_t v1 = lane_from(v0, 4 * (lane ^ 16)), v2 = lane_from(v0, 4 * (lane ^ 32)), v3 = lane_from(v0, 4 * (lane ^ 48));
    const uint32_t va = (v1 << 16) | v0, vb = (v3 << 16) | v2;
    uint16_t* row = pb + b * 2 * PB8_RSTRIDE * 8;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const uint32_t pp = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(pe[t][b], pe[t][b]));
      const uint32_t xa = pk_mul(pp, va), xb = pk_mul(pp, vb);
      row[c0 + 32 * t] = static_cast<uint16_t>(xa);
      row[c1 + 32 * t] = static_cast<uint16_t>(xa >> 16);
      row[c2 + 32 * t] = static_cast<uint16_t>(xb);
      row[c3 + 32 * t] = static_cast<uint16_t>(xb >> 16);
    }
    if constexpr (QM != QM_SYM4) zb[b * 2 * ZB_RSTRIDE * 8] = static_cast<uint16_t>((r.vs[b] & ZM) << zsh);
  }
  return wide;
}

template <int QM, class SM>
DEVI void value_phase8(const SM& S, WaveState8& st, const VRegs<QM>& r, int lane, int wave, bool wide) {
  // column n = lane & 15 = (group n >> 2, head n & 3 of the half); a masked entry word is multiplied with the strip
  // rows of both halves (entries 8 g + head and 8 g + 4 + head; lanes of foreign groups read the zero pad entry)
  const int n = lane & 15, kc = lane >> 4;
  const uint4* rowg = reinterpret_cast<const uint4*>(S.pb(wave)) + kc * PB8_RSTRIDE;
#pragma unroll
  for (int s2 = 0; s2 < QBLK<QM> / 2; ++s2) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {            // strip group g = entries of half eh = g & 1, word pair g >> 1
      const int eh = g & 1;
      const uint4* src = rowg + 4 * s2 * PB8_RSTRIDE;
      const half8 b0 = __builtin_bit_cast(half8, src[(n >> 2) == g ? 8 * g + (n & 3) : 32]);
      const half8 b1 = __builtin_bit_cast(half8, src[(n >> 2) == g ? 8 * g + 4 + (n & 3) : 32]);
#pragma unroll
      for (int y = 0; y < 2; ++y) {
        const int sub = 2 * (g >> 1) + y;
        uint32_t x[4];
        if constexpr (QM == QM_ASYM2) {
          if (sub & 1) UnpackD<QM>::run_hi(r.vc[2 * s2 + eh][sub >> 1], x); else UnpackD<QM>::run(r.vc[2 * s2 + eh][sub >> 1], x);
        }
        else UnpackD<QM>::run(r.vc[2 * s2 + eh][sub], x);
        const half8 aq = __builtin_bit_cast(half8, make_uint4(x[0], x[1], x[2], x[3]));
        st.ot[0][y] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aq, b0, st.ot[0][y], 0, 0, 0);
        st.ot[1][y] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aq, b1, st.ot[1][y], 0, 0, 0);
      }
    }
  }
  if constexpr (QM != QM_SYM4) {   // sum p' zero point: lane = (row group, group, head pair), both halves
    const int rg = lane >> 3, g = (lane >> 1) & 3, hp = lane & 1;
    const uint4 zq = (reinterpret_cast<const uint4*>(S.zb(wave)) + rg * ZB_RSTRIDE)[g];
    const uint4* pp = reinterpret_cast<const uint4*>(S.pb(wave)) + rg * PB8_RSTRIDE + g * 8 + 2 * hp;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const uint4 pq = pp[4 * t + e];
        float a = st.z[t][e];
        a = dot2(zq.x, pq.x, a); a = dot2(zq.y, pq.y, a); a = dot2(zq.z, pq.z, a); a = dot2(zq.w, pq.w, a);
        st.z[t][e] = a;
      }
  }
  // quads with a wide V scale: the other 255/256 of the value products and of the zero-point sums (value_phase)
  if (__builtin_expect(wide, 0)) {
    int again = 0;
    asm volatile("" : "+s"(again));
    const int n2 = (lane + again) & 15, kc2 = (lane + again) >> 4;
    const uint4* rowg2 = reinterpret_cast<const uint4*>(S.pb(wave)) + kc2 * PB8_RSTRIDE;
#pragma unroll
    for (int s2 = 0; s2 < QBLK<QM> / 2; ++s2) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int eh = g & 1;
        const uint4* src = rowg2 + 4 * s2 * PB8_RSTRIDE;
#pragma unroll
        for (int y = 0; y < 2; ++y) {
          const int sub = 2 * (g >> 1) + y;
          uint32_t w = QM == QM_ASYM2 ? r.vc[2 * s2 + eh][sub >> 1] : r.vc[2 * s2 + eh][sub];
          asm volatile("" : "+v"(w));
          uint32_t x[4];
          if constexpr (QM == QM_ASYM2) {
            if (sub & 1) UnpackD<QM>::run_hi(w, x); else UnpackD<QM>::run(w, x);
          }
          else UnpackD<QM>::run(w, x);
          const half8 aq = __builtin_bit_cast(half8, make_uint4(x[0], x[1], x[2], x[3]));
          const half8 a256 = __builtin_bit_cast(half8, make_uint4(pk_mul(x[0], WideFold<QM>::up), pk_mul(x[1], WideFold<QM>::up), pk_mul(x[2], WideFold<QM>::up), pk_mul(x[3], WideFold<QM>::up)));
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            uint4 bq = src[(n2 >> 2) == g ? 8 * g + 4 * t + (n2 & 3) : 32];
            st.ot[t][y] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a256, __builtin_bit_cast(half8, bq), st.ot[t][y], 0, 0, 0);
            bq = make_uint4(bq.x ^ 0x80008000u, bq.y ^ 0x80008000u, bq.z ^ 0x80008000u, bq.w ^ 0x80008000u);
            st.ot[t][y] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aq, __builtin_bit_cast(half8, bq), st.ot[t][y], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);      // one step's operands at a time: this path is rare and must not claim registers
          }
        }
      }
    }
    if constexpr (QM != QM_SYM4) {
      const int l2 = lane + again;
      const int rg = l2 >> 3, g = (l2 >> 1) & 3, hp = l2 & 1;
      const uint4 zq = (reinterpret_cast<const uint4*>(S.zb(wave)) + rg * ZB_RSTRIDE)[g];
      const uint4* pp = reinterpret_cast<const uint4*>(S.pb(wave)) + rg * PB8_RSTRIDE + g * 8 + 2 * hp;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const uint4 pq = pp[4 * t + e];
          float a = dot2(zq.x, pq.x, 0.f);
          a = dot2(zq.y, pq.y, a); a = dot2(zq.z, pq.z, a); a = dot2(zq.w, pq.w, a);
          st.z[t][e] += WideFold<QM>::rest * a;
        }
    }
  }
}

// BF16 sink / window rows of one sequence: partial softmax over tail_len rows, lanes own 2 dims of the outputs.
// A wavefront takes 16 rows per step.  Scores on the matrix pipe: A = the tile's four query rows (rows 4..15 of the
// operand are zero), B = the 16 key rows as they lie in memory (a lane's 16 bytes are 8 channels of row lane & 15),
// four products of 32 channels -- lanes 0..15 then hold the four heads' scores of row `lane`, with no cross-lane sum.
// One maximum per head and step (a row reduction), one exponential per (row, head), column sums kept per lane until
// the end.  The weights pass through 256 bytes of LDS (`pw`, this wavefront's own) and come back as broadcast reads,
// one per row, for the value products on the vector pipe: 8 multiply-adds and 2 conversions per row.
// q and the rows are read 16 bytes at a time: the caller has checked their alignment (fr_v2_attn).
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
template <int NW>
DEVI void tail_partial(const DecodeParams& p, int b, int kvh, int tile, float* pw, float (&m)[4], float (&l)[4], float (&o)[4][2]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kb = lane >> 4;
  const int n = p.tail_len[b];
  const int row = p.tail_idx != nullptr ? p.tail_idx[b] : b;
  const uint16_t* base = static_cast<const uint16_t*>(p.tail) + static_cast<long long>(row) * p.tail_bs;
  uint4 qa[4];
  {
    const int hq = tile * 4 + col;
    const bool live = col < 4 && hq < p.gqa;
    const uint16_t* qr = static_cast<const uint16_t*>(p.q) + static_cast<long long>(b) * p.q_bs +
                         (static_cast<long long>(kvh) * p.gqa + (live ? hq : 0)) * 128 + 8 * kb;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint4 v = *reinterpret_cast<const uint4*>(qr + 32 * s);
      qa[s] = live ? v : make_uint4(0u, 0u, 0u, 0u);
    }
  }
  float lp[4];
#pragma unroll
  for (int h = 0; h < 4; ++h) { m[h] = -INFINITY; lp[h] = 0.f; o[h][0] = o[h][1] = 0.f; }
  for (int t0 = wave * 16; t0 < n; t0 += NW * 16) {
    const uint16_t* kr = base + static_cast<long long>(min(t0 + col, n - 1)) * p.tail_ts + kvh * 128 + 8 * kb;
    uint4 kk[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) kk[s] = *reinterpret_cast<const uint4*>(kr + 32 * s);
    uint32_t vr[16];
#pragma unroll
    for (int r = 0; r < 16; ++r)
      vr[r] = *reinterpret_cast<const uint32_t*>(base + static_cast<long long>(min(t0 + r, n - 1)) * p.tail_ts + (p.Hkv + kvh) * 128 + 2 * lane);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s)
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, qa[s]), __builtin_bit_cast(bf16x8, kk[s]), acc, 0, 0, 0);
    const bool in = t0 + col < n;
    float pe[4];
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const float sc = in ? acc[h] * p.qscale : -INFINITY;
      // (lane 0 is in the row of the scores; row t0 exists, so the maximum is a number)
      const float mx = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, row_max16(sc))));
      const float mn = fmaxf(m[h], mx);
      const float alpha = fexp2(m[h] - mn);
      pe[h] = fexp2(sc - mn);
      m[h] = mn;
      lp[h] = lp[h] * alpha + pe[h];
      o[h][0] *= alpha; o[h][1] *= alpha;
    }
    if (lane < 16) *reinterpret_cast<float4*>(pw + 4 * lane) = make_float4(pe[0], pe[1], pe[2], pe[3]);
    wave_lds_sync();
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float4 w = *reinterpret_cast<const float4*>(pw + 4 * r);
      const float v0 = bf16_lo(vr[r]), v1 = bf16_hi(vr[r]);
      o[0][0] += w.x * v0; o[0][1] += w.x * v1;
      o[1][0] += w.y * v0; o[1][1] += w.y * v1;
      o[2][0] += w.z * v0; o[2][1] += w.z * v1;
      o[3][0] += w.w * v0; o[3][1] += w.w * v1;
    }
    wave_lds_sync();      // the weights have been read before the next step replaces them
  }
#pragma unroll
  for (int h = 0; h < 4; ++h)
    l[h] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, row_sum16(lp[h]))));
}

// H32 (Sylvester order, factor 1/sqrt(32)) over the 32 channels of a group held two per lane by a row of 16 lanes
// (channel 2 (lane & 15) + e): what brings a share of the BF16 rows into the basis the static formats store V in
DEVI void h32_row16(float& a, float& b, int lane) {
  float y0 = a + b, y1 = a - b;
  { const float p0 = dpp_xor1(y0), p1 = dpp_xor1(y1); y0 = (lane & 1) ? p0 - y0 : y0 + p0; y1 = (lane & 1) ? p1 - y1 : y1 + p1; }
  { const float p0 = dpp_xor2(y0), p1 = dpp_xor2(y1); y0 = (lane & 2) ? p0 - y0 : y0 + p0; y1 = (lane & 2) ? p1 - y1 : y1 + p1; }
  { const float p0 = swz_xor<4>(y0), p1 = swz_xor<4>(y1); y0 = (lane & 4) ? p0 - y0 : y0 + p0; y1 = (lane & 4) ? p1 - y1 : y1 + p1; }
  { const float p0 = swz_xor<8>(y0), p1 = swz_xor<8>(y1); y0 = (lane & 8) ? p0 - y0 : y0 + p0; y1 = (lane & 8) ? p1 - y1 : y1 + p1; }
  a = y0 * kC32; b = y1 * kC32;
}
// ... for the lane's four heads where the group's mask asks for it (every lane runs the exchanges)
DEVI void tail_to_stored_basis(float (&o)[4][2], bool rotated, int lane) {
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    float a = o[h][0], b = o[h][1];
    h32_row16(a, b, lane);
    o[h][0] = rotated ? a : o[h][0];
    o[h][1] = rotated ? b : o[h][1];
  }
}

}  // namespace dec
}  // namespace fr
