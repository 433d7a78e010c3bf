// Building blocks of the multi-query prefill kernels (mq_prefill.hip: head dim 128; mq_wide.hip: head dim 256 as two
// 128-d halves): the plan records a workgroup reads, the fp16 tile converters (page words -> K tile, V^T tile in LDS),
// and the 64-key block step on the matrix cores (scores, online softmax, values).  Everything is inlined device code.
#pragma once
#include "fr_common.hpp"
#include "fr_unpack.hpp"

namespace frmq {
using namespace fr;


typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int D = 128, PAGE = 16, BN = 64, TILE_INTS = 9, ITEM_INTS = 4;
constexpr int KROW = 272;                    // bytes per K tile row: 256 + 16 pad
constexpr int VROW = 144;                    // bytes per V^T tile row: 128 + 16 pad
constexpr int KT_BYTES = BN * KROW, VT_BYTES = D * VROW;
constexpr int QROW = 264;                    // bytes per staged q row (natural order)
constexpr int PG_CACHE = 1024;               // page ids kept in LDS (256 blocks of 64 keys)

struct Smem {
  alignas(16) uint8_t kt[KT_BYTES];
  alignas(16) uint8_t vt[VT_BYTES];
  alignas(16) uint32_t vsc[4][8][4];         // per (group, run): scale pairs (t0,t4) (t1,t5) (t2,t6) (t3,t7)
  alignas(16) uint32_t vnz[4][8][4];         // per (group, run): -(1024 + zero point) pairs
  int pages[PG_CACHE];                       // page ids of the blocks [cb, cb + PG_CACHE / 4) of the item
};
static_assert(128 * QROW <= KT_BYTES + VT_BYTES, "q staging aliases the tiles");

struct Params {
  const uint16_t* q;
  const uint8_t* pool;
  long long page_stride;
  const int* bt;
  long long bt_stride;
  const int* tiles;
  const int* items;
  int Hkv, G, shift, kmin;
  float* opart;
  float* ml;
};

// What one workgroup (item, KV head) has to do, read from its item record (tile, first block, end block, 0) and the tile
// record that names (block-table row, first compact query row, first output row, tokens, position of the first token,
// page keys of the request, first item, items, reach).  `reach`: a key index every row may see on top of its causal
// range (a large negative number when there is none).
struct Work {
  const int* block_table;
  int compact_row, tokens, first_pos, reach;
  int key_end;              // keys at or past it are invisible to the whole tile or belong to a later item
  int block0, block1;       // 64-key blocks [block0, block1) to read (empty when the item starts past key_end)
  int rows_used;            // query rows of the tile that hold a token's head: whole tokens only
  int shift;

  DEVI Work(const Params& p, int item, int rows) {
    const int* irec = p.items + ITEM_INTS * item;
    const int* trec = p.tiles + TILE_INTS * irec[0];
    block_table = p.bt + static_cast<long long>(trec[0]) * p.bt_stride;
    compact_row = trec[1]; tokens = trec[3]; first_pos = trec[4]; reach = trec[8];
    shift = p.shift;
    const int causal_end = max(first_pos + tokens - shift, reach + 1);      // what the tile's last token sees
    key_end = min(min(trec[5], irec[2] * BN), causal_end);
    block0 = irec[1];
    block1 = key_end > block0 * BN ? (key_end + BN - 1) / BN : block0;
    rows_used = min(rows / p.G, tokens) * p.G;
  }
  DEVI bool has_row(int row) const { return row < rows_used; }
  DEVI int last_key(int token) const { return min(key_end - 1, max(first_pos + token - shift, reach)); }
};


template <typename T> DEVI T gload(const void* p) {
  return *reinterpret_cast<const __attribute__((address_space(1))) T*>(reinterpret_cast<uintptr_t>(p));
}
DEVI float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }
DEVI half8 as_h8(u32x4 v) { return __builtin_bit_cast(half8, v); }
DEVI uint32_t pack_h2(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}
DEVI uint32_t pack_h2_rn(float a, float b) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  h2 v = {static_cast<_Float16>(a), static_cast<_Float16>(b)};
  return __builtin_bit_cast(uint32_t, v);
}

// token (0..31 inside a 32-key tile) -> K tile row, and accumulator index -> token
DEVI int krow_of_token(int tk) {
  const int run = tk >> 3, t8 = tk & 7, e = 2 * (t8 & 3) + (t8 >> 2);
  return 16 * (run >> 1) + 8 * (e >> 2) + 4 * (run & 1) + (e & 3);
}
DEVI constexpr int token_of_acc(int i, int hh) {   // accumulator i of the lane half hh
  const int s = i >> 3, e = i & 7;
  const int t8 = (e >> 1) + 4 * (e & 1);           // run order t0 t4 t1 t5 t2 t6 t3 t7
  return 8 * (2 * s + hh) + t8;
}

template <int QM> struct Fmt {
  static constexpr int CB = QM == QM_ASYM2 ? 32 : 64;
  static constexpr int V_OFF = CB * PAGE, KS_OFF = 2 * CB * PAGE, VS_OFF = KS_OFF + 8 * PAGE, CHUNK = VS_OFF + 8 * PAGE;
  static constexpr uint32_t ZM = QM == QM_ASYM2 ? 3u : 15u;
};

// ------------------------------------------------------------------------------------------------ key-only pages
// Inverse transform of one token's keys while they are fp16 pairs in registers.  A thread holds, per 32-group, the 8
// elements d = 4 tg + i (A_i) and 16 + 4 tg + i (B_i) as (A0 A2) (B0 B2) (A1 A3) (B1 B3); the four threads of a quad
// (tg = lane & 3) hold the group.  Index bits of d: bit 0 = registers 0,1 <-> 2,3; bit 1 = low <-> high half; bits 2,3 =
// the quad lanes (DPP); bit 4 = registers 0 <-> 1, 2 <-> 3; the two group bits of the whole-head transform = registers of
// different groups.  The five stages inside a group run on the integers code - zero point (exact in fp16), then the
// group scale times the transform's whole normalisation is applied -- as an fp16 value + remainder pair (scale x
// 2^-2.5 is not an fp16 number; a single rounded factor would be off by up to 2^-12 for all 32 channels of the group
// alike, which moves the group's share of every score the same way), two packed operations per register -- then the
// whole-head stages.
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
DEVI h2_t h2(uint32_t u) { return __builtin_bit_cast(h2_t, u); }
DEVI uint32_t u2(h2_t v) { return __builtin_bit_cast(uint32_t, v); }
DEVI void bfly(uint32_t& a, uint32_t& b) {
  const h2_t x = h2(a), y = h2(b);
  a = u2(x + y); b = u2(x - y);
}
DEVI uint32_t bfly_halves(uint32_t a) {                       // (lo, hi) -> (lo + hi, lo - hi)
  const uint32_t sw = (a >> 16) | (a << 16);
  const h2_t sg = h2(0xBC003C00u);                            // (1, -1)
  return u2(__builtin_elementwise_fma(h2(a), sg, h2(sw)));
}
template <int CTRL> DEVI uint32_t bfly_lanes(uint32_t a, uint32_t sgn) {   // sgn = (1,1) on the lower lane, (-1,-1) on the upper
  const uint32_t o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(a), CTRL, 0xF, 0xF, true));
  return u2(__builtin_elementwise_fma(h2(a), h2(sgn), h2(o)));
}
DEVI void h32_group(uint32_t (&x)[4], uint32_t sgn1, uint32_t sgn2) {
  bfly(x[0], x[2]); bfly(x[1], x[3]);                          // d bit 0
#pragma unroll
  for (int r = 0; r < 4; ++r) x[r] = bfly_halves(x[r]);        // d bit 1
#pragma unroll
  for (int r = 0; r < 4; ++r) x[r] = bfly_lanes<0xB1>(x[r], sgn1);   // d bit 2: quad lanes xor 1
#pragma unroll
  for (int r = 0; r < 4; ++r) x[r] = bfly_lanes<0x4E>(x[r], sgn2);   // d bit 3: quad lanes xor 2
  bfly(x[0], x[1]); bfly(x[2], x[3]);                          // d bit 4
}

// ------------------------------------------------------------------------------------------------ tile converters
// Page ids of the blocks [cb, cb + PG_CACHE / 4) of an item into the LDS window.  Only the item's own pages are read
// (entries past them are 0) and every load is unconditional, its index clamped to the item's last page: a thread's
// loads are in flight together, one memory latency per fill (as loads under a condition each was waited for in turn).
template <int NT>
DEVI void fill_page_window(int* pages, const int* bt, int cb, int kb1, int kend, int tid) {
  constexpr int NF = PG_CACHE / NT;
  const int last = min(4 * kb1, (kend + PAGE - 1) / PAGE) - 1;     // the item's last page
  int v[NF];
#pragma unroll
  for (int k = 0; k < NF; ++k) v[k] = 0;
  if (last >= 4 * cb) {                                              // (uniform over the workgroup)
#pragma unroll
    for (int k = 0; k < NF; ++k) v[k] = bt[min(4 * cb + tid + k * NT, last)];
  }
#pragma unroll
  for (int k = 0; k < NF; ++k) pages[tid + k * NT] = 4 * cb + tid + k * NT <= last ? v[k] : 0;
}

// The thread index as a value the compiler must take as new at every use site: what a converter derives from it (tile
// addresses, lane offsets) is recomputed per block with a few integer operations instead of being kept in registers
// across the whole key loop, where the accumulators leave no room for it.
DEVI int tid_now() {
  int t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

// The raw page words of a 64-key block are fetched into registers one block ahead (load_raw) and turned into the
// fp16 tiles after the previous block's matrix work (convert_k, v_tables, convert_v).
template <int NT> struct Raw {
  static constexpr int NI = 256 / NT;
  u32x4 kc[NI];      // K code words of (token, tg): INT4 four groups, INT2 two words in .x .y
  u32x2 ks[NI];      // the token's four K scale words
  uint32_t vf[NI];   // the token's group-0 V scale word (whole-head flag of key-only pages)
  u32x4 vc[NI];      // V^T entry (e, c8) of a page
  u32x4 vs;          // threads < 32: V scale words of (group, run)
};

// `h` is the index of the chunk inside a page: the KV head at head dim 128, 2 head + half at head dim 256
// FRESH: the lane offsets are recomputed per block from the thread index (a few integer operations) instead of being
// kept as 64-bit addresses across the key loop -- for the kernels whose registers are short (there the kept addresses
// were spilled, and a spilled register's reload waits for every fetch in flight); where there is room, keeping them is
// the faster form.
template <int QM, bool K2, int NT, bool FRESH = false>
DEVI void load_raw_k(Raw<NT>& R, const Params& p, const int* pg, int h, int kb, int kend) {   // pg[0] = first page of block kb
  using F = Fmt<QM>;
  const int tnow = FRESH ? tid_now() : static_cast<int>(threadIdx.x);
#pragma unroll
  for (int it = 0; it < Raw<NT>::NI; ++it) {
    const int idx = tnow + it * NT;
    {
      const int tk = idx >> 2, tg = idx & 3, j = kb * BN + tk;
      if (j < kend) {
        const uint8_t* ch = p.pool + static_cast<long long>(pg[tk >> 4]) * p.page_stride + static_cast<long long>(h) * F::CHUNK;
        const int pos = j & 15;
        if constexpr (QM == QM_ASYM2) {
          const u32x2 c = gload<u32x2>(ch + 32 * (pos ^ ((pos >> 1) & 2)) + 8 * tg);
          R.kc[it] = u32x4{c.x, c.y, 0u, 0u};
        } else {
          R.kc[it] = gload<u32x4>(ch + 64 * pos + 16 * tg);
        }
        R.ks[it] = gload<u32x2>(ch + F::KS_OFF + 8 * pos);
        if constexpr (K2) R.vf[it] = gload<uint16_t>(ch + F::VS_OFF + (8 * (pos >> 3) + vs_slot8(pos)) * 2);
      }
    }
  }
}
template <int QM, int NT, bool FRESH = false>
DEVI void load_raw_v(Raw<NT>& R, const Params& p, const int* pg, int h, int kb, int kend) {
  using F = Fmt<QM>;
  const int tnow = FRESH ? tid_now() : static_cast<int>(threadIdx.x);
#pragma unroll
  for (int it = 0; it < Raw<NT>::NI; ++it) {
    const int idx = tnow + it * NT;
    {
      const int pgi = idx >> 6, e = (idx & 63) >> 1, c8 = idx & 1, j0 = kb * BN + PAGE * pgi;
      if (j0 < kend) {
        const uint8_t* ch = p.pool + static_cast<long long>(pg[pgi]) * p.page_stride + static_cast<long long>(h) * F::CHUNK;
        if constexpr (QM == QM_ASYM2) {
          const u32x2 c = gload<u32x2>(ch + F::V_OFF + (e * 2 + c8) * 8);
          R.vc[it] = u32x4{c.x, c.y, 0u, 0u};
        } else {
          R.vc[it] = gload<u32x4>(ch + F::V_OFF + (e * 2 + c8) * 16);
        }
      }
    }
  }
  if (tnow < 32) {
    const int g = tnow >> 3, run = tnow & 7, j0 = kb * BN + 8 * run;
    if (j0 < kend) {
      const uint8_t* ch = p.pool + static_cast<long long>(pg[run >> 1]) * p.page_stride + static_cast<long long>(h) * F::CHUNK;
      R.vs = gload<u32x4>(ch + F::VS_OFF + (g * PAGE + 8 * (run & 1)) * 2);   // t0 t2 | t4 t6 | t1 t3 | t5 t7
    }
  }
}
template <int QM, bool K2, int NT, bool FRESH = false>
DEVI void load_raw(Raw<NT>& R, const Params& p, const int* pg, int h, int kb, int kend) {
  load_raw_k<QM, K2, NT, FRESH>(R, p, pg, h, kb, kend);
  load_raw_v<QM, NT, FRESH>(R, p, pg, h, kb, kend);
}

// Key-only pages, one 128-d (half) chunk: the keys of (token, quarter tg) per group g as four fp16 pairs, either final
// (rot[g] false: (code - zero point) * scale, one rounding) or rotated back (rot[g] true): the five in-group stages on
// the exact integers, the group scale times 2^-2.5 (H32 alone) or times the whole-head normalisation (`whole`: 2^-3.5
// at head dim 128, 2^-4 at head dim 256), and for `whole` the two stages across the four groups.  Head dim 256 leaves
// the stage across the two halves to the caller.
template <int QM, int HD>
DEVI void k2_values(const u32x4 kc, const u32x2 sw, bool whole, int tg, const Consts& cst, uint32_t (&v)[4][4], bool (&rot)[4]) {
  using F = Fmt<QM>;
  uint32_t w[4];
  if constexpr (QM == QM_ASYM2) {
    w[0] = kc.x; w[1] = kc.x >> 4; w[2] = kc.y; w[3] = kc.y >> 4;
  } else {
    w[0] = kc.x; w[1] = kc.y; w[2] = kc.z; w[3] = kc.w;
  }
  const uint32_t s16[4] = {sw.x & 0xFFFFu, sw.x >> 16, sw.y & 0xFFFFu, sw.y >> 16};
  const uint32_t sgn1 = (tg & 1) ? 0xBC00BC00u : 0x3C003C00u, sgn2 = (tg & 2) ? 0xBC00BC00u : 0x3C003C00u;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    rot[g] = whole || ((s16[g] >> 15) & 1u);
    const uint32_t z = negz16(s16[g] & F::ZM) * 0x10001u, sc = (s16[g] & 0x7FFFu) * 0x10001u;
    // normalisation as fp16 value + remainder: 2^-2.5 = 0x31A8 + 0x013D, 2^-3.5 = 0x2DA8 + 0x009E, 2^-4 = 0x2C00 (exact)
    const uint32_t ch = whole ? (HD == 128 ? 0x2DA82DA8u : 0x2C002C00u) : 0x31A831A8u;
    const uint32_t cl = whole ? (HD == 128 ? 0x009E009Eu : 0u) : 0x013D013Du;
    const uint32_t fh = pk_mul(sc, ch);
    const uint32_t fl = u2(__builtin_elementwise_fma(h2(sc), h2(cl), __builtin_elementwise_fma(h2(sc), h2(ch), h2(fh ^ 0x80008000u))));
    const uint32_t nz[4] = {z, z, z, z};
    uint32_t c[4], y[4];
    Unpack<QM>::run(w[g], nz, cst, c);
#pragma unroll
    for (int r = 0; r < 4; ++r) y[r] = c[r];
    h32_group(y, sgn1, sgn2);                 // on the integers code - zero point: exact (|sum| <= 32 * 15)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      v[g][r] = rot[g] ? u2(__builtin_elementwise_fma(h2(y[r]), h2(fl), h2(y[r]) * h2(fh))) : pk_mul(c[r], sc);
  }
  if (__any(whole)) {                                          // the two group bits of the whole-head transform
    uint32_t f[4][4];                                          // (whole: every group is rotated, v holds the y of all four)
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int r = 0; r < 4; ++r) f[g][r] = v[g][r];
#pragma unroll
    for (int r = 0; r < 4; ++r) { bfly(f[0][r], f[1][r]); bfly(f[2][r], f[3][r]); }
#pragma unroll
    for (int r = 0; r < 4; ++r) { bfly(f[0][r], f[2][r]); bfly(f[1][r], f[3][r]); }
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int r = 0; r < 4; ++r) v[g][r] = whole ? f[g][r] : v[g][r];
  }
}

// K tile entry idx = (token tk = idx >> 2 of the block, quarter tg = idx & 3) from the token's raw words
template <int QM, bool K2>
DEVI void convert_k_entry(uint8_t* kt, int idx, const u32x4 kc, const u32x2 sw, uint32_t vf, int kb, int kend, const Consts& cst) {
  using F = Fmt<QM>;
  {
    const int tk = idx >> 2, tg = idx & 3;
    const int j = kb * BN + tk;
    const int row = 32 * (tk >> 5) + krow_of_token(tk & 31);
    u32x4* dst = reinterpret_cast<u32x4*>(kt + row * KROW);
    if (j >= kend) {
#pragma unroll
      for (int g = 0; g < 4; ++g) dst[4 * g + tg] = u32x4{0u, 0u, 0u, 0u};
      return;
    }
    uint32_t w[4];
    if constexpr (QM == QM_ASYM2) {
      w[0] = kc.x; w[1] = kc.x >> 4; w[2] = kc.y; w[3] = kc.y >> 4;
    } else {
      w[0] = kc.x; w[1] = kc.y; w[2] = kc.z; w[3] = kc.w;
    }
    const uint32_t s16[4] = {sw.x & 0xFFFFu, sw.x >> 16, sw.y & 0xFFFFu, sw.y >> 16};
    if constexpr (!K2) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const uint32_t z = negz16(s16[g] & F::ZM) * 0x10001u, sc = (s16[g] & 0x7FFFu) * 0x10001u;
        const uint32_t nz[4] = {z, z, z, z};
        uint32_t x[4];
        Unpack<QM>::run(w[g], nz, cst, x);
        dst[4 * g + tg] = u32x4{pk_mul(x[0], sc), pk_mul(x[1], sc), pk_mul(x[2], sc), pk_mul(x[3], sc)};
      }
    } else {
      // key-only pages: the token's flags select identity / H32 per group / whole-head H128 (the quad of a token agrees)
      const bool ff = (vf >> 15) & 1u;
      uint32_t v[4][4];
      bool rot[4];
      k2_values<QM, 128>(kc, sw, ff, tg, cst, v, rot);
#pragma unroll
      for (int g = 0; g < 4; ++g) dst[4 * g + tg] = u32x4{v[g][0], v[g][1], v[g][2], v[g][3]};
    }
  }
}

template <int QM, bool K2, int NT>
DEVI void convert_k(Smem& S, const Raw<NT>& R, int kb, int kend, const Consts& cst) {
#pragma unroll
  for (int it = 0; it < Raw<NT>::NI; ++it)
    convert_k_entry<QM, K2>(S.kt, threadIdx.x + it * NT, R.kc[it], R.ks[it], K2 ? R.vf[it] : 0u, kb, kend, cst);
}

// per (group, run) scale / zero point pairs in the run order; tokens at or beyond kend get scale 0
template <int QM, int NT>
DEVI void v_tables(Smem& S, const Raw<NT>& R, int kb, int kend) {
  using F = Fmt<QM>;
  if (threadIdx.x < 32) {
    const int g = threadIdx.x >> 3, run = threadIdx.x & 7;
    const int j0 = kb * BN + 8 * run;
    u32x4 sc = {0u, 0u, 0u, 0u}, nz = {0u, 0u, 0u, 0u};
    if (j0 < kend) {
      const u32x4 w = R.vs;
      const uint32_t t[8] = {w.x & 0xFFFFu, w.z & 0xFFFFu, w.x >> 16, w.z >> 16, w.y & 0xFFFFu, w.w & 0xFFFFu, w.y >> 16, w.w >> 16};
      uint32_t s[8], z[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        s[k] = j0 + k < kend ? (t[k] & 0x7FFFu) : 0u;
        z[k] = negz16(t[k] & F::ZM);
      }
      sc = u32x4{s[0] | (s[4] << 16), s[1] | (s[5] << 16), s[2] | (s[6] << 16), s[3] | (s[7] << 16)};
      nz = u32x4{z[0] | (z[4] << 16), z[1] | (z[5] << 16), z[2] | (z[6] << 16), z[3] | (z[7] << 16)};
    }
    *reinterpret_cast<u32x4*>(S.vsc[g][run]) = sc;
    *reinterpret_cast<u32x4*>(S.vnz[g][run]) = nz;
  }
}

template <int QM, int NT>
DEVI void convert_v(Smem& S, const Raw<NT>& R, int kb, int kend, const Consts& cst) {
#pragma unroll
  for (int it = 0; it < Raw<NT>::NI; ++it) {
    const int idx = threadIdx.x + it * NT;
    const int pgi = idx >> 6, e = (idx & 63) >> 1, c8 = idx & 1, run = 2 * pgi + c8;
    const int j0 = kb * BN + PAGE * pgi;
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    if (j0 < kend) {
      if constexpr (QM == QM_ASYM2) {
        w[0] = R.vc[it].x; w[1] = R.vc[it].x >> 4; w[2] = R.vc[it].y; w[3] = R.vc[it].y >> 4;
      } else {
        w[0] = R.vc[it].x; w[1] = R.vc[it].y; w[2] = R.vc[it].z; w[3] = R.vc[it].w;
      }
    }
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) {
      const int d = 64 * (sub >> 1) + 16 * (e >> 3) + 8 * (sub & 1) + (e & 7), g = d >> 5;
      const u32x4 sc = *reinterpret_cast<const u32x4*>(S.vsc[g][run]);
      const u32x4 z = *reinterpret_cast<const u32x4*>(S.vnz[g][run]);
      const uint32_t nz[4] = {z.x, z.y, z.z, z.w};
      uint32_t x[4];
      Unpack<QM>::run(w[sub], nz, cst, x);
      *reinterpret_cast<u32x4*>(S.vt + d * VROW + 16 * run) =
          u32x4{pk_mul(x[0], sc.x), pk_mul(x[1], sc.y), pk_mul(x[2], sc.z), pk_mul(x[3], sc.w)};
    }
  }
}

// ------------------------------------------------------------------------------------------------ one 64-key block
// scores, mask, online softmax and values of the wavefront's 32 rows against the tiles in LDS, in three parts
// S^T = K q^T: two 32-key tiles (two independent accumulator chains), eight 16-element steps; the K operands of four
// steps are requested ahead, and the scheduler is told to keep the reads that far in front of the matrix instructions
// (ADD: on top of what sacc holds -- the second 128-d half of a 256-d head)
template <bool ADD = false>
DEVI void qk_block(const uint8_t* kt, const u32x4 (&qf)[8], f32x16 (&sacc)[2], int l32, int hh) {
  if (!ADD) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[t][i] = 0.f;
  }
  const uint8_t* k0 = kt + l32 * KROW + 16 * hh;
  const uint8_t* k1 = k0 + 32 * KROW;
  u32x4 a0[8], a1[8];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    a0[s] = *reinterpret_cast<const u32x4*>(k0 + 64 * (s >> 1) + 32 * (s & 1));
    a1[s] = *reinterpret_cast<const u32x4*>(k1 + 64 * (s >> 1) + 32 * (s & 1));
  }
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    if (s + 4 < 8) {
      a0[s + 4] = *reinterpret_cast<const u32x4*>(k0 + 64 * ((s + 4) >> 1) + 32 * (s & 1));
      a1[s + 4] = *reinterpret_cast<const u32x4*>(k1 + 64 * ((s + 4) >> 1) + 32 * (s & 1));
    }
    sacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_h8(a0[s]), as_h8(qf[s]), sacc[0], 0, 0, 0);
    sacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_h8(a1[s]), as_h8(qf[s]), sacc[1], 0, 0, 0);
  }
  __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);       // 8 LDS reads
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);     // 2 MFMA
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);     // 2 LDS reads
  }
  __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
}

// max over lanes l and l + 32, in both: one v_permlane32_swap, no trip through the LDS queue (which the other group's
// matrix operand reads keep full)
DEVI float max_halves(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);   // (lo, lo), (hi, hi)
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// mask + online softmax (lane = row; lanes l and l + 32 hold the two halves of its keys); the probabilities leave as the
// fp16 B operands of the value product, in the V^T token order
DEVI void softmax_block(f32x16 (&sacc)[2], u32x4 (&pb)[4], f32x16 (&o)[4], float& mrow, float& lrow, int kb, int lim,
                        bool rvalid, int kmin, int hh) {
  const int jb = kb * BN;
  const bool full = __all(rvalid && jb + BN - 1 <= lim) && jb >= kmin;
  if (!full) {
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int j = jb + 32 * kt + token_of_acc(i, hh);
        if (!(j <= lim && j >= kmin)) sacc[kt][i] = -INFINITY;
      }
  }
  float mx = -INFINITY;
#pragma unroll
  for (int kt = 0; kt < 2; ++kt)
#pragma unroll
    for (int i = 0; i < 16; ++i) mx = fmaxf(mx, sacc[kt][i]);
  mx = max_halves(mx);
  const float mnew = fmaxf(mrow, mx);
  const float base = mnew == -INFINITY ? 0.f : mnew;
  const float alpha = fexp2(mrow - base);
  float sum = 0.f;
#pragma unroll
  for (int kt = 0; kt < 2; ++kt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      sacc[kt][i] = fexp2(sacc[kt][i] - base);
      sum += sacc[kt][i];
    }
  lrow = lrow * alpha + sum;
  if (!__all(mnew == mrow)) {
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
  }
  mrow = mnew;
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {      // ks = 2 kt + s
    const int kt = ks >> 1, s2 = ks & 1;
    pb[ks] = u32x4{pack_h2_rn(sacc[kt][8 * s2], sacc[kt][8 * s2 + 1]), pack_h2_rn(sacc[kt][8 * s2 + 2], sacc[kt][8 * s2 + 3]),
                   pack_h2_rn(sacc[kt][8 * s2 + 4], sacc[kt][8 * s2 + 5]), pack_h2_rn(sacc[kt][8 * s2 + 6], sacc[kt][8 * s2 + 7])};
  }
}

// O^T += V^T P^T: four independent accumulator chains (the 32-dim blocks); V^T operands requested two steps ahead
DEVI void pv_block(const uint8_t* vt, const u32x4 (&pb)[4], f32x16 (&o)[4], int l32, int hh) {
  u32x4 va[4][4];
  const uint8_t* v0 = vt + l32 * VROW + 16 * hh;
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int db = 0; db < 4; ++db) va[ks][db] = *reinterpret_cast<const u32x4*>(v0 + 32 * db * VROW + 32 * ks);
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    if (ks + 2 < 4) {
#pragma unroll
      for (int db = 0; db < 4; ++db) va[ks + 2][db] = *reinterpret_cast<const u32x4*>(v0 + 32 * db * VROW + 32 * (ks + 2));
    }
#pragma unroll
    for (int db = 0; db < 4; ++db) o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_h8(va[ks][db]), as_h8(pb[ks]), o[db], 0, 0, 0);
  }
  __builtin_amdgcn_sched_group_barrier(0x100, 8, 1);
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    __builtin_amdgcn_sched_group_barrier(0x008, 4, 1);
    __builtin_amdgcn_sched_group_barrier(0x100, 4, 1);
  }
  __builtin_amdgcn_sched_group_barrier(0x008, 8, 1);
}

DEVI void attend_block(const Smem& S, const u32x4 (&qf)[8], f32x16 (&o)[4], float& mrow, float& lrow, int kb, int lim,
                       bool rvalid, int kmin, int l32, int hh) {
  f32x16 sacc[2];
  u32x4 pb[4];
  qk_block(S.kt, qf, sacc, l32, hh);
  softmax_block(sacc, pb, o, mrow, lrow, kb, lim, rvalid, kmin, hh);
  pv_block(S.vt, pb, o, l32, hh);
}

}  // namespace frmq
