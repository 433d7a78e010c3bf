// Prefix-cached multi-query prefill attention straight from FlagRot INT4 / INT2 pages for gfx950 (wave64, MFMA), and the
// extern "C" surface of libflagrot_mq.so (declared in include/flagrot_mq.h).
//
// Workgroup = (work item, KV head): a q tile of ROWS = 32 x waves rows (row r = token r / G, q head h G + r % G) against
// the item's 64-key blocks.  Per block the workgroup turns the four page chunks into two fp16 tiles in LDS,
//   K  [64 keys][128]  (code - zero point) * scale, one rounding; elements in code-word order, rows permuted so that
//                      the score accumulators come out in the V^T token order;
//   V^T [128 dims][64] eight-token runs exactly as the page stores them;
// and every wavefront runs v_mfma_f32_32x32x16_f16 transposed: S^T = K q^T (lane = one query row, 32 keys in
// registers: the softmax needs one cross-lane step), P^T straight from the accumulators as the B operand of
// O^T = V^T P^T.  Key-only pages (per-token H32 / H128 flags): the conversion applies the token's inverse transform to
// the fp16 pairs in registers (packed butterflies, the quad of a token exchanging by DPP) before the tile is stored, so
// the matrix part is the same for every format.
// Two kernels: k_mq (64 / 128 rows, two or four wavefronts that convert, then attend, with barriers in between; the
// reference's selectors 1 - 3) and k_mq8 (256 rows, selector 4: eight wavefronts in two groups half a block apart, the
// matrix instructions of one group under the vector instructions of the other; described at its definition).
// Causal rule: key j is visible to the row at position p iff kmin <= j <= max(p - shift, ext), j < nk.
// Partials (unnormalised O, running maximum in log2 units, sum) per (item, KV head, row); k_fold_items combines the
// items of a tile.  Semantics follow integrations/vllm_flagrot/csrc/mq_prefill.cu:345-498 (k_mq), :716-772 (merge),
// :789-823 (q preparation), :1350-1465 (BF16 window gather / sink merge), :1469-1601 (C ABI).
#include <cstdio>
#include <cstring>

#include "../../include/flagrot_mq.h"
#include "fr_common.hpp"
#include "fr_unpack.hpp"
#include "mq_launch.hpp"
#include "mq_tiles.hpp"

namespace frmq {
using namespace fr;
namespace {

char g_err[512] = "";

// ------------------------------------------------------------------------------------------------ main kernel
template <int QM, bool K2, int NW>
__global__ void __launch_bounds__(64 * NW, 2) k_mq(const Params p) {
  constexpr int NT = 64 * NW, ROWS = 32 * NW;
  extern __shared__ __align__(16) uint8_t lds[];
  Smem& S = *reinterpret_cast<Smem*>(lds);
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
  const int item = blockIdx.x, h = blockIdx.y;
  const Work work(p, item, ROWS);
  const int G = p.G, Hq = p.Hkv * G;
  const int* bt = work.block_table;
  const int kend = work.key_end, kb0 = work.block0, kb1 = work.block1;
  const Consts cst = make_consts();

  // this lane's query row
  const int r = 32 * wv + l32;
  const bool rvalid = work.has_row(r);
  const int lim = rvalid ? work.last_key(r / G) : -1;

  // page ids of the first blocks (published by the barriers of the q staging below)
  int cb = kb0;
  auto fill_pages = [&]() { fill_page_window<NT>(S.pages, bt, cb, kb1, kend, tid); };
  fill_pages();

  // q fragments: the tile through LDS (natural order), gathered in code-word order
  u32x4 qf[8];
  for (int row = tid >> 5; row < ROWS; row += NT / 32) {
    const int t = row / G, lq = tid & 31;
    u32x2 raw = {0u, 0u};
    if (work.has_row(row)) raw = gload<u32x2>(p.q + (static_cast<long long>(work.compact_row + t) * Hq + h * G + row % G) * D + 4 * lq);
    *reinterpret_cast<u32x2*>(lds + row * QROW + 8 * lq) = raw;
  }
  __syncthreads();
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const int dA = 32 * (s >> 1) + 4 * (2 * (s & 1) + hh);
    const u32x2 a = *reinterpret_cast<const u32x2*>(lds + r * QROW + 2 * dA);
    const u32x2 b = *reinterpret_cast<const u32x2*>(lds + r * QROW + 2 * (dA + 16));
    // (A0 A1)(A2 A3), (B0 B1)(B2 B3) -> (A0 A2)(B0 B2)(A1 A3)(B1 B3)
    qf[s] = u32x4{(a.x & 0xFFFFu) | (a.y << 16), (b.x & 0xFFFFu) | (b.y << 16),
                  (a.x >> 16) | (a.y & 0xFFFF0000u), (b.x >> 16) | (b.y & 0xFFFF0000u)};
  }

  f32x16 o[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float mrow = -INFINITY, lrow = 0.f;

  // Raw words in flight: two blocks ahead in two register sets; the 64-row kernel (two entries per thread and set) has
  // room for one set only and fetches one block ahead -- a second set there is spilled as it arrives, and a spilled
  // register's reload waits for every fetch in flight.
  constexpr int AHEAD = NW == 2 ? 1 : 2;
  Raw<NT> rawA, rawB;
  if (kb0 < kb1) load_raw<QM, K2, NT, NW == 2>(rawA, p, S.pages, h, kb0, kend);
  if constexpr (AHEAD == 2) {
    if (kb0 + 1 < kb1) load_raw<QM, K2, NT, NW == 2>(rawB, p, S.pages + 4, h, kb0 + 1, kend);
  }
  auto block_step = [&](Raw<NT>& raw, int kb) {
    __syncthreads();                                   // the tiles (or the q staging) are no longer read
    convert_k<QM, K2, NT>(S, raw, kb, kend, cst);
    v_tables<QM, NT>(S, raw, kb, kend);
    if (kb + AHEAD < kb1 && kb + AHEAD >= cb + PG_CACHE / 4) {   // the next fetch leaves the cached window: slide it
      cb = kb + AHEAD;
      fill_pages();
    }
    __syncthreads();
    convert_v<QM, NT>(S, raw, kb, kend, cst);
    __syncthreads();
    if (kb + AHEAD < kb1) load_raw<QM, K2, NT, NW == 2>(raw, p, S.pages + 4 * (kb + AHEAD - cb), h, kb + AHEAD, kend);
    attend_block(S, qf, o, mrow, lrow, kb, lim, rvalid, p.kmin, l32, hh);
  };
  if constexpr (AHEAD == 2) {
    for (int kb = kb0; kb < kb1; kb += 2) {
      block_step(rawA, kb);
      if (kb + 1 < kb1) block_step(rawB, kb + 1);
    }
  } else {
    for (int kb = kb0; kb < kb1; ++kb) block_step(rawA, kb);
  }
  // partials
  const float l = lrow + __shfl_xor(lrow, 32, 64);
  if (rvalid) {
    const long long base = (static_cast<long long>(item) * p.Hkv + h) * ROWS + r;
    float* op = p.opart + base * D;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *reinterpret_cast<float4*>(op + 32 * db + 8 * q4 + 4 * hh) =
            make_float4(o[db][4 * q4], o[db][4 * q4 + 1], o[db][4 * q4 + 2], o[db][4 * q4 + 3]);
    if (hh == 0) *reinterpret_cast<float2*>(p.ml + base * 2) = make_float2(mrow, l);
  }
}

// ------------------------------------------------------------------------------------------------ 256-row kernel
// Eight wavefronts, 256 rows, two groups of four wavefronts (one of each group per SIMD) that alternate between a
// matrix slot and a vector slot, half a block apart, so that the matrix instructions of one group run under the vector
// instructions of the other:
//   slot 2k      group A: O += P(k-1) V(k-1), S = K(k) q      group B: softmax(k-1), V(k) -> tile
//   slot 2k + 1  group A: softmax(k), K(k+1) -> tile          group B: O += P(k-1) V(k-1), S = K(k) q
// One barrier per slot; a wavefront raises its issue priority for its matrix slot (the arbiter otherwise serves the
// older wavefronts' vector instructions first and the matrix pipe starves).  Group A converts the K tiles, group B the V^T tiles, each into the buffer the other block
// parity is not reading; a tile is complete one barrier before its first reader.  The raw words of a tile are fetched
// by the converting group right after the previous conversion (two slots ahead).
struct Smem8 {
  alignas(16) uint8_t kt[2][KT_BYTES];
  alignas(16) uint8_t vt[2][VT_BYTES];
  int pages[PG_CACHE];
};
static_assert(256 * QROW <= 2 * (KT_BYTES + VT_BYTES), "q staging aliases the tiles");

// Raw page words of a thread's tile entry, one register set for both groups (a set per group would let the compiler
// reuse the other group's registers for LDS operands and guard them with waits on outstanding fetches):
//   group A  w[0] = K code words of (token, tg) (INT2: .x .y), w[1].xy = the token's four K scale words,
//            w[1].z = the token's group-0 V scale word (whole-head flag of key-only pages)
//   group B  w[0] = V^T entry (e, c8) of a page, w[1], w[2] = V scale words of the entry's run (eight tokens) in its
//            two groups: t0 t2 | t4 t6 | t1 t3 | t5 t7
struct Raw8 {
  u32x4 w[3];
};

// A wavefront of the group fetches one page of the block (page = its index in the group): the page base is
// wave-uniform, the lane adds a 32-bit offset.  Lane = (token pos = lane >> 2, quarter tg) for the K words.
template <int QM, bool K2>
DEVI void load_k8(Raw8& R, const Params& p, const int* pg, int h, int kb, int kend, int t256) {
  using F = Fmt<QM>;
  const uint32_t lane = t256 & 63, pos = lane >> 2, tg = lane & 3u;
  const int pgi = __builtin_amdgcn_readfirstlane(t256 >> 6);
  const int j0 = kb * BN + PAGE * pgi;
  if (j0 + static_cast<int>(pos) < kend) {
    const int page = __builtin_amdgcn_readfirstlane(pg[pgi]);
    const uint8_t* ch = p.pool + static_cast<long long>(page) * p.page_stride + static_cast<long long>(h) * F::CHUNK;
    if constexpr (QM == QM_ASYM2) {
      const u32x2 c = gload<u32x2>(ch + (32u * (pos ^ ((pos >> 1) & 2u)) + 8u * tg));
      R.w[0] = u32x4{c.x, c.y, 0u, 0u};
    } else {
      R.w[0] = gload<u32x4>(ch + 16u * lane);
    }
    const u32x2 ks = gload<u32x2>(ch + (F::KS_OFF + 8u * pos));
    R.w[1].x = ks.x; R.w[1].y = ks.y;
    if constexpr (K2) R.w[1].z = gload<uint16_t>(ch + (F::VS_OFF + (8u * (pos >> 3) + static_cast<uint32_t>(vs_slot8(pos))) * 2u));
  }
}
template <int QM>
DEVI void load_v8(Raw8& R, const Params& p, const int* pg, int h, int kb, int kend, int t256) {
  using F = Fmt<QM>;
  const uint32_t lane = t256 & 63, g = lane >> 5, c8 = lane & 1u;      // entry e = lane >> 1: its dims lie in groups g, g + 2
  const int pgi = __builtin_amdgcn_readfirstlane(t256 >> 6);
  const int j0 = kb * BN + PAGE * pgi;
  if (j0 < kend) {
    const int page = __builtin_amdgcn_readfirstlane(pg[pgi]);
    const uint8_t* ch = p.pool + static_cast<long long>(page) * p.page_stride + static_cast<long long>(h) * F::CHUNK;
    if constexpr (QM == QM_ASYM2) {
      const u32x2 c = gload<u32x2>(ch + (F::V_OFF + 8u * lane));
      R.w[0] = u32x4{c.x, c.y, 0u, 0u};
    } else {
      R.w[0] = gload<u32x4>(ch + (F::V_OFF + 16u * lane));
    }
    R.w[1] = gload<u32x4>(ch + (F::VS_OFF + (g * PAGE + 8u * c8) * 2u));
    R.w[2] = gload<u32x4>(ch + (F::VS_OFF + ((g + 2u) * PAGE + 8u * c8) * 2u));
  }
}

// V^T tile entry: the scale / zero point pairs of the entry's run come from the thread's own scale words, in the run
// order (t0,t4) (t1,t5) (t2,t6) (t3,t7); tokens at or beyond kend get scale 0
template <int QM>
DEVI void convert_v8(uint8_t* vt, const Raw8& R, int kb, int kend, const Consts& cst, int t256) {
  using F = Fmt<QM>;
  const int pgi = t256 >> 6, e = (t256 & 63) >> 1, c8 = t256 & 1, run = 2 * pgi + c8;
  const bool have = kb * BN + PAGE * pgi < kend;
  const bool ragged = kb * BN + BN > kend;                         // uniform: only the last block of an item
  uint32_t w[4] = {0u, 0u, 0u, 0u};
  if (have) {
    if constexpr (QM == QM_ASYM2) {
      w[0] = R.w[0].x; w[1] = R.w[0].x >> 4; w[2] = R.w[0].y; w[3] = R.w[0].y >> 4;
    } else {
      w[0] = R.w[0].x; w[1] = R.w[0].y; w[2] = R.w[0].z; w[3] = R.w[0].w;
    }
  }
  uint32_t sc[2][4], nz[2][4];
#pragma unroll
  for (int gg = 0; gg < 2; ++gg) {
    const u32x4 v = R.w[1 + gg];
    const uint32_t pr[4] = {__builtin_amdgcn_perm(v.y, v.x, 0x05040100u), __builtin_amdgcn_perm(v.w, v.z, 0x05040100u),
                            __builtin_amdgcn_perm(v.y, v.x, 0x07060302u), __builtin_amdgcn_perm(v.w, v.z, 0x07060302u)};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sc[gg][i] = have ? pr[i] & 0x7FFF7FFFu : 0u;
      nz[gg][i] = (pr[i] & (F::ZM * 0x10001u)) | 0xE400E400u;
    }
  }
  if (ragged) {
    const int t0 = kb * BN + 8 * run;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t m = (t0 + i < kend ? 0xFFFFu : 0u) | (t0 + i + 4 < kend ? 0xFFFF0000u : 0u);
      sc[0][i] &= m; sc[1][i] &= m;
    }
  }
#pragma unroll
  for (int sub = 0; sub < 4; ++sub) {
    const int d = 64 * (sub >> 1) + 16 * (e >> 3) + 8 * (sub & 1) + (e & 7);   // group d >> 5 = 2 (sub >> 1) + (e >> 4)
    uint32_t x[4];
    Unpack<QM>::run(w[sub], nz[sub >> 1], cst, x);
    *reinterpret_cast<u32x4*>(vt + d * VROW + 16 * run) =
        u32x4{pk_mul(x[0], sc[sub >> 1][0]), pk_mul(x[1], sc[sub >> 1][1]), pk_mul(x[2], sc[sub >> 1][2]), pk_mul(x[3], sc[sub >> 1][3])};
  }
}

// The 256-row kernel keeps a per-row REFERENCE instead of the running maximum: the score accumulators start at
// -reference (qk8), so that exp2 applies to them as they are; the reference moves (and O, l are rescaled) only when a
// score exceeds it by more than 2^8, which keeps p <= 256 in fp16.  Any reference gives the same O / l; the partial's
// (m, l) carry it to the merge.
DEVI void qk8(const uint8_t* kt, const u32x4 (&qf)[8], f32x16 (&sacc)[2], float ref, int l32, int hh) {
  f32x16 init;
  const float c0 = ref == -INFINITY ? 0.f : -ref;
#pragma unroll
  for (int i = 0; i < 16; ++i) init[i] = c0;
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
    sacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_h8(a0[s]), as_h8(qf[s]), s ? sacc[0] : init, 0, 0, 0);
    sacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_h8(a1[s]), as_h8(qf[s]), s ? sacc[1] : init, 0, 0, 0);
  }
  __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);       // 8 LDS reads
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);     // 2 MFMA
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);     // 2 LDS reads
  }
  __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
}

// lane = row, lanes l and l + 32 hold the two halves of its 64 keys; sacc = score - reference.  full: no key of the
// block is masked for any row of the wavefront.
DEVI void softmax8(f32x16 (&sacc)[2], u32x4 (&pb)[4], f32x16 (&o)[4], float& ref, float& lrow, bool full, int kb, int lim,
                   int kmin, int hh) {
  if (!full) {
    const int jb = kb * BN;
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
  const bool bump = (mx > 8.f || ref == -INFINITY) && mx != -INFINITY;
  if (__any(bump)) {                                     // rare after the first blocks: move the reference to the row maximum
    const float delta = bump ? mx : 0.f;
    const float alpha = ref == -INFINITY ? 0.f : fexp2(-delta);   // no reference yet: O and l are still zero
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[kt][i] -= delta;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
    lrow *= alpha;
    if (bump) ref = (ref == -INFINITY ? 0.f : ref) + delta;
  }
  typedef _Float16 h2v __attribute__((ext_vector_type(2)));
  const h2v ones = {static_cast<_Float16>(1.f), static_cast<_Float16>(1.f)};
  float s4[4] = {0.f, 0.f, 0.f, 0.f};                   // the sum of what the value product uses
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {      // ks = 2 kt + s
    const int kt = ks >> 1, s2 = ks & 1;
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = pack_h2_rn(fexp2(sacc[kt][8 * s2 + 2 * j]), fexp2(sacc[kt][8 * s2 + 2 * j + 1]));
#pragma unroll
    for (int j = 0; j < 4; ++j) s4[j] = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2v, w[j]), ones, s4[j], false);
    pb[ks] = u32x4{w[0], w[1], w[2], w[3]};
  }
  lrow += (s4[0] + s4[1]) + (s4[2] + s4[3]);
}

template <int QM, bool K2>
__global__ void __launch_bounds__(512, 1) k_mq8(const Params p) {
  constexpr int NT = 512, ROWS = 256;
  extern __shared__ __align__(16) uint8_t lds[];
  Smem8& S = *reinterpret_cast<Smem8*>(lds);
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
  const int grp = __builtin_amdgcn_readfirstlane(wv >> 2);
  const int item = blockIdx.x, h = blockIdx.y;
  const Work work(p, item, ROWS);
  const int G = p.G, Hq = p.Hkv * G;
  const int* bt = work.block_table;
  const int kend = work.key_end, kb0 = work.block0, kb1 = work.block1;
  const Consts cst = make_consts();

  const int r = 32 * wv + l32;
  const bool rvalid = work.has_row(r);
  const int lim = rvalid ? work.last_key(r / G) : -1;

  int cb = kb0;
  auto fill_pages = [&]() { fill_page_window<NT>(S.pages, bt, cb, kb1, kend, tid); };
  fill_pages();

  u32x4 qf[8];
  for (int row = tid >> 5; row < ROWS; row += NT / 32) {
    const int t = row / G, lq = tid & 31;
    u32x2 raw = {0u, 0u};
    if (work.has_row(row)) raw = gload<u32x2>(p.q + (static_cast<long long>(work.compact_row + t) * Hq + h * G + row % G) * D + 4 * lq);
    *reinterpret_cast<u32x2*>(lds + row * QROW + 8 * lq) = raw;
  }
  __syncthreads();
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const int dA = 32 * (s >> 1) + 4 * (2 * (s & 1) + hh);
    const u32x2 a = *reinterpret_cast<const u32x2*>(lds + r * QROW + 2 * dA);
    const u32x2 b = *reinterpret_cast<const u32x2*>(lds + r * QROW + 2 * (dA + 16));
    qf[s] = u32x4{(a.x & 0xFFFFu) | (a.y << 16), (b.x & 0xFFFFu) | (b.y << 16),
                  (a.x >> 16) | (a.y & 0xFFFF0000u), (b.x >> 16) | (b.y & 0xFFFF0000u)};
  }

  f32x16 o[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float mrow = -INFINITY, lrow = 0.f;                  // mrow: the row's reference (see qk8)
  // no key of block kb is masked for any row of the wavefront iff kmin <= 64 kb and 64 kb + 63 <= the smallest limit
  const int lim_min = -static_cast<int>(wave_max64(-static_cast<float>(rvalid ? lim : -1)));   // exact: key indices < 2^24
  auto is_full = [&](int kb) { return kb * BN >= p.kmin && kb * BN + BN - 1 <= lim_min; };
  // The pipeline starts and drains through harmless work instead of branches: probabilities 0 against zeroed V^T
  // tiles add nothing, scores of -inf leave the running maximum and sum alone.
  f32x16 sacc[2];
  u32x4 pb[4];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[t][i] = -INFINITY;
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) pb[ks] = u32x4{0u, 0u, 0u, 0u};
  Raw8 raw;                                            // fetched at the end of a matrix slot, converted in the next vector slot
  const int nb = kb1 - kb0;                            // blocks of the item
  __syncthreads();                                     // the q staging is no longer read
  for (int i = tid; i < 2 * VT_BYTES / 16; i += NT) reinterpret_cast<u32x4*>(&S.vt[0][0])[i] = u32x4{0u, 0u, 0u, 0u};
  if (grp == 0) {                                      // K(0) before the first slot
    load_k8<QM, K2>(raw, p, S.pages, h, kb0, kend, tid_now() & 255);
    convert_k_entry<QM, K2>(S.kt[0], tid_now() & 255, raw.w[0], u32x2{raw.w[1].x, raw.w[1].y}, K2 ? raw.w[1].z : 0u, kb0, kend, cst);
  } else {
    load_v8<QM>(raw, p, S.pages, h, kb0, kend, tid_now() & 255);
  }
  __syncthreads();

  auto slot_barrier = [&]() {                          // nothing of a slot may move into the next one
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };
  // The packed probabilities are pure register values: without this the compiler sinks their conversion past the
  // barrier to their use, between the matrix instructions of the next slot, where a vector instruction stalls them.
  auto pin = [&]() {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) asm volatile("" : "+v"(pb[ks]));
  };
  auto slide = [&](int kb) {
    if (kb + 1 >= cb + PG_CACHE / 4) {                 // block kb + 1 is fetched in this step: slide the window
      slot_barrier();
      cb = kb + 1;
      fill_pages();
      slot_barrier();
    }
  };
  // One loop per group (the same number of barriers in both): the register allocation of one path does not bind the
  // other.  A wavefront issues no vector work between its matrix instructions (on this chip a vector instruction behind
  // a matrix instruction of the same wavefront waits for it); the fetch of the next raw words, mostly latency, follows
  // the last matrix instruction, and nothing is outstanding when the next matrix slot starts.
  if (grp == 0) {
    for (int k = 0; k < nb; ++k) {
      const int kb = kb0 + k;
      slide(kb);
      pv_block(S.vt[(k & 1) ^ 1], pb, o, l32, hh);     // slot 2k: matrix.  V(k - 1), K(k)
      __builtin_amdgcn_sched_barrier(0);
      qk8(S.kt[k & 1], qf, sacc, mrow, l32, hh);
      __builtin_amdgcn_sched_barrier(0);
      load_k8<QM, K2>(raw, p, S.pages + 4 * (kb + 1 - cb), h, kb + 1, kend, tid_now() & 255);
      slot_barrier();
      softmax8(sacc, pb, o, mrow, lrow, is_full(kb), kb, lim, p.kmin, hh);   // slot 2k + 1: vector; K(k + 1) is written
      pin();
      __builtin_amdgcn_sched_barrier(0);
      convert_k_entry<QM, K2>(S.kt[(k & 1) ^ 1], tid_now() & 255, raw.w[0], u32x2{raw.w[1].x, raw.w[1].y}, K2 ? raw.w[1].z : 0u, kb + 1, kend, cst);
      slot_barrier();
    }
    if (nb > 0) pv_block(S.vt[(nb - 1) & 1], pb, o, l32, hh);
  } else {
    for (int k = 0; k < nb; ++k) {
      const int kb = kb0 + k;
      slide(kb);
      softmax8(sacc, pb, o, mrow, lrow, is_full(kb - 1), kb - 1, lim, p.kmin, hh);   // slot 2k: vector (block k - 1); V(k) is written
      pin();
      __builtin_amdgcn_sched_barrier(0);
      convert_v8<QM>(S.vt[k & 1], raw, kb, kend, cst, tid_now() & 255);
      slot_barrier();
      pv_block(S.vt[(k & 1) ^ 1], pb, o, l32, hh);     // slot 2k + 1: matrix.  V(k - 1), K(k)
      __builtin_amdgcn_sched_barrier(0);
      qk8(S.kt[k & 1], qf, sacc, mrow, l32, hh);
      __builtin_amdgcn_sched_barrier(0);
      load_v8<QM>(raw, p, S.pages + 4 * (kb + 1 - cb), h, kb + 1, kend, tid_now() & 255);
      slot_barrier();
    }
    if (nb > 0) {                                      // group B is one slot behind
      softmax8(sacc, pb, o, mrow, lrow, is_full(kb1 - 1), kb1 - 1, lim, p.kmin, hh);
      pin();
      pv_block(S.vt[(nb - 1) & 1], pb, o, l32, hh);
    }
  }

  const float l = lrow + __shfl_xor(lrow, 32, 64);
  if (rvalid) {
    const long long base = (static_cast<long long>(item) * p.Hkv + h) * ROWS + r;
    float* op = p.opart + base * D;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *reinterpret_cast<float4*>(op + 32 * db + 8 * q4 + 4 * hh) =
            make_float4(o[db][4 * q4], o[db][4 * q4 + 1], o[db][4 * q4 + 2], o[db][4 * q4 + 3]);
    if (hh == 0) *reinterpret_cast<float2*>(p.ml + base * 2) = make_float2(mrow, l);
  }
}

// ------------------------------------------------------------------------------------------------ items of a tile, folded
// A wavefront folds FOLD_ROWS consecutive query rows of a tile for one KV head, a lane per channel pair.  The items'
// (maximum, sum) pairs are read one item per lane (64 at a time), so the common maximum, every item's weight
// 2^(m - M) and the total sum come from three wave reductions instead of two serial passes; the accumulation loop then
// takes each weight from its lane.  A tile with a single item (the common case when the requests fill the GPU) needs
// neither: its partial is divided by its own sum.
constexpr int FOLD_ROWS = 4;

// W consecutive floats per lane: W = 2 covers a 128-d row with one wavefront, W = 4 a 256-d row
template <int W> DEVI void ldw(const float* p, float (&x)[W]) {
  if constexpr (W == 2) { const float2 v = *reinterpret_cast<const float2*>(p); x[0] = v.x; x[1] = v.y; }
  else { const float4 v = *reinterpret_cast<const float4*>(p); x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w; }
}
template <int W> DEVI void stw(float* p, const float (&x)[W]) {
  if constexpr (W == 2) *reinterpret_cast<float2*>(p) = make_float2(x[0], x[1]);
  else *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
}
template <int W> DEVI void ldw_bf16(const uint16_t* p, float (&x)[W]) {
  if constexpr (W == 2) { const uint32_t v = *reinterpret_cast<const uint32_t*>(p); x[0] = bf16_lo(v); x[1] = bf16_hi(v); }
  else { const uint2 v = *reinterpret_cast<const uint2*>(p); x[0] = bf16_lo(v.x); x[1] = bf16_hi(v.x); x[2] = bf16_lo(v.y); x[3] = bf16_hi(v.y); }
}
template <int W> DEVI void stw_bf16(uint16_t* p, const float (&x)[W]) {
  if constexpr (W == 2) *reinterpret_cast<uint32_t*>(p) = bf16_rn(x[0]) | (bf16_rn(x[1]) << 16);
  else *reinterpret_cast<uint2*>(p) = make_uint2(bf16_rn(x[0]) | (bf16_rn(x[1]) << 16), bf16_rn(x[2]) | (bf16_rn(x[3]) << 16));
}

template <bool FP32_OUT, int W>
__global__ void __launch_bounds__(256) k_fold_items(const int* __restrict__ tiles, const float* __restrict__ opart,
                                                    const float* __restrict__ ml, int Hkv, int G, int rows,
                                                    void* __restrict__ out, long long out_stride, float* __restrict__ lse,
                                                    long long lse_stride) {
  const int lane = threadIdx.x & 63, head = blockIdx.y;
  const int* rec = tiles + TILE_INTS * blockIdx.x;
  const int first = rec[6], count = rec[7];
  const int used = min(rows / G, rec[3]) * G;                            // rows of the tile that hold a token's head
  const long long per_item = static_cast<long long>(Hkv) * rows;         // partial rows from one item to the next
  const int row0 = (blockIdx.z * 4 + (threadIdx.x >> 6)) * FOLD_ROWS;
#pragma unroll
  for (int i = 0; i < FOLD_ROWS; ++i) {
    const int row = row0 + i;
    if (row >= used) break;                                              // wave uniform
    constexpr int DW = 64 * W;                                           // the head dim
    const long long at = (static_cast<long long>(first) * Hkv + head) * rows + row;
    float sum[W];
#pragma unroll
    for (int k = 0; k < W; ++k) sum[k] = 0.f;
    float top, total;
    if (count == 1) {
      const float2 st = *reinterpret_cast<const float2*>(ml + 2 * at);
      top = st.x; total = st.y;
      if (top != -INFINITY) ldw<W>(opart + at * DW + W * lane, sum);
    } else {
      top = -INFINITY; total = 0.f;
      for (int s0 = 0; s0 < count; s0 += 64)
        top = fmaxf(top, wave_max64(s0 + lane < count ? ml[2 * (at + (s0 + lane) * per_item)] : -INFINITY));
      if (top != -INFINITY) {
        for (int s0 = 0; s0 < count; s0 += 64) {
          float weight = 0.f, mass = 0.f;
          if (s0 + lane < count) {
            const float2 st = *reinterpret_cast<const float2*>(ml + 2 * (at + (s0 + lane) * per_item));
            weight = st.x == -INFINITY ? 0.f : fexp2(st.x - top);
            mass = weight * st.y;
          }
          total += wave_sum64(mass);
          const int n = min(64, count - s0);
          for (int s = 0; s < n; ++s) {
            const float w = __shfl(weight, s, 64);
            if (w == 0.f) continue;                                      // an item that saw no key: nothing to read
            float x[W];
            ldw<W>(opart + (at + (s0 + s) * per_item) * DW + W * lane, x);
#pragma unroll
            for (int k = 0; k < W; ++k) sum[k] += w * x[k];
          }
        }
      }
    }
    if (top != -INFINITY) {
      const float inv = 1.f / total;
#pragma unroll
      for (int k = 0; k < W; ++k) sum[k] *= inv;
    }
    const int token = row / G, qhead = head * G + row % G;
    if (FP32_OUT) {                                                      // compact rows, dense [m, Hq, D]
      float* dst = static_cast<float*>(out) + (static_cast<long long>(rec[1] + token) * Hkv * G + qhead) * DW;
      stw<W>(dst + W * lane, sum);
    } else {                                                             // rows of the layer output
      uint16_t* dst = static_cast<uint16_t*>(out) + static_cast<long long>(rec[2] + token) * out_stride + qhead * DW;
      stw_bf16<W>(dst + W * lane, sum);
    }
    if (lse != nullptr && lane == 0)
      lse[qhead * lse_stride + rec[1] + token] = top == -INFINITY ? -INFINITY : (top + log2f(total)) * 0.6931471805599453f;
  }
}

// ------------------------------------------------------------------------------------------------ query rows for the kernel
// A workgroup takes one query row and walks its heads, eight at a time: a half wave per head, four channels per lane
// (the shape the Hadamard helpers work on).  Where the head's keys are stored whole-head rotated the row becomes
// H128 x / 8 (unnormalised butterflies, then one multiply), then the groups stored H32-rotated get the orthonormal H32,
// then the softmax factor, then one rounding to fp16 -- each step rounded to fp32 on its own, in this order.
template <typename T> DEVI void read4(const T* p, float (&x)[4]);
template <> DEVI void read4<float>(const float* p, float (&x)[4]) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
}
template <> DEVI void read4<uint16_t>(const uint16_t* p, float (&x)[4]) {     // bf16
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  x[0] = bf16_lo(v.x); x[1] = bf16_hi(v.x); x[2] = bf16_lo(v.y); x[3] = bf16_hi(v.y);
}

template <typename T>
__global__ void __launch_bounds__(256) k_query_rows(const T* __restrict__ q, long long q_stride, const int* __restrict__ pick,
                                                    int Hq, int G, const uint8_t* __restrict__ whole,
                                                    const uint8_t* __restrict__ rotated, float factor,
                                                    uint16_t* __restrict__ q16) {
  const int l32 = threadIdx.x & 31, sub = l32 >> 3;
  const long long src = pick != nullptr ? pick[blockIdx.x] : blockIdx.x;
  for (int head = threadIdx.x >> 5; head < Hq; head += 8) {
    const int kv = head / G;
    float x[4];
    read4<T>(q + src * q_stride + head * D + 4 * l32, x);
    if (whole != nullptr && whole[kv]) {
      butterflies<128>(x, l32);
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] *= 0.125f;
    }
    if (rotated != nullptr) {                    // every lane takes part in the exchange; the flagged groups keep the result
      float y[4] = {x[0], x[1], x[2], x[3]};
      fwht<32>(y, l32);
      if (rotated[kv * 4 + sub]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) x[i] = y[i];
      }
    }
    uint32_t h[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) h[i] = f16_bits_rn(x[i] * factor);
    *reinterpret_cast<uint2*>(q16 + (static_cast<long long>(blockIdx.x) * Hq + head) * D + 4 * l32) =
        make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
  }
}

// ------------------------------------------------------------------------------------------------ BF16 window / sink rows
// Collects the K and V rows of the window call: a flat grid over the 16-byte pieces of all rows (a row is Hkv x 128 bf16
// = 16 Hkv pieces per tensor), so the launch fills the GPU whatever Hkv is.  map[d] = (source << 32) | row.
__global__ void __launch_bounds__(256) k_collect_rows(const long long* __restrict__ map, int nrows, const uint4* __restrict__ sinks,
                                                      const uint4* __restrict__ earlier, const uint16_t* __restrict__ kbatch,
                                                      long long k_stride, const uint16_t* __restrict__ vbatch, long long v_stride,
                                                      int pieces, uint4* __restrict__ kdst, uint4* __restrict__ vdst) {
  const long long e = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= static_cast<long long>(nrows) * pieces) return;
  const long long d = e / pieces;
  const int i = static_cast<int>(e - d * pieces);
  const long long code = map[d];
  const unsigned from = static_cast<unsigned>(code >> 32);
  const long long row = code & 0xffffffffLL;
  uint4 k, v;
  if (from == 2u) {                              // this batch's own rows: K and V in separate tensors
    k = reinterpret_cast<const uint4*>(kbatch + row * k_stride)[i];
    v = reinterpret_cast<const uint4*>(vbatch + row * v_stride)[i];
  } else {                                       // kept rows: [K heads | V heads] side by side
    const uint4* both = (from == 0u ? sinks : earlier) + row * 2 * pieces;
    k = both[i];
    v = both[pieces + i];
  }
  kdst[e] = k;
  vdst[e] = v;
}

// Mixes the parts of a compact row's attention by their log-sum-exps and writes the bf16 output row: one wavefront per
// (row, query head), a lane per channel pair.  Page part fp32 (o, lse); window part bf16 (o, lse) or absent; sink part
// computed here over the keys j < min(S, length of the request's sinks), j <= position - W: first every key's score
// (one wave reduction each, key j's score parked in lane j), then the softmax across lanes, then the weighted rows.
// An lse of +-inf or NaN means the part is empty.  S <= 64.
DEVI bool usable(float lse) { return lse == lse && lse != INFINITY && lse != -INFINITY; }

template <int W>
__global__ void __launch_bounds__(256) k_mix_parts(int m, int Hq, int Hkv, const uint16_t* __restrict__ q, long long q_stride,
                                                   const long long* __restrict__ out_row, const float* __restrict__ o_pages,
                                                   const float* __restrict__ lse_pages, const uint16_t* __restrict__ o_win,
                                                   const float* __restrict__ lse_win, const uint16_t* __restrict__ sinks,
                                                   const long long* __restrict__ req_of, const long long* __restrict__ pos_of,
                                                   const long long* __restrict__ sink_len, int S, int W_keep, float scale,
                                                   uint16_t* __restrict__ out, long long out_stride) {
  const int lane = threadIdx.x & 63;
  const int c = blockIdx.x, head = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (head >= Hq) return;
  constexpr int DW = 64 * W;                     // the head dim: W channels per lane
  const int kv = head / (Hq / Hkv);
  const long long dst_row = out_row[c], flat = (static_cast<long long>(c) * Hq + head) * DW + W * lane;

  float lp = lse_pages[static_cast<long long>(head) * m + c];
  float vp[W], vw[W], vs[W];
#pragma unroll
  for (int k = 0; k < W; ++k) vp[k] = vw[k] = vs[k] = 0.f;
  if (usable(lp)) ldw<W>(o_pages + flat, vp); else lp = -INFINITY;

  float lw = -INFINITY;
  if (o_win != nullptr) {
    const float l = lse_win[static_cast<long long>(head) * m + c];
    if (usable(l)) { lw = l; ldw_bf16<W>(o_win + flat, vw); }
  }

  float ls = -INFINITY;
  if (sinks != nullptr) {
    const long long req = req_of[c];
    const int n = static_cast<int>(min(min(static_cast<long long>(S), sink_len[req]), pos_of[c] - W_keep + 1));
    if (n > 0) {
      float qv[W];
      ldw_bf16<W>(q + dst_row * q_stride + static_cast<long long>(head) * DW + W * lane, qv);
      const uint16_t* base = sinks + (req * S * 2 * Hkv + kv) * DW + W * lane;      // K head kv of sink row 0
      const long long step = 2LL * Hkv * DW, to_v = static_cast<long long>(Hkv) * DW;
      float mine = -INFINITY;                                                      // lane j: score of key j
      for (int j = 0; j < n; ++j) {
        float kk[W];
        ldw_bf16<W>(base + j * step, kk);
        float dot = 0.f;
#pragma unroll
        for (int k = 0; k < W; ++k) dot += qv[k] * kk[k];
        const float sc = wave_sum64(dot) * scale;
        if (lane == j) mine = sc;
      }
      const float top = wave_max64(mine);
      const float p = lane < n ? expf(mine - top) : 0.f;
      const float mass = wave_sum64(p);
      for (int j = 0; j < n; ++j) {
        const float w = __shfl(p, j, 64);
        float vv[W];
        ldw_bf16<W>(base + j * step + to_v, vv);
#pragma unroll
        for (int k = 0; k < W; ++k) vs[k] += w * vv[k];
      }
#pragma unroll
      for (int k = 0; k < W; ++k) vs[k] /= mass;
      ls = top + logf(mass);
    }
  }

  const float top = fmaxf(lp, fmaxf(lw, ls));
  float o[W];
#pragma unroll
  for (int k = 0; k < W; ++k) o[k] = 0.f;
  if (top != -INFINITY) {
    const float wp = lp == -INFINITY ? 0.f : expf(lp - top), ww = lw == -INFINITY ? 0.f : expf(lw - top),
                wsk = ls == -INFINITY ? 0.f : expf(ls - top);
    const float inv = 1.f / (wp + ww + wsk);
#pragma unroll
    for (int k = 0; k < W; ++k) o[k] = (wp * vp[k] + ww * vw[k] + wsk * vs[k]) * inv;
  }
  stw_bf16<W>(out + dst_row * out_stride + static_cast<long long>(head) * DW + W * lane, o);
}

template <int QM, bool K2, int NW> int launch_mq(const Params& p, int nitems, hipStream_t st) {
  static bool attr = false;
  if (!attr) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_mq<QM, K2, NW>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(sizeof(Smem))) != hipSuccess) return -1;
    attr = true;
  }
  hipLaunchKernelGGL((k_mq<QM, K2, NW>), dim3(nitems, p.Hkv), dim3(64 * NW), sizeof(Smem), st, p);
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

template <int QM, bool K2> int launch_mq8(const Params& p, int nitems, hipStream_t st) {
  static bool attr = false;
  if (!attr) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_mq8<QM, K2>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(sizeof(Smem8))) != hipSuccess) return -1;
    attr = true;
  }
  hipLaunchKernelGGL((k_mq8<QM, K2>), dim3(nitems, p.Hkv), dim3(512), sizeof(Smem8), st, p);
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

int done(int rc, const char* what) {
  if (rc == -1) std::snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(hipGetLastError()));
  return rc;
}
int bad(int rc, const char* msg) {
  std::strncpy(g_err, msg, sizeof(g_err) - 1);
  return rc;
}

}  // namespace
}  // namespace frmq

using namespace frmq;

extern "C" {

int frmq_abi_version(void) { return 7; }
const char* frmq_last_error(void) { return g_err; }
int frmq_smem_bytes(void) {
  const int a = static_cast<int>(sizeof(Smem8) > sizeof(Smem) ? sizeof(Smem8) : sizeof(Smem)), b = wide_smem_bytes();
  return a > b ? a : b;
}

int frmq_prep_q(const void* q, int q_fp32, long long q_ts, const int* idx, int m, int Hq, int G, const uint8_t* kfull,
                const uint8_t* kmask, float qscale, void* q16, int Dh, void* stream) {
  if (m <= 0) return 0;
  if (Dh != D && Dh != 256) return bad(-4, "frmq_prep_q: head dim 128 or 256");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (Dh == 256) return done(wide_query_rows_launch(q, q_fp32, q_ts, idx, m, Hq, G, kfull, kmask, qscale, q16, st), "frmq_prep_q");
  uint16_t* dst = static_cast<uint16_t*>(q16);
  if (q_fp32) hipLaunchKernelGGL(k_query_rows<float>, dim3(m), dim3(256), 0, st, static_cast<const float*>(q), q_ts, idx, Hq, G,
                                 kfull, kmask, qscale, dst);
  else hipLaunchKernelGGL(k_query_rows<uint16_t>, dim3(m), dim3(256), 0, st, static_cast<const uint16_t*>(q), q_ts, idx, Hq, G,
                          kfull, kmask, qscale, dst);
  return done(hipPeekAtLastError() == hipSuccess ? 0 : -1, "frmq_prep_q");
}

int frmq_attn(const void* q16, const uint8_t* pool, long long page_stride, const int* bt, long long bt_stride,
              const int* tiles, const int* items, int nitems, int Hkv, int G, int shift, int konly, float* opart,
              float* ml, int kernel, int Dh, void* stream, int kmin) {
  if (nitems <= 0) return 0;
  if (Dh != D && Dh != 256) return bad(-4, "frmq_attn: head dim 128 or 256");
  const int rows = Dh == 256 ? 128 : kernel == 1 ? 64 : kernel == 4 ? 256 : 128;     // head dim 256: one kernel, 128 rows
  if (G < 1 || G > rows) return bad(-3, "frmq_attn: G out of range");
  if (kernel < 1 || kernel > 4) return bad(-2, "frmq_attn: kernel must be 1, 2, 3 or 4");
  Params p{};
  p.q = static_cast<const uint16_t*>(q16); p.pool = pool; p.page_stride = page_stride; p.bt = bt; p.bt_stride = bt_stride;
  p.tiles = tiles; p.items = items; p.Hkv = Hkv; p.G = G; p.shift = shift; p.kmin = kmin; p.opart = opart; p.ml = ml;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool k2 = konly & 1, i2 = konly & 2;
  int rc;
  if (Dh == 256) {
    rc = wide_attn_launch(p, nitems, konly, st);
  } else if (rows == 256) {
    rc = i2 ? (k2 ? launch_mq8<QM_ASYM2, true>(p, nitems, st) : launch_mq8<QM_ASYM2, false>(p, nitems, st))
            : (k2 ? launch_mq8<QM_ASYM4, true>(p, nitems, st) : launch_mq8<QM_ASYM4, false>(p, nitems, st));
  } else if (rows == 64) {
    rc = i2 ? (k2 ? launch_mq<QM_ASYM2, true, 2>(p, nitems, st) : launch_mq<QM_ASYM2, false, 2>(p, nitems, st))
            : (k2 ? launch_mq<QM_ASYM4, true, 2>(p, nitems, st) : launch_mq<QM_ASYM4, false, 2>(p, nitems, st));
  } else {
    rc = i2 ? (k2 ? launch_mq<QM_ASYM2, true, 4>(p, nitems, st) : launch_mq<QM_ASYM2, false, 4>(p, nitems, st))
            : (k2 ? launch_mq<QM_ASYM4, true, 4>(p, nitems, st) : launch_mq<QM_ASYM4, false, 4>(p, nitems, st));
  }
  return done(rc, "frmq_attn");
}

int frmq_merge(const int* tiles, int ntiles, const float* opart, const float* ml, int Hkv, int G, int rows, void* out,
               long long o_ts, int out_fp32, float* lse, long long lse_ts, int Dh, void* stream) {
  if (ntiles <= 0) return 0;
  if (Dh != D && Dh != 256) return bad(-4, "frmq_merge: head dim 128 or 256");
  const dim3 grid(ntiles, Hkv, (rows + 4 * FOLD_ROWS - 1) / (4 * FOLD_ROWS));      // four wavefronts x FOLD_ROWS rows per workgroup
  hipStream_t st = static_cast<hipStream_t>(stream);
  const auto kern = Dh == 256 ? (out_fp32 ? k_fold_items<true, 4> : k_fold_items<false, 4>)
                              : (out_fp32 ? k_fold_items<true, 2> : k_fold_items<false, 2>);
  hipLaunchKernelGGL(kern, grid, dim3(256), 0, st, tiles, opart, ml, Hkv, G, rows, out, o_ts, lse, lse_ts);
  return done(hipPeekAtLastError() == hipSuccess ? 0 : -1, "frmq_merge");
}

int frmq_win_gather(const long long* map, int nk, const void* sinkb, const void* preb, const void* kch, long long k_ts,
                    const void* vch, long long v_ts, int Hkv, void* kw, void* vw, int Dh, void* stream) {
  if (nk <= 0) return 0;
  if (Dh != D && Dh != 256) return bad(-4, "frmq_win_gather: head dim 128 or 256");
  const int pieces = Hkv * Dh / 8;                         // 16-byte pieces of one K (or V) row
  const long long total = static_cast<long long>(nk) * pieces;
  hipLaunchKernelGGL(k_collect_rows, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), map, nk, static_cast<const uint4*>(sinkb), static_cast<const uint4*>(preb),
                     static_cast<const uint16_t*>(kch), k_ts, static_cast<const uint16_t*>(vch), v_ts, pieces,
                     static_cast<uint4*>(kw), static_cast<uint4*>(vw));
  return done(hipPeekAtLastError() == hipSuccess ? 0 : -1, "frmq_win_gather");
}

int frmq_bf_merge(int m, int Hq, int Hkv, const void* q, long long q_ts, const long long* idx, const float* o_p,
                  const float* lse_p, const void* o_w, const float* lse_w, const void* sk, const long long* row_req,
                  const long long* row_pos, const long long* sk_len, int S, int W, float scale, void* out, long long o_ts,
                  int Dh, void* stream) {
  if (m <= 0) return 0;
  if (Dh != D && Dh != 256) return bad(-4, "frmq_bf_merge: head dim 128 or 256");
  if (sk != nullptr && S > 64) return bad(-5, "frmq_bf_merge: at most 64 sink tokens");
  using U = uint16_t;
  const auto kern = Dh == 256 ? k_mix_parts<4> : k_mix_parts<2>;
  hipLaunchKernelGGL(kern, dim3(m, (Hq + 3) / 4), dim3(256), 0, static_cast<hipStream_t>(stream), m, Hq, Hkv,
                     static_cast<const U*>(q), q_ts, idx, o_p, lse_p, static_cast<const U*>(o_w), lse_w,
                     static_cast<const U*>(sk), row_req, row_pos, sk_len, S, W, scale, static_cast<U*>(out), o_ts);
  return done(hipPeekAtLastError() == hipSuccess ? 0 : -1, "frmq_bf_merge");
}

}  // extern "C"
