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
#include "decode_tiles.hpp"

// FLAGROT_STRICT_MERGE=1 (a build flag: `FLAGROT_STRICT_MERGE=1 python -m flagrot_releaser_amd.build kernels`) gives the
// split-merge ticket the orders the HIP memory model asks for -- an agent-scope release on the ticket, an agent-scope
// acquire in the last arriver -- instead of relying on what write-through stores and read-through loads do on gfx950.
// Same results; each workgroup then pays a write-back and an invalidate of its XCD's L2.
#ifndef FLAGROT_STRICT_MERGE
#define FLAGROT_STRICT_MERGE 0
#endif

namespace fr {
using namespace dec;
namespace {
constexpr bool STRICT_MERGE = FLAGROT_STRICT_MERGE != 0;

template <int QM, bool K2, int P, int NW>
__global__ void __launch_bounds__(64 * NW, 4) k_decode(const DecodeParams p, int ntile, int nparts) {
  using L = Lay<QM, P>;
  __shared__ Smem<QM, NW> S;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int kvh = blockIdx.x / ntile, tile = blockIdx.x % ntile;
  // Workgroups are dispatched in linear order and the CU's arbiter favours the older wavefronts: the splits of one
  // sequence are spread over the whole dispatch order (split slowest) so that every sequence gets the same mix.
  int lin = blockIdx.z * gridDim.y + blockIdx.y;
  if (ntile > 1 && (p.Hkv * static_cast<int>(gridDim.y * gridDim.z)) % 8 == 0) {
    // Workgroups go to the 8 XCDs round robin in dispatch order and each XCD has its own L2.  The q tiles of one (KV
    // head, split, sequence) read the same pages: they are made neighbours on ONE XCD (dispatch positions 8 apart), so
    // that the second reader finds the first one's lines in that L2 -- whoever runs ahead waits for HBM, whoever
    // follows catches up.
    const int pos = blockIdx.x + gridDim.x * lin;
    const int slot = pos >> 3, t3 = (slot / ntile) * 8 + (pos & 7);
    tile = slot % ntile;
    kvh = t3 % p.Hkv;
    lin = t3 / p.Hkv;
  }
  // Where the body workgroups of a sequence draw from one shared range, the BF16 rows' workgroups (the last split) go
  // first in dispatch order: short ones that start with the launch instead of trailing it, and a body workgroup that
  // starts later for it just draws what is left.  (With fixed ranges per split a late start is a late end: there the
  // body goes first; measured both ways.)
  const int nsp = static_cast<int>(gridDim.y * gridDim.z) / p.B;
  int split = lin / p.B;
  if (p.tail != nullptr && p.dyn != 0) split = split == 0 ? nsp - 1 : split - 1;
  const int b = lin % p.B;
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
  // q tiles per counter slot: always 1.  The value is hidden from the compiler on purpose: folded in as a constant it
  // turns the final merge into straight-line code, the register allocation of the page loop changes with it, and the
  // loops of two formats spill (a reload from scratch waits for every page fetch in flight).
  int tpc = 1;
  asm volatile("" : "+s"(tpc));
  int* const ctr = p.counter + (static_cast<long long>(b) * p.Hkv + kvh) * (ntile / tpc) + tile / tpc;
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
      // (their tokens are masked).  The quad's entries come from LDS in ONE read (lane k < PPQ takes the k-th, the other
      // lanes repeat them); past the cached window they are read from memory.
      auto chunks_of = [&](int quad, const uint8_t* (&ch)[QB]) {
        const int i = min(PPQ * quad + (lane & (PPQ - 1)), npg - 1);
        int entry = S.btc[min(i, BT_CACHE - 1)];
        // (the value is made opaque here so that this stays an LDS read of its own: merged with the memory path below
        // into one load through a selected pointer it becomes a flat access, and a flat access is awaited together
        // with every fetch in flight -- the value loads of this quad, and whatever of the next keys was requested)
        asm volatile("" : "+v"(entry));
        if (__builtin_expect(PPQ * quad + PPQ > BT_CACHE, 0)) {
          if (i >= BT_CACHE) entry = bt[pg0 + i];
          asm volatile("" : "+v"(entry));      // awaited inside the branch: after the join nothing of it is pending
        }
#pragma unroll
        for (int k = 0; k < PPQ; ++k) {
          const int page = __builtin_amdgcn_readlane(entry, k);
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
        const bool wide = softmax_phase<QM>(S, st, cur, sc, valid, qs20, sc0, lane, wave, [&](float (&raw)[QB]) {
          // (the quad's page ids are read again, behind an opaque value, and each chunk address is formed when its
          // block's turn comes: kept from the loads they would occupy eight scalar registers across the key phase)
          int quad = __builtin_amdgcn_readfirstlane(qi);
          asm volatile("" : "+s"(quad));
          const int i = min(PPQ * quad + (lane & (PPQ - 1)), npg - 1);
          int entry = i < BT_CACHE ? S.btc[min(i, BT_CACHE - 1)] : bt[pg0 + i];
          rescore_fine<QM, K2, P, 1>(S, cur.vs, lane, raw, [&](int blk) {
            const int page = __builtin_amdgcn_readlane(entry, P == 16 ? blk : blk >> 1);
            return (const uint8_t*)(pool + (static_cast<long long>(page) * p.Hkv + kvh) * L::CHUNK);
          });
        });
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
        value_phase<QM>(S, st, vr, lane, wave, wide);
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
    // head x = lane >> 4 lives in a row of 16 lanes.  Every wavefront leaves its maxima, its sums and its outputs
    // relative to its OWN maxima (its strips are dead: the outputs take their place); the output threads scale while
    // they add -- one barrier and one LDS round trip between the last quad and the result.
    const float lsum = row_sum16(st.l * unfold);
    if ((lane & 15) == 0) { S.m[wave][lane >> 4] = st.m; S.l[wave][lane >> 4] = lsum; }
    {
      const int kc = lane >> 4;      // the lane's four entry rows: 4 kc + r
      float* o = S.o(wave, hl);
#pragma unroll
      for (int y = 0; y < 2; ++y) {
        // entry e = 16 (gl & 1) + 4 kc + r, word sub = 2 (gl >> 1) + y: dim 64 (sub >> 1) + 16 (e >> 3) + 8 (sub & 1) + (e & 7)
        const int d = 32 * gl + 16 * (kc >> 1) + 8 * y + 4 * (kc & 1);
        *reinterpret_cast<float4*>(o + d) = make_float4(st.ot[y][0], st.ot[y][1], st.ot[y][2], st.ot[y][3]);
      }
    }
    if (p.fuse_tail && split == 0) {      // uniform over the workgroup
      // The BF16 rows of the sequence, this wavefront's share, folded into what it has just left in LDS (the first
      // split's workgroup takes them): a workgroup of their own costs its whole life -- arguments, rows, epilogue,
      // partial, ticket, merge: 10 us behind the 43-53 us of the body at B = 32 x 8 k -- where these rows are a few
      // hundred KB per sequence.
      // (more rows per step -- nine, so that 144 rows are one step of 16 wavefronts -- measured no better: 62.1 against
      // 60.4 us)
      float m[4], l[4], o[4][2];
      tail_partial<NW>(p, b, kvh, tile, S.tailw[wave], m, l, o);
      // static formats merge in the stored basis: the rows' share is rotated on the groups the writer rotated
      if constexpr (!K2) {
        if (p.vmask != nullptr) tail_to_stored_basis(o, p.vmask[kvh * 4 + (lane >> 4)] != 0, lane);
      }
      wave_lds_sync();
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        const float mp = S.m[wave][h], lp = S.l[wave][h];
        float2* slot = reinterpret_cast<float2*>(S.o(wave, h)) + lane;
        const float2 op = *slot;
        const float top = fmaxf(mp, m[h]);
        const float fp = mp == -INFINITY ? 0.f : fexp2(mp - top), ft = m[h] == -INFINITY ? 0.f : fexp2(m[h] - top);
        *slot = make_float2(op.x * fp + o[h][0] * ft, op.y * fp + o[h][1] * ft);
        wave_lds_sync();      // every lane has read the pair before lane 0 replaces it
        if (lane == 0) { S.m[wave][h] = top; S.l[wave][h] = lp * fp + l[h] * ft; }
      }
    }
  } else {
    float m[4], l[4], o[4][2];
    tail_partial<NW>(p, b, kvh, tile, S.tailw[wave], m, l, o);
    if (lane < 4) { S.m[wave][lane] = pick4(m[0], m[1], m[2], m[3], lane); S.l[wave][lane] = pick4(l[0], l[1], l[2], l[3], lane); }
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      float* so = S.o(wave, h);
      so[2 * lane] = o[h][0];
      so[2 * lane + 1] = o[h][1];
    }
  }
  __syncthreads();
  // ---- workgroup partial: (o[4][128] relative to M, M, L); thread = (head, 2 dims) for the first 4 wavefronts
  float po[2] = {0.f, 0.f}, pm = -INFINITY, pl = 0.f;
  const int oh = wave & 3;           // head of this thread's two outputs
  if (act) {
    // lane w holds wavefront w's maximum and sum of head oh: the workgroup's maximum, every wavefront's factor
    // 2^(m_w - M) and the scaled sum come from two row reductions
    const float mw = lane < NW ? S.m[lane][oh] : -INFINITY;
    const float lw = lane < NW ? S.l[lane][oh] : 0.f;
    pm = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, row_max16(mw))));
    const float fw = mw == -INFINITY ? 0.f : fexp2(mw - pm);
    pl = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, row_sum16(fw * lw))));
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float f = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, fw), w));
      const float2 v = *reinterpret_cast<const float2*>(S.o(w, oh) + 2 * lane);
      po[0] += f * v.x; po[1] += f * v.y;
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
      const int prev = __hip_atomic_fetch_add(ctr, dyn ? DRAW_MASK + 1 : 1, STRICT_MERGE ? __ATOMIC_RELEASE : __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
      S.last = (dyn ? static_cast<int>(static_cast<unsigned>(prev) >> DRAW_BITS) : prev) == tpc * nparts - 1;
      if (S.last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!S.last) return;
    if constexpr (STRICT_MERGE) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    else __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
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
      merge_parts(p.mlpart, p.opart, base, nparts, oh, lane, M, Lsum, o0, o1);
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
  const int nparts = p.nsplit + ((p.tail != nullptr && !p.fuse_tail) ? 1 : 0);
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

}  // namespace

int decode_launch(int fmt, const DecodeParams& p, hipStream_t st) {
  return p.tile8 ? decode8_launch(fmt, p, st) : decode_dispatch(fmt, p, st);
}
int decode_waves(int chunk_tokens) { return waves_for(chunk_tokens); }
int decode_big_chunk() {      // FLAGROT_BIG_CHUNK overrides (experiments)
  static const int v = getenv("FLAGROT_BIG_CHUNK") != nullptr ? atoi(getenv("FLAGROT_BIG_CHUNK")) : BIG_CHUNK;
  return v;
}

}  // namespace fr
