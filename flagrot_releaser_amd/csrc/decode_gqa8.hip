// Paged split-K GQA decode attention over FlagRot INT4 / INT2 pages for gfx950 (wave64): tiles of 8 query heads.
//
// GQA groups of 5 .. 8 query heads per KV head (variant GEN | GT8 of fr_v2_attn; the reference's GT = 8 kernels,
// kernels/csrc/attn_decode_v2g.cuh:5-10).  One workgroup serves all 8 heads of a (KV head, split, sequence): every
// quad of pages is fetched and unpacked ONCE and multiplied with the query operands of both 4-head halves (key phase)
// and with both halves' p * V-scale strip rows (value phase).  The launch shapes, the page loop (quads drawn from a
// counter, block table in LDS, next keys in flight during the value phase), the single-barrier wave merge, the split
// merge with its ticket and the BF16 rows' extra split are those of decode.hip; the phases are the *8 templates of
// decode_tiles.hpp.  Two sets of accumulators, softmax states and score registers need up to 168 registers per lane:
// three wavefronts per SIMD (large workgroup: 12 wavefronts) instead of four.  Partials, outputs and merges are per
// 4-head half (slot (tile * 2 + half) * nparts + split): the workspace layout a caller sizes for tiles of 8.
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

constexpr int NT = 2;             // 4-head halves of a tile
// Static formats whose unpacking needs the most registers (sign-magnitude INT4; INT2 with 32-token pages) get two
// wavefronts per SIMD instead of three, so that no page loop spills.
template <int QM, bool K2, int P> constexpr int MINW8 = (!K2 && (QM == QM_SYM4 || (QM == QM_ASYM2 && P == 32))) ? 2 : 3;

template <int QM, bool K2, int P, int NW>
__global__ void __launch_bounds__(64 * NW, (MINW8<QM, K2, P>)) k_decode8(const DecodeParams p, int ntile, int nparts) {
  using L = Lay<QM, P>;
  __shared__ Smem8<QM, NW> S;
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
  constexpr int SPEC = (BT_CACHE + 64 * NW - 1) / (64 * NW);      // entries per thread
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
  // partials of the workgroup's 4-head halves: slots (tile * NT + half) * nparts + split of the (sequence, KV head)
  const long long part0 = ((static_cast<long long>(b) * p.Hkv + kvh) * ntile + tile) * NT * nparts + split;
  const bool act = wave < 4;      // the 256 threads that own the 4 x 128 outputs of a half

  // the (sequence, KV head, q tile)'s counter slot: merge ticket, and in the dynamic mode the quad draw counter
  int* const ctr = p.counter + (static_cast<long long>(b) * p.Hkv + kvh) * ntile + tile;
  if (!is_tail) {
    const int lo = dyn ? min(p.kv_start, len) : max(split * p.chunk, min(p.kv_start, len));
    const int hi = dyn ? len : min(len, (split + 1) * p.chunk);
    WaveState8 st;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      st.m[t] = -INFINITY; st.l[t] = 0.f;
      st.z[t][0] = st.z[t][1] = 0.f;
      st.ot[t][0] = st.ot[t][1] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  
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
      constexpr int RSTR = PB8_RSTRIDE;
      for (int i = threadIdx.x; i < NW * Strip8<QM>::ROWS; i += 64 * NW)
        (reinterpret_cast<uint4*>(S.pb(i / Strip8<QM>::ROWS)) + (i % Strip8<QM>::ROWS) * RSTR)[RSTR - 1] = make_uint4(0u, 0u, 0u, 0u);
      q_prologue8<QM, K2, NW>(S, p, b, kvh, tile);
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
        float sc[2][QB];
        key_phase8<QM, K2>(S, cur, lane, sc);
        const bool wide = softmax_phase8<QM>(S, st, cur, sc, valid, qs20, sc0, lane, wave, [&](float (&raw)[2 * QB]) {
          // (as in k_decode: page ids read again behind an opaque value, a chunk address per block when its turn comes)
          int quad = __builtin_amdgcn_readfirstlane(qi);
          asm volatile("" : "+s"(quad));
          const int i = min(PPQ * quad + (lane & (PPQ - 1)), npg - 1);
          int entry = i < BT_CACHE ? S.btc[min(i, BT_CACHE - 1)] : bt[pg0 + i];
          rescore_fine<QM, K2, P, 2>(S, cur.vs, lane, raw, [&](int blk) {
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
        value_phase8<QM>(S, st, vr, lane, wave, wide);
        wave_lds_sync();
        qi = qn;
      }
      // the last draw is never used: it must have reached the counter before this workgroup takes its ticket (the
      // last arriver clears the word)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    // ---- fold the wave: zero-point sums per (head, group) through the wave's strip, codes -> values:
    //      2^24 (acc - sum p' zero point)
    const float unfold = (lane & 1) ? static_cast<float>(1 << UnpackD<QM>::SH) : 1.f;   // lane & 1 = token parity
    const int hl = lane & 3, gl = (lane >> 2) & 3;      // the lane's accumulator column: head hl, group gl
    // the same per half of the tile: zero-point sums [half][head][group] through the strip, then maxima, sums, outputs
    if constexpr (QM != QM_SYM4) {
      float* zs = reinterpret_cast<float*>(S.pb(wave));
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        float z0 = st.z[t][0], z1 = st.z[t][1];
        z0 += swz_xor<8>(z0); z1 += swz_xor<8>(z1);
        z0 += swz_xor<16>(z0); z1 += swz_xor<16>(z1);
        z0 += xor32(z0); z1 += xor32(z1);
        if (lane < 8) { zs[16 * t + (2 * (lane & 1)) * 4 + (lane >> 1)] = z0; zs[16 * t + (2 * (lane & 1) + 1) * 4 + (lane >> 1)] = z1; }
      }
      wave_lds_sync();
    }
    float zg[2] = {0.f, 0.f};
    if constexpr (QM != QM_SYM4) {
      zg[0] = reinterpret_cast<const float*>(S.pb(wave))[hl * 4 + gl];
      zg[1] = reinterpret_cast<const float*>(S.pb(wave))[16 + hl * 4 + gl];
      wave_lds_sync();               // the outputs below overwrite the sums
    }
    const int kc = lane >> 4;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if constexpr (QM == QM_ASYM2) st.ot[t][1] *= 0.0625f;
      const float lsum = row_sum16(st.l[t] * unfold);
      if ((lane & 15) == 0) { S.m[wave][4 * t + (lane >> 4)] = st.m[t]; S.l[wave][4 * t + (lane >> 4)] = lsum; }
      float* o = S.o(wave, 4 * t + hl);
#pragma unroll
      for (int y = 0; y < 2; ++y) {
        const int d = 32 * gl + 16 * (kc >> 1) + 8 * y + 4 * (kc & 1);
        *reinterpret_cast<float4*>(o + d) = make_float4((st.ot[t][y][0] - zg[t]) * 16777216.f, (st.ot[t][y][1] - zg[t]) * 16777216.f,
                                                        (st.ot[t][y][2] - zg[t]) * 16777216.f, (st.ot[t][y][3] - zg[t]) * 16777216.f);
      }
    }
    if (p.fuse_tail && split == 0) {      // uniform over the workgroup: as in k_decode, half by half
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        float m[4], l[4], o[4][2];
        tail_partial<NW>(p, b, kvh, tile * NT + t, S.tailw[wave], m, l, o);
        // static formats merge in the stored basis: the rows' share is rotated on the groups the writer rotated
        if constexpr (!K2) {
          if (p.vmask != nullptr) tail_to_stored_basis(o, p.vmask[kvh * 4 + (lane >> 4)] != 0, lane);
        }
        wave_lds_sync();
#pragma unroll
        for (int h = 0; h < 4; ++h) {
          const float mp = S.m[wave][4 * t + h], lp = S.l[wave][4 * t + h];
          float2* slot = reinterpret_cast<float2*>(S.o(wave, 4 * t + h)) + lane;
          const float2 op = *slot;
          const float top = fmaxf(mp, m[h]);
          const float fp = mp == -INFINITY ? 0.f : fexp2(mp - top), ft = m[h] == -INFINITY ? 0.f : fexp2(m[h] - top);
          *slot = make_float2(op.x * fp + o[h][0] * ft, op.y * fp + o[h][1] * ft);
          wave_lds_sync();
          if (lane == 0) { S.m[wave][4 * t + h] = top; S.l[wave][4 * t + h] = lp * fp + l[h] * ft; }
        }
      }
    }
  } else {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float m[4], l[4], o[4][2];
      tail_partial<NW>(p, b, kvh, tile * NT + t, S.tailw[wave], m, l, o);
      if (lane < 4) { S.m[wave][4 * t + lane] = pick4(m[0], m[1], m[2], m[3], lane); S.l[wave][4 * t + lane] = pick4(l[0], l[1], l[2], l[3], lane); }
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        float* so = S.o(wave, 4 * t + h);
        so[2 * lane] = o[h][0];
        so[2 * lane + 1] = o[h][1];
      }
    }
  }
  __syncthreads();
  // ---- workgroup partial per half: (o[4][128] relative to M, M, L); thread = (head, 2 dims) for the first 4 wavefronts
  float po[NT][2], pm[NT], pl[NT];
  const int oh = wave & 3;           // head (within a half) of this thread's two outputs
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    po[t][0] = po[t][1] = 0.f; pm[t] = -INFINITY; pl[t] = 0.f;
    if (act) {
      // lane w holds wavefront w's maximum and sum of the head: the workgroup's maximum, every wavefront's factor
      // 2^(m_w - M) and the scaled sum come from two row reductions
      const float mw = lane < NW ? S.m[lane][4 * t + oh] : -INFINITY;
      const float lw = lane < NW ? S.l[lane][4 * t + oh] : 0.f;
      pm[t] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, row_max16(mw))));
      const float fw = mw == -INFINITY ? 0.f : fexp2(mw - pm[t]);
      pl[t] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, row_sum16(fw * lw))));
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float f = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, fw), w));
        const float2 v = *reinterpret_cast<const float2*>(S.o(w, 4 * t + oh) + 2 * lane);
        po[t][0] += f * v.x; po[t][1] += f * v.y;
      }
    }
  }
  // a value group's 32 outputs of a head rotated back (static formats): through the head's row in LDS
  auto unrotate = [&](float (&v2)[2]) {
    __syncthreads();
    if (act) { S.o(0, oh)[2 * lane] = v2[0]; S.o(0, oh)[2 * lane + 1] = v2[1]; }
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
          v2[e] = a * kC32;
        }
      }
    }
  };
  if (is_tail && p.vmask != nullptr) {  // the merged sum is rotated back once: bring the tail into the stored basis
#pragma unroll
    for (int t = 0; t < NT; ++t) unrotate(po[t]);
  }
  if (nparts > 1) {
    // Partials cross workgroups (and XCDs, each with its own L2) through device-scope relaxed atomic stores / loads,
    // which are write-through / read-through; a device-scope fence here would write back and invalidate the whole
    // L2 once per workgroup.  Order: every storing wavefront waits until its stores are acknowledged (an explicit
    // wait on the vector memory counter, which counts stores on this target: a workgroup-scope fence emits no such
    // wait), barrier, ticket; the last arriver reads (device-scope loads) after its ticket has returned.
    if (act) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const long long part_id = part0 + static_cast<long long>(t) * nparts;
        float* op = p.opart + part_id * 512 + oh * 128 + 2 * lane;
        __hip_atomic_store(op, po[t][0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(op + 1, po[t][1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (lane == 0) {
          __hip_atomic_store(p.mlpart + part_id * 8 + 2 * oh, pm[t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(p.mlpart + part_id * 8 + 2 * oh + 1, pl[t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // this wavefront's partial stores have been acknowledged
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) {    // every draw of this workgroup precedes its ticket: the last arriver may clear the slot
      const int prev = __hip_atomic_fetch_add(ctr, dyn ? DRAW_MASK + 1 : 1, STRICT_MERGE ? __ATOMIC_RELEASE : __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
      S.last = (dyn ? static_cast<int>(static_cast<unsigned>(prev) >> DRAW_BITS) : prev) == nparts - 1;
      if (S.last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!S.last) return;
    if constexpr (STRICT_MERGE) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    else __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  } else if (dyn && threadIdx.x == 0) {
    __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // the only workgroup of the slot
  }
  // ---- final merge (last arriving workgroup, or the only one), half by half
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    float M = pm[t], Lsum = pl[t], o0 = po[t][0], o1 = po[t][1];
    if (nparts > 1 && act) {
      const long long base = part0 - split + static_cast<long long>(t) * nparts;
      merge_parts(p.mlpart, p.opart, base, nparts, oh, lane, M, Lsum, o0, o1);
    }
    const float inv = Lsum > 0.f ? 1.f / Lsum : 0.f;
    float r[2] = {o0 * inv, o1 * inv};
    if (p.vmask != nullptr) unrotate(r);
    const int hq = (tile * NT + t) * 4 + oh;
    if (act && hq < p.gqa) {
      uint16_t* orow = static_cast<uint16_t*>(p.out) + static_cast<long long>(b) * p.o_bs +
                       (static_cast<long long>(kvh) * p.gqa + hq) * 128 + 2 * lane;
      *reinterpret_cast<uint32_t*>(orow) = bf16_rn(r[0]) | (bf16_rn(r[1]) << 16);
    }
  }
}

// Wavefronts per workgroup: 4, or one large workgroup that fills a CU's register file: 12 (three per SIMD), 8 where a
// format runs two per SIMD.
template <int QM, bool K2, int P>
void launch_shape(const DecodeParams& p, dim3 grid, int ntile, int nparts, hipStream_t st) {
  constexpr int NWB = 4 * MINW8<QM, K2, P>;
  if (p.wg_waves > 4) hipLaunchKernelGGL((k_decode8<QM, K2, P, NWB>), grid, dim3(64 * NWB), 0, st, p, ntile, nparts);
  else hipLaunchKernelGGL((k_decode8<QM, K2, P, 4>), grid, dim3(256), 0, st, p, ntile, nparts);
}

template <int QM, bool K2>
int launch_qm(const DecodeParams& p, hipStream_t st) {
  if (p.page != 16 && p.page != 32) return -5;
  const int ntile = (p.gqa + 7) / 8;
  const int nparts = p.nsplit + ((p.tail != nullptr && !p.fuse_tail) ? 1 : 0);
  if (nparts <= 0 || p.B <= 0) return 0;
  dim3 grid(p.Hkv * ntile, nparts, p.B);
  if (p.page == 32) launch_shape<QM, K2, 32>(p, grid, ntile, nparts, st);
  else launch_shape<QM, K2, 16>(p, grid, ntile, nparts, st);
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

int decode8_launch(int fmt, const DecodeParams& p, hipStream_t st) {
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

}  // namespace fr
