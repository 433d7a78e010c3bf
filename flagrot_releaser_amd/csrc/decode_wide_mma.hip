// Paged decode attention for 256-d heads on the matrix pipe (`variant | 4096` of fr_v2_attn / fr_cb_attn; reference
// kernels/csrc/attn_decode_v2g.cuh:11-25, 276): the body splits.  The chunk of a (page, KV head) is two 128-d half
// chunks, each in the 128-d layout (half s = dims [128 s, 128 s + 128), virtual head 2 kvh + s of the pool), so a wave
// iteration is the 128-d kernel's (decode_tiles.hpp) worked through the head in halves:
//   keys     the quad's scores are the sum of the two halves' score products; per half the query operand tables of
//            the 128-d kernel (identity / H32 per group / whole head = H256 here, value + remainder, zero-point sums),
//            made once per workgroup; the tokens' whole-head flags sit in half 0's value scale words;
//   softmax  once per quad;
//   values   per half: p * V-scale strips of that half's four groups, then its value products into its own accumulators.
// One workgroup of 4 wavefronts per (KV head x q tile of 4 heads, split, sequence), wavefront = head in the prologue;
// the wavefronts draw quads of 64 tokens from a counter in LDS.  Partials go out in the format of k_wide_parts
// (decode_wide.hip: o [4][256] relative to the part's maxima, (maximum, sum) per head), whose merge kernel serves
// both; the BF16 sink / window rows are one more split of this grid (plain fp32, a wavefront per row).
#include <cstddef>

#include "decode_tiles.hpp"

namespace fr {
using namespace dec;
namespace {

constexpr int NWW = 4;

template <int QM> struct WideMma {
  static constexpr int STRIP_BYTES = Strip<QM>::BYTES;
  alignas(16) uint4 qhi[2][4][64];                   // [half][group][lane of the matrix instruction]: as Smem::qhi
  alignas(16) uint4 qlo[2][4][64];
  alignas(16) uint4 qz[2][4][64];
  alignas(16) uint8_t work[NWW * (STRIP_BYTES > 2048 ? STRIP_BYTES : 2048)];
  float m[NWW][4], l[NWW][4];
  int next;
  DEVI float* o(int w, int h) { return reinterpret_cast<float*>(work) + (w * 4 + h) * 128; }
};
// what the phases of decode_tiles.hpp see of it: one half's operand tables, the wave strips
template <int QM> struct HalfView {
  const uint4 (*qhi)[64];
  const uint4 (*qlo)[64];
  const uint4 (*qz)[64];
  uint8_t* work;
  DEVI uint8_t* pb(int w) const { return work + w * Strip<QM>::BYTES; }
  DEVI uint8_t* zb(int w) const { return work + w * Strip<QM>::BYTES + Strip<QM>::PB_BYTES; }
};


// The 128-d prologue per half (decode_tiles.hpp q_prologue): wavefront = head, half wave 0 writes the rows of variants
// 0 (identity, or the static kmask rotation) and 1 (H32), half wave 1 those of variant 2 (H256) and the idle row 3.
template <int QM, bool K2>
DEVI void q_prologue_wide(WideMma<QM>& S, const DecodeParams& p, int b, int kvh, int tile) {
  const int w = threadIdx.x >> 6, half = (threadIdx.x >> 5) & 1, l32 = threadIdx.x & 31;
  const int hq = tile * 4 + w;
  float x[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  if (hq < p.gqa) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const uint16_t* qr = static_cast<const uint16_t*>(p.q) + static_cast<long long>(b) * p.q_bs +
                           (static_cast<long long>(kvh) * p.gqa + hq) * 256 + 128 * s + 4 * l32;
      const uint2 raw = *reinterpret_cast<const uint2*>(qr);
      x[s][0] = bf16_lo(raw.x); x[s][1] = bf16_hi(raw.x); x[s][2] = bf16_lo(raw.y); x[s][3] = bf16_hi(raw.y);
    }
  }
  const int g = l32 >> 3, isB = (l32 >> 2) & 1, tg = l32 & 3;   // the lane's dims 128 s + 4 l32 + i: group, word half, quarter
  float y[2][4];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < 4; ++i) y[s][i] = x[s][i];
  if (half == 0) { fwht<32>(y[0], l32); fwht<32>(y[1], l32); } else h256(y, l32);
  const float beta = (isB ? static_cast<float>(1 << UnpackD<QM>::SH) : 1.f) * ((QM == QM_ASYM2 && (g & 1)) ? 16.f : 1.f);
#pragma unroll
  for (int s = 0; s < 2; ++s) {
#pragma unroll
    for (int vi = 0; vi < 2; ++vi) {
      const int var = 2 * half + vi;
      float v[4];
      bool live;
      if (K2) {
        live = var < 3;
        const uint32_t rot = var != 0 ? 0xFFFFFFFFu : 0u;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = __uint_as_float((__float_as_uint(y[s][i]) & rot) | (__float_as_uint(x[s][i]) & ~rot));
      } else {
        live = var == 0;
        const uint32_t rot = (p.kmask != nullptr && p.kmask[kvh * 8 + 4 * s + g] != 0) ? 0xFFFFFFFFu : 0u;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = __uint_as_float((__float_as_uint(y[s][i]) & rot) | (__float_as_uint(x[s][i]) & ~rot));
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
      uint32_t* dh = reinterpret_cast<uint32_t*>(&S.qhi[s][g][ln]);
      uint32_t* dl = reinterpret_cast<uint32_t*>(&S.qlo[s][g][ln]);
      dh[isB] = hb[0] | (hb[2] << 16); dh[2 + isB] = hb[1] | (hb[3] << 16);
      dl[isB] = lb[0] | (lb[2] << 16); dl[2 + isB] = lb[1] | (lb[3] << 16);
      if constexpr (QM != QM_SYM4) {
        qs += hx(qs, 1); qs += hx(qs, 2); qs += hx(qs, 4);
        if ((l32 & 7) == 0) {
          const _Float16 zh = static_cast<_Float16>(-qs);
          const _Float16 zl = static_cast<_Float16>(-qs - static_cast<float>(zh));
          const int sh = 16 * (g & 1);
          S.qz[s][g][m] = make_uint4(static_cast<uint32_t>(__builtin_bit_cast(uint16_t, zh)) << sh, 0u, 0u, 0u);
          S.qz[s][g][m + 16] = make_uint4(static_cast<uint32_t>(__builtin_bit_cast(uint16_t, zl)) << sh, 0u, 0u, 0u);
          S.qz[s][g][m + 32] = make_uint4(0u, 0u, 0u, 0u);
          S.qz[s][g][m + 48] = make_uint4(0u, 0u, 0u, 0u);
        }
      }
    }
  }
}

// The BF16 sink / window rows of one sequence (the split after the body splits): a wavefront takes every fourth row,
// lanes own 4 dims (lanes 0..31 half 0, 32..63 half 1), eight rows in flight; the wavefronts are merged through LDS and
// the partial leaves in the body splits' format.  Static formats merge in the stored basis: the rows' share is rotated
// on the vmask groups (H32 inside the eight lanes of a group).
template <int QM, bool K2>
DEVI void tail_split_wide(WideMma<QM>& S, const DecodeParams& p, int b, int kvh, int tile, float* __restrict__ op,
                          float* __restrict__ mlp) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = p.tail_len != nullptr ? p.tail_len[b] : 0;
  if (n <= 0) {                                       // uniform
    if (threadIdx.x < 4) { mlp[2 * threadIdx.x] = -INFINITY; mlp[2 * threadIdx.x + 1] = 0.f; }
    return;
  }
  const uint16_t* base = static_cast<const uint16_t*>(p.tail) + static_cast<long long>(p.tail_idx != nullptr ? p.tail_idx[b] : b) * p.tail_bs;
  float q[4][4], m[4], l[4], o[4][4];
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    const int hq = tile * 4 + h;
#pragma unroll
    for (int i = 0; i < 4; ++i) q[h][i] = o[h][i] = 0.f;
    if (hq < p.gqa) {
      const uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(p.q) + static_cast<long long>(b) * p.q_bs +
                                                        (static_cast<long long>(kvh) * p.gqa + hq) * 256 + 4 * lane);
      q[h][0] = bf16_lo(raw.x) * p.qscale; q[h][1] = bf16_hi(raw.x) * p.qscale;
      q[h][2] = bf16_lo(raw.y) * p.qscale; q[h][3] = bf16_hi(raw.y) * p.qscale;
    }
    m[h] = -INFINITY; l[h] = 0.f;
  }
  for (int tb = wave; tb < n; tb += 4 * 8) {
    uint2 kr[8], vr[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint16_t* row = base + static_cast<long long>(min(tb + 4 * i, n - 1)) * p.tail_ts;
      kr[i] = *reinterpret_cast<const uint2*>(row + kvh * 256 + 4 * lane);
      vr[i] = *reinterpret_cast<const uint2*>(row + (p.Hkv + kvh) * 256 + 4 * lane);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (tb + 4 * i >= n) break;
      const float k[4] = {bf16_lo(kr[i].x), bf16_hi(kr[i].x), bf16_lo(kr[i].y), bf16_hi(kr[i].y)};
      const float v[4] = {bf16_lo(vr[i].x), bf16_hi(vr[i].x), bf16_lo(vr[i].y), bf16_hi(vr[i].y)};
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        const float sc = wave_sum64(q[h][0] * k[0] + q[h][1] * k[1] + q[h][2] * k[2] + q[h][3] * k[3]);
        const float mn = fmaxf(m[h], sc);
        const float alpha = m[h] == -INFINITY ? 0.f : fexp2(m[h] - mn), pe = fexp2(sc - mn);
        l[h] = l[h] * alpha + pe;
#pragma unroll
        for (int c = 0; c < 4; ++c) o[h][c] = o[h][c] * alpha + pe * v[c];
        m[h] = mn;
      }
    }
  }
  if (lane < 4) S.m[wave][lane] = pick4(m[0], m[1], m[2], m[3], lane);
  __syncthreads();
  float Mwg[4];
  workgroup_max<NWW>(S, lane, Mwg);
  // [wave][head][256] fp32 = 16 KB in place of the operand tables (24 KB, contiguous), which this split never builds
  static_assert(sizeof(S.qhi) + sizeof(S.qlo) >= NWW * 4 * 256 * 4 && offsetof(WideMma<QM>, qlo) == sizeof(S.qhi), "merge buffer");
  float* buf = reinterpret_cast<float*>(&S.qhi[0][0][0]);
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    const float f = m[h] == -INFINITY ? 0.f : fexp2(m[h] - Mwg[h]);
    if (lane == 0) S.l[wave][h] = f * l[h];
    *reinterpret_cast<float4*>(buf + (wave * 4 + h) * 256 + 4 * lane) = make_float4(f * o[h][0], f * o[h][1], f * o[h][2], f * o[h][3]);
  }
  __syncthreads();
  {   // wavefront = head: sum over the wavefronts, rotate (static formats), store
    const int h = wave;
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int w = 0; w < NWW; ++w) {
      const float4 v = *reinterpret_cast<const float4*>(buf + (w * 4 + h) * 256 + 4 * lane);
      a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
    }
    if (!K2 && p.vmask != nullptr) {
      float y[4] = {a.x, a.y, a.z, a.w};
      fwht<32>(y, lane & 31);
      if (p.vmask[kvh * 8 + (lane >> 3)]) a = make_float4(y[0], y[1], y[2], y[3]);
    }
    *reinterpret_cast<float4*>(op + h * 256 + 4 * lane) = a;
    if (lane == 0) {
      mlp[2 * h] = pick4(Mwg[0], Mwg[1], Mwg[2], Mwg[3], h);
      mlp[2 * h + 1] = (S.l[0][h] + S.l[1][h]) + (S.l[2][h] + S.l[3][h]);
    }
  }
}

template <int QM, bool K2, int P>
__global__ void __launch_bounds__(64 * NWW, 2) k_wide_parts_mma(const DecodeParams p, int ntile, int nparts) {
  using L = Lay<QM, P>;
  constexpr int QB = QBLK<QM>, PPQ = 16 * QB / P;
  __shared__ WideMma<QM> S;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // Workgroups go to the 8 XCDs round robin in dispatch order, and each XCD has its own L2.  The q tiles of one (KV
  // head, split, sequence) read the same pages: they are made neighbours ON ONE XCD (dispatch positions 8 apart), so
  // that the second reader finds the first one's lines in that L2 -- whoever runs ahead waits for HBM, whoever follows
  // catches up.  (Needs the number of (KV head, split, sequence) triples to be a multiple of 8.)
  int kvh = blockIdx.x / ntile, tile = blockIdx.x % ntile, split = blockIdx.y, b = blockIdx.z;
  {
    const int triples = p.Hkv * nparts * p.B;
    if (ntile > 1 && triples % 8 == 0) {
      const int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
      const int slot = lin >> 3, t3 = (slot / ntile) * 8 + (lin & 7);
      tile = slot % ntile;
      kvh = t3 % p.Hkv; split = (t3 / p.Hkv) % nparts; b = t3 / (p.Hkv * nparts);
    }
  }
  const long long part_id = ((static_cast<long long>(b) * p.Hkv + kvh) * ntile + tile) * nparts + split;
  float* const op = p.opart + part_id * 4 * 256;
  float* const mlp = p.mlpart + part_id * 8;
  if (p.tail != nullptr && split == p.nsplit) {
    tail_split_wide<QM, K2>(S, p, b, kvh, tile, op, mlp);
    return;
  }
  const int len = p.seq_lens[b];
  const int lo = max(split * p.chunk, min(p.kv_start, len)), hi = min(len, (split + 1) * p.chunk);
  if (lo >= hi) {                                     // uniform: nothing of the range is visible
    if (threadIdx.x < 4) { mlp[2 * threadIdx.x] = -INFINITY; mlp[2 * threadIdx.x + 1] = 0.f; }
    return;
  }
  if (threadIdx.x == 0) S.next = NWW;
  // the pad entry of every strip row group: what the value phase reads for the columns of foreign groups
  for (int i = threadIdx.x; i < NWW * Strip<QM>::ROWS; i += 64 * NWW)
    (reinterpret_cast<uint4*>(S.work + (i / Strip<QM>::ROWS) * Strip<QM>::BYTES) + (i % Strip<QM>::ROWS) * PB_RSTRIDE)[16] = make_uint4(0u, 0u, 0u, 0u);
  q_prologue_wide<QM, K2>(S, p, b, kvh, tile);
  __syncthreads();
  const HalfView<QM> H0{S.qhi[0], S.qlo[0], S.qz[0], S.work}, H1{S.qhi[1], S.qlo[1], S.qz[1], S.work};

  const int pg0 = lo / P, pg1 = (hi + P - 1) / P, npg = pg1 - pg0, nquad = (npg + PPQ - 1) / PPQ;
  const int* bt = p.block_table + static_cast<long long>(b) * p.bt_stride;
  typedef const __attribute__((address_space(1))) uint8_t* gptr;
  const gptr pool = (gptr)p.pool;
  const KOffs<QM, P> koff = key_offsets<QM, P>(lane);
  const float sc0 = (lane & 1) ? -static_cast<float>(UnpackD<QM>::SH) : 0.f;
  const float qs20 = p.qscale * (16777216.f / QPRE);
  WaveState st0, st1;                                 // per half: accumulators and zero-point sums; m and l live in st0
  st0.m = -INFINITY; st0.l = 0.f;
  st0.z[0] = st0.z[1] = st1.z[0] = st1.z[1] = 0.f;
  st0.ot[0] = st0.ot[1] = st1.ot[0] = st1.ot[1] = f32x4{0.f, 0.f, 0.f, 0.f};
  st1.m = -INFINITY; st1.l = 0.f;

  // chunk addresses of a quad's blocks, half 0 (half 1: CHUNK further).  Pages past the range name its last page again.
  auto chunks_of = [&](int quad, const uint8_t* (&ch)[QB]) {
#pragma unroll
    for (int k = 0; k < PPQ; ++k) {
      const int page = __builtin_amdgcn_readfirstlane(bt[pg0 + min(PPQ * quad + k, npg - 1)]);
      const uint8_t* c = (const uint8_t*)(pool + (static_cast<long long>(page) * (2 * p.Hkv) + 2 * kvh) * L::CHUNK);
      if constexpr (P == 16) ch[k] = c;
      else { ch[2 * k] = c; ch[2 * k + 1] = c; }
    }
  };
  int qi = wave;
  const uint8_t* ch0[QB];
  const uint8_t* ch1[QB];
  KRegs<QM> k0, k1;
  if (qi < nquad) {
    chunks_of(qi, ch0);
#pragma unroll
    for (int k = 0; k < QB; ++k) ch1[k] = ch0[k] + L::CHUNK;
    load_k<QM, P, false>(k0, ch0, koff);
    load_k<QM, P, false>(k1, ch1, koff);
  }
  while (qi < nquad) {
    int take = 0;
    if (lane == 0) take = atomicAdd(&S.next, 1);
    VRegs<QM> v0, v1;                                  // this quad's V^T entries: in flight during the key phase
    load_v<QM, P, false>(v0, ch0, lane);
    load_v<QM, P, false>(v1, ch1, lane);
    bool valid[QB];
    {
      const int tok0 = (pg0 + PPQ * qi) * P + (lane & 15);
#pragma unroll
      for (int k = 0; k < QB; ++k) valid[k] = tok0 + 16 * k >= lo && tok0 + 16 * k < hi;
    }
    // ---- scores: both halves into one sum; the whole-head flags come with half 0
    bool full[QB];
    whole_head_flags<QM, K2>(k0, lane, full);
    float sc[QB];
#pragma unroll
    for (int k = 0; k < QB; ++k) sc[k] = 0.f;
    key_scores<QM, K2>(H0, k0, lane, full, sc);
    key_scores<QM, K2>(H1, k1, lane, full, sc);
    // ---- softmax step (decode_tiles.hpp softmax_phase, with the accumulators of both halves)
    float pe[QB];
    {
      float mx = -INFINITY;
#pragma unroll
      for (int k = 0; k < QB; ++k) {
        sc[k] = valid[k] ? sc[k] * qs20 + sc0 : -INFINITY;
        mx = fmaxf(mx, sc[k]);
      }
      const bool beat = mx > st0.m;
      float al = 1.f, az0 = 1.f, az1 = 1.f, am = 1.f;
      if (__builtin_expect(__any(beat), 0)) {
        const float mn = fmaxf(st0.m, row_max16(mx));
        am = mn == -INFINITY ? 1.f : fexp2(st0.m - mn);
        st0.m = mn;
        const float a0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am), 0));
        const float a1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am), 16));
        const float a2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am), 32));
        const float a3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, am), 48));
        al = (lane & 2) ? ((lane & 1) ? a3 : a2) : ((lane & 1) ? a1 : a0);
        az0 = (lane & 1) ? a2 : a0;
        az1 = (lane & 1) ? a3 : a1;
      }
      st0.l *= am;
      st0.ot[0] *= al; st0.ot[1] *= al; st1.ot[0] *= al; st1.ot[1] *= al;
      st0.z[0] *= az0; st0.z[1] *= az1; st1.z[0] *= az0; st1.z[1] *= az1;
#pragma unroll
      for (int k = 0; k < QB; ++k) {
        pe[k] = fexp2(sc[k] - st0.m);
        st0.l += pe[k];
      }
    }
    // the value scale words outlive the key registers, which take the next quad's keys now
    uint16_t vs0[QB], vs1[QB];
#pragma unroll
    for (int k = 0; k < QB; ++k) { vs0[k] = k0.vs[k]; vs1[k] = k1.vs[k]; }
    const int qn = __builtin_amdgcn_readfirstlane(take);
    chunks_of(qn, ch0);
#pragma unroll
    for (int k = 0; k < QB; ++k) ch1[k] = ch0[k] + L::CHUNK;
    load_k<QM, P, false>(k0, ch0, koff);
    load_k<QM, P, false>(k1, ch1, koff);
    // ---- values, half by half through the same strips
    const bool wide0 = quad_is_wide<QM>(vs0);
    write_strips<QM>(H0, vs0, pe, valid, lane, wave, wide0);
    wave_lds_sync();
    value_phase<QM>(H0, st0, v0, lane, wave, wide0);
    wave_lds_sync();
    const bool wide1 = quad_is_wide<QM>(vs1);
    write_strips<QM>(H1, vs1, pe, valid, lane, wave, wide1);
    wave_lds_sync();
    value_phase<QM>(H1, st1, v1, lane, wave, wide1);
    wave_lds_sync();
    qi = qn;
  }

  // ---- fold the wave and merge the wavefronts, half by half (the epilogue of the 128-d kernel)
  const float unfold = (lane & 1) ? static_cast<float>(1 << UnpackD<QM>::SH) : 1.f;
  const int hl = lane & 3, gl = (lane >> 2) & 3;
  const float lsum = row_sum16(st0.l * unfold);
  if ((lane & 15) == 0) S.m[wave][lane >> 4] = st0.m;
  float Mwg[4], f[4];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    WaveState& t = s ? st1 : st0;
    if constexpr (QM != QM_SYM4) {
      float z0 = t.z[0], z1 = t.z[1];
      z0 += swz_xor<8>(z0); z1 += swz_xor<8>(z1);
      z0 += swz_xor<16>(z0); z1 += swz_xor<16>(z1);
      z0 += xor32(z0); z1 += xor32(z1);
      float* zs = reinterpret_cast<float*>(H0.pb(wave));          // [head][group]; the strips are dead by now
      if (lane < 8) { zs[(2 * (lane & 1)) * 4 + (lane >> 1)] = z0; zs[(2 * (lane & 1) + 1) * 4 + (lane >> 1)] = z1; }
      wave_lds_sync();
    }
    {
      float zg = 0.f;
      if constexpr (QM != QM_SYM4) zg = reinterpret_cast<const float*>(H0.pb(wave))[hl * 4 + gl];
      if constexpr (QM == QM_ASYM2) t.ot[1] *= 0.0625f;
#pragma unroll
      for (int y = 0; y < 2; ++y)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) t.ot[y][r4] = (t.ot[y][r4] - zg) * 16777216.f;
    }
    __syncthreads();     // every wave is done with its strip (and the maxima are in S.m): the partial outputs may overwrite them
    if (s == 0) {
      workgroup_max<NWW>(S, lane, Mwg);
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        const float mh = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, st0.m), 16 * h));
        f[h] = mh == -INFINITY ? 0.f : fexp2(mh - Mwg[h]);
      }
      if ((lane & 15) == 0) S.l[wave][lane >> 4] = pick4(f[0], f[1], f[2], f[3], lane >> 4) * lsum;
    }
    {
      const float fl = pick4(f[0], f[1], f[2], f[3], hl);
      const int kc = lane >> 4;
      float* o = S.o(wave, hl);
#pragma unroll
      for (int y = 0; y < 2; ++y) {
        const int d = 32 * gl + 16 * (kc >> 1) + 8 * y + 4 * (kc & 1);
        *reinterpret_cast<float4*>(o + d) = make_float4(fl * t.ot[y][0], fl * t.ot[y][1], fl * t.ot[y][2], fl * t.ot[y][3]);
      }
    }
    __syncthreads();
    {   // thread = (head `wave`, 2 dims of the half)
      float2 acc = make_float2(0.f, 0.f);
#pragma unroll
      for (int w = 0; w < NWW; ++w) {
        const float2 v = *reinterpret_cast<const float2*>(S.o(w, wave) + 2 * lane);
        acc.x += v.x; acc.y += v.y;
      }
      *reinterpret_cast<float2*>(op + wave * 256 + 128 * s + 2 * lane) = acc;
    }
    __syncthreads();
  }
  if (lane == 0) {
    mlp[2 * wave] = pick4(Mwg[0], Mwg[1], Mwg[2], Mwg[3], wave);
    mlp[2 * wave + 1] = (S.l[0][wave] + S.l[1][wave]) + (S.l[2][wave] + S.l[3][wave]);
  }
}

template <int QM, bool K2>
int wide_mma_qm(const DecodeParams& p, int ntile, int nparts, hipStream_t st) {
  const dim3 grid(p.Hkv * ntile, nparts, p.B);
  if (p.page == 16) hipLaunchKernelGGL((k_wide_parts_mma<QM, K2, 16>), grid, dim3(64 * NWW), 0, st, p, ntile, nparts);
  else if (p.page == 32) hipLaunchKernelGGL((k_wide_parts_mma<QM, K2, 32>), grid, dim3(64 * NWW), 0, st, p, ntile, nparts);
  else return -5;
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

// every split of a head dim 256 launch; nparts = nsplit (+ 1 with BF16 window rows)
int decode_wide_mma_launch(int fmt, const DecodeParams& p, int ntile, int nparts, hipStream_t st) {
  if (nparts <= 0) return 0;
  switch (fmt) {
    case FMT_INT4: return wide_mma_qm<QM_SYM4, false>(p, ntile, nparts, st);
    case FMT_INT4A: return wide_mma_qm<QM_ASYM4, false>(p, ntile, nparts, st);
    case FMT_INT2A: return wide_mma_qm<QM_ASYM2, false>(p, ntile, nparts, st);
    case FMT_KONLY: return wide_mma_qm<QM_SYM4, true>(p, ntile, nparts, st);
    case FMT_KONLYA: return wide_mma_qm<QM_ASYM4, true>(p, ntile, nparts, st);
    case FMT_KONLYA2: return wide_mma_qm<QM_ASYM2, true>(p, ntile, nparts, st);
  }
  return -4;
}

}  // namespace fr
