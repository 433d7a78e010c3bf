// Paged decode attention for 256-d heads (`variant | 4096` of fr_v2_attn; reference kernels/csrc/attn_decode_v2g.cuh:
// 11-25, 276): the chunk of a (page, KV head) is two 128-d half chunks, each in the 128-d layout, half s = dims
// [128 s, 128 s + 128); q tiles of 4 heads; static formats (q rotated by kmask, output rotated back by vmask) and
// key-only kinds (H32 flag of key group g = sign bit of its K scale word, whole-head H256 flag = sign bit of the
// token's group-0 V scale word of half 0; the inverse key transforms are applied to the query: three variants, chosen
// per (token, group)).
//
// Correctness first: plain fp32 vector code, no matrix pipe, two launches.  k_wide_parts: a workgroup of 256 threads per
// (KV head x q tile, split, sequence) walks its tokens 64 at a time in three phases --
//   scores   thread = (token, quarter of the key groups): the token's code words of its groups against the query
//            variant the flags select (queries in LDS, fp32, pre-multiplied by the softmax factor);
//   softmax  wavefront = head, lane = token: running maximum / sum, probabilities to LDS;
//   values   thread = channel: its V^T words of the 64 tokens, (code - zero point) * scale * p into four accumulators
//            (one per head of the tile);
// and writes the unnormalised partial (o [4][256], maximum, sum); the BF16 window rows are one more split of the same
// grid.  k_wide_merge combines the splits, rotates static formats back and writes bf16.  The caller's counter words
// are not used (they stay zero).  Byte positions follow the page layout as the writers store it (fr_common.hpp Lay,
// place4 / store_v_codes) and as the torch parser of the front end reads it.
#include <cstdlib>

#include "fr_common.hpp"
#include "fr_launch.hpp"

namespace fr {
int decode_wide_mma_launch(int fmt, const DecodeParams& p, int ntile, int nparts, hipStream_t st);   // decode_wide_mma.hip
namespace {

constexpr int WD = 256, WG = 8;                 // head dim, 32-channel groups per head

DEVI float fexp2w(float x) { return __builtin_amdgcn_exp2f(x); }
DEVI float sylv(int a, int b) { return (__builtin_popcount(a & b) & 1) ? -1.f : 1.f; }

// one stored code as a number (zero point not yet subtracted): element `isB` of byte i of `word`
template <int QM> DEVI float code4(uint32_t word, int i, bool isB) {
  const uint32_t by = (word >> (8 * i)) & 0xFFu;
  if constexpr (QM == QM_ASYM4) return static_cast<float>(isB ? by >> 4 : by & 15u);
  else {   // sign-magnitude: A = sign bit 7, magnitude bits 0-2 of its byte; B = sign bit 3 of its byte, magnitude
           // bits 4-6 of byte (i + 3) % 4 of the same word
    const uint32_t other = (word >> (8 * ((i + 3) & 3))) & 0xFFu;
    const float mag = static_cast<float>(isB ? (other >> 4) & 7u : by & 7u);
    const bool neg = isB ? (by >> 3) & 1u : by >> 7;
    return neg ? -mag : mag;
  }
}

struct WideSmem {
  float qv[3][4][WD];          // query variants (identity / H32 per group / H256) of the tile's heads, times qscale
  float qsum[3][4][WG];        // their sums per key group (zero-point term of the asymmetric formats)
  float sc[4][4][64];          // partial scores per (quarter of the groups, head, token)
  float pr[4][64];             // probabilities per (head, token)
  float vsc[64][WG], vz[64][WG];   // value scale and zero point per (token, group); scale 0 outside the range
  float alpha[4];
  int page[4];
};

template <int QM, bool K2, int P>
__global__ void __launch_bounds__(256) k_wide_parts(const DecodeParams p, int ntile, int nparts) {
  using L = Lay<QM, P>;
  constexpr uint32_t ZMASK = QM == QM_ASYM4 ? 15u : QM == QM_ASYM2 ? 3u : 0u;
  __shared__ WideSmem S;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int kvh = blockIdx.x / ntile, tile = blockIdx.x % ntile, split = blockIdx.y, b = blockIdx.z;
  const bool is_tail = p.tail != nullptr && split == p.nsplit;
  const long long part_id = ((static_cast<long long>(b) * p.Hkv + kvh) * ntile + tile) * nparts + split;
  float* const op = p.opart + part_id * 4 * WD;
  float* const mlp = p.mlpart + part_id * 8;
  const int len = p.seq_lens[b];
  // ---- query variants.  Static formats: variant 0 = q rotated on the kmask groups, variant 1 = q as it is (the BF16
  //      rows are in the original basis).  Key-only kinds: 0 = q, 1 = H32 per group, 2 = H256.
  for (int e = tid; e < 4 * WD; e += 256) {
    const int h = e / WD, d = e % WD, hq = tile * 4 + h;
    float x = 0.f;
    if (hq < p.gqa) x = bf16_lo(static_cast<const uint16_t*>(p.q)[static_cast<long long>(b) * p.q_bs + (static_cast<long long>(kvh) * p.gqa + hq) * WD + d]) * p.qscale;
    S.qv[K2 ? 0 : 1][h][d] = x;
  }
  __syncthreads();
  for (int e = tid; e < 4 * WD; e += 256) {
    const int h = e / WD, d = e % WD, g = d >> 5;
    const float* src = S.qv[K2 ? 0 : 1][h];
    float a32 = 0.f;
    for (int k = 0; k < 32; ++k) a32 += sylv(d & 31, k) * src[32 * g + k];
    a32 *= kC32;
    if constexpr (K2) {
      float a256 = 0.f;
      for (int k = 0; k < WD; ++k) a256 += sylv(d, k) * src[k];
      S.qv[1][h][d] = a32;
      S.qv[2][h][d] = a256 * 0.0625f;
    } else {
      S.qv[0][h][d] = (p.kmask != nullptr && p.kmask[kvh * WG + g]) ? a32 : src[d];
    }
  }
  __syncthreads();
  if (tid < 3 * 4 * WG) {
    const int v = tid / (4 * WG), h = (tid / WG) & 3, g = tid % WG;
    float a = 0.f;
    for (int k = 0; k < 32; ++k) a += S.qv[v][h][32 * g + k];
    S.qsum[v][h][g] = a;
  }
  __syncthreads();

  float m_run = -INFINITY, l_run = 0.f;       // of head `wave`, uniform over the wavefront
  float o[4] = {0.f, 0.f, 0.f, 0.f};          // channel tid of the four heads
  const int lo = is_tail ? 0 : max(split * p.chunk, min(p.kv_start, len));
  const int hi = is_tail ? (p.tail_len != nullptr ? p.tail_len[b] : 0) : min(len, (split + 1) * p.chunk);
  const int* bt = p.block_table + static_cast<long long>(b) * p.bt_stride;
  const uint16_t* rows = nullptr;              // BF16 rows of this sequence: [slot][2 Hkv][256]
  if (is_tail) rows = static_cast<const uint16_t*>(p.tail) + static_cast<long long>(p.tail_idx != nullptr ? p.tail_idx[b] : b) * p.tail_bs;

  for (int base = (lo / 64) * 64; base < hi; base += 64) {
    if (!is_tail && tid < 64 / P) S.page[tid] = bt[min(base / P + tid, (hi - 1) / P)];
    __syncthreads();
    // ---- scores: thread = (token, quarter q4 of the key groups)
    {
      const int t = lane, q4 = wave, pos = base + t;
      const bool valid = pos >= lo && pos < hi;
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
      if (valid && is_tail) {
        const uint16_t* kr = rows + static_cast<long long>(pos) * p.tail_ts + static_cast<long long>(kvh) * WD + 64 * q4;
        for (int d = 0; d < 64; ++d) {
          const float k = bf16_lo(kr[d]);
#pragma unroll
          for (int h = 0; h < 4; ++h) acc[h] += k * S.qv[K2 ? 0 : 1][h][64 * q4 + d];       // the query as it came
        }
      } else if (valid) {
        const int tp = pos % P;
        const long long pg = S.page[(pos - base) / P];
        const uint8_t* c0 = p.pool + (pg * (2 * p.Hkv) + 2 * kvh) * L::CHUNK;      // half chunk 0 of this (page, head)
        bool whole = false;
        if constexpr (K2) whole = *reinterpret_cast<const uint16_t*>(c0 + L::VS_OFF + (8 * (tp >> 3) + vs_slot8(tp)) * 2) >> 15;
#pragma unroll
        for (int gg = 0; gg < 2; ++gg) {
          const int G8 = 2 * q4 + gg, s = G8 >> 2, g = G8 & 3;                     // group G8 of the head: half s, group g
          const uint8_t* ch = c0 + s * L::CHUNK;
          const uint32_t kw = *reinterpret_cast<const uint16_t*>(ch + L::KS_OFF + 8 * tp + 2 * g);
          const float mag = f16_value(kw & 0x7FFFu);
          const int var = K2 ? (whole ? 2 : static_cast<int>(kw >> 15)) : 0;
          float dot[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int tg = 0; tg < 4; ++tg) {
            uint32_t word;
            if constexpr (QM == QM_ASYM2) word = *reinterpret_cast<const uint32_t*>(ch + 32 * (tp ^ ((tp >> 1) & 2)) + 8 * tg + 4 * (g >> 1));
            else word = *reinterpret_cast<const uint32_t*>(ch + 64 * tp + 16 * tg + 4 * g);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
              for (int isB = 0; isB < 2; ++isB) {
                float c;
                if constexpr (QM == QM_ASYM2) c = static_cast<float>((word >> (8 * i + 4 * (g & 1) + 2 * isB)) & 3u);
                else c = code4<QM>(word, i, isB);
                const int d = 32 * G8 + 16 * isB + 4 * tg + i;
#pragma unroll
                for (int h = 0; h < 4; ++h) dot[h] += c * S.qv[var][h][d];
              }
          }
          const float z = static_cast<float>(kw & ZMASK);
#pragma unroll
          for (int h = 0; h < 4; ++h) acc[h] += mag * (dot[h] - z * S.qsum[var][h][G8]);
        }
      }
#pragma unroll
      for (int h = 0; h < 4; ++h) S.sc[q4][h][t] = valid ? acc[h] : -INFINITY;
      // value scales / zero points of this thread's two groups
      if (!is_tail) {
#pragma unroll
        for (int gg = 0; gg < 2; ++gg) {
          const int G8 = 2 * q4 + gg, s = G8 >> 2, g = G8 & 3;
          float vs = 0.f, vz = 0.f;
          if (valid) {
            const int tp = pos % P;
            const uint8_t* ch = p.pool + (static_cast<long long>(S.page[(pos - base) / P]) * (2 * p.Hkv) + 2 * kvh + s) * L::CHUNK;
            const uint32_t vw = *reinterpret_cast<const uint16_t*>(ch + L::VS_OFF + (g * P + 8 * (tp >> 3) + vs_slot8(tp)) * 2);
            vs = f16_value(vw & 0x7FFFu);
            vz = static_cast<float>(vw & ZMASK);
          }
          S.vsc[t][G8] = vs; S.vz[t][G8] = vz;
        }
      }
    }
    __syncthreads();
    // ---- softmax: wavefront = head
    {
      const int h = wave, t = lane;
      const float s = ((S.sc[0][h][t] + S.sc[1][h][t]) + S.sc[2][h][t]) + S.sc[3][h][t];   // -inf outside the range
      const float mn = fmaxf(m_run, wave_max64(s));
      float pv = 0.f, al = 1.f;
      if (mn != -INFINITY) {
        pv = fexp2w(s - mn);
        al = m_run == -INFINITY ? 0.f : fexp2w(m_run - mn);
      }
      l_run = l_run * al + wave_sum64(pv);
      m_run = mn;
      S.pr[h][t] = pv;
      if (lane == 0) S.alpha[h] = al;
    }
    __syncthreads();
    // ---- values: thread = channel d of the head
    {
      const int d = tid, s = d >> 7, dd = d & 127, g = dd >> 5, G8 = d >> 5;
#pragma unroll
      for (int h = 0; h < 4; ++h) o[h] *= S.alpha[h];
      if (is_tail) {
        for (int t = 0; t < 64 && base + t < hi; ++t) {
          if (base + t < lo) continue;
          const float v = bf16_lo(rows[static_cast<long long>(base + t) * p.tail_ts + (static_cast<long long>(p.Hkv) + kvh) * WD + d]);
#pragma unroll
          for (int h = 0; h < 4; ++h) o[h] += S.pr[h][t] * v;
        }
      } else {
        const int e = ((dd & 63) >> 4) * 8 + (dd & 7);          // V^T entry of the channel inside its half
        for (int r = 0; r < 8; ++r) {                           // runs of 8 tokens
          const int t0 = 8 * r;
          if (base + t0 >= hi || base + t0 + 8 <= lo) continue;
          const uint8_t* ch = p.pool + (static_cast<long long>(S.page[t0 / P]) * (2 * p.Hkv) + 2 * kvh + s) * L::CHUNK;
          const int c8 = (t0 % P) >> 3;
          uint32_t word;
          if constexpr (QM == QM_ASYM2) word = *reinterpret_cast<const uint32_t*>(ch + L::V_OFF + (e * (P / 8) + c8) * 8 + 4 * (dd >> 6));
          else word = *reinterpret_cast<const uint32_t*>(ch + L::V_OFF + (e * (P / 8) + c8) * 16 + 4 * (2 * (dd >> 6) + ((dd & 15) >> 3)));
#pragma unroll
          for (int ii = 0; ii < 4; ++ii)
#pragma unroll
            for (int odd = 0; odd < 2; ++odd) {
              const int t = t0 + 2 * ii + odd;
              float c;
              if constexpr (QM == QM_ASYM2) c = static_cast<float>((word >> (8 * ii + 4 * ((dd & 15) >> 3) + 2 * odd)) & 3u);
              else c = code4<QM>(word, ii, odd);
              const float v = (c - S.vz[t][G8]) * S.vsc[t][G8];   // scale 0 outside the range
#pragma unroll
              for (int h = 0; h < 4; ++h) o[h] += S.pr[h][t] * v;
            }
        }
      }
      (void)g;
    }
    __syncthreads();
  }
  // ---- the partial.  Static formats merge in the stored basis: the BF16 rows' share is rotated on the vmask groups.
  if (is_tail && !K2 && p.vmask != nullptr) {
    float* buf = &S.qv[0][0][0];                               // [4][256], free by now
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 4; ++h) buf[h * WD + tid] = o[h];
    __syncthreads();
    if (p.vmask[kvh * WG + (tid >> 5)]) {
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        float a = 0.f;
        for (int k = 0; k < 32; ++k) a += sylv(tid & 31, k) * buf[h * WD + (tid & ~31) + k];
        o[h] = a * kC32;
      }
    }
  }
#pragma unroll
  for (int h = 0; h < 4; ++h) op[h * WD + tid] = o[h];
  if (lane == 0) { mlp[2 * wave] = m_run; mlp[2 * wave + 1] = l_run; }
}

__global__ void __launch_bounds__(256) k_wide_merge(const DecodeParams p, int ntile, int nparts, int rotate_back) {
  __shared__ float buf[WD];
  const int kvh = blockIdx.x / ntile, tile = blockIdx.x % ntile, b = blockIdx.y, d = threadIdx.x;
  const long long part0 = ((static_cast<long long>(b) * p.Hkv + kvh) * ntile + tile) * nparts;
  for (int h = 0; h < 4; ++h) {
    const int hq = tile * 4 + h;
    if (hq >= p.gqa) break;                                     // uniform
    float M = -INFINITY;
    for (int s = 0; s < nparts; ++s) M = fmaxf(M, p.mlpart[(part0 + s) * 8 + 2 * h]);
    float acc = 0.f, Lsum = 0.f;
    if (M != -INFINITY) {
      for (int s = 0; s < nparts; ++s) {
        const float ms = p.mlpart[(part0 + s) * 8 + 2 * h];
        if (ms == -INFINITY) continue;
        const float f = fexp2w(ms - M);
        Lsum += f * p.mlpart[(part0 + s) * 8 + 2 * h + 1];
        acc += f * p.opart[(part0 + s) * 4 * WD + h * WD + d];
      }
    }
    float v = Lsum > 0.f ? acc / Lsum : 0.f;
    if (rotate_back) {
      __syncthreads();
      buf[d] = v;
      __syncthreads();
      if (p.vmask[kvh * WG + (d >> 5)]) {
        float a = 0.f;
        for (int k = 0; k < 32; ++k) a += sylv(d & 31, k) * buf[(d & ~31) + k];
        v = a * kC32;
      }
    }
    static_cast<uint16_t*>(p.out)[static_cast<long long>(b) * p.o_bs + (static_cast<long long>(kvh) * p.gqa + hq) * WD + d] =
        static_cast<uint16_t>(bf16_rn(v));
  }
}

template <int QM, bool K2, int FMT>
int wide_qm(const DecodeParams& p, hipStream_t st) {
  const int ntile = (p.gqa + 3) / 4;
  const int nparts = p.nsplit + (p.tail != nullptr ? 1 : 0);
  if (p.page != 16 && p.page != 32) return -5;
  // every split through the matrix-pipe kernel file (decode_wide_mma.hip) unless FLAGROT_WIDE_PLAIN=1 (read at every
  // call) asks for the plain kernel of this file
  const char* env = std::getenv("FLAGROT_WIDE_PLAIN");
  if (env != nullptr && env[0] == '1') {
    const dim3 grid(p.Hkv * ntile, nparts, p.B);
    if (p.page == 16) hipLaunchKernelGGL((k_wide_parts<QM, K2, 16>), grid, dim3(256), 0, st, p, ntile, nparts);
    else hipLaunchKernelGGL((k_wide_parts<QM, K2, 32>), grid, dim3(256), 0, st, p, ntile, nparts);
    if (hipPeekAtLastError() != hipSuccess) return -1;
  } else {
    const int rc = decode_wide_mma_launch(FMT, p, ntile, nparts, st);
    if (rc) return rc;
  }
  hipLaunchKernelGGL(k_wide_merge, dim3(p.Hkv * ntile, p.B), dim3(256), 0, st, p, ntile, nparts, (!K2 && p.vmask != nullptr) ? 1 : 0);
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

int decode_wide_launch(int fmt, const DecodeParams& p, hipStream_t st) {
  switch (fmt) {
    case FMT_INT4: return wide_qm<QM_SYM4, false, FMT_INT4>(p, st);
    case FMT_INT4A: return wide_qm<QM_ASYM4, false, FMT_INT4A>(p, st);
    case FMT_INT2A: return wide_qm<QM_ASYM2, false, FMT_INT2A>(p, st);
    case FMT_KONLY: return wide_qm<QM_SYM4, true, FMT_KONLY>(p, st);
    case FMT_KONLYA: return wide_qm<QM_ASYM4, true, FMT_KONLYA>(p, st);
    case FMT_KONLYA2: return wide_qm<QM_ASYM2, true, FMT_KONLYA2>(p, st);
  }
  return -4;
}

}  // namespace fr
