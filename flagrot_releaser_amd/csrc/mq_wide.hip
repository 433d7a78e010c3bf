// Multi-query prefill attention at head dim 256 for gfx950 (integrations/vllm_flagrot/csrc/mq_prefill.cu:825-1203 k_mq3,
// :1275-1339 k_mq_prep256).  A (page, KV head) chunk is two 128-d half chunks, half s = dims [128 s, 128 s + 128), each
// in the 128-d layout, so the tile converters and the 64-key block step of mq_tiles.hpp serve each half as they are:
//   scores   S^T = K_0 q_0^T + K_1 q_1^T: two K tiles, the second product on top of the first accumulators;
//   values   the workgroups of grid z = 0, 1 each own one V half (128 output dims): both compute the same scores and
//            probabilities, each converts and multiplies its own V^T tile, so a wavefront keeps the 128-d kernel's
//            accumulators and registers (a single workgroup with 256 output dims per row would hold 128 accumulator
//            registers more and run one wavefront per SIMD).  Price: the score product and the K conversion twice.
// Key-only pages: the H32 flag of group g (0..7) is the sign of its K scale word in half g / 4, the whole-head H256
// flag the sign of the token's group-0 V scale word of half 0.  A thread converts both halves of its (token, quarter):
// the in-half stages as at 128 (k2_values, with the whole normalisation 2^-4 = 1/16 of H256 applied there), then the
// stage across the halves in registers.
// 128 rows per workgroup whatever the selector, like the reference at this head dim.
#include "mq_launch.hpp"
#include "mq_tiles.hpp"

namespace frmq {
using namespace fr;
namespace {

constexpr int DW = 256;

struct SmemW {
  Smem a;                                   // K tile of half 0, V^T tile of this workgroup's half, tables, page ids
  alignas(16) uint8_t kt1[KT_BYTES];        // K tile of half 1
};

template <int QM>
DEVI void convert_k2_wide(uint8_t* kt0, uint8_t* kt1, int idx, const u32x4 kc0, const u32x2 sw0, const u32x4 kc1,
                          const u32x2 sw1, uint32_t vf, int kb, int kend, const Consts& cst) {
  const int tk = idx >> 2, tg = idx & 3;
  const int j = kb * BN + tk;
  const int row = 32 * (tk >> 5) + krow_of_token(tk & 31);
  u32x4* d0 = reinterpret_cast<u32x4*>(kt0 + row * KROW);
  u32x4* d1 = reinterpret_cast<u32x4*>(kt1 + row * KROW);
  if (j >= kend) {
#pragma unroll
    for (int g = 0; g < 4; ++g) { d0[4 * g + tg] = u32x4{0u, 0u, 0u, 0u}; d1[4 * g + tg] = u32x4{0u, 0u, 0u, 0u}; }
    return;
  }
  const bool ff = (vf >> 15) & 1u;
  uint32_t v0[4][4], v1[4][4];
  bool r0[4], r1[4];
  k2_values<QM, 256>(kc0, sw0, ff, tg, cst, v0, r0);
  k2_values<QM, 256>(kc1, sw1, ff, tg, cst, v1, r1);
  if (__any(ff)) {                                             // the stage across the halves
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        uint32_t a = v0[g][r], b = v1[g][r];
        bfly(a, b);
        v0[g][r] = ff ? a : v0[g][r];
        v1[g][r] = ff ? b : v1[g][r];
      }
  }
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    d0[4 * g + tg] = u32x4{v0[g][0], v0[g][1], v0[g][2], v0[g][3]};
    d1[4 * g + tg] = u32x4{v1[g][0], v1[g][1], v1[g][2], v1[g][3]};
  }
}

template <int QM, bool K2>
__global__ void __launch_bounds__(256, 2) k_mq256(const Params p) {
  constexpr int NT = 256, ROWS = 128;
  extern __shared__ __align__(16) uint8_t lds[];
  SmemW& SW = *reinterpret_cast<SmemW*>(lds);
  Smem& S = SW.a;
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
  const int item = blockIdx.x, h = blockIdx.y, vz = blockIdx.z;
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

  // q fragments of both halves: the tile through LDS (natural order), gathered in code-word order
  u32x4 qf[2][8];
#pragma unroll
  for (int s2 = 0; s2 < 2; ++s2) {
    if (s2) __syncthreads();
    for (int row = tid >> 5; row < ROWS; row += NT / 32) {
      const int t = row / G, lq = tid & 31;
      u32x2 raw = {0u, 0u};
      if (work.has_row(row))
        raw = gload<u32x2>(p.q + (static_cast<long long>(work.compact_row + t) * Hq + h * G + row % G) * DW + 128 * s2 + 4 * lq);
      *reinterpret_cast<u32x2*>(lds + row * QROW + 8 * lq) = raw;
    }
    __syncthreads();
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int dA = 32 * (s >> 1) + 4 * (2 * (s & 1) + hh);
      const u32x2 a = *reinterpret_cast<const u32x2*>(lds + r * QROW + 2 * dA);
      const u32x2 b = *reinterpret_cast<const u32x2*>(lds + r * QROW + 2 * (dA + 16));
      qf[s2][s] = u32x4{(a.x & 0xFFFFu) | (a.y << 16), (b.x & 0xFFFFu) | (b.y << 16),
                        (a.x >> 16) | (a.y & 0xFFFF0000u), (b.x >> 16) | (b.y & 0xFFFF0000u)};
    }
  }

  f32x16 o[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float mrow = -INFINITY, lrow = 0.f;

  // raw words of one block: K of both halves, V of this workgroup's half.  One block in
  // flight (the 128-d kernels keep two): requested when the previous block's tiles are complete, used after its matrix
  // work -- the registers of a second set are what the second half's q fragments take here.
  struct RawW { Raw<NT> half[2], val; };                // (K fields of half[], V fields of val are the ones used)
  RawW raw;
  auto fetch = [&](RawW& R, const int* pg, int kb) {
    load_raw_k<QM, K2, NT, true>(R.half[0], p, pg, 2 * h, kb, kend);
    load_raw_k<QM, K2, NT, true>(R.half[1], p, pg, 2 * h + 1, kb, kend);
    load_raw_v<QM, NT, true>(R.val, p, pg, 2 * h + vz, kb, kend);
  };
  if (kb0 < kb1) fetch(raw, S.pages, kb0);
  auto block_step = [&](RawW& R, int kb) {
    __syncthreads();                                   // the tiles (or the q staging) are no longer read
#pragma unroll
    for (int it = 0; it < Raw<NT>::NI; ++it) {
      const int idx = tid + it * NT;
      if constexpr (K2)
        convert_k2_wide<QM>(S.kt, SW.kt1, idx, R.half[0].kc[it], R.half[0].ks[it], R.half[1].kc[it], R.half[1].ks[it],
                            R.half[0].vf[it], kb, kend, cst);
      else {
        convert_k_entry<QM, false>(S.kt, idx, R.half[0].kc[it], R.half[0].ks[it], 0u, kb, kend, cst);
        convert_k_entry<QM, false>(SW.kt1, idx, R.half[1].kc[it], R.half[1].ks[it], 0u, kb, kend, cst);
      }
    }
    v_tables<QM, NT>(S, R.val, kb, kend);
    if (kb + 1 < kb1 && kb + 1 >= cb + PG_CACHE / 4) {   // the next fetch leaves the cached window: slide it
      cb = kb + 1;
      fill_pages();
    }
    __syncthreads();
    convert_v<QM, NT>(S, R.val, kb, kend, cst);
    __syncthreads();
    if (kb + 1 < kb1) fetch(R, S.pages + 4 * (kb + 1 - cb), kb + 1);   // the next block
    f32x16 sacc[2];
    u32x4 pb[4];
    qk_block<false>(S.kt, qf[0], sacc, l32, hh);
    qk_block<true>(SW.kt1, qf[1], sacc, l32, hh);
    softmax_block(sacc, pb, o, mrow, lrow, kb, lim, rvalid, p.kmin, hh);
    pv_block(S.vt, pb, o, l32, hh);
  };
  for (int kb = kb0; kb < kb1; ++kb) block_step(raw, kb);
  // partials: this workgroup's 128 dims of the row; (maximum, sum) once
  const float l = lrow + __shfl_xor(lrow, 32, 64);
  if (rvalid) {
    const long long base = (static_cast<long long>(item) * p.Hkv + h) * ROWS + r;
    float* op = p.opart + base * DW + 128 * vz;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *reinterpret_cast<float4*>(op + 32 * db + 8 * q4 + 4 * hh) =
            make_float4(o[db][4 * q4], o[db][4 * q4 + 1], o[db][4 * q4 + 2], o[db][4 * q4 + 3]);
    if (hh == 0 && vz == 0) *reinterpret_cast<float2*>(p.ml + base * 2) = make_float2(mrow, l);
  }
}

// ------------------------------------------------------------------------------------------------ query rows
// One half wave per (row, head): lane l holds channels 128 s + 4 l + i.  Whole-head keys: the eight butterfly stages in
// distance order (the seven of each half, then the one across the halves) and one multiply by 1/16; H32 groups: the
// orthonormal transform on the flagged ones of the eight groups; the softmax factor; one rounding to fp16 -- every
// step rounded to fp32 on its own, in this order.
template <typename T> DEVI void read4w(const T* p, float (&x)[4]);
template <> DEVI void read4w<float>(const float* p, float (&x)[4]) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
}
template <> DEVI void read4w<uint16_t>(const uint16_t* p, float (&x)[4]) {     // bf16
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  x[0] = bf16_lo(v.x); x[1] = bf16_hi(v.x); x[2] = bf16_lo(v.y); x[3] = bf16_hi(v.y);
}

template <typename T>
__global__ void __launch_bounds__(256) k_query_rows256(const T* __restrict__ q, long long q_stride, const int* __restrict__ pick,
                                                       int Hq, int G, const uint8_t* __restrict__ whole,
                                                       const uint8_t* __restrict__ rotated, float factor,
                                                       uint16_t* __restrict__ q16) {
  const int l32 = threadIdx.x & 31, sub = l32 >> 3;
  const long long src = pick != nullptr ? pick[blockIdx.x] : blockIdx.x;
  for (int head = threadIdx.x >> 5; head < Hq; head += 8) {
    const int kv = head / G;
    float x[2][4];
    read4w<T>(q + src * q_stride + head * DW + 4 * l32, x[0]);
    read4w<T>(q + src * q_stride + head * DW + 128 + 4 * l32, x[1]);
    if (whole != nullptr && whole[kv]) {
      butterflies<128>(x[0], l32);
      butterflies<128>(x[1], l32);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float a = x[0][i], b = x[1][i];
        x[0][i] = (a + b) * 0.0625f;
        x[1][i] = (a - b) * 0.0625f;
      }
    }
    if (rotated != nullptr) {                    // every lane takes part in the exchange; the flagged groups keep the result
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        float y[4] = {x[s][0], x[s][1], x[s][2], x[s][3]};
        fwht<32>(y, l32);
        if (rotated[kv * 8 + 4 * s + sub]) {
#pragma unroll
          for (int i = 0; i < 4; ++i) x[s][i] = y[i];
        }
      }
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      uint32_t hb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) hb[i] = f16_bits_rn(x[s][i] * factor);
      *reinterpret_cast<uint2*>(q16 + (static_cast<long long>(blockIdx.x) * Hq + head) * DW + 128 * s + 4 * l32) =
          make_uint2(hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16));
    }
  }
}

template <int QM, bool K2> int launch_mq256(const Params& p, int nitems, hipStream_t st) {
  static bool attr = false;
  if (!attr) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_mq256<QM, K2>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(sizeof(SmemW))) != hipSuccess) return -1;
    attr = true;
  }
  hipLaunchKernelGGL((k_mq256<QM, K2>), dim3(nitems, p.Hkv, 2), dim3(256), sizeof(SmemW), st, p);
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

int wide_smem_bytes() { return static_cast<int>(sizeof(SmemW)); }

int wide_attn_launch(const Params& p, int nitems, int konly, hipStream_t st) {
  const bool k2 = konly & 1, i2 = konly & 2;
  return i2 ? (k2 ? launch_mq256<QM_ASYM2, true>(p, nitems, st) : launch_mq256<QM_ASYM2, false>(p, nitems, st))
            : (k2 ? launch_mq256<QM_ASYM4, true>(p, nitems, st) : launch_mq256<QM_ASYM4, false>(p, nitems, st));
}

int wide_query_rows_launch(const void* q, int q_fp32, long long q_ts, const int* idx, int m, int Hq, int G, const uint8_t* kfull,
                           const uint8_t* kmask, float qscale, void* q16, hipStream_t st) {
  uint16_t* dst = static_cast<uint16_t*>(q16);
  if (q_fp32) hipLaunchKernelGGL(k_query_rows256<float>, dim3(m), dim3(256), 0, st, static_cast<const float*>(q), q_ts, idx, Hq,
                                 G, kfull, kmask, qscale, dst);
  else hipLaunchKernelGGL(k_query_rows256<uint16_t>, dim3(m), dim3(256), 0, st, static_cast<const uint16_t*>(q), q_ts, idx, Hq,
                          G, kfull, kmask, qscale, dst);
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

}  // namespace frmq
