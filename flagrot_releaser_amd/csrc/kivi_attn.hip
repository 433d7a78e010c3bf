// Paged split-K decode attention over KIVI-style FlagRot INT2 pages (gfx950, wave64, no matrix cores), the split merge,
// and the extern "C" surface of libflagrot_kivi.so (declared in include/flagrot_kivi.h).
//
// Workgroup (256 threads) per (sequence, KV head, split); split index NS is the BF16 sink / window rows.  Per
// 32-token group (two pages):
//   q' * scale   the query is rotated three ways once (identity, H32, H128); per group the channel scales are folded
//                into the variant its flags select, and q' . min becomes a per-head bias;
//   scores       thread = (token, 16-channel word): 2-bit codes against q' * scale, partials through LDS;
//   softmax      thread = (head, token): exp2-domain online softmax, half-wave reductions;
//   values       thread = (4 channels, token slice): d = code * |scale| + min accumulated into one of three classes
//                (stored as is / H32 / H128, by the value flags); the classes are inverse-transformed once at the end:
//                o = accI + H32(accH) + H128(accF).
// Semantics follow integrations/vllm_flagrot/csrc/kivi.cu:729-980 (k_attn) and :1908-1931 (k_merge).
#include <cstdio>
#include <cstring>

#include "../../include/flagrot_kivi.h"
#include "fr_common.hpp"
#include "kivi_launch.hpp"

namespace frkv {
using namespace fr;
namespace {

char g_err[512] = "";
int bad(const char* msg) {
  std::strncpy(g_err, msg, sizeof(g_err) - 1);
  return 2;
}

template <int G> struct ASmem {
  float q[3][G][128];
  float qs[G][128];
  float acc[3][G][128];
  uint32_t km[32][4];
  float part[8][G][32];
  float bias[G];
  float p[G][32];
  float alpha[G];
  int flags[2];
  int changed;
};

template <int G>
__global__ void __launch_bounds__(256) k_attn(const uint16_t* __restrict__ q, long long q_rs, const uint8_t* __restrict__ pool,
                                              const int* __restrict__ bt, long long bt_rs, const int* __restrict__ cached,
                                              int kv_start, int Hkv, int NS, int chunk, float qscale,
                                              const uint16_t* __restrict__ ring, const int* __restrict__ tail_len,
                                              const int* __restrict__ tail_idx, int T, float* __restrict__ opart,
                                              float* __restrict__ ml) {
  extern __shared__ __align__(16) uint8_t lds[];
  ASmem<G>& S = *reinterpret_cast<ASmem<G>*>(lds);
  const int b = blockIdx.x, h = blockIdx.y, sp = blockIdx.z;
  const int tid = threadIdx.x, hw = tid >> 5, l32 = tid & 31;
  const long long pidx = (static_cast<long long>(b) * Hkv + h) * (NS + 1) + sp;
  float* op = opart + pidx * G * 128;
  float* mlp = ml + pidx * G * 2;
  const bool tail = sp == NS;
  int t0, t1;
  if (tail) { t0 = 0; t1 = tail_len != nullptr ? tail_len[b] : 0; }
  else { t0 = max(sp * chunk, kv_start); t1 = min((sp + 1) * chunk, cached[b]); }
  if (t1 <= t0) {
    if (tid < G) { mlp[2 * tid] = -INFINITY; mlp[2 * tid + 1] = 0.f; }
    return;
  }
  // query variants: half wave per (variant, head) row
  for (int r = hw; r < 3 * G; r += 8) {
    const int var = r / G, g = r % G;
    const uint2 raw = *reinterpret_cast<const uint2*>(q + static_cast<long long>(b) * q_rs + (static_cast<long long>(h) * G + g) * 128 + 4 * l32);
    float x[4] = {bf16_lo(raw.x), bf16_hi(raw.x), bf16_lo(raw.y), bf16_hi(raw.y)};
    if (!tail && var == 1) fwht<32>(x, l32);
    if (!tail && var == 2) fwht<128>(x, l32);
    *reinterpret_cast<float4*>(&S.q[var][g][4 * l32]) = make_float4(x[0], x[1], x[2], x[3]);
  }
  for (int e = tid; e < 3 * G * 128; e += 256) (&S.acc[0][0][0])[e] = 0.f;
  float accI[G][4], accH[G][4], accF[G][4];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i) { accI[g][i] = 0.f; accH[g][i] = 0.f; accF[g][i] = 0.f; }
  float m_run = -INFINITY, l_run = 0.f;               // of head tid >> 5 (softmax mapping), replicated over the half wave
  const int* btb = bt + static_cast<long long>(b) * bt_rs;
  const uint16_t* rbase = ring + static_cast<long long>(tail ? (tail_idx != nullptr ? tail_idx[b] : 0) : 0) * T * 2 * Hkv * 128;
  __syncthreads();

  for (int base = tail ? 0 : (t0 / 32) * 32; base < t1; base += 32) {
    const uint8_t* chA = nullptr;
    const uint8_t* chB = nullptr;
    if (!tail) {
      const int g32 = base / 32;
      chA = pool + (static_cast<long long>(btb[2 * g32]) * Hkv + h) * 1552ll;
      chB = pool + (static_cast<long long>(btb[2 * g32 + 1]) * Hkv + h) * 1552ll;
      if (tid < 128) S.km[tid >> 2][tid & 3] = reinterpret_cast<const uint32_t*>(((tid >> 2) < 16 ? chA : chB) + 512 + ((tid >> 2) & 15) * 16)[tid & 3];
      if (tid < G) S.bias[tid] = 0.f;
      __syncthreads();
      if (tid == 0) {
        int lm = 0;
        for (int j = 0; j < 4; ++j) lm |= ((S.km[0][j] >> 15) & 1) << j;
        S.flags[0] = lm;
        S.flags[1] = (S.km[1][0] >> 15) & 1;
      }
      __syncthreads();
      {   // q' * scale and q' . min: thread = (channel, head parity)
        const int c = tid & 127, gp = tid >> 7;
        const uint32_t w = S.km[c >> 2][c & 3];
        const float s = f16_value(w & 0x7FFFu), mn = f16_value(w >> 16);
        const int which = S.flags[1] ? 2 : ((S.flags[0] >> (c >> 5)) & 1);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          if ((g & 1) != gp && G > 1) continue;
          if (G == 1 && gp) continue;
          const float qp = S.q[which][g][c];
          S.qs[g][c] = qp * s;
          float v = qp * mn;
#pragma unroll
          for (int m = 1; m < 32; m <<= 1) v += hx(v, m);
          v += __shfl_xor(v, 32, 64);
          if ((tid & 63) == 0) atomicAdd(&S.bias[g], v);
        }
      }
      __syncthreads();
      {   // partial scores: thread = (token l32, word hw of 16 channels)
        const uint8_t* ch = l32 < 16 ? chA : chB;
        const uint32_t word = reinterpret_cast<const uint32_t*>(ch + (l32 & 15) * 32)[hw];
        float cv[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) cv[i] = static_cast<float>((word >> (2 * (i >> 1) + 16 * (i & 1))) & 3u);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          float a = 0.f;
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            const float4 qv = *reinterpret_cast<const float4*>(&S.qs[g][16 * hw + 4 * i4]);
            a += qv.x * cv[4 * i4] + qv.y * cv[4 * i4 + 1] + qv.z * cv[4 * i4 + 2] + qv.w * cv[4 * i4 + 3];
          }
          S.part[hw][g][l32] = a;
        }
      }
    } else {
      if (tid < G) S.bias[tid] = 0.f;
      const int j = base + l32;
      float a[G];
#pragma unroll
      for (int g = 0; g < G; ++g) a[g] = 0.f;
      if (j < t1) {
        const uint16_t* kr = rbase + static_cast<long long>(j) * 2 * Hkv * 128 + h * 128 + 16 * hw;
#pragma unroll
        for (int i2 = 0; i2 < 8; ++i2) {
          const uint32_t w = reinterpret_cast<const uint32_t*>(kr)[i2];
          const float k0 = bf16_lo(w), k1 = bf16_hi(w);
#pragma unroll
          for (int g = 0; g < G; ++g) a[g] += S.q[0][g][16 * hw + 2 * i2] * k0 + S.q[0][g][16 * hw + 2 * i2 + 1] * k1;
        }
      }
#pragma unroll
      for (int g = 0; g < G; ++g) S.part[hw][g][l32] = a[g];
    }
    if (tid == 0) S.changed = 0;
    __syncthreads();
    if (hw < G) {   // online softmax: thread = (head hw, token l32)
      const int g = hw, pos = base + l32;
      const bool valid = pos >= t0 && pos < t1;
      float sc = S.bias[g];
#pragma unroll
      for (int w8 = 0; w8 < 8; ++w8) sc += S.part[w8][g][l32];
      sc = valid ? sc * qscale : -INFINITY;
      float mx = sc;
#pragma unroll
      for (int m = 1; m < 32; m <<= 1) mx = fmaxf(mx, hx(mx, m));
      const float mnew = fmaxf(m_run, mx);
      const float p = (mnew == -INFINITY || !valid) ? 0.f : exp2f(sc - mnew);
      const float al = m_run == -INFINITY ? 0.f : exp2f(m_run - mnew);
      float ps = p;
#pragma unroll
      for (int m = 1; m < 32; m <<= 1) ps += hx(ps, m);
      l_run = l_run * al + ps;
      if (l32 == 0) { S.alpha[g] = al; if (mnew != m_run) S.changed = 1; }
      m_run = mnew;
      S.p[g][l32] = p;
    }
    __syncthreads();
    if (S.changed) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float al = S.alpha[g];
#pragma unroll
        for (int i = 0; i < 4; ++i) { accI[g][i] *= al; accH[g][i] *= al; accF[g][i] *= al; }
      }
    }
    // values: thread = (channels 4 l32 .. 4 l32 + 3, tokens hw, hw + 8, hw + 16, hw + 24 of the group)
    const int nt = min(32, t1 - base), i0 = max(0, t0 - base);
    for (int i = hw; i < nt; i += 8) {
      if (i < i0) continue;
      float d[4];
      int cls = 0;
      if (!tail) {
        const uint8_t* ch = i < 16 ? chA : chB;
        const int cell = i & 15;
        const uint32_t byte = ch[768 + cell * 32 + l32];
        const uint32_t w = reinterpret_cast<const uint32_t*>(ch + 1280 + cell * 16)[l32 >> 3];
        const float s = f16_value(w & 0x7FFFu), mn = f16_value(w >> 16);
        cls = ch[1536 + cell] ? 2 : static_cast<int>((w >> 15) & 1u);
#pragma unroll
        for (int k = 0; k < 4; ++k) d[k] = static_cast<float>((byte >> (2 * k)) & 3u) * s + mn;
      } else {
        const uint2 raw = *reinterpret_cast<const uint2*>(rbase + static_cast<long long>(base + i) * 2 * Hkv * 128 + (Hkv + h) * 128 + 4 * l32);
        d[0] = bf16_lo(raw.x); d[1] = bf16_hi(raw.x); d[2] = bf16_lo(raw.y); d[3] = bf16_hi(raw.y);
      }
      if (cls == 2) {
#pragma unroll
        for (int g = 0; g < G; ++g) { const float pv = S.p[g][i];
#pragma unroll
          for (int k = 0; k < 4; ++k) accF[g][k] += pv * d[k]; }
      } else if (cls == 1) {
#pragma unroll
        for (int g = 0; g < G; ++g) { const float pv = S.p[g][i];
#pragma unroll
          for (int k = 0; k < 4; ++k) accH[g][k] += pv * d[k]; }
      } else {
#pragma unroll
        for (int g = 0; g < G; ++g) { const float pv = S.p[g][i];
#pragma unroll
          for (int k = 0; k < 4; ++k) accI[g][k] += pv * d[k]; }
      }
    }
    __syncthreads();
  }
  // fold the 8 token slices, inverse-transform the classes, store the partial
  for (int r = 0; r < 8; ++r) {   // in slice order: the sum does not depend on scheduling
    if (hw == r) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float4* pI = reinterpret_cast<float4*>(&S.acc[0][g][4 * l32]);
        float4* pH = reinterpret_cast<float4*>(&S.acc[1][g][4 * l32]);
        float4* pF = reinterpret_cast<float4*>(&S.acc[2][g][4 * l32]);
        float4 a = *pI, bh = *pH, cf = *pF;
        a.x += accI[g][0]; a.y += accI[g][1]; a.z += accI[g][2]; a.w += accI[g][3];
        bh.x += accH[g][0]; bh.y += accH[g][1]; bh.z += accH[g][2]; bh.w += accH[g][3];
        cf.x += accF[g][0]; cf.y += accF[g][1]; cf.z += accF[g][2]; cf.w += accF[g][3];
        *pI = a; *pH = bh; *pF = cf;
      }
    }
    __syncthreads();
  }
  for (int g = hw; g < G; g += 8) {
    const float4 a = *reinterpret_cast<const float4*>(&S.acc[0][g][4 * l32]);
    const float4 bh = *reinterpret_cast<const float4*>(&S.acc[1][g][4 * l32]);
    const float4 cf = *reinterpret_cast<const float4*>(&S.acc[2][g][4 * l32]);
    float yh[4] = {bh.x, bh.y, bh.z, bh.w}, yf[4] = {cf.x, cf.y, cf.z, cf.w};
    if (!tail) { fwht<32>(yh, l32); fwht<128>(yf, l32); }
    *reinterpret_cast<float4*>(op + g * 128 + 4 * l32) = make_float4(a.x + yh[0] + yf[0], a.y + yh[1] + yf[1], a.z + yh[2] + yf[2], a.w + yh[3] + yf[3]);
  }
  if (hw < G && l32 == 0) { mlp[2 * hw] = m_run; mlp[2 * hw + 1] = l_run; }
}

__global__ void __launch_bounds__(128) k_merge(const float* __restrict__ opart, const float* __restrict__ ml, int Hkv, int G,
                                               int NS, uint16_t* __restrict__ out, long long out_rs) {
  const int b = blockIdx.x, hq = blockIdx.y, h = hq / G, g = hq % G;
  const long long p0 = (static_cast<long long>(b) * Hkv + h) * (NS + 1);
  float M = -INFINITY;
  for (int s = 0; s <= NS; ++s) M = fmaxf(M, ml[((p0 + s) * G + g) * 2]);
  float o = 0.f, L = 0.f;
  if (M != -INFINITY) {
    for (int s = 0; s <= NS; ++s) {
      const float m = ml[((p0 + s) * G + g) * 2];
      if (m == -INFINITY) continue;
      const float f = exp2f(m - M);
      L += f * ml[((p0 + s) * G + g) * 2 + 1];
      o += f * opart[((p0 + s) * G + g) * 128 + threadIdx.x];
    }
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  out[static_cast<long long>(b) * out_rs + static_cast<long long>(hq) * 128 + threadIdx.x] = static_cast<uint16_t>(bf16_rn(o * inv));
}

template <int G>
int attn_g(const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs, const void* cached, int kv_start,
           int B, int Hkv, int NS, int chunk, float qscale, const void* ring, const void* tail_len, const void* tail_idx,
           int T, void* opart, void* ml, hipStream_t st) {
  static bool attr = false;
  if (!attr) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_attn<G>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(sizeof(ASmem<G>))) != hipSuccess) return 1;
    attr = true;
  }
  hipLaunchKernelGGL(k_attn<G>, dim3(B, Hkv, NS + 1), dim3(256), sizeof(ASmem<G>), st, static_cast<const uint16_t*>(q), q_rs,
                     static_cast<const uint8_t*>(pool), static_cast<const int*>(bt), bt_rs, static_cast<const int*>(cached),
                     kv_start, Hkv, NS, chunk, qscale, static_cast<const uint16_t*>(ring), static_cast<const int*>(tail_len),
                     static_cast<const int*>(tail_idx), T, static_cast<float*>(opart), static_cast<float*>(ml));
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

int launched(int rc, const char* what) {
  if (rc == 1) std::snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(hipGetLastError()));
  return rc;
}

}  // namespace
}  // namespace frkv

using namespace frkv;

extern "C" {

int kv_abi_version(void) { return 9; }
const char* kv_last_error(void) { return g_err; }
int kv_chunk_bytes(int D) { return 12 * D + 16; }
int kv_chunk_bytes8(int D) { return 10 * D; }

int kv_v_write(const void* kv, long long kv_rs, int n, int Hkv, int D, const void* slots, const void* co, const void* M,
               void* pool, int ident, const void* vfix, int f8, void* stream) {
  if (n <= 0) return 0;
  if (D != 128) return bad("kv_v_write: head dim 128 only");
  if (f8) return bad("kv_v_write: FP8-meta pages are not built");
  if (M != nullptr) return bad("kv_v_write: matrix weighting M is not built (diag co only)");
  return launched(v_write_launch(kv, kv_rs, n, Hkv, static_cast<const long long*>(slots), static_cast<const float*>(co),
                                 static_cast<uint8_t*>(pool), ident, static_cast<const int*>(vfix),
                                 static_cast<hipStream_t>(stream)), "kv_v_write");
}

int kv_k_encode(const void* src, long long src_rs, const void* src2, long long src2_rs, const void* sidx,
                const void* dslot, int N, int Hkv, int D, const void* qs, const void* lz, int NQ, float qsc, void* pool,
                int ident, const void* kfix, int f8, void* stream) {
  if (N <= 0) return 0;
  if (D != 128) return bad("kv_k_encode: head dim 128 only");
  if (f8) return bad("kv_k_encode: FP8-meta pages are not built");
  return launched(k_encode_launch(src, src_rs, src2, src2_rs, static_cast<const long long*>(sidx),
                                  static_cast<const long long*>(dslot), N, Hkv, static_cast<const float*>(qs),
                                  static_cast<const float*>(lz), NQ, qsc, static_cast<uint8_t*>(pool), ident,
                                  static_cast<const int*>(kfix), static_cast<hipStream_t>(stream)), "kv_k_encode");
}

int kv_attn(const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs, const void* cached,
            int kv_start, int B, int Hkv, int G, int D, int NS, int chunk, float qscale, const void* ring,
            const void* tail_len, const void* tail_idx, int T, void* opart, void* ml, void* out, long long out_rs, int f8,
            void* stream) {
  if (B <= 0) return 0;
  if (G > 8 || G < 1 || chunk % 32 || chunk <= 0) { std::snprintf(g_err, sizeof(g_err), "kv_attn: G %d chunk %d", G, chunk); return 2; }
  if (D != 128) return bad("kv_attn: head dim 128 only");
  if (f8 & 1) return bad("kv_attn: FP8-meta pages are not built");
  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc;
#define FRKV_G(GG) case GG: rc = attn_g<GG>(q, q_rs, pool, bt, bt_rs, cached, kv_start, B, Hkv, NS, chunk, qscale, ring, tail_len, tail_idx, T, opart, ml, st); break;
  switch (G) {
    FRKV_G(1) FRKV_G(2) FRKV_G(3) FRKV_G(4) FRKV_G(5) FRKV_G(6) FRKV_G(7) FRKV_G(8)
    default: rc = 2;
  }
#undef FRKV_G
  if (rc) return launched(rc, "kv_attn");
  hipLaunchKernelGGL(k_merge, dim3(B, Hkv * G), dim3(128), 0, st, static_cast<const float*>(opart), static_cast<const float*>(ml),
                     Hkv, G, NS, static_cast<uint16_t*>(out), out_rs);
  return launched(hipPeekAtLastError() == hipSuccess ? 0 : 1, "kv_attn (merge)");
}

int kv_dequant(const void* pool, const void* bt, int g0, int g1, int nvalid, int Hkv, int D, int fp32, void* ok, void* ov,
               int f8, void* stream) {
  if (g1 <= g0) return 0;
  if (D != 128) return bad("kv_dequant: head dim 128 only");
  if (f8 & 1) return bad("kv_dequant: FP8-meta pages are not built");
  return launched(dequant_launch(static_cast<const uint8_t*>(pool), static_cast<const int*>(bt), g0, g1, nvalid, Hkv, fp32, ok,
                                 ov, static_cast<hipStream_t>(stream)), "kv_dequant");
}

int kv_lse_merge(const void* oa, const void* la, long long la_hs, const void* ob, const void* lb, long long lb_hs,
                 void* out, long long out_rs, int na, int H, int D, void* stream) {
  if (na <= 0) return 0;
  return launched(lse_merge_launch(oa, static_cast<const float*>(la), la_hs, ob, static_cast<const float*>(lb), lb_hs, out,
                                   out_rs, na, H, D, static_cast<hipStream_t>(stream)), "kv_lse_merge");
}

}  // extern "C"
