// Paged split-K decode attention over KIVI-style FlagRot INT2 pages for gfx950 (wave64, matrix pipe for both products):
// the page splits and the BF16 ring rows (one more split).  (The split merge and the C ABI live in kivi_attn.hip.)
//
// Workgroup = 4 wavefronts per (sequence, KV head with its whole GQA group of up to 8 query heads, split); a wavefront
// owns whole 32-token groups (two pages) and keeps its own running maxima, sums and accumulators; the wavefronts are
// merged through LDS at the end.  Per group:
//   q' * scale   lane = channel pair: the group's channel scales times the query rotation the group's flags select
//                (identity / H32 per sub-vector / H128; the three rotations are made once per workgroup and kept as
//                fp16 value + fp16 remainder: 22 bits).  The product enters the matrix pipe as TWO fp16 operands per
//                channel: the rounded product and its exact remainder (one packed fused multiply-add gives it: the
//                product of two fp16 numbers has 22 bits, the rounded product takes the upper 11), plus the
//                remainder part of the query -- so the scores carry no 2^-11 rounding of terms that can be a hundred
//                times larger than their sum (heavy outlier channels).  Written to two LDS strips (values, remainders).
//   bias         sum q' * min per (group, head): four more matrix products whose A operand is the channel mins (the
//                same for every token row, from a 256-byte LDS strip) and whose B operand is the query rotation
//                itself, value and remainder, straight from the workgroup's table -- exact fp16 x fp16 products summed
//                in fp32, no per-head vector work; added to the scores as one term per lane.
//   scores       v_mfma_f32_16x16x32_f16, rows = the 16 tokens of a page, columns = heads (0..7 against the value
//                strips, 8..15 against the remainder strips; the two halves are added afterwards), 128 channels in
//                four steps per page: a 2-bit code field masked in place is an fp16
//                DENORMAL whose value is code * 2^(shift - 24) (the matrix pipe keeps denormal inputs); the power of
//                two is folded into the query operand.
//   softmax      exp2-domain, lane = (head, 8 tokens); the running maximum is re-reduced only when some token beats it.
//   values       v_mfma_f32_32x32x16_f16, rows = the 32 channels of a sub-vector, columns = (class, head) with class =
//                stored as is / H32 / H128, 32 tokens in two steps.  B = p * scale of the token if it belongs to the
//                column's class, else 0 (class-masked scale strips written by the token lanes); A = the tokens' code
//                bytes (transposed through LDS as zero-extended 16-bit values, so a 128-bit read is four token pairs)
//                masked in place to the row's 2-bit field.  sum p * min per (head, class, sub-vector): one more
//                16x16x32 product.  o = accI + H32(accH) + H128(accF) once per workgroup.
// FP8-meta pages (template flag F8; 1280-byte chunks, kivi.cu:28-35): scale and min are E4M3 bytes.  An E4M3 pattern
// shifted left by 7 is the fp16 pattern of value / 256 (same mantissa position, exponent bias 15 instead of 7; E4M3
// subnormals land on fp16 subnormals), so one packed fp16 multiply by 256 -- folded into a factor the f16 path applies
// anyway where there is one -- gives the exact value, and the rest of the loop is shared with the FP16-meta pages.
// Semantics follow integrations/vllm_flagrot/csrc/kivi.cu:729-980 (k_attn).
#include "fr_common.hpp"
#include "kivi_launch.hpp"
#include "kivi_mma.hpp"

namespace frkv {
using namespace fr;
using namespace mma;
namespace {

constexpr int KM_OFF = 512, VF_OFF = 1536;                                     // VF: FP16-meta pages only
template <bool F8> constexpr int CHUNK = F8 ? 1280 : 1552;
template <bool F8> constexpr int VC_OFF = F8 ? 640 : 768;
template <bool F8> constexpr int VM_OFF = F8 ? 1152 : 1280;
constexpr int OROW = 132;                       // floats per row of the merged accumulators: 128 + 4 pad

struct Scr {                                    // per wavefront, rewritten for every 32-token group
  alignas(16) uint32_t qs[GT][QROW];            // fp16 pairs of q' * scale * 2^-shift per (head, channel pair)
  alignas(16) uint32_t ql[GT][QROW];            // fp16 pairs of what the rounding of those products dropped
  alignas(16) uint32_t mn[64];                  // fp16 pair of the channel mins per channel pair
  // rows and blocks padded so that the 128-bit rows one instruction reads fall into different banks
  alignas(16) _Float16 pst[GT][PROW];           // p per (head, token)
  alignas(16) uint16_t vsm[3][4 * 32 + 8];      // value scale (fp16 bits) per (class, sub-vector * 32 + token), 0 off its class
  alignas(16) uint16_t vmm[3][4 * 32 + 8];      // value min likewise
  alignas(16) uint16_t vt[4][8 * PROW + 16];    // value code bytes (zero-extended) per (sub-vector, byte * PROW + token)
};
struct Smem {
  alignas(16) uint32_t qh[3][GT][QROW];         // query rotations as fp16 pairs per (variant, head, channel pair)
  alignas(16) uint32_t qr[3][GT][QROW];         // their remainders (rotation - fp16 value) as fp16 pairs
  union {
    Scr w[4];
    float ob[3][GT][OROW];                      // merged accumulators per class (after the page loop)
  };
  float ams[4][GT][12];                         // per wavefront: sum p * min per (head, class, sub-vector)
  float mw[4][GT], lw[4][GT];
};

struct GroupRegs {
  u32x2 ka, kb;  // lane (token m = lane & 15 of page A / B, quarter kc = lane >> 4): code words 2 kc, 2 kc + 1 of the token
  u32x2 km;      // lane = channel pair: (scale | min << 16) of channels 2 l, 2 l + 1; F8: .x = bytes (s, m, s, m) of the pair
  u32x4 vc;      // lane (token, half): the token's code bytes of sub-vectors 2 half, 2 half + 1
  u32x2 vm;      // lane (token, half): (scale | min << 16) of sub-vectors 2 half, 2 half + 1; F8: .x = bytes (s, m, s, m)
  uint32_t vf;   // the token's whole-head flag: non-zero = H128
};

template <bool F8>
DEVI void load_group(GroupRegs& r, const uint8_t* chA, const uint8_t* chB, int lane) {
  const int t = lane & 31, hh = lane >> 5;
  const uint8_t* cht = t < 16 ? chA : chB;
  r.ka = gload<u32x2>(chA + (lane & 15) * 32 + 8 * (lane >> 4));
  r.kb = gload<u32x2>(chB + (lane & 15) * 32 + 8 * (lane >> 4));
  r.vc = gload<u32x4>(cht + VC_OFF<F8> + (t & 15) * 32 + 16 * hh);
  if (F8) {
    // channels 2 l, 2 l + 1 = slots 2 (l & 1), 2 (l & 1) + 1 of cell l >> 1: four bytes at 4 l
    r.km = u32x2{gload<uint32_t>((lane < 32 ? chA : chB) + KM_OFF + (lane & 31) * 4), 0u};
    r.vm = u32x2{gload<uint32_t>(cht + VM_OFF<true> + (t & 15) * 8 + 4 * hh), 0u};
    r.vf = gload<uint8_t>(cht + KM_OFF + (t & 15) * 8 + 6) & 0x80u;      // bit 7 of the key scale byte in slot 3 of the token's cell
  } else {
    r.km = gload<u32x2>((lane < 32 ? chA : chB) + KM_OFF + (lane & 31) * 8);
    r.vm = gload<u32x2>(cht + VM_OFF<false> + (t & 15) * 16 + 8 * hh);
    r.vf = gload<uint8_t>(cht + VF_OFF + (t & 15));
  }
}

// all-reduce over the 16 lanes of a row (DPP: quad permutes, then the mirrors of 8 and of 16 lanes)
DEVI float row16_max(float v) {
  v = fmaxf(v, dpp_xor1(v)); v = fmaxf(v, dpp_xor2(v));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true)));
  return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true)));
}
DEVI float row16_sum(float v) {
  v += dpp_xor1(v); v += dpp_xor2(v);
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));
  return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));
}
DEVI float lane_value(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// The BF16 ring rows of one sequence (split index NS): rows [0, tail_len) of ring block tail_idx, K row h, V row Hkv + h,
// original basis; same partial format as the page splits.  A wavefront takes 16 rows per step.  Scores on the matrix
// pipe: A = the GQA group's query rows as BF16 (rows G..15 of the operand zero), B = the 16 key rows as they lie in
// memory (a lane's 16 bytes are 8 channels of row lane & 15), four products of 32 channels: lanes 0..15 then hold the
// scores of heads 0..3 for row `lane`, lanes 16..31 those of heads 4..7 -- no cross-lane sums.  One maximum per head
// and step, one exponential per (row, head); the weights pass through LDS (the wavefront's own scratch block, idle in
// this split) and come back as broadcast reads for the value products on the vector pipe, lanes owning 2 dims.
// q and the ring are read 16 bytes at a time (kv_attn checks their alignment).
template <int G>
DEVI void tail_split(Smem& S, const uint16_t* __restrict__ q, long long q_rs, const uint16_t* __restrict__ ring,
                     const int* __restrict__ tail_len, const int* __restrict__ tail_idx, int T, int Hkv, int Gq, int b, int h,
                     int g0, float qscale, float* __restrict__ op, float* __restrict__ mlp) {
  static_assert(G == 8, "two rows of 16 lanes carry the heads");
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
  const int n = tail_len != nullptr ? tail_len[b] : 0;
  if (n <= 0) {
    if (tid < G && g0 + tid < Gq) { mlp[2 * tid] = -INFINITY; mlp[2 * tid + 1] = 0.f; }
    return;
  }
  const int col = lane & 15, kb = lane >> 4;
  uint4 qa[4];
  {
    const bool live = col < G && g0 + col < Gq;
    const uint16_t* qr = q + static_cast<long long>(b) * q_rs + (static_cast<long long>(h) * Gq + (live ? g0 + col : 0)) * 128 + 8 * kb;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint4 v = *reinterpret_cast<const uint4*>(qr + 32 * s);
      qa[s] = live ? v : make_uint4(0u, 0u, 0u, 0u);
    }
  }
  // the lane's four heads 4 kb + i (kb < 2; the other lanes carry the operand's zero rows): maxima (alike over the
  // lane's row of 16), column sums of the weights
  float mr[4], lp[4], oa[G], ob[G];
#pragma unroll
  for (int i = 0; i < 4; ++i) { mr[i] = -INFINITY; lp[i] = 0.f; }
#pragma unroll
  for (int g = 0; g < G; ++g) oa[g] = ob[g] = 0.f;
  float* pw = reinterpret_cast<float*>(&S.w[wv]);            // [head quad kb][row][4]
  const uint16_t* rbase = ring + static_cast<long long>(tail_idx != nullptr ? tail_idx[b] : 0) * T * 2 * Hkv * 128;
  const long long rs = 2ll * Hkv * 128;
  for (int t0 = wv * 16; t0 < n; t0 += 64) {
    const uint16_t* kr = rbase + min(t0 + col, n - 1) * rs + h * 128 + 8 * kb;
    uint4 kk[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) kk[s] = *reinterpret_cast<const uint4*>(kr + 32 * s);
    uint32_t vr[16];
#pragma unroll
    for (int r = 0; r < 16; ++r)
      vr[r] = *reinterpret_cast<const uint32_t*>(rbase + min(t0 + r, n - 1) * rs + (Hkv + h) * 128 + 2 * lane);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s)
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, qa[s]), __builtin_bit_cast(bf16x8, kk[s]), acc, 0, 0, 0);
    const bool in = t0 + col < n;
    float pe[4], al[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float sc = in ? acc[i] * qscale : -INFINITY;
      const float mn = fmaxf(mr[i], row16_max(sc));          // a number: row t0 exists
      al[i] = fexp2(mr[i] - mn);
      pe[i] = fexp2(sc - mn);
      mr[i] = mn;
      lp[i] = lp[i] * al[i] + pe[i];
    }
    if (lane < 32) *reinterpret_cast<float4*>(pw + 4 * lane) = make_float4(pe[0], pe[1], pe[2], pe[3]);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float a = lane_value(al[g & 3], 16 * (g >> 2));
      oa[g] *= a; ob[g] *= a;
    }
    wave_lds_sync();
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float4 w0 = *reinterpret_cast<const float4*>(pw + 4 * r);
      const float4 w1 = *reinterpret_cast<const float4*>(pw + 64 + 4 * r);
      const float v0 = bf16_lo(vr[r]), v1 = bf16_hi(vr[r]);
      oa[0] += w0.x * v0; ob[0] += w0.x * v1; oa[1] += w0.y * v0; ob[1] += w0.y * v1;
      oa[2] += w0.z * v0; ob[2] += w0.z * v1; oa[3] += w0.w * v0; ob[3] += w0.w * v1;
      oa[4] += w1.x * v0; ob[4] += w1.x * v1; oa[5] += w1.y * v0; ob[5] += w1.y * v1;
      oa[6] += w1.z * v0; ob[6] += w1.z * v1; oa[7] += w1.w * v0; ob[7] += w1.w * v1;
    }
    wave_lds_sync();      // the weights have been read before the next step replaces them
  }
  float m[G], l[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = lane_value(mr[g & 3], 16 * (g >> 2));
    l[g] = lane_value(row16_sum(lp[g & 3]), 16 * (g >> 2));
  }
  if (lane == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g) { S.mw[wv][g] = m[g]; S.lw[wv][g] = l[g]; }
  }
  __syncthreads();
  for (int r = 0; r < 4; ++r) {
    if (wv == r) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float M = fmaxf(fmaxf(S.mw[0][g], S.mw[1][g]), fmaxf(S.mw[2][g], S.mw[3][g]));
        const float f = m[g] == -INFINITY ? 0.f : fexp2(m[g] - M);
        float2* dst = reinterpret_cast<float2*>(&S.ob[0][g][2 * lane]);
        float2 acc = make_float2(0.f, 0.f);
        if (r) acc = *dst;
        *dst = make_float2(acc.x + f * oa[g], acc.y + f * ob[g]);
      }
    }
    __syncthreads();
  }
  for (int g = wv; g < G && g0 + g < Gq; g += 4) {
    *reinterpret_cast<float2*>(op + g * 128 + 2 * lane) = *reinterpret_cast<const float2*>(&S.ob[0][g][2 * lane]);
    if (lane == 0) {
      const float M = fmaxf(fmaxf(S.mw[0][g], S.mw[1][g]), fmaxf(S.mw[2][g], S.mw[3][g]));
      float L = 0.f;
      for (int w = 0; w < 4; ++w) L += S.mw[w][g] == -INFINITY ? 0.f : fexp2(S.mw[w][g] - M) * S.lw[w][g];
      mlp[2 * g] = M; mlp[2 * g + 1] = L;
    }
  }
}

template <bool F8>
__global__ void __launch_bounds__(256, 3) k_attn_pages(const uint16_t* __restrict__ q, long long q_rs,
                                                    const uint8_t* __restrict__ pool, const int* __restrict__ bt,
                                                    long long bt_rs, const int* __restrict__ cached, int kv_start, int Hkv,
                                                    int NS, int chunk, float qscale, float* __restrict__ opart,
                                                    float* __restrict__ ml, int Gq,
                                                    const uint16_t* __restrict__ ring, const int* __restrict__ tail_len,
                                                    const int* __restrict__ tail_idx, int T) {
  constexpr int G = GT;
  extern __shared__ __align__(16) uint8_t lds[];
  Smem& S = *reinterpret_cast<Smem*>(lds);
  const int b = blockIdx.x, h = blockIdx.y, g0 = 0, sp = blockIdx.z;
  const int tid = threadIdx.x, wv = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
  const long long pidx = (static_cast<long long>(b) * Hkv + h) * (NS + 1) + sp;
  float* op = opart + pidx * Gq * 128;
  float* mlp = ml + pidx * Gq * 2;
  if (sp == NS) {
    tail_split<G>(S, q, q_rs, ring, tail_len, tail_idx, T, Hkv, Gq, b, h, g0, qscale, op, mlp);
    return;
  }
  const int t0 = max(sp * chunk, kv_start), t1 = min((sp + 1) * chunk, cached[b]);
  if (t1 <= t0) {
    if (tid < Gq) { mlp[2 * tid] = -INFINITY; mlp[2 * tid + 1] = 0.f; }
    return;
  }
  // query rotations: half wave per (variant, head); heads past the group are zero
  for (int r = tid >> 5; r < 3 * G; r += 8) {
    const int var = r / G, g = r % G, lq = tid & 31;
    float x[4] = {0.f, 0.f, 0.f, 0.f};
    if (g < Gq) {
      const uint2 raw = *reinterpret_cast<const uint2*>(q + static_cast<long long>(b) * q_rs + (static_cast<long long>(h) * Gq + g) * 128 + 4 * lq);
      x[0] = bf16_lo(raw.x); x[1] = bf16_hi(raw.x); x[2] = bf16_lo(raw.y); x[3] = bf16_hi(raw.y);
    }
    if (var == 1) fwht<32>(x, lq);
    if (var == 2) fwht<128>(x, lq);
    {
      const uint32_t h01 = pack_rn(x[0], x[1]), h23 = pack_rn(x[2], x[3]);
      const uint32_t l01 = pack_rn(x[0] - f16_value(h01 & 0xFFFFu), x[1] - f16_value(h01 >> 16));
      const uint32_t l23 = pack_rn(x[2] - f16_value(h23 & 0xFFFFu), x[3] - f16_value(h23 >> 16));
      *reinterpret_cast<u32x2*>(&S.qh[var][g][2 * lq]) = u32x2{h01, h23};
      *reinterpret_cast<u32x2*>(&S.qr[var][g][2 * lq]) = u32x2{l01, l23};
    }
  }
  __syncthreads();

  Scr& W = S.w[wv];
  // Score layout: lane = (head sn = lane & 15 (heads 8..15 repeat 0..7 and are ignored), token quarter kc = lane >> 4);
  // value layout: lane = (column vn = lane & 31 = (class vn >> 3, head vn & 7; columns 24..31 ignored), token half lane >> 5).
  const int sn = lane & 15, kc = lane >> 4, sh = sn & 7;
  const int vcl = min(l32 >> 3, 2), vh = l32 & 7;
  float m_run = -INFINITY, l_run = 0.f;          // of head sh, over this lane's tokens
  f32x16 accv[4];                                // [sub-vector]: rows = the 32 channels, this lane's column; codes * 2^-24 * 2^(2 field)
  f32x4 amd = {0.f, 0.f, 0.f, 0.f};              // score layout: sum p * min, rows = heads 4 kc + r, column sn = (class sn >> 2, sub-vector sn & 3)
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma unroll
    for (int i = 0; i < 16; ++i) accv[j][i] = 0.f;
  }
  const int* btb = bt + static_cast<long long>(b) * bt_rs;
  const int g_first = t0 / 32, g_end = (t1 + 31) / 32;
  // power of two folded into the query operand of this lane's channel pair (pair k = lane & 7 of its word):
  // fields 0..4 are masked in place (code * 2^(2k - 24)), fields 5..7 after a shift by 10 (code * 2^(2(k-5) - 24))
  const int kq = lane & 7;
  const float qfold = __uint_as_float((127u - 2u * static_cast<uint32_t>(kq < 5 ? kq : kq - 5)) << 23);
  const uint32_t vmask = 0x00030003u << (2 * (l32 & 3));      // value layout row = channel l32: field l32 & 3 of byte l32 >> 2
  const uint32_t qfold8 = pack_rn(256.f * qfold, 256.f * qfold);

  GroupRegs cur;
  int gi = g_first + wv;
  if (gi < g_end) load_group<F8>(cur, pool + (static_cast<long long>(btb[2 * gi]) * Hkv + h) * CHUNK<F8>,
                                 pool + (static_cast<long long>(btb[2 * gi + 1]) * Hkv + h) * CHUNK<F8>, lane);
  for (; gi < g_end; gi += 4) {
    const bool full = gi * 32 >= t0 && gi * 32 + 32 <= t1;     // every token of the group is inside the range (wave uniform)
    // The next group is requested on every path (past the range: the range's last group again, a cache hit nobody
    // uses).  Were the requests inside a branch, the wait counts after the join would be those of the path without
    // them, and this group's first use would wait for the next group's data as well.
    GroupRegs nxt;
    {
      const int gn = min(gi + 4, g_end - 1);
      load_group<F8>(nxt, pool + (static_cast<long long>(btb[2 * gn]) * Hkv + h) * CHUNK<F8>,
                     pool + (static_cast<long long>(btb[2 * gn + 1]) * Hkv + h) * CHUNK<F8>, lane);
    }
    // ---- group flags; q' * scale strip and the channel mins: lane = channel pair
    int wkc;                                    // the rotation this lane's B operands of the bias product come from
    {
      // flag channels: 0 .. 3 and 4 (F8: 0, 4, 8, 12 and 16, the first byte of lanes 0, 2, 4, 6 and 8)
      const uint32_t s0 = __builtin_amdgcn_readlane(cur.km.x, 0), s1 = F8 ? __builtin_amdgcn_readlane(cur.km.x, 2) : __builtin_amdgcn_readlane(cur.km.y, 0),
                     s2 = __builtin_amdgcn_readlane(cur.km.x, F8 ? 4 : 1), s3 = F8 ? __builtin_amdgcn_readlane(cur.km.x, 6) : __builtin_amdgcn_readlane(cur.km.y, 1),
                     s4 = __builtin_amdgcn_readlane(cur.km.x, F8 ? 8 : 2);
      constexpr int FB = F8 ? 7 : 15;
      const bool useF = (s4 >> FB) & 1u;
      const uint32_t lmask = ((s0 >> FB) & 1u) | (((s1 >> FB) & 1u) << 1) | (((s2 >> FB) & 1u) << 2) | (((s3 >> FB) & 1u) << 3);
      const int which = useF ? 2 : static_cast<int>((lmask >> (lane >> 4)) & 1u);
      // fp16 products of the fp16 query pair with (scale * 2^-shift) and with min
      uint32_t spair, mpair;
      if (F8) {
        const uint32_t mb = (cur.km.x >> 8) & 0x00FF00FFu;
        spair = pk_mul((cur.km.x & 0x007F007Fu) << 7, qfold8);
        mpair = pk_mul(((mb & 0x007F007Fu) << 7) | ((mb & 0x00800080u) << 8), X256);
      } else {
        spair = pack_rn(f16_value(cur.km.x & 0x7FFFu) * qfold, f16_value(cur.km.y & 0x7FFFu) * qfold);
        mpair = (cur.km.x >> 16) | (cur.km.y & 0xFFFF0000u);
      }
      wkc = useF ? 2 : static_cast<int>((lmask >> kc) & 1u);               // sub-vector kc = channel pairs 16 kc .. 16 kc + 15
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const uint32_t qv = S.qh[which][g][lane], qrem = S.qr[which][g][lane];
        const uint32_t b1 = pk_mul(qv, spair);
        const uint32_t rem = pk_fma(qv, spair, b1 ^ 0x80008000u);        // exact: what the rounding of b1 dropped
        W.qs[g][lane] = b1;
        W.ql[g][lane] = pk_fma(qrem, spair, rem);
      }
      W.mn[lane] = mpair;
    }
    // ---- value strips: lane = (token l32, half hh) serves sub-vectors 2 hh, 2 hh + 1.  Scale and min go to the strip of
    //      the token's class (0 in the other two; tokens outside the range have no class), the code bytes to byte rows.
    // Groups that hold a value scale above WIDE_SCALE (wave uniform) keep their scales times 2^-8 in the strips and
    // run a second pass of value products (below, where the reason is given).
    bool wide_scales;
    {
      const int pos = gi * 32 + l32;
      const bool vF = cur.vf != 0;
      uint32_t w2[2];                                  // fp16 scale (bit 15 = H32) | fp16 min << 16 of sub-vectors 2 hh, 2 hh + 1
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        if (F8) {
          const uint32_t b2 = jj ? cur.vm.x >> 16 : cur.vm.x;                         // s8 | m8 << 8
          w2[jj] = pk_mul(((b2 & 0x7Fu) << 7) | ((b2 & 0x7F00u) << 15) | ((b2 & 0x8000u) << 16), X256) | ((b2 & 0x80u) << 8);
        } else w2[jj] = jj ? cur.vm.y : cur.vm.x;
      }
      wide_scales = __any(max(w2[0] & 0x7FFFu, w2[1] & 0x7FFFu) > WIDE_SCALE);
      const uint32_t sfold = wide_scales ? 0x1C00u : 0x3C00u;                          // fp16 2^-8 or 1
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const uint32_t w = w2[jj];
        const int j = 2 * hh + jj;
        int cls = vF ? 2 : static_cast<int>((w >> 15) & 1u);
        if (!full) cls = (pos >= t0 && pos < t1) ? cls : 3;
        const uint16_t sc16 = static_cast<uint16_t>(pk_mul(w & 0x7FFFu, sfold));
#pragma unroll
        for (int c = 0; c < 3; ++c) {
          W.vsm[c][32 * j + l32] = cls == c ? sc16 : static_cast<uint16_t>(0);
          W.vmm[c][32 * j + l32] = cls == c ? static_cast<uint16_t>(w >> 16) : static_cast<uint16_t>(0);
        }
        const uint32_t c0 = jj ? cur.vc.z : cur.vc.x, c1 = jj ? cur.vc.w : cur.vc.y;
        // bytes 0, 1 and 2, 3 of a word side by side in the two halves of one register: one permute per pair
        const uint32_t c01 = __builtin_amdgcn_perm(0u, c0, 0x0C010C00u), c23 = __builtin_amdgcn_perm(0u, c0, 0x0C030C02u);
        const uint32_t c45 = __builtin_amdgcn_perm(0u, c1, 0x0C010C00u), c67 = __builtin_amdgcn_perm(0u, c1, 0x0C030C02u);
        uint16_t* vt = &W.vt[j][l32];
        vt[0 * PROW] = static_cast<uint16_t>(c01); vt[1 * PROW] = static_cast<uint16_t>(c01 >> 16);
        vt[2 * PROW] = static_cast<uint16_t>(c23); vt[3 * PROW] = static_cast<uint16_t>(c23 >> 16);
        vt[4 * PROW] = static_cast<uint16_t>(c45); vt[5 * PROW] = static_cast<uint16_t>(c45 >> 16);
        vt[6 * PROW] = static_cast<uint16_t>(c67); vt[7 * PROW] = static_cast<uint16_t>(c67 >> 16);
      }
    }
    wave_lds_sync();
    // ---- bias: sum q' * min of head sh (every row of the product is that sum)
    float bq;
    {
      // columns 0..7 of the product take the rotations' values, columns 8..15 their remainders: one product where
      // there were two, and the halves of a row of 16 lanes are added afterwards
      f32x4 bacc = {0.f, 0.f, 0.f, 0.f};
      const uint32_t* qsel = sn < 8 ? &S.qh[wkc][sh][0] : &S.qr[wkc][sh][0];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const u32x4 m4 = *reinterpret_cast<const u32x4*>(&W.mn[16 * kc + 4 * s]);
        const u32x4 q0 = *reinterpret_cast<const u32x4*>(qsel + 16 * kc + 4 * s);
        bacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, m4), __builtin_bit_cast(half8, q0), bacc, 0, 0, 0);
      }
      bq = (bacc[0] + ror8(bacc[0])) * qscale;
    }
    // ---- scores on the matrix pipe: rows = the 16 tokens of a page, columns = heads, 128 channels in four steps of 32.
    //      A code field masked in place is an fp16 denormal (code * 2^(shift - 24)); the bias sum q' * min enters as
    //      2^-24 * (q' * min) through the same accumulators.
    f32x4 sa0, sa1;
    {
      sa0 = f32x4{0.f, 0.f, 0.f, 0.f}; sa1 = sa0;
      const uint32_t* bsel = sn < 8 ? &W.qs[sh][0] : &W.ql[sh][0];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const uint32_t wa = (s >> 1) ? cur.ka.y : cur.ka.x, wb = (s >> 1) ? cur.kb.y : cur.kb.x;
        u32x4 xa, xb;
        if (s & 1) {
          const uint32_t wa10 = wa >> 10, wb10 = wb >> 10;
          xa = u32x4{wa & 0x03000300u, wa10 & 0x00030003u, wa10 & 0x000C000Cu, wa10 & 0x00300030u};
          xb = u32x4{wb & 0x03000300u, wb10 & 0x00030003u, wb10 & 0x000C000Cu, wb10 & 0x00300030u};
        } else {
          xa = u32x4{wa & 0x00030003u, wa & 0x000C000Cu, wa & 0x00300030u, wa & 0x00C000C0u};
          xb = u32x4{wb & 0x00030003u, wb & 0x000C000Cu, wb & 0x00300030u, wb & 0x00C000C0u};
        }
        // the code operands against the products (columns 0..7) and against their remainders (columns 8..15)
        const u32x4 b0 = *reinterpret_cast<const u32x4*>(bsel + 16 * kc + 4 * s);
        sa0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, xa), __builtin_bit_cast(half8, b0), sa0, 0, 0, 0);
        sa1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, xb), __builtin_bit_cast(half8, b0), sa1, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) { sa0[i] += ror8(sa0[i]); sa1[i] += ror8(sa1[i]); }      // value part + remainder part
    }
    // ---- softmax: lane = (head sh, tokens 4 kc + r of page A (columns 0..7) or of page B (columns 8..15))
    {
      // after the halves were added both column halves hold the totals: the lanes of columns 0..7 go on with page A's
      // four tokens, those of columns 8..15 with page B's
      const int pgb = sn >> 3;
      float sc[4];                       // raw accumulators: score = sc * 2^24 * qscale (a positive factor)
      const float up = 16777216.f * qscale;
#pragma unroll
      for (int i = 0; i < 4; ++i) sc[i] = pgb ? sa1[i] : sa0[i];
      if (!full) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int pos = gi * 32 + 16 * pgb + 4 * kc + i;
          sc[i] = (pos >= t0 && pos < t1) ? sc[i] : -INFINITY;
        }
      }
      float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])) * up + bq;
      if (__any(mx > m_run)) {
        mx = fmaxf(mx, ror8(mx));
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mn = fmaxf(m_run, mx);
        const float alpha = m_run == -INFINITY ? 0.f : fexp2(m_run - mn);
        m_run = mn;
        l_run *= alpha;
        const float av = __shfl(alpha, vh, 64);          // the factor of this lane's value column (head vh)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
          for (int i = 0; i < 16; ++i) accv[j][i] *= av;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) amd[r] *= __shfl(alpha, 4 * kc + r, 64);      // rows = heads 4 kc + r (8..15 repeat 0..7)
      }
      // a wavefront's group always holds a token of the range: the maximum is finite from its first group on
      float p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p[i] = fexp2(__builtin_fmaf(sc[i], up, bq - m_run));
        l_run += p[i];
      }
      *reinterpret_cast<u32x2*>(&W.pst[sh][16 * pgb + 4 * kc]) = u32x2{pack_rn(p[0], p[1]), pack_rn(p[2], p[3])};
    }
    wave_lds_sync();
    // ---- values on the matrix pipe: rows = the 32 channels of a sub-vector, columns = (class, head), 32 tokens in two
    //      steps of 16; B = p * scale of the column's class (0 for tokens of another class), A = the tokens' code fields
    //      masked in place.  sum p * min per (class, head, sub-vector) by v_dot2.
    {   // sum p * min: rows = heads, columns = (class, sub-vector), the 32 tokens in one step
      const u32x4 pa = *reinterpret_cast<const u32x4*>(&W.pst[sh][8 * kc]);
      const u32x4 mb = *reinterpret_cast<const u32x4*>(&W.vmm[min(sn >> 2, 2)][32 * (sn & 3) + 8 * kc]);
      amd = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, pa), __builtin_bit_cast(half8, mb), amd, 0, 0, 0);
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int tk = 16 * s + 8 * hh;
      const u32x4 pr = *reinterpret_cast<const u32x4*>(&W.pst[vh][tk]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const u32x4 sv = *reinterpret_cast<const u32x4*>(&W.vsm[vcl][32 * j + tk]);
        const u32x4 by = *reinterpret_cast<const u32x4*>(&W.vt[j][(l32 >> 2) * PROW + tk]);     // (token 2 i | token 2 i + 1 << 16) per word
        const u32x4 bo = u32x4{pk_mul(pr.x, sv.x), pk_mul(pr.y, sv.y), pk_mul(pr.z, sv.z), pk_mul(pr.w, sv.w)};
        const u32x4 ao = u32x4{by.x & vmask, by.y & vmask, by.z & vmask, by.w & vmask};
        accv[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, ao), __builtin_bit_cast(half8, bo), accv[j], 0, 0, 0);
      }
    }
    // The code fields enter the matrix pipe as fp16 denormals (a field masked in place is code * 2^(2 f - 24)).  The pipe
    // aligns the addends of an instruction -- products and accumulator -- to the largest NOMINAL exponent, for which a
    // denormal counts as 2^-14 whatever its leading zeros, and keeps 24 bits from there: 14.6 + 2 f bits below the
    // largest product survive.  Ordinary data is far inside the bar with that.  A token whose p * scale is hundreds of
    // times its neighbours' (a row scaled x200) lifts the window of its whole instruction: neighbours and accumulator
    // lose up to 2^-13 / 4^f of ITS p * scale, 0.08 at scale 680, which shows where the exact output is near zero.
    // In such groups the strips hold scale * 2^-8, so the products above came to 1/256 of their value with the window
    // 8 bits lower; here the other 255/256 follow with the code operands times 255 (exact: 10 bits), and what the fp16
    // rounding of p * scale dropped (one fused multiply-add per pair, exact) with the code operands times 256.
    if (__builtin_expect(wide_scales, 0)) {
      // (the strips are read again through an offset the compiler cannot see through: recognised as the reads of the
      // pass above, they would keep every operand of that pass in registers until here)
      int again = 0;
      asm volatile("" : "+s"(again));
      constexpr uint32_t X255 = 0x5BF85BF8u;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int tk = 16 * s + 8 * hh + again;
        const u32x4 pr = *reinterpret_cast<const u32x4*>(&W.pst[vh][tk]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const u32x4 sv = *reinterpret_cast<const u32x4*>(&W.vsm[vcl][32 * j + tk]);
          const u32x4 by = *reinterpret_cast<const u32x4*>(&W.vt[j][(l32 >> 2) * PROW + tk]);
          const u32x4 bo = u32x4{pk_mul(pr.x, sv.x), pk_mul(pr.y, sv.y), pk_mul(pr.z, sv.z), pk_mul(pr.w, sv.w)};
          const u32x4 br = u32x4{pk_fma(pr.x, sv.x, bo.x ^ 0x80008000u), pk_fma(pr.y, sv.y, bo.y ^ 0x80008000u),
                                 pk_fma(pr.z, sv.z, bo.z ^ 0x80008000u), pk_fma(pr.w, sv.w, bo.w ^ 0x80008000u)};
          const u32x4 ao = u32x4{by.x & vmask, by.y & vmask, by.z & vmask, by.w & vmask};
          const u32x4 a255 = u32x4{pk_mul(ao.x, X255), pk_mul(ao.y, X255), pk_mul(ao.z, X255), pk_mul(ao.w, X255)};
          const u32x4 a256 = u32x4{pk_mul(ao.x, X256), pk_mul(ao.y, X256), pk_mul(ao.z, X256), pk_mul(ao.w, X256)};
          accv[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a255), __builtin_bit_cast(half8, bo), accv[j], 0, 0, 0);
          accv[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a256), __builtin_bit_cast(half8, br), accv[j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);      // one step's operands at a time: this path is rare and must not claim registers
        }
      }
    }
    wave_lds_sync();
    cur = nxt;
  }

  // ---- merge of the wavefronts: maxima, sums, accumulators per class (in wavefront order), inverse transforms
  {
    float lt = l_run + ror8(l_run);
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    if (lane < G) { S.mw[wv][lane] = m_run; S.lw[wv][lane] = lt; }
    if (sn < 12 && kc < 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r) S.ams[wv][4 * kc + r][sn] = amd[r];
    }
  }
  __syncthreads();          // every wavefront is done with its strips: the merged accumulators take their place
  float fac;
  {
    const float M = fmaxf(fmaxf(S.mw[0][vh], S.mw[1][vh]), fmaxf(S.mw[2][vh], S.mw[3][vh]));
    const float mine = S.mw[wv][vh];
    fac = mine == -INFINITY ? 0.f : fexp2(mine - M);
  }
  for (int r = 0; r < 4; ++r) {
    if (wv == r && l32 < 24) {
      float* orow = &S.ob[l32 >> 3][vh][0];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float mj = S.ams[wv][vh][4 * (l32 >> 3) + j];
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          float4* dst = reinterpret_cast<float4*>(orow + 32 * j + 8 * i4 + 4 * hh);      // row = 8 (i >> 2) + 4 hh + (i & 3)
          float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
          if (r) acc = *dst;
          // field f = i & 3 of its byte: code * 2^(2 f - 24) was accumulated
          acc.x += fac * (accv[j][4 * i4 + 0] * 16777216.f + mj);
          acc.y += fac * (accv[j][4 * i4 + 1] * 4194304.f + mj);
          acc.z += fac * (accv[j][4 * i4 + 2] * 1048576.f + mj);
          acc.w += fac * (accv[j][4 * i4 + 3] * 262144.f + mj);
          *dst = acc;
        }
      }
    }
    __syncthreads();
  }
  for (int g = tid >> 5; g < Gq; g += 8) {
    const int lq = tid & 31;
    const float4 a4 = *reinterpret_cast<const float4*>(&S.ob[0][g][4 * lq]);
    const float4 b4 = *reinterpret_cast<const float4*>(&S.ob[1][g][4 * lq]);
    const float4 c4 = *reinterpret_cast<const float4*>(&S.ob[2][g][4 * lq]);
    float yh[4] = {b4.x, b4.y, b4.z, b4.w}, yf[4] = {c4.x, c4.y, c4.z, c4.w};
    fwht<32>(yh, lq);
    fwht<128>(yf, lq);
    *reinterpret_cast<float4*>(op + g * 128 + 4 * lq) = make_float4(a4.x + yh[0] + yf[0], a4.y + yh[1] + yf[1], a4.z + yh[2] + yf[2], a4.w + yh[3] + yf[3]);
    if (lq == 0) {
      const float M = fmaxf(fmaxf(S.mw[0][g], S.mw[1][g]), fmaxf(S.mw[2][g], S.mw[3][g]));
      float L = 0.f;
      for (int w = 0; w < 4; ++w) L += S.mw[w][g] == -INFINITY ? 0.f : fexp2(S.mw[w][g] - M) * S.lw[w][g];
      mlp[2 * g] = M; mlp[2 * g + 1] = L;
    }
  }
}

int launch_pages(int Gq, const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs, const void* cached,
                 int kv_start, int B, int Hkv, int NS, int chunk, float qscale, const void* ring, const void* tail_len,
                 const void* tail_idx, int T, void* opart, void* ml, int f8, hipStream_t st) {
  static bool attr = false;
  if (!attr) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_attn_pages<false>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(sizeof(Smem))) != hipSuccess) return 1;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_attn_pages<true>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(sizeof(Smem))) != hipSuccess) return 1;
    attr = true;
  }
  const auto kern = f8 ? k_attn_pages<true> : k_attn_pages<false>;
  hipLaunchKernelGGL(kern, dim3(B, Hkv, NS + 1), dim3(256), sizeof(Smem), st, static_cast<const uint16_t*>(q), q_rs,
                     static_cast<const uint8_t*>(pool), static_cast<const int*>(bt), bt_rs, static_cast<const int*>(cached),
                     kv_start, Hkv, NS, chunk, qscale, static_cast<float*>(opart), static_cast<float*>(ml), Gq,
                     static_cast<const uint16_t*>(ring), static_cast<const int*>(tail_len), static_cast<const int*>(tail_idx), T);
  return hipPeekAtLastError() == hipSuccess ? 0 : 1;
}

}  // namespace

int attn_splits_launch(int G, const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs,
                       const void* cached, int kv_start, int B, int Hkv, int NS, int chunk, float qscale, const void* ring,
                       const void* tail_len, const void* tail_idx, int T, void* opart, void* ml, int f8, hipStream_t st) {
  if (G < 1 || G > GT) return 2;
  return launch_pages(G, q, q_rs, pool, bt, bt_rs, cached, kv_start, B, Hkv, NS, chunk, qscale, ring, tail_len, tail_idx, T, opart, ml, f8, st);
}

}  // namespace frkv
