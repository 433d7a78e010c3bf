// Split merge of the KIVI-style decode attention (both head dims): workgroup = (sequence, query head), thread = channel.
// The NS + 1 partials of the query head's (sequence, KV head) are folded eight at a time; the (maximum, sum) pairs and
// the thread's channel of all eight are requested together, so a call with up to eight partials is ONE memory round
// trip (maxima first and the rest afterwards is two).  Semantics: integrations/vllm_flagrot/csrc/kivi.cu:1908-1931.
#pragma once
#include "fr_common.hpp"

namespace frkv {
using namespace fr;

template <int D>
__global__ void __launch_bounds__(D) k_merge_parts(const float* __restrict__ opart, const float* __restrict__ ml, int Hkv, int G,
                                                   int NS, uint16_t* __restrict__ out, long long out_rs) {
  const int b = blockIdx.x, hq = blockIdx.y, h = hq / G, g = hq % G;
  const long long p0 = (static_cast<long long>(b) * Hkv + h) * (NS + 1);
  float M = -INFINITY, L = 0.f, o = 0.f;
  for (int s0 = 0; s0 <= NS; s0 += 8) {
    float m8[8], l8[8], o8[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {      // past the last partial: the last one again, skipped below
      const long long at = (p0 + min(s0 + i, NS)) * G + g;
      m8[i] = ml[at * 2]; l8[i] = ml[at * 2 + 1]; o8[i] = opart[at * D + threadIdx.x];
    }
    float top = M;
#pragma unroll
    for (int i = 0; i < 8; ++i) top = fmaxf(top, s0 + i <= NS ? m8[i] : -INFINITY);
    if (top == -INFINITY) continue;                       // nothing but empty partials so far
    const float keep = M == -INFINITY ? 0.f : exp2f(M - top);
    L *= keep; o *= keep; M = top;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (s0 + i > NS || m8[i] == -INFINITY) continue;
      const float f = exp2f(m8[i] - M);
      L += f * l8[i];
      o += f * o8[i];
    }
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  out[static_cast<long long>(b) * out_rs + static_cast<long long>(hq) * D + threadIdx.x] = static_cast<uint16_t>(bf16_rn(o * inv));
}

}  // namespace frkv
