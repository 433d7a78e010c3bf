// extern "C" surface of libflagrot_kivi.so (declared in include/flagrot_kivi.h) and the split merge of the decode
// attention.  The writers, the dequantiser and the LSE merge are in kivi_write.hip, the decode splits in kivi_decode.hip, everything of head dim 256 in kivi_wide.hip.
// Semantics follow integrations/vllm_flagrot/csrc/kivi.cu:1908-1931 (k_merge) and :1933-2342 (C ABI).
#include <cstdio>
#include <cstring>

#include "../../include/flagrot_kivi.h"
#include "fr_common.hpp"
#include "kivi_launch.hpp"
#include "kivi_merge.hpp"

namespace frkv {
using namespace fr;
namespace {

char g_err[512] = "";
int bad(const char* msg) {
  std::strncpy(g_err, msg, sizeof(g_err) - 1);
  return 2;
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
  if (D != 128 && D != 256) return bad("kv_v_write: head dim 128 or 256");
  if (D == 256)
    return launched(v_write256_launch(kv, kv_rs, n, Hkv, static_cast<const long long*>(slots), static_cast<const float*>(co),
                                      static_cast<uint8_t*>(pool), static_cast<const float*>(M), ident,
                                      static_cast<const int*>(vfix), f8 & 1, static_cast<hipStream_t>(stream)), "kv_v_write");
  return launched(v_write_launch(kv, kv_rs, n, Hkv, static_cast<const long long*>(slots), static_cast<const float*>(co),
                                 static_cast<uint8_t*>(pool), static_cast<const float*>(M), ident, static_cast<const int*>(vfix), f8 & 1,
                                 static_cast<hipStream_t>(stream)), "kv_v_write");
}

int kv_k_encode(const void* src, long long src_rs, const void* src2, long long src2_rs, const void* sidx,
                const void* dslot, int N, int Hkv, int D, const void* qs, const void* lz, int NQ, float qsc, void* pool,
                int ident, const void* kfix, int f8, void* stream) {
  if (N <= 0) return 0;
  if (D != 128 && D != 256) return bad("kv_k_encode: head dim 128 or 256");
  if (D == 256)
    return launched(k_encode256_launch(src, src_rs, src2, src2_rs, static_cast<const long long*>(sidx),
                                       static_cast<const long long*>(dslot), N, Hkv, static_cast<const float*>(qs),
                                       static_cast<const float*>(lz), NQ, qsc, static_cast<uint8_t*>(pool), ident,
                                       static_cast<const int*>(kfix), f8 & 1, static_cast<hipStream_t>(stream)), "kv_k_encode");
  return launched(k_encode_launch(src, src_rs, src2, src2_rs, static_cast<const long long*>(sidx),
                                  static_cast<const long long*>(dslot), N, Hkv, static_cast<const float*>(qs),
                                  static_cast<const float*>(lz), NQ, qsc, static_cast<uint8_t*>(pool), ident,
                                  static_cast<const int*>(kfix), f8 & 1, static_cast<hipStream_t>(stream)), "kv_k_encode");
}

int kv_attn(const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs, const void* cached,
            int kv_start, int B, int Hkv, int G, int D, int NS, int chunk, float qscale, const void* ring,
            const void* tail_len, const void* tail_idx, int T, void* opart, void* ml, void* out, long long out_rs, int f8,
            void* stream) {
  if (B <= 0) return 0;
  if (G > 8 || G < 1 || chunk % 32 || chunk <= 0) { std::snprintf(g_err, sizeof(g_err), "kv_attn: G %d chunk %d", G, chunk); return 2; }
  if (D != 128 && D != 256) return bad("kv_attn: head dim 128 or 256");
  hipStream_t st = static_cast<hipStream_t>(stream);
  // the head-dim-128 kernel reads q and the ring rows 16 bytes at a time (operands of matrix instructions)
  if (D == 128 && ring != nullptr &&
      (((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(ring)) & 15u) != 0 || (q_rs & 7) != 0))
    return bad("kv_attn: with ring rows, q and the ring must be 16-byte aligned and q_rs a multiple of 8 elements");
  if (D == 256)
    return launched(attn256_launch(G, q, q_rs, pool, bt, bt_rs, cached, kv_start, B, Hkv, NS, chunk, qscale, ring, tail_len,
                                   tail_idx, T, opart, ml, out, out_rs, f8 & 1, st), "kv_attn");
  const int rc = attn_splits_launch(G, q, q_rs, pool, bt, bt_rs, cached, kv_start, B, Hkv, NS, chunk, qscale, ring, tail_len,
                                    tail_idx, T, opart, ml, f8 & 1, st);
  if (rc) return launched(rc, "kv_attn");
  hipLaunchKernelGGL(k_merge_parts<128>, dim3(B, Hkv * G), dim3(128), 0, st, static_cast<const float*>(opart), static_cast<const float*>(ml),
                     Hkv, G, NS, static_cast<uint16_t*>(out), out_rs);
  return launched(hipPeekAtLastError() == hipSuccess ? 0 : 1, "kv_attn (merge)");
}

int kv_dequant(const void* pool, const void* bt, int g0, int g1, int nvalid, int Hkv, int D, int fp32, void* ok, void* ov,
               int f8, void* stream) {
  if (g1 <= g0) return 0;
  if (D != 128 && D != 256) return bad("kv_dequant: head dim 128 or 256");
  if (D == 256)
    return launched(dequant256_launch(static_cast<const uint8_t*>(pool), static_cast<const int*>(bt), g0, g1, nvalid, Hkv, fp32,
                                      ok, ov, f8 & 1, static_cast<hipStream_t>(stream)), "kv_dequant");
  return launched(dequant_launch(static_cast<const uint8_t*>(pool), static_cast<const int*>(bt), g0, g1, nvalid, Hkv, fp32, ok,
                                 ov, f8 & 1, static_cast<hipStream_t>(stream)), "kv_dequant");
}

int kv_lse_merge(const void* oa, const void* la, long long la_hs, const void* ob, const void* lb, long long lb_hs,
                 void* out, long long out_rs, int na, int H, int D, void* stream) {
  if (na <= 0) return 0;
  return launched(lse_merge_launch(oa, static_cast<const float*>(la), la_hs, ob, static_cast<const float*>(lb), lb_hs, out,
                                   out_rs, na, H, D, static_cast<hipStream_t>(stream)), "kv_lse_merge");
}

}  // extern "C"
