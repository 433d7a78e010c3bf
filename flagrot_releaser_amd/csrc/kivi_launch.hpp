// Launcher prototypes shared by the translation units of libflagrot_kivi.so (f8: FP8-meta pages).  The plain names are
// the 128-d kernels (kivi_write.hip, kivi_decode.hip), the *256 ones the 256-d kernels (kivi_wide.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace frkv {

int v_write_launch(const void* kv, long long kv_rs, int n, int Hkv, const long long* slots, const float* co, uint8_t* pool,
                   const float* M, int ident, const int* vfix, int f8, hipStream_t st);
int k_encode_launch(const void* src, long long src_rs, const void* src2, long long src2_rs, const long long* sidx,
                    const long long* dslot, int N, int Hkv, const float* qs, const float* lz, int NQ, float qsc,
                    uint8_t* pool, int ident, const int* kfix, int f8, hipStream_t st);
int dequant_launch(const uint8_t* pool, const int* bt, int g0, int g1, int nvalid, int Hkv, int fp32, void* ok, void* ov,
                   int f8, hipStream_t st);
int lse_merge_launch(const void* oa, const float* la, long long la_hs, const void* ob, const float* lb, long long lb_hs,
                     void* out, long long out_rs, int na, int H, int D, hipStream_t st);
// splits [0, NS) over the pages and split NS over the BF16 ring rows (kivi_decode.hip): partials per (sequence, KV head,
// split): opart fp32 [.., G, 128] unnormalised, ml fp32 [.., G, 2] = (maximum in log2 units, sum)
int attn_splits_launch(int G, const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs,
                       const void* cached, int kv_start, int B, int Hkv, int NS, int chunk, float qscale, const void* ring,
                       const void* tail_len, const void* tail_idx, int T, void* opart, void* ml, int f8, hipStream_t st);


int v_write256_launch(const void* kv, long long kv_rs, int n, int Hkv, const long long* slots, const float* co, uint8_t* pool,
                      const float* M, int ident, const int* vfix, int f8, hipStream_t st);
int k_encode256_launch(const void* src, long long src_rs, const void* src2, long long src2_rs, const long long* sidx,
                       const long long* dslot, int N, int Hkv, const float* qs, const float* lz, int NQ, float qsc,
                       uint8_t* pool, int ident, const int* kfix, int f8, hipStream_t st);
int dequant256_launch(const uint8_t* pool, const int* bt, int g0, int g1, int nvalid, int Hkv, int fp32, void* ok, void* ov,
                      int f8, hipStream_t st);
// splits and merge in one call: out bf16 rows of Hkv G 256 values
int attn_pages256_launch(int Gq, const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs,
                         const void* cached, int kv_start, int B, int Hkv, int NS, int chunk, float qscale, const void* ring,
                         const void* tail_len, const void* tail_idx, int T, void* opart, void* ml, int f8, hipStream_t st);
int attn256_launch(int G, const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs, const void* cached,
                   int kv_start, int B, int Hkv, int NS, int chunk, float qscale, const void* ring, const void* tail_len,
                   const void* tail_idx, int T, void* opart, void* ml, void* out, long long out_rs, int f8, hipStream_t st);

}  // namespace frkv
