/* C ABI of libflagrot_kivi.so for MI355X (gfx950): KIVI-style FlagRot INT2 pages (keys quantised per channel over
 * 32-token groups, values per token in groups of 32 channels, identity / H32 / whole-head Hadamard chosen per group /
 * token, flags in the sign bits of the FP16 scales).
 *
 * Drop-in for the entry points the reference plugin binds with ctypes (integrations/vllm_flagrot/vllm_flagrot/kivi.py:
 * 49-77 of the reference; definitions in integrations/vllm_flagrot/csrc/kivi.cu:1933-2342).  Raw device pointers,
 * `stream` is a hipStream_t, asynchronous, no allocation.  Return codes: 0 ok, 1 launch failure, 2 bad / unsupported
 * argument (message from kv_last_error()).  Built for head dim 128 and 256 (kivi.cu's <128> and <256> instantiations;
 * at 256 a chunk has eight sub-vectors and key cells of eight channels; kv_attn serves G <= 8 at both head dims), FP16 scale / min pages (f8 bit 0 clear) and FP8 E4M3 scale / min pages (f8 bit 0 set: 10 D-byte chunks, codes
 * computed from the stored values, the value rows' whole-head flags in bit 7 of key scale bytes; kivi.cu:28-35, 84-88,
 * 123-128), diagonal (co) and matrix (M) value weighting at both head dims.
 */
#ifndef FLAGROT_KIVI_H
#define FLAGROT_KIVI_H
#ifdef __cplusplus
extern "C" {
#endif

/* kivi.cu:63 -- == 9 */
int kv_abi_version(void);
/* kivi.cu:62 */
const char* kv_last_error(void);
/* kivi.cu:91-92 -- bytes per (16-token page, KV head): 12 D + 16 (FP16 meta), 10 D (FP8 meta) */
int kv_chunk_bytes(int D);
int kv_chunk_bytes8(int D);

/* kivi.cu:1934-1949.  kv bf16 [n, 2*Hkv, D] (row stride kv_rs elements; V rows Hkv..2Hkv-1); slots int64 [n]
 * (< 0 skipped); co fp32 [Hkv, D]; M fp32 [Hkv, D, D] or null (null: a candidate's error is sum d^2 co; else d^T M d,
 * the diagonal 32-blocks of M for the sub-vector choices, kivi.cu:213-287); vfix int32 [Hkv] or null (bits 0..3 = H32
 * per sub-vector, bit 16 = H_D); ident: identity only. */
int kv_v_write(const void* kv, long long kv_rs, int n, int Hkv, int D, const void* slots, const void* co, const void* M,
               void* pool, int ident, const void* vfix, int f8, void* stream);

/* kivi.cu:1951-1977.  src / src2 bf16 rows (K row of head h at + h*D); sidx int64 [N, 32]: r >= 0 src row, r <= -2
 * src2 row -r-2, -1 not in the group; dslot int64 [N, 32] page slots (dslot[n][0] < 0: inactive item); qs fp32
 * [Hkv, NQ, D], lz fp32 [Hkv, NQ]; kfix int32 [Hkv] or null. */
int kv_k_encode(const void* src, long long src_rs, const void* src2, long long src2_rs, const void* sidx,
                const void* dslot, int N, int Hkv, int D, const void* qs, const void* lz, int NQ, float qsc, void* pool,
                int ident, const void* kfix, int f8, void* stream);

/* kivi.cu:1987-2039.  q bf16 [B, Hkv*G, D] (row stride q_rs); bt int32 [B, bt_rs]; cached int32 [B] (page tokens
 * [kv_start, cached[b]) are attended); ring bf16 [(R+1)*T, 2*Hkv, D] with tail_len / tail_idx int32 [B]; opart fp32
 * [B*Hkv*(NS+1)*G*D], ml fp32 [B*Hkv*(NS+1)*G*2]; out bf16 [B, Hkv*G*D] (row stride out_rs).  G <= 8, chunk % 32 == 0.
 * f8 bit 1 (the reference's fast variant) is accepted and ignored.  At D = 128 with ring rows, q and ring must be
 * 16-byte aligned and q_rs a multiple of 8 elements (the rows are operands of matrix instructions; contiguous torch
 * tensors are): 2 if not. */
int kv_attn(const void* q, long long q_rs, const void* pool, const void* bt, long long bt_rs, const void* cached,
            int kv_start, int B, int Hkv, int G, int D, int NS, int chunk, float qscale, const void* ring,
            const void* tail_len, const void* tail_idx, int T, void* opart, void* ml, void* out, long long out_rs, int f8,
            void* stream);

/* kivi.cu:2325-2342.  groups [g0, g1) of one request (block-table row bt) -> K, V [(g1-g0)*32 (first nvalid rows),
 * Hkv, D] in the original basis, bf16 or fp32. */
int kv_dequant(const void* pool, const void* bt, int g0, int g1, int nvalid, int Hkv, int D, int fp32, void* ok, void* ov,
               int f8, void* stream);

/* kivi.cu:2315-2323.  out = bf16 LSE merge of (oa bf16 [na, H, D], la fp32 [H, na]) and (ob, lb). */
int kv_lse_merge(const void* oa, const void* la, long long la_hs, const void* ob, const void* lb, long long lb_hs,
                 void* out, long long out_rs, int na, int H, int D, void* stream);

#ifdef __cplusplus
}
#endif
#endif
