/* C ABI of libflagrot_mq.so for MI355X (gfx950): prefix-cached multi-query prefill attention straight from FlagRot
 * INT4 / INT2 pages (asymmetric codes, static or key-only 2x2), MFMA f16 with fp32 accumulation.
 *
 * Drop-in for the entry points the reference plugin binds with ctypes (integrations/vllm_flagrot/vllm_flagrot/
 * prefill_mq.py:57-86 of the reference; definitions in integrations/vllm_flagrot/csrc/mq_prefill.cu:1469-1601).  Raw
 * device pointers, `stream` is a hipStream_t, asynchronous, no allocation.  Return codes: 0 ok, -1 launch failure,
 * -2 bad kernel selector, -3 bad G, -4 unsupported head dim (128 and 256 are built; at 256 one kernel
 * with 128-row tiles serves every selector, like the reference's k_mq3).  frmq_last_error() returns this library's
 * last message.
 *
 * Plan buffers (host planner, prefill_mq.py:128-210): tiles int32 [nt][9] = (block-table row, compact row0, output
 * row0, tokens, position of the first token, page keys nk, first item, items, ext); items int32 [ni][4] = (tile,
 * first 64-key block, end block, 0).  Row r of a tile = token r / G, q head h G + r % G; rows per tile = 64 for
 * kernel 1, 128 for kernel 2 / 3 (the reference's selectors), 256 for kernel 4 (this library only: eight wavefronts in
 * two groups that alternate between the matrix and the vector half of a block).  Key j is visible to the row at position p iff kmin <= j <= max(p - shift, ext)
 * and j < nk.
 */
#ifndef FLAGROT_MQ_H
#define FLAGROT_MQ_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* mq_prefill.cu:1471 -- == 7 */
int frmq_abi_version(void);
/* mq_prefill.cu:1600 */
const char* frmq_last_error(void);
/* mq_prefill.cu:1598 -- dynamic LDS bytes of the attention kernel */
int frmq_smem_bytes(void);

/* mq_prefill.cu:1474-1488.  q bf16 or fp32 (q_fp32) rows [*, Hq, Dh] with row stride q_ts elements; idx int32 [m]
 * rows to take (null: 0..m-1); kfull uint8 [Hkv] (whole-head H_128 / 8) and kmask uint8 [Hkv][4] (orthonormal H32 per
 * flagged group), either may be null; q16 fp16 [m, Hq, Dh] = rotated q * qscale. */
int frmq_prep_q(const void* q, int q_fp32, long long q_ts, const int* idx, int m, int Hq, int G, const uint8_t* kfull,
                const uint8_t* kmask, float qscale, void* q16, int Dh, void* stream);

/* mq_prefill.cu:1490-1544.  q16 from frmq_prep_q (pre-scaled by softmax scale * log2 e); pool uint8 pages with byte
 * stride page_stride, KV head h at + h * chunk bytes; konly bit 0: key-only 2x2 pages (per-token H32 / H128 flags),
 * bit 1: INT2 pages (80 B per token) instead of INT4 (144 B); opart fp32 [nitems, Hkv, rows, Dh] unnormalised, ml fp32
 * [nitems, Hkv, rows, 2] = (running maximum in log2 units, sum); kernel 1 | 2 | 3 | 4 selects rows per tile (64 | 128 | 128 | 256). */
int frmq_attn(const void* q16, const uint8_t* pool, long long page_stride, const int* bt, long long bt_stride,
              const int* tiles, const int* items, int nitems, int Hkv, int G, int shift, int konly, float* opart,
              float* ml, int kernel, int Dh, void* stream, int kmin);

/* mq_prefill.cu:1546-1559.  Combines the items of each tile: out_fp32 = 0: bf16 rows out[(orow0 + t) * o_ts + hq * Dh];
 * 1: fp32 compact rows out[((crow0 + t) * Hq + hq) * Dh]; lse (or null): natural-log sums [Hq][lse_ts], -inf for rows
 * without a visible key. */
int frmq_merge(const int* tiles, int ntiles, const float* opart, const float* ml, int Hkv, int G, int rows, void* out,
               long long o_ts, int out_fp32, float* lse, long long lse_ts, int Dh, void* stream);

/* mq_prefill.cu:1561-1577.  K / V rows of the BF16 window call: destination row d from map[d] = (kind << 32) | row;
 * kind 0: sinkb [*, 2 Hkv, Dh], 1: preb [*, 2 Hkv, Dh], 2: the batch rows kch / vch (row strides k_ts / v_ts). */
int frmq_win_gather(const long long* map, int nk, const void* sinkb, const void* preb, const void* kch, long long k_ts,
                    const void* vch, long long v_ts, int Hkv, void* kw, void* vw, int Dh, void* stream);

/* mq_prefill.cu:1579-1596.  out[idx[c]] = LSE merge of the page part (o_p fp32 [m, Hq, Dh], lse_p [Hq, m]), the window
 * part (o_w bf16, lse_w; may be null) and the sink part (sk bf16 [nreq, S, 2 Hkv, Dh], keys j < min(S, sk_len[req]) with
 * j <= row_pos[c] - W; may be null). */
int frmq_bf_merge(int m, int Hq, int Hkv, const void* q, long long q_ts, const long long* idx, const float* o_p,
                  const float* lse_p, const void* o_w, const float* lse_w, const void* sk, const long long* row_req,
                  const long long* row_pos, const long long* sk_len, int S, int W, float scale, void* out, long long o_ts,
                  int Dh, void* stream);

#ifdef __cplusplus
}
#endif
#endif
