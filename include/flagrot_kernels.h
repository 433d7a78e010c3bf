/* C ABI of libflagrot_kernels.so for MI355X (gfx950): paged FlagRot KV-cache writers and paged decode attention.
 *
 * Drop-in for the entry points the reference plugin binds with ctypes
 * (integrations/vllm_flagrot/vllm_flagrot/kernels.py:140-177 of the reference; definitions in
 * integrations/vllm_flagrot/csrc/flagrot_capi.cu).  All pointers are raw device addresses, `stream` is a
 * hipStream_t, every call is asynchronous on that stream, allocates nothing and may be captured in a HIP graph.
 * Return codes: 0 ok; -1 launch error; -2 LDS request refused; -3 unsupported variant / stages; -4 unknown fmt /
 * kind; -5 page not in {16, 32}; -7 gqa out of range; -8 head dim not supported.
 *
 * fmt  (static / generalised decode): 4 int4, 5 int4a, 6 konly, 7 konlya, 8 int2a, 9 konlya2
 * kind (key-only 2x2 codebooks):      6 konly, 10 konlya, 11 konlya2
 */
#ifndef FLAGROT_KERNELS_H
#define FLAGROT_KERNELS_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* flagrot_capi.cu:21 -- == 9 */
int fr_abi_version(void);

/* flagrot_capi.cu:42-64.  q bf16 [B, gqa*Hkv, 128] (row stride q_bs elements); pool [num_pages, Hkv, chunk];
 * block_table int32 [B, bt_stride] (bt_stride may be 0); seq_lens int32 [B]; out bf16 [B, gqa*Hkv*128] (row stride
 * o_bs); kmask / vmask uint8 [Hkv, 4] or null (honoured if qrot / if vrot or tail); tail bf16
 * [rows, W, 2*Hkv, 128] (strides tail_bs / tail_ts elements) + tail_len int32 [B] (+ tail_idx int32 [B]) or null.
 * With a tail at head dim 128, q and tail must be 16-byte aligned and q_bs, tail_bs, tail_ts multiples of 8 elements
 * (the rows are operands of matrix instructions, read 16 bytes at a time; contiguous torch tensors always are): -3 if not.
 * nsplit counts the body splits; with a tail the workspace must hold B*Hkv*ceil(gqa/GT)*(nsplit+1) partials of
 * GT*128 floats (GT = 8 when variant has bits 1024|2048, else 4); counter int32 [B*Hkv*ceil(gqa/GT)] zeroed once by the
 * caller (merge tickets and, when the body workgroups of a sequence share its page range, their page draws; the last
 * arriving workgroup leaves the word at 0).  If B*Hkv*ceil(gqa/GT)*nsplit fits the CUs and chunk >= 1024, split s owns
 * tokens [s, s+1)*chunk and one large workgroup per CU runs it; otherwise nsplit only counts the workgroups per
 * (sequence, KV head, q tile); nsplit*chunk must cover the longest sequence either way.
 * variant bit 4096 (kernels/csrc/attn_decode_v2g.cuh:11-25, 276): head dim 256 -- q, out and tail rows have 256 channels,
 * the pool chunk is two 128-d half chunks per (page, KV head), kmask / vmask are [Hkv, 8], partials are GT*256 floats
 * with GT = 4, split s owns tokens [s, s+1)*chunk and the counter words are not used. */
int fr_v2_attn(int fmt, const void* q, long long q_bs, const uint8_t* pool, const int* block_table, int bt_stride,
               const int* seq_lens, int B, int Hkv, int page, int nsplit, int chunk, float qscale,
               const uint8_t* kmask, const uint8_t* vmask, int rb, int qrot, int vrot, int variant, int stages,
               float* opart, float* mlpart, int* counter, void* out, long long o_bs, const void* tail,
               const int* tail_len, const int* tail_idx, long long tail_bs, long long tail_ts, void* stream,
               int gqa, int kv_start);

/* flagrot_capi.cu:68-77.  kv bf16 [T, 2*Hkv, hd] (token stride kv_ts elements) -> pool at slots int64 [T]
 * (< 0 skipped); mask uint8 [2*Hkv, hd/32]; kmu fp32 [Hkv, hd] or null; fmt 4 | 5 | 8; rb must be 32. */
int fr_v2_write(int fmt, const void* kv, long long kv_ts, const long long* slots, int T, int Hkv, int page,
                const uint8_t* mask, int rb, uint8_t* pool, void* stream, int hd, const float* kmu);

/* flagrot_capi.cu:79-80.  Resident 4-wavefront workgroups per CU (for the host split planner); bytes per (page, head)
 * chunk. */
int fr_v2_occupancy(int fmt, int variant, int stages, int page);
int fr_v2_chunk_bytes(int fmt, int page);

/* flagrot_capi.cu:84 -- == 15 (rows of the sign table `sg`; unused by the key-only kinds) */
int fr_cb_nsg(void);

/* flagrot_capi.cu:86-98.  Selecting writer.  CT fp32 [Hkv, hd, hd] = C_q transposed; co fp32 [Hkv, hd] (unused by
 * the key-only kinds: values carry no transform); sg uint32 [15*4] (unused); tg: scheduling hint (ignored).
 * hd 0 | 128, or 256 (kernels/csrc/attn_codebook.cu:384-392, 432: eight key groups, whole-head H256, the page chunk two
 * 128-d half chunks, the H256 flag in the group-0 V scale word of half 0). */
int fr_cb_write(const void* kv, long long kv_ts, const long long* slots, int slot_ph, int T, int Hkv, int page, int tg,
                const float* CT, const float* co, const unsigned* sg, int kind, uint8_t* pool, void* stream, int hd,
                const float* kmu);

/* flagrot_capi.cu:104-115.  Same bytes as fr_cb_write.  nchunk < 0 skips the key pass, nchunk_v < 0 the value
 * pass; the two passes own disjoint bits of the token's group-0 V scale word, so they may run on two streams.
 * Key passes of more than 1024 (token, head) rows run the screened kernel: the weighted errors are estimated on the
 * matrix pipe and a token is decided from the estimates only where the exactly ordered evaluation cannot decide
 * otherwise; the rest is evaluated exactly.  The error bound is computed from CT by the kernel itself: C1 / beta (the
 * screening constants of the reference's tensor-core writer) are accepted and ignored (may be null). */
int fr_cb_write3(const void* kv, long long kv_ts, const long long* slots, int slot_ph, int T, int Hkv, int page,
                 const float* CT, const float* co, const void* C1, const float* beta, const unsigned* sg, int kind,
                 uint8_t* pool, int nchunk, int nchunk_v, void* stream, const float* kmu);

/* flagrot_capi.cu:120-129.  = fr_head_fwht(kv, hfull, 1/16) then fr_v2_write(rb 32) in one kernel, byte for byte.
 * asym 0 int4 | 1 int4a | 2 int2a; path is a scheduling hint (ignored). */
int fr_w3_static_write(const void* kv, long long kv_ts, const long long* slots, int T, int Hkv, int page,
                       const uint8_t* mask, const uint8_t* hfull, int asym, uint8_t* pool, int path, void* stream,
                       const float* kmu);

/* flagrot_capi.cu:131-149.  Key-only 2x2 decode, 4 q heads per KV head, head dim 128. */
int fr_cb_attn(const void* q, long long q_bs, const uint8_t* pool, const int* block_table, int bt_stride,
               const int* seq_lens, int B, int Hkv, int page, int nsplit, int chunk, float qscale, const unsigned* sg,
               int kind, int variant, int stages, float* opart, float* mlpart, int* counter, void* out, long long o_bs,
               const void* tail, const int* tail_len, const int* tail_idx, long long tail_bs, long long tail_ts,
               void* stream, int kv_start);

/* No counterpart in the reference.  For callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): fr_cb_attn for any gqa (<= 64) without the workspace
 * arguments.  Partials, (max, sum) pairs and counters live in an array built into the library (about 16.3 MiB per GPU,
 * held until the process ends); the call allocates nothing and clears its counters itself.  Limit:
 * B*Hkv*ceil(gqa/4)*(nsplit+1) <= FR_NOALLOC_MAX_PARTS, else -2 with a message in fr_last_error().  All calls on one
 * GPU share the array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream are safe.
 * The first call on a device looks the array's address up (a host-side query: no stream work, no allocation); make it
 * outside a stream capture -- every later call on that device may be captured into a HIP graph. */
#define FR_NOALLOC_MAX_PARTS 8192
int fr_cb_attn_noalloc(const void* q, long long q_bs, const uint8_t* pool, const int* block_table, int bt_stride,
                       const int* seq_lens, int B, int Hkv, int page, int nsplit, int chunk, float qscale, int kind,
                       void* out, long long o_bs, const void* tail, const int* tail_len, const int* tail_idx,
                       long long tail_bs, long long tail_ts, void* stream, int gqa, int kv_start);

/* flagrot_capi.cu:151-153 */
int fr_cb_occupancy(int kind, int variant, int stages, int page);
int fr_cb_chunk_bytes(int kind, int page);
int fr_cb_write_smem(int kind, int tg, int hd);

/* flagrot_capi.cu:155 */
const char* fr_last_error(void);

/* flagrot_capi.cu:250-265.  out[t, h, :] = flags[h] ? scale * (+-1 Sylvester H_D) x[t, h, :] : x[t, h, :];
 * x, out bf16 (may alias), D 128 | 256. */
int fr_head_fwht(const void* x, long long x_ts, void* out, long long o_ts, int T, int H, const uint8_t* flags,
                 float scale, void* stream, int D);

#ifdef __cplusplus
}
#endif
#endif
