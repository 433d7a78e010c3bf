/* libflagrot_probe.so: a measurement aid with no counterpart in the reference and no place in the drop-in boundary.
 * fr_probe_read launches a kernel that only reads the (page, KV head) chunks a paged decode launch over the same block
 * table reads, with the decode kernel's workgroup layout; bench.py times it beside the decode kernel, so that the rate
 * this memory system gives that access pattern is measured in the same run; fr_probe_mfma does the same for the matrix
 * pipe beside the multi-query prefill kernel.  Raw device pointers, asynchronous on
 * `stream`, no allocation.  Return codes: 0 ok, -1 launch error, -2 bad argument (message: fr_probe_last_error()). */
#ifndef FLAGROT_PROBE_H
#define FLAGROT_PROBE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

int fr_probe_abi_version(void);
const char* fr_probe_last_error(void);
/* pool [num_pages, Hkv, chunk_bytes] (chunk_bytes a multiple of 16, at most 5120: a 32-token INT4 page is 4608); block_table int32 [B, bt_stride];
 * seq_lens int32 [B]; page 16 | 32; sink: one writable 32-bit word (practically never written). */
int fr_probe_read(const uint8_t* pool, const int* block_table, int bt_stride, const int* seq_lens, int B, int Hkv, int page,
                  int chunk_bytes, uint32_t* sink, void* stream);

/* The matrix pipe's reachable rate: `workgroups` workgroups of 8 wavefronts each issue iters x 4
 * v_mfma_f32_32x32x16_f16 per wavefront and nothing else; mode 0: operands in registers, mode 1: one operand of every
 * instruction read from LDS (1 KB per wavefront and instruction).  fr_probe_mfma_flops: the flops of such a launch. */
int fr_probe_mfma(int mode, int iters, int workgroups, uint32_t* sink, void* stream);
long long fr_probe_mfma_flops(int iters, int workgroups);

#ifdef __cplusplus
}
#endif
#endif
