/* A C caller of the three boundary libraries, compiled as C99 against the headers under include/ and linked against the built .so
 * files: the headers are valid C, every declared entry point resolves at link time, and the calls that need no GPU
 * (versions, sizes, argument checks that return before any launch) behave as the headers say.  Exit code 0 = all good;
 * otherwise the number of the first failed check.  Built and run by tests/test_capi_load.py. */
#include <stdio.h>
#include <string.h>

#include "flagrot_kernels.h"
#include "flagrot_kivi.h"
#include "flagrot_mq.h"

#define CHECK(n, cond) do { if (!(cond)) { fprintf(stderr, "check %d failed: %s\n", (n), #cond); return (n); } } while (0)

int main(void) {
  /* addresses of every entry point: a missing export is a link error */
  typedef void (*entry_t)(void);
  const entry_t all[] = {
      (entry_t)fr_abi_version, (entry_t)fr_v2_attn, (entry_t)fr_v2_write, (entry_t)fr_v2_occupancy,
      (entry_t)fr_v2_chunk_bytes, (entry_t)fr_cb_nsg, (entry_t)fr_cb_write, (entry_t)fr_cb_write3,
      (entry_t)fr_w3_static_write, (entry_t)fr_cb_attn, (entry_t)fr_cb_attn_noalloc, (entry_t)fr_cb_occupancy,
      (entry_t)fr_cb_chunk_bytes, (entry_t)fr_cb_write_smem, (entry_t)fr_last_error, (entry_t)fr_head_fwht,
      (entry_t)kv_abi_version, (entry_t)kv_last_error, (entry_t)kv_chunk_bytes, (entry_t)kv_chunk_bytes8,
      (entry_t)kv_v_write, (entry_t)kv_k_encode, (entry_t)kv_attn, (entry_t)kv_dequant, (entry_t)kv_lse_merge,
      (entry_t)frmq_abi_version, (entry_t)frmq_last_error, (entry_t)frmq_smem_bytes, (entry_t)frmq_prep_q,
      (entry_t)frmq_attn, (entry_t)frmq_merge, (entry_t)frmq_win_gather, (entry_t)frmq_bf_merge};
  size_t i;
  for (i = 0; i < sizeof(all) / sizeof(all[0]); ++i) CHECK(1, all[i] != (entry_t)0);

  CHECK(2, fr_abi_version() == 9 && kv_abi_version() == 9 && frmq_abi_version() == 7);
  CHECK(3, fr_cb_nsg() == 15);
  /* bytes per (page, KV head): 144 P (INT4) / 80 P (INT2) */
  CHECK(4, fr_v2_chunk_bytes(4, 16) == 2304 && fr_v2_chunk_bytes(5, 16) == 2304 && fr_v2_chunk_bytes(8, 16) == 1280);
  CHECK(5, fr_v2_chunk_bytes(5, 32) == 4608 && fr_cb_chunk_bytes(6, 16) == 2304 && fr_cb_chunk_bytes(10, 16) == 2304 &&
               fr_cb_chunk_bytes(11, 16) == 1280);
  CHECK(6, kv_chunk_bytes(128) == 1552 && kv_chunk_bytes8(128) == 1280 && kv_chunk_bytes(256) == 3088 && kv_chunk_bytes8(256) == 2560);
  CHECK(7, fr_v2_occupancy(5, 264, 4, 16) == 1 && fr_cb_occupancy(10, 0, 4, 16) == 1);
  CHECK(8, fr_cb_write_smem(10, 128, 128) > 0 && fr_cb_write_smem(10, 128, 256) > 0 && fr_cb_write_smem(10, 128, 64) == 0);
  CHECK(9, frmq_smem_bytes() > 0);

  /* empty work returns 0 without touching a device */
  CHECK(10, fr_v2_write(5, NULL, 0, NULL, 0, 8, 16, NULL, 32, NULL, NULL, 128, NULL) == 0);
  CHECK(11, fr_cb_write(NULL, 0, NULL, 0, 0, 8, 16, 128, NULL, NULL, NULL, 10, NULL, NULL, 128, NULL) == 0);
  CHECK(12, kv_v_write(NULL, 0, 0, 8, 128, NULL, NULL, NULL, NULL, 0, NULL, 0, NULL) == 0);
  CHECK(13, kv_attn(NULL, 0, NULL, NULL, 0, NULL, 0, 0, 8, 8, 128, 1, 256, 1.0f, NULL, NULL, NULL, 0, NULL, NULL, NULL, 0, 0, NULL) == 0);

  /* argument checks come before any launch: the documented codes, and a message behind *_last_error */
  CHECK(14, fr_v2_write(5, NULL, 0, NULL, 4, 8, 16, NULL, 32, NULL, NULL, 64, NULL) == -8);      /* head dim */
  CHECK(15, strlen(fr_last_error()) > 0);
  CHECK(16, fr_v2_write(5, NULL, 0, NULL, 4, 8, 16, NULL, 16, NULL, NULL, 128, NULL) == -3);     /* rotation block */
  CHECK(17, kv_v_write(NULL, 0, 4, 8, 64, NULL, NULL, NULL, NULL, 0, NULL, 0, NULL) == 2);       /* head dim */
  CHECK(18, strlen(kv_last_error()) > 0);
  CHECK(19, kv_attn(NULL, 0, NULL, NULL, 0, NULL, 0, 1, 8, 9, 128, 1, 256, 1.0f, NULL, NULL, NULL, 0, NULL, NULL, NULL, 0, 0, NULL) == 2);   /* G > 8 */
  CHECK(20, kv_attn(NULL, 0, NULL, NULL, 0, NULL, 0, 1, 8, 8, 128, 1, 250, 1.0f, NULL, NULL, NULL, 0, NULL, NULL, NULL, 0, 0, NULL) == 2);   /* chunk % 32 */
  printf("abi_check: %u entry points, all checks passed\n", (unsigned)(sizeof(all) / sizeof(all[0])));
  return 0;
}
