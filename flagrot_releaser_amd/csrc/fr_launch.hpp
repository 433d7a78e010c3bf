// Host-side parameter blocks and launcher prototypes shared by the translation units of libflagrot_kernels.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fr {

struct StaticWriteParams {
  const void* kv;          // bf16 [T, rows, 128] (rows = 2 * Hkv half-head rows, K rows first), token stride kv_ts
  long long kv_ts;
  const long long* slots;  // [T], < 0: skip
  int T, Hkv, page;        // Hkv counts 128-d (half) heads
  const uint8_t* mask;     // [2 * Hkv, 4] or null
  const uint8_t* hfull;    // [2 * Hkv] whole-head +-1 Hadamard / 16 with a bf16 rounding first, or null
  const float* kmu;        // [Hkv, 128] or null
  uint8_t* pool;
};
int static_write_launch(int fmt, const StaticWriteParams& p, hipStream_t st);

struct K2WriteParams {
  const void* kv;
  long long kv_ts;
  const long long* slots;
  int slot_ph;
  int T, Hkv, page;
  const float* CT;         // [Hkv, hd (k), hd (i)] = C_q[h][i][k]
  const float* kmu;
  uint8_t* pool;
  int passes;              // bit 0: key rows, bit 1: value rows
  int screen;              // 1: large key passes may run the screened kernel (same bytes; fr_cb_write3)
  int hd;                  // head dim: 0 | 128, or 256 (fr_cb_write only)
};
int k2_write_launch(int kind, const K2WriteParams& p, hipStream_t st);
int k2_write_lds_bytes(int hd);

int head_fwht_launch(const void* x, long long x_ts, void* out, long long o_ts, int T, int H, const uint8_t* flags,
                     float scale, hipStream_t st, int D);

struct DecodeParams {
  const void* q;
  long long q_bs;
  const uint8_t* pool;
  const int* block_table;
  int bt_stride;
  const int* seq_lens;
  int B, Hkv, page, nsplit, chunk;   // nsplit: body splits (the tail adds one partial)
  float qscale;
  const uint8_t* kmask;    // static formats: q rotated on flagged key groups, or null
  const uint8_t* vmask;    // static formats: output (and tail partial) rotated on flagged value groups, or null
  float* opart;
  float* mlpart;
  int* counter;
  int tile8;               // 1: a workgroup serves a tile of 8 query heads (both 4-head halves on one unpacking), 0: tiles of 4
  void* out;
  long long o_bs;
  const void* tail;
  const int* tail_len;
  const int* tail_idx;
  long long tail_bs, tail_ts;
  int gqa;
  int kv_start;
  int dyn;                 // 1: the nsplit body workgroups of a (sequence, KV head, q tile) share its whole page range and
                           //    draw quads of 4 pages from the slot's counter; 0: split s owns tokens [s, s + 1) * chunk
  int wg_waves;            // wavefronts per workgroup: 4, or the large workgroup that fills a CU
  int fuse_tail;           // 1: no workgroup of their own for the BF16 rows -- the wavefronts of the first body split take
                           //    them after their pages and fold them into their own partials (k_decode, k_decode8; key-only formats)
};
int decode_launch(int fmt, const DecodeParams& p, hipStream_t st);
int decode8_launch(int fmt, const DecodeParams& p, hipStream_t st);       // tiles of 8 query heads (decode_gqa8.hip)
int decode_wide_launch(int fmt, const DecodeParams& p, hipStream_t st);   // head dim 256 (decode_wide.hip)
int decode_big_chunk();                     // tokens per split from which the large workgroup is worth launching
int decode_waves(int chunk_tokens);          // wavefronts per workgroup the launcher picks for a split of that many tokens

void set_error(const char* msg);

}  // namespace fr
