// Launchers of the head-dim-256 kernels of libflagrot_mq.so (mq_wide.hip), called from the C ABI in mq_prefill.hip.
// Return 0, or -1 when the launch failed.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace frmq {

struct Params;
int wide_smem_bytes();
int wide_attn_launch(const Params& p, int nitems, int konly, hipStream_t st);
int wide_query_rows_launch(const void* q, int q_fp32, long long q_ts, const int* idx, int m, int Hq, int G, const uint8_t* kfull,
                           const uint8_t* kmask, float qscale, void* q16, hipStream_t st);

}  // namespace frmq
