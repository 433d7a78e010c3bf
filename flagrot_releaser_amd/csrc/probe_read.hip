// Measurement aid, not part of the drop-in boundary: a kernel that ONLY READS the pages a paged decode launch reads,
// through the same block table and with the same workgroup layout (one workgroup of 16 wavefronts per (sequence, KV
// head), KV head fastest in dispatch order, a wavefront takes every sixteenth page, four pages in flight, 16-byte loads
// per lane over the contiguous chunk of a (page, KV head), with the non-temporal hint as in the decode kernels: 46.9 us
// for the 302 MB of the 32 x 8192-token launch, 52.6 us without the hint).  What it reaches on a cache is the rate this memory system
// gives any kernel with that access pattern: the yardstick the decode kernel's time is read against.
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>

#include "../../include/flagrot_probe.h"

namespace {

char g_err[256] = "";
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int KU>      // 1 KB slices (64 lanes x 16 bytes) per chunk: 3 covers pages of 16 tokens, 5 pages of 32 (4608 bytes)
__global__ void __launch_bounds__(1024) k_probe_read(const uint8_t* __restrict__ pool, const int* __restrict__ bt, int bt_stride,
                                                     const int* __restrict__ seq_lens, int Hkv, int page, int chunk_bytes,
                                                     uint32_t* __restrict__ sink) {
  const int kvh = blockIdx.x, b = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int npg = (seq_lens[b] + page - 1) / page;
  const int* row = bt + static_cast<long long>(b) * bt_stride;
  const int units = chunk_bytes / 16;                       // 16-byte units of a chunk
  uint32_t acc = 0;
  for (int pg = wave; pg < npg; pg += 64) {
    u32x4 v[4][KU];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int pi = min(pg + 16 * u, npg - 1);             // past the end: the last page again (a cache hit)
      const uint8_t* ch = pool + (static_cast<long long>(row[pi]) * Hkv + kvh) * chunk_bytes;
#pragma unroll
      for (int k = 0; k < KU; ++k) {
        const int at = k * 64 + lane;
        v[u][k] = at < units ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(ch + 16 * at)) : u32x4{0u, 0u, 0u, 0u};
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int k = 0; k < KU; ++k) acc |= v[u][k].x | v[u][k].y | v[u][k].z | v[u][k].w;
  }
  // keeps the loads alive; on real pages practically never taken (a test plants the value in a pool of zeros)
  if (acc == 0x9E3779B9u) sink[0] = acc;
}

}  // namespace

extern "C" {

int fr_probe_abi_version(void) { return 1; }
const char* fr_probe_last_error(void) { return g_err; }

int fr_probe_read(const uint8_t* pool, const int* block_table, int bt_stride, const int* seq_lens, int B, int Hkv, int page,
                  int chunk_bytes, uint32_t* sink, void* stream) {
  if (B <= 0) return 0;
  if (chunk_bytes <= 0 || chunk_bytes % 16 || chunk_bytes > 5 * 64 * 16 || (page != 16 && page != 32)) {
    std::snprintf(g_err, sizeof(g_err), "fr_probe_read: chunk of %d bytes / page %d", chunk_bytes, page);
    return -2;
  }
  if (chunk_bytes <= 3 * 64 * 16)
    hipLaunchKernelGGL(k_probe_read<3>, dim3(Hkv, B), dim3(1024), 0, static_cast<hipStream_t>(stream), pool, block_table,
                       bt_stride, seq_lens, Hkv, page, chunk_bytes, sink);
  else
    hipLaunchKernelGGL(k_probe_read<5>, dim3(Hkv, B), dim3(1024), 0, static_cast<hipStream_t>(stream), pool, block_table,
                       bt_stride, seq_lens, Hkv, page, chunk_bytes, sink);
  if (hipPeekAtLastError() != hipSuccess) {
    std::snprintf(g_err, sizeof(g_err), "fr_probe_read: %s", hipGetErrorString(hipGetLastError()));
    return -1;
  }
  return 0;
}

}  // extern "C"
