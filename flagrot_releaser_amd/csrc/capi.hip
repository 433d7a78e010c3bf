// extern "C" surface of libflagrot_kernels.so (declared in include/flagrot_kernels.h): argument checks, the
// reference's return codes, and dispatch to the launchers of writer.hip / decode.hip.
#include <cstdlib>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "../../include/flagrot_kernels.h"
#include "fr_common.hpp"
#include "fr_launch.hpp"

namespace fr {
namespace {
char g_err[512] = "";
}
void set_error(const char* msg) {
  std::strncpy(g_err, msg, sizeof(g_err) - 1);
  g_err[sizeof(g_err) - 1] = 0;
}
namespace {
int fail(int code, const char* msg) {
  set_error(msg);
  return code;
}
int launched(int rc, const char* what) {
  if (rc == -1) {
    char buf[400];
    std::snprintf(buf, sizeof(buf), "%s: %s", what, hipGetErrorString(hipGetLastError()));
    set_error(buf);
  } else if (rc == -4) set_error("unknown format / kind");
  else if (rc == -5) set_error("page size not supported");
  return rc;
}
constexpr int GEN = 1024, GT8 = 2048, HD256 = 4096;

int fmt_of_kind(int kind) {
  return kind == KIND_KONLY ? FMT_KONLY : kind == KIND_KONLYA ? FMT_KONLYA : kind == KIND_KONLYA2 ? FMT_KONLYA2 : -1;
}
bool fmt_int2(int fmt) { return fmt == FMT_INT2A || fmt == FMT_KONLYA2; }
}  // namespace
}  // namespace fr

using namespace fr;

namespace {
int device_cus() {
  static int n = 0;
  if (n == 0) {
    int dev = 0;
    hipDeviceProp_t pr;
    n = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&pr, dev) == hipSuccess) ? pr.multiProcessorCount : 256;
  }
  return n;
}
}  // namespace

extern "C" {

int fr_abi_version(void) { return 9; }

int fr_v2_attn(int fmt, const void* q, long long q_bs, const uint8_t* pool, const int* block_table, int bt_stride,
               const int* seq_lens, int B, int Hkv, int page, int nsplit, int chunk, float qscale,
               const uint8_t* kmask, const uint8_t* vmask, int rb, int qrot, int vrot, int variant, int stages,
               float* opart, float* mlpart, int* counter, void* out, long long o_bs, const void* tail,
               const int* tail_len, const int* tail_idx, long long tail_bs, long long tail_ts, void* stream,
               int gqa, int kv_start) {
  if (B <= 0) return 0;
  if (fmt < FMT_INT4 || fmt > FMT_KONLYA2) return fail(-4, "fr_v2_attn: unknown format");
  if ((variant & HD256) && (variant & GT8)) return fail(-3, "fr_v2_attn: head dim 256 takes q tiles of 4 heads");
  if ((variant & ~(GEN | GT8 | HD256)) != 264 && (variant & ~(GEN | GT8 | HD256)) != 0)
    return fail(-3, "fr_v2_attn: unsupported variant");
  if (stages < 1 || stages > 8) return fail(-3, "fr_v2_attn: unsupported stages");
  if (page != 16 && page != 32) return fail(-5, "fr_v2_attn: page size 16 or 32");
  if (gqa <= 0) gqa = 4;
  if (gqa > 64) return fail(-7, "fr_v2_attn: gqa out of range");
  if (gqa != 4 && !(variant & GEN)) return fail(-7, "fr_v2_attn: gqa != 4 needs the generalised variant");
  if (rb != 32 && (qrot || vrot)) return fail(-3, "fr_v2_attn: rotation block 32 only");
  if (nsplit < 1 || chunk <= 0 || chunk % page) return fail(-3, "fr_v2_attn: bad split plan");
  const bool k2 = fmt == FMT_KONLY || fmt == FMT_KONLYA || fmt == FMT_KONLYA2;
  DecodeParams p{};
  p.q = q; p.q_bs = q_bs; p.pool = pool; p.block_table = block_table; p.bt_stride = bt_stride; p.seq_lens = seq_lens;
  p.B = B; p.Hkv = Hkv; p.page = page; p.nsplit = nsplit; p.chunk = chunk; p.qscale = qscale;
  p.kmask = (!k2 && qrot) ? kmask : nullptr;
  p.vmask = (!k2 && (vrot || tail != nullptr)) ? vmask : nullptr;
  p.opart = opart; p.mlpart = mlpart; p.counter = counter;
  // tiles of 8 query heads (GEN | GT8): one workgroup per (KV head, 8 heads), one counter slot and two 4-head partial
  // slots per tile -- the layout a caller sizes with tile_of(variant) = 8; heads past gqa are padding
  p.tile8 = ((variant & GEN) && (variant & GT8)) ? 1 : 0;
  const int ntile = p.tile8 ? (gqa + 7) / 8 : (gqa + 3) / 4;
  p.out = out; p.o_bs = o_bs;
  p.tail = tail; p.tail_len = tail_len; p.tail_idx = tail_idx; p.tail_bs = tail_bs; p.tail_ts = tail_ts;
  p.gqa = gqa; p.kv_start = kv_start;
  // the head-dim-128 kernels read q and the BF16 rows 16 bytes at a time (operands of the matrix instructions)
  if (tail != nullptr && !(variant & HD256) &&
      (((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(tail)) & 15u) != 0 || ((q_bs | tail_bs | tail_ts) & 7) != 0))
    return fail(-3, "fr_v2_attn: with BF16 rows, q and the rows must be 16-byte aligned and their strides multiples of 8 elements");
  // Two launch shapes.  (a) The split plan fills the CUs at most once with long chunks: one large workgroup per CU, each
  // owning its chunk, its wavefronts drawing quads of pages from a counter in LDS.  (b) Otherwise workgroups of 4
  // wavefronts, and where the slot's counter word can hold both (one q tile per slot, tickets above the draw bits) the
  // body workgroups of a (sequence, KV head, q tile) share its whole page range and draw quads from the slot's
  // counter: the split plan then only says how many workgroups there are.  FLAGROT_DECODE_STATIC=1 keeps fixed
  // ranges, FLAGROT_WG_WAVES=4 | 16 forces a workgroup size (above 4: the large one).
  static const bool force_static = getenv("FLAGROT_DECODE_STATIC") != nullptr && getenv("FLAGROT_DECODE_STATIC")[0] == '1';
  static const int env_waves = getenv("FLAGROT_WG_WAVES") != nullptr ? atoi(getenv("FLAGROT_WG_WAVES")) : 0;
  // (read at every call, unlike the others: the tests run the same cases with and without it in one process)
  const char* const replan_env = getenv("FLAGROT_REPLAN");
  const bool replan = !(replan_env != nullptr && replan_env[0] == '0');
  // A plan of more workgroups than CUs is run as fewer, longer splits where shape (a) then applies.  The reference front
  // end caps a chunk at 8192 tokens (vllm_flagrot/kernels.py:74, MAX_CHUNK), so a context beyond 8192 tokens always
  // arrives as two or more splits per (sequence, KV head, q tile) pair -- also where 256 pairs fill the CUs by
  // themselves (B = 32, 8 KV heads), the case in which one large workgroup per CU streaming the whole sequence is the
  // fastest shape there is (B = 32, L = 16 k ... 64 k on the 4-bit pages: 0.59-0.65 -> 0.76-0.79 of the bandwidth).
  //  * pairs <= CUs: CUs / pairs splits per pair, one round of large workgroups (every format);
  //  * pairs > CUs, 4-bit pages (launches bound by memory; the 2-bit ones are bound by vector issue and gain nothing):
  //    the fewest splits (the longest chunks, >= 4096 tokens) whose large workgroups fill their last round of CUs to
  //    90 % -- B = 64, L = 8 k ... 32 k: 0.61-0.67 -> 0.72-0.79; a round and a quarter of them would be slower than the
  //    small workgroups (B = 40: 82 -> 89 us), so such plans stay as they are.
  // The splits that are run are the first `nsplit` of the caller's layout: never more than the caller planned, so
  // partials and tickets stay inside what the caller sized.  FLAGROT_REPLAN=0 switches this off (experiments).
  const long long pairs = static_cast<long long>(B) * Hkv * ntile;
  const long long cus = device_cus();
  bool rounds = false;                       // large workgroups although there are more of them than CUs
  if (replan && env_waves == 0 && !(variant & HD256) && pairs * nsplit > cus) {
    const long long span = static_cast<long long>(nsplit) * chunk;
    auto chunk_for = [&](long long ns) { return static_cast<int>(((span + ns - 1) / ns + 63) / 64 * 64); };   // a multiple of both page sizes
    int fewer = 0;
    if (span < (1ll << 30)) {
      if (pairs <= cus) {
        if (chunk_for(cus / pairs) >= decode_big_chunk()) fewer = static_cast<int>(cus / pairs);   // >= 1 and < nsplit
      } else if (!fmt_int2(fmt)) {
        for (int ns = 1; ns <= nsplit && ns <= 8 && chunk_for(ns) >= 4096; ++ns) {
          const long long wg = pairs * ns, full = (wg + cus - 1) / cus * cus;
          if (wg * 10 >= full * 9) { fewer = ns; rounds = true; break; }
        }
      }
    }
    if (fewer > 0) {
      chunk = chunk_for(fewer); nsplit = fewer;
      p.nsplit = nsplit; p.chunk = chunk;
    }
  }
  // Short splits (below the large workgroups' threshold; the reference planner makes them for short contexts on few
  // pairs: one sequence of 2048 tokens arrives as 6 x 384) are run as large workgroups too where those fit the CUs once:
  // a single one up to 1024 tokens, splits of 512 tokens beyond -- these launches are chains of latencies, and a
  // workgroup whose 16 wavefronts take one quad each has the shortest one (one sequence: 512 tokens 10.3 -> 9.6 us,
  // 1536 14.5 -> 11.8, 2048 15.0 -> 11.9; 32 sequences of 512 14.7 -> 11.0; tiles of 8 heads, one sequence of 2048
  // 20.8 -> 15.3).  From 512 tokens: below, the four wavefronts of a small workgroup are as fast or faster (256 tokens:
  // 7.9 against 8.8 us).  Never more splits than the caller's.
  bool short_big = false;
  if (replan && env_waves == 0 && !(variant & HD256) && chunk < decode_big_chunk()) {
    const long long span = static_cast<long long>(nsplit) * chunk;
    if (span >= 512 && span < (1ll << 30)) {
      const int ns = span <= 1024 ? 1 : static_cast<int>((span + 511) / 512);
      const int ch = span <= 1024 ? static_cast<int>(span) : 512;
      if (ns <= nsplit && pairs * ns <= cus) {
        nsplit = ns; chunk = ch; short_big = true;
        p.nsplit = nsplit; p.chunk = chunk;
      }
    }
  }
  const long long wgs = pairs * nsplit;
  const bool big = env_waves > 4 || short_big || (env_waves == 0 && chunk >= decode_big_chunk() && (wgs <= cus || rounds));
  // BF16 rows: the wavefronts of the first split take them themselves (static formats: rotated into the stored basis
  // wavefront by wavefront) -- one partial less, and with a single split no ticket and no merge at all.  Their cost is small
  // (scores on the matrix pipe, tail_partial), a workgroup of their own costs its whole life: arguments, rows, epilogue,
  // partial, ticket, merge.
  static const bool fuse_ok = !(getenv("FLAGROT_FUSE_TAIL") != nullptr && getenv("FLAGROT_FUSE_TAIL")[0] == '0');
  // (several splits: only where a split is long -- 4096 tokens -- since the first split's workgroup ends later than
  // the others; with 32 splits of 1024 tokens of one sequence the rows' own workgroups were faster)
  p.fuse_tail = (fuse_ok && tail != nullptr && env_waves == 0 && !(variant & HD256) &&
                 (nsplit == 1 || chunk >= 4096)) ? 1 : 0;
  const int nparts = nsplit + ((tail != nullptr && !p.fuse_tail) ? 1 : 0);
  const bool can_draw = !force_static && counter != nullptr && nparts <= 1023;
  // the split merge goes through the caller's workspace: partials, their (max, sum) pairs and, at head dim 128, the ticket
  if (nparts > 1 && (opart == nullptr || mlpart == nullptr || (!(variant & HD256) && counter == nullptr)))
    return fail(-3, "fr_v2_attn: more than one partial per (sequence, KV head) needs opart, mlpart and counter");
  if ((variant & HD256) && (opart == nullptr || mlpart == nullptr))
    return fail(-3, "fr_v2_attn: the head dim 256 kernels need opart and mlpart");
  p.wg_waves = big ? decode_waves(1 << 30) : 4;
  p.dyn = (can_draw && (!big || env_waves > 4)) ? 1 : 0;
  if (variant & HD256) return launched(decode_wide_launch(fmt, p, static_cast<hipStream_t>(stream)), "fr_v2_attn (head dim 256)");
  return launched(decode_launch(fmt, p, static_cast<hipStream_t>(stream)), "fr_v2_attn");
}

int fr_v2_write(int fmt, const void* kv, long long kv_ts, const long long* slots, int T, int Hkv, int page,
                const uint8_t* mask, int rb, uint8_t* pool, void* stream, int hd, const float* kmu) {
  if (T <= 0) return 0;
  if (hd != 0 && hd != 128 && hd != 256) return fail(-8, "fr_v2_write: head dim 128 | 256");
  if (rb != 32) return fail(-3, "fr_v2_write: rotation block 32 only");
  StaticWriteParams p{};
  p.kv = kv; p.kv_ts = kv_ts; p.slots = slots; p.T = T; p.Hkv = hd == 256 ? 2 * Hkv : Hkv; p.page = page;
  p.mask = mask; p.hfull = nullptr; p.kmu = kmu; p.pool = pool;
  return launched(static_write_launch(fmt, p, static_cast<hipStream_t>(stream)), "fr_v2_write");
}

// What the host split planner multiplies by the CU count to get the number of workgroups that run at once.  The answer
// is 1: the fastest launch shape is ONE large workgroup per CU (decode_launch takes it whenever the plan's workgroups
// fit the CUs once with >= 1024 tokens each), and a planner that fills "1 x CUs" slots with the longest chunks that
// fit (the reference front end's cost model, vllm_flagrot/kernels.py:247-265) lands on exactly that shape: 256
// (sequence, KV head) pairs of 8192 tokens -> nsplit 1, chunk 8192; 8 pairs of 32768 tokens -> 32 splits of 1024.
// When more workgroups than CUs are asked for, the library runs 4-wavefront workgroups, of which up to 4 are
// resident per CU; it then treats nsplit only as the number of workgroups per (sequence, KV head, q tile).
int fr_v2_occupancy(int fmt, int variant, int stages, int page) {
  (void)variant; (void)stages;
  if ((page != 16 && page != 32) || fmt < FMT_INT4 || fmt > FMT_KONLYA2) return 0;
  return 1;
}
int fr_v2_chunk_bytes(int fmt, int page) { return page * (fmt_int2(fmt) ? 80 : 144); }

int fr_cb_nsg(void) { return 15; }

int fr_cb_write(const void* kv, long long kv_ts, const long long* slots, int slot_ph, int T, int Hkv, int page, int tg,
                const float* CT, const float* co, const unsigned* sg, int kind, uint8_t* pool, void* stream, int hd,
                const float* kmu) {
  (void)tg; (void)co; (void)sg;
  if (T <= 0) return 0;
  if (hd != 0 && hd != 128 && hd != 256) return fail(-8, "fr_cb_write: head dim 128 | 256");
  K2WriteParams p{};
  p.kv = kv; p.kv_ts = kv_ts; p.slots = slots; p.slot_ph = slot_ph; p.T = T; p.Hkv = Hkv; p.page = page;
  p.CT = CT; p.kmu = kmu; p.pool = pool; p.passes = 3; p.hd = hd == 256 ? 256 : 128;
  return launched(k2_write_launch(kind, p, static_cast<hipStream_t>(stream)), "fr_cb_write");
}

int fr_cb_write3(const void* kv, long long kv_ts, const long long* slots, int slot_ph, int T, int Hkv, int page,
                 const float* CT, const float* co, const void* C1, const float* beta, const unsigned* sg, int kind,
                 uint8_t* pool, int nchunk, int nchunk_v, void* stream, const float* kmu) {
  (void)co; (void)C1; (void)beta; (void)sg;
  if (T <= 0) return 0;
  K2WriteParams p{};
  p.kv = kv; p.kv_ts = kv_ts; p.slots = slots; p.slot_ph = slot_ph; p.T = T; p.Hkv = Hkv; p.page = page;
  p.CT = CT; p.kmu = kmu; p.pool = pool;
  p.passes = (nchunk >= 0 ? 1 : 0) | (nchunk_v >= 0 ? 2 : 0);
  p.screen = 1;
  if (p.passes == 0) return 0;
  return launched(k2_write_launch(kind, p, static_cast<hipStream_t>(stream)), "fr_cb_write3");
}

int fr_w3_static_write(const void* kv, long long kv_ts, const long long* slots, int T, int Hkv, int page,
                       const uint8_t* mask, const uint8_t* hfull, int asym, uint8_t* pool, int path, void* stream,
                       const float* kmu) {
  (void)path;
  if (T <= 0) return 0;
  if (asym < 0 || asym > 2) return fail(-4, "fr_w3_static_write: asym must be 0, 1 or 2");
  StaticWriteParams p{};
  p.kv = kv; p.kv_ts = kv_ts; p.slots = slots; p.T = T; p.Hkv = Hkv; p.page = page;
  p.mask = mask; p.hfull = hfull; p.kmu = kmu; p.pool = pool;
  const int fmt = asym == 0 ? FMT_INT4 : asym == 1 ? FMT_INT4A : FMT_INT2A;
  return launched(static_write_launch(fmt, p, static_cast<hipStream_t>(stream)), "fr_w3_static_write");
}

int fr_cb_attn(const void* q, long long q_bs, const uint8_t* pool, const int* block_table, int bt_stride,
               const int* seq_lens, int B, int Hkv, int page, int nsplit, int chunk, float qscale, const unsigned* sg,
               int kind, int variant, int stages, float* opart, float* mlpart, int* counter, void* out, long long o_bs,
               const void* tail, const int* tail_len, const int* tail_idx, long long tail_bs, long long tail_ts,
               void* stream, int kv_start) {
  (void)sg;
  if (B <= 0) return 0;
  const int fmt = fmt_of_kind(kind);
  if (fmt < 0) return fail(-4, "fr_cb_attn: kind must be 6 (konly), 10 (konlya) or 11 (konlya2)");
  if (variant != 0 && variant != 1) return fail(-3, "fr_cb_attn: unsupported variant");
  return fr_v2_attn(fmt, q, q_bs, pool, block_table, bt_stride, seq_lens, B, Hkv, page, nsplit, chunk, qscale, nullptr,
                    nullptr, 32, 0, 0, 264, stages, opart, mlpart, counter, out, o_bs, tail, tail_len, tail_idx,
                    tail_bs, tail_ts, stream, 4, kv_start);
}

// ---- the entry point that allocates nothing --------------------------------------------------------------------
// Split partials, their (max, sum) pairs and the ticket / draw counters of fr_cb_attn_noalloc live in this array
// instead of a caller-owned workspace.  Every GPU the library runs on holds its own copy, at its own address, until
// the process ends.  Host code must never use the array's name as a device address: the address is asked for once
// per device (scratch_of) and only that pointer is handed to kernels.
}  // extern "C"
namespace {
constexpr int NA_MAX_PARTS = FR_NOALLOC_MAX_PARTS;            // partials of 4 heads x 128 floats
constexpr size_t NA_OPART = size_t(NA_MAX_PARTS) * 512 * 4;   // bytes
constexpr size_t NA_MLPART = size_t(NA_MAX_PARTS) * 8 * 4;
constexpr size_t NA_COUNTER = size_t(NA_MAX_PARTS) * 4;
static __device__ __align__(256) unsigned char scratch[NA_OPART + NA_MLPART + NA_COUNTER];

constexpr int NA_MAX_DEV = 64;
std::mutex g_scratch_mu;
unsigned char* g_scratch_ptr[NA_MAX_DEV] = {nullptr};

// device address of `scratch` on the current device (asked for once per device), or null with the error text set
unsigned char* scratch_of() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= NA_MAX_DEV) {
    (void)hipGetLastError();
    set_error("fr_cb_attn_noalloc: no current device");
    return nullptr;
  }
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      char buf[200];
      std::snprintf(buf, sizeof(buf), "fr_cb_attn_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
      (void)hipGetLastError();
      set_error(buf);
      return nullptr;
    }
    g_scratch_ptr[dev] = static_cast<unsigned char*>(ptr);
  }
  return g_scratch_ptr[dev];
}

// a fill kernel and not hipMemsetAsync: memset nodes recorded into a HIP graph are not reliable on replays
__global__ void k_clear_words(int* w, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) w[i] = 0;
}
}  // namespace
extern "C" {

int fr_cb_attn_noalloc(const void* q, long long q_bs, const uint8_t* pool, const int* block_table, int bt_stride,
                       const int* seq_lens, int B, int Hkv, int page, int nsplit, int chunk, float qscale, int kind,
                       void* out, long long o_bs, const void* tail, const int* tail_len, const int* tail_idx,
                       long long tail_bs, long long tail_ts, void* stream, int gqa, int kv_start) {
  if (B <= 0) return 0;
  const int fmt = fmt_of_kind(kind);
  if (fmt < 0) return fail(-4, "fr_cb_attn_noalloc: kind must be 6 (konly), 10 (konlya) or 11 (konlya2)");
  if (gqa <= 0) gqa = 4;
  if (gqa > 64 || Hkv <= 0 || nsplit < 1) return fail(-7, "fr_cb_attn_noalloc: bad gqa / Hkv / nsplit");
  const long long ntile = (gqa + 3) / 4;
  const long long parts = static_cast<long long>(B) * Hkv * ntile * (nsplit + 1);
  if (parts > NA_MAX_PARTS) {
    char buf[200];
    std::snprintf(buf, sizeof(buf), "fr_cb_attn_noalloc: B*Hkv*ceil(gqa/4)*(nsplit+1) = %lld partials exceed the built-in "
                  "workspace of %d", parts, NA_MAX_PARTS);
    return fail(-2, buf);
  }
  unsigned char* base = scratch_of();
  if (base == nullptr) return -1;
  float* opart = reinterpret_cast<float*>(base);
  float* mlpart = reinterpret_cast<float*>(base + NA_OPART);
  int* counter = reinterpret_cast<int*>(base + NA_OPART + NA_MLPART);
  // The counters are left at zero by every completed call; they are cleared all the same, so that a call that was cut
  // short (a failed launch, a device reset of another context) cannot poison the next one.
  const int nctr = static_cast<int>(static_cast<long long>(B) * Hkv * ntile);
  hipLaunchKernelGGL(k_clear_words, dim3((nctr + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), counter, nctr);
  if (hipPeekAtLastError() != hipSuccess) return launched(-1, "fr_cb_attn_noalloc (clear)");
  // groups of 5 .. 8 heads (and whole multiples of 8) run tiles of 8 heads: same partial slots, half the counter words
  const int variant = 264 | GEN | (((gqa > 4 && gqa <= 8) || gqa % 8 == 0) ? GT8 : 0);
  return fr_v2_attn(fmt, q, q_bs, pool, block_table, bt_stride, seq_lens, B, Hkv, page, nsplit, chunk, qscale, nullptr,
                    nullptr, 32, 0, 0, variant, 4, opart, mlpart, counter, out, o_bs, tail, tail_len, tail_idx,
                    tail_bs, tail_ts, stream, gqa, kv_start);
}

int fr_cb_occupancy(int kind, int variant, int stages, int page) {
  (void)variant; (void)stages;
  if ((page != 16 && page != 32) || fmt_of_kind(kind) < 0) return 0;
  return 1;      // as fr_v2_occupancy: one large workgroup per CU is the shape a planner should aim at
}
int fr_cb_chunk_bytes(int kind, int page) { return page * (kind == KIND_KONLYA2 ? 80 : 144); }
int fr_cb_write_smem(int kind, int tg, int hd) {
  (void)tg;
  if (fmt_of_kind(kind) < 0 || (hd != 0 && hd != 128 && hd != 256)) return 0;
  return k2_write_lds_bytes(hd);
}

const char* fr_last_error(void) { return g_err; }

int fr_head_fwht(const void* x, long long x_ts, void* out, long long o_ts, int T, int H, const uint8_t* flags,
                 float scale, void* stream, int D) {
  if (T <= 0) return 0;
  if (D != 128 && D != 256) return fail(-8, "fr_head_fwht: head dim 128 | 256");
  return launched(head_fwht_launch(x, x_ts, out, o_ts, T, H, flags, scale, static_cast<hipStream_t>(stream), D),
                  "fr_head_fwht");
}

}  // extern "C"
