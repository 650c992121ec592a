// Shared host/device helpers for the gfx950 kernels behind include/ssc.h.
#ifndef SSC_COMMON_H_
#define SSC_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "ssc.h"

namespace ssc {

// Thread-local message returned by ssc_last_error().
int fail(int code, const char *fmt, ...);

#define SSC_CHECK(cond, code, ...)                        \
  do {                                                    \
    if (!(cond)) return ::ssc::fail((code), __VA_ARGS__); \
  } while (0)

#define SSC_HIP(expr)                                                                   \
  do {                                                                                  \
    hipError_t e__ = (expr);                                                            \
    if (e__ != hipSuccess)                                                              \
      return ::ssc::fail(SSC_EHIP, "%s failed: %s", #expr, hipGetErrorString(e__));     \
  } while (0)

#define SSC_LAUNCH_CHECK(name)                                                          \
  do {                                                                                  \
    hipError_t e__ = hipGetLastError();                                                 \
    if (e__ != hipSuccess)                                                              \
      return ::ssc::fail(SSC_EHIP, "launch of %s failed: %s", name, hipGetErrorString(e__)); \
  } while (0)

static inline size_t align_up(size_t x, size_t a = 256) { return (x + a - 1) / a * a; }
static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Carves 256-byte aligned regions out of a caller-provided workspace.
struct Carver {
  char *base;
  size_t used;
  explicit Carver(void *p) : base(static_cast<char *>(p)), used(0) {}
  template <typename T> T *take(size_t count) {
    T *p = reinterpret_cast<T *>(base + used);
    used += align_up(count * sizeof(T));
    return p;
  }
};

// ---- rank/select over a bit table -------------------------------------------------------
// A set of integer keys in [0, n_bits) is held as a bit table.  After
// popcount_scan(), rank(key) = prefix[key >> 5] + popc(bits[key >> 5] below key)
// numbers the keys in ascending order: a minimal perfect hash whose order is
// the sorted order, so no sort and no probing are needed.
constexpr int kScanThreads = 256;
constexpr int kScanItems = 8;  // words per thread
constexpr int kScanBlockWords = kScanThreads * kScanItems;

struct BitTable {
  uint32_t *bits;     // [n_words]
  int32_t *prefix;    // [n_words] exclusive popcount prefix
  int32_t *blocksum;  // [n_scan_blocks]
  int32_t *total;     // [4]: popcount of the table; a flag word; two words for the table's user
  int64_t n_words;
  int64_t n_scan_blocks;
};

static inline int64_t bit_words(int64_t n_bits) { return ceil_div(n_bits, 32); }
size_t bit_table_bytes(int64_t n_bits);
BitTable bit_table_carve(Carver &c, int64_t n_bits);
// Enqueue: zero the table and total[]; with blocksum_too also blocksum[] (for a first scan
// pass that adds into it); with per_word also that array of one counter for every word.
int bit_table_clear(const BitTable &t, hipStream_t s, bool blocksum_too = false,
                    int32_t *per_word = nullptr);
// Enqueue: prefix[], total[0] from bits[].  With `mirror` (memory the device can write and
// the host can read, see read_back_mirror), the kernel that writes total[0] also copies
// total[0..3] there, which saves the copy a host that waits for them would otherwise queue.
int bit_table_scan(const BitTable &t, hipStream_t s, int32_t *mirror = nullptr, int ticket = 0);
// The second pass of bit_table_scan alone (the first one, popc_blocksum_block, is then run
// by a kernel of the caller that has other work to do beside it).
int bit_table_scan_prefix(const BitTable &t, hipStream_t s, int32_t *mirror = nullptr,
                          int ticket = 0);

// Block-wide exclusive scan of one int per thread (kScanThreads threads).
__device__ __forceinline__ int block_exclusive_scan(int v, int *lds /* [kScanThreads/64 + 1] */,
                                                    int *block_total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    int o = __shfl_up(incl, d, 64);
    if (lane >= d) incl += o;
  }
  if (lane == 63) lds[wave] = incl;
  __syncthreads();
  int wave_off = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < kScanThreads / 64; ++w) {
    int x = lds[w];
    if (w < wave) wave_off += x;
    tot += x;
  }
  __syncthreads();
  *block_total = tot;
  return wave_off + incl - v;
}

// First pass of the popcount scan for scan block `b` (kScanThreads threads):
// blocksum[b] = popcount of the block's kScanBlockWords words.
__device__ __forceinline__ void popc_blocksum_block(const uint32_t *__restrict__ bits,
                                                    int64_t n_words, int64_t b,
                                                    int32_t *__restrict__ blocksum, int *lds) {
  int64_t base = b * kScanBlockWords + (int64_t)threadIdx.x * kScanItems;
  int v = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i)
    if (base + i < n_words) v += __popc(bits[base + i]);
  int tot;
  block_exclusive_scan(v, lds, &tot);
  if (threadIdx.x == 0) blocksum[b] = tot;
}

// Second pass of the popcount scan for scan block blockIdx.x (kScanThreads threads):
// exclusive prefix per word.  Every block first adds up the sums of the blocks before it
// (at most 2^31 / 32 / kScanBlockWords = 32768 values), which saves the launch of a scan
// over blocksum[]; the table's last block (`last`) also writes the total, and with `mirror`
// copies total[0..3] there (total[1..3] were written by kernels before this one).
constexpr int kMirrorTicket = 8;  // where in the host mirror a ticket goes (see read_back_mirror_ticket)
__device__ __forceinline__ void popc_prefix_block(const uint32_t *__restrict__ bits,
                                                  int64_t n_words,
                                                  const int32_t *__restrict__ blocksum,
                                                  int32_t *__restrict__ prefix,
                                                  int32_t *__restrict__ total,
                                                  int32_t *__restrict__ mirror, bool last,
                                                  int ticket = 0) {
  __shared__ int lds[kScanThreads / 64 + 1];
  int before = 0;
  for (int64_t b = threadIdx.x; b < (int64_t)blockIdx.x; b += kScanThreads) before += blocksum[b];
  int block_off;
  block_exclusive_scan(before, lds, &block_off);
  int64_t base = (int64_t)blockIdx.x * kScanBlockWords + (int64_t)threadIdx.x * kScanItems;
  int c[kScanItems];
  int v = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    c[i] = base + i < n_words ? __popc(bits[base + i]) : 0;
    v += c[i];
  }
  int tot;
  int ex = block_exclusive_scan(v, lds, &tot) + block_off;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    if (base + i < n_words) prefix[base + i] = ex;
    ex += c[i];
  }
  if (last && threadIdx.x == 0) {
    total[0] = block_off + tot;
    if (mirror != nullptr) {
      mirror[0] = block_off + tot;
      mirror[1] = total[1];
      mirror[2] = total[2];
      mirror[3] = total[3];
      // (a host that spins on the ticket sees the four values with it: read_back_end)
      if (ticket != 0)
        __hip_atomic_store(mirror + kMirrorTicket, ticket, __ATOMIC_RELEASE,
                           __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

__device__ __forceinline__ int bit_rank(const uint32_t *__restrict__ bits,
                                        const int32_t *__restrict__ prefix, uint32_t key) {
  uint32_t w = key >> 5;
  uint32_t below = bits[w] & ((1u << (key & 31u)) - 1u);
  return prefix[w] + __popc(below);
}

// Decode every set bit of word w into its (b,x,y,z) row, written at the bit's rank.
__device__ __forceinline__ void emit_rows_of_word_at(uint32_t b, int r, int64_t w, int d1,
                                                     int d2, int d3,
                                                     int32_t *__restrict__ out);
__device__ __forceinline__ void emit_rows_of_word(const uint32_t *__restrict__ bits,
                                                  const int32_t *__restrict__ prefix, int64_t w,
                                                  int d1, int d2, int d3,
                                                  int32_t *__restrict__ out) {
  const uint32_t b = bits[w];
  if (b == 0) return;
  emit_rows_of_word_at(b, prefix[w], w, d1, d2, d3, out);
}
// The same for a word b whose first set bit has rank r.
__device__ __forceinline__ void emit_rows_of_word_at(uint32_t b, int r, int64_t w, int d1,
                                                     int d2, int d3,
                                                     int32_t *__restrict__ out) {
  // the word's first cell is decoded once; its other cells differ in z only, unless
  // the word runs over the end of a z row (extents that are not multiples of 32)
  uint32_t key0 = (uint32_t)(w * 32);
  const int z0 = key0 % d3;
  key0 /= d3;
  const int y0 = key0 % d2;
  key0 /= d2;
  const int x0 = key0 % d1;
  const int b0 = key0 / d1;
  while (b) {
    int bit = __ffs(b) - 1;
    b &= b - 1;
    int z = z0 + bit;
    if (z < d3) {
      reinterpret_cast<int4 *>(out)[r++] = make_int4(b0, x0, y0, z);
    } else {
      uint32_t key = (uint32_t)(w * 32 + bit);
      z = key % d3;
      key /= d3;
      int y = key % d2;
      key /= d2;
      int x = key % d1;
      int bb = key / d1;
      reinterpret_cast<int4 *>(out)[r++] = make_int4(bb, x, y, z);
    }
  }
}

// ---- work split of a convolution, seeded by the rulebook ----------------------------------
// A regular rulebook knows, word by word of its output table, how many output rows and how
// many pairs lie below the word (at stride 1 the popcounts its dilation step takes anyway;
// otherwise the marking kernel counts the pairs of every word on its way).  That is the work
// measure the convolution's plan deals its output rows to the workgroups by, so the rulebook
// can place the ranges' boundaries itself, in a launch it makes anyway: the plan is then
// built without its own passes over the pairs for that purpose.
constexpr int kMaxRanges = 512;       // two for each of at most 256 workgroups
constexpr int kSeedMaxBlocks = 512;   // scan blocks of a table whose block sums are scanned in LDS by
                                      // every block that needs them (512: 33 M cells)
struct SplitRequest {
  int n_rng;           // ranges to cut the output rows into (<= kMaxRanges)
  int tile_rows;       // weight of a pair relative to tile_cost (see split_work in conv.hip)
  long long tile_cost; // cost of a row's share of a tile, in the same unit
  int32_t *range_row0; // [n_rng + 1] device: first output row of every range
  // A second cut of the same rows (n_rng_alt = 0: none), for a caller whose plan depends on
  // the number of output rows, which only the rulebook's totals will tell: it asks for the
  // cut of either plan and uses the one that applies.
  int n_rng_alt, tile_rows_alt;
  int32_t *range_row0_alt;
};
// Blocks of kScanThreads threads that place the boundaries of a request (16 lanes to a range).
static inline int split_request_blocks(const SplitRequest &rq) {
  return (int)(ceil_div(rq.n_rng, kScanThreads / 16) + ceil_div(rq.n_rng_alt, kScanThreads / 16));
}
// ssc_rulebook_begin with an optional split request.  *seeded = whether range_row0 will be
// written (a regular convolution whose table has at most kSeedMaxBlocks scan blocks).  `job`
// (optional, conv_pack.h): synthesis and packing of a layer's filters, enqueued with the
// rulebook's first launch where that has room for it and before it otherwise.
struct CombineJob;
int rulebook_begin_impl(const int32_t *indices, int64_t n_in, const ssc_geometry *g,
                        void *workspace, size_t workspace_bytes, int32_t *pairs,
                        int32_t *pair_num, int32_t *out_indices, int64_t out_capacity,
                        void *clean_table, size_t clean_table_bytes, const SplitRequest *split,
                        bool *seeded, hipStream_t s, const CombineJob *job);

// Enqueue: fill an int32 array (a kernel, so the call may be graph-captured).
int fill_i32(int32_t *p, int64_t n, int32_t v, hipStream_t s);
int fill_f32(float *p, int64_t n, float v, hipStream_t s);

// Bring `bytes` (at most kReadBackBytes) of device memory to the host behind the work queued
// on `s` and wait for it.  The copy lands in a block of pinned host memory that each host
// thread keeps for the life of the process, so nothing is staged through a pageable buffer;
// `*view` points into that block and holds until the thread's next read-back.
constexpr size_t kReadBackBytes = 64 << 10;
int read_back_view(const void **view, const void *src_dev, size_t bytes, hipStream_t s);
// The same in two steps: read_back_begin queues the copy and an event behind the work on
// `s` and returns; read_back_end, on the same host thread, waits for that event only, so
// work queued on `s` after read_back_begin keeps the GPU busy while the host wakes up.
int read_back_begin(const void *src_dev, size_t bytes, hipStream_t s);
int read_back_end(const void **view);
// The same without a copy: *mirror is the calling thread's pinned block as the device sees
// it; a kernel queued on `s` writes its results there, read_back_mirror_queued records the
// event behind that kernel, and read_back_end waits for it and returns the block.
int read_back_mirror(int32_t **mirror);
int read_back_mirror_queued(hipStream_t s, int ticket = 0);
// For a kernel that stores its results into the mirror while it still has other work to
// do: the kernel stores the results, then `ticket` (read_back_mirror_ticket(), never 0) into
// mirror[kMirrorTicket] with a release at system scope; read_back_mirror_queued(s, ticket)
// behind the launch; read_back_end then returns as soon as the ticket shows up in the host's
// view of the block, not when the kernel ends.
int read_back_mirror_ticket();
// The same, moved on to `dst_host`.
int read_back(void *dst_host, const void *src_dev, size_t bytes, hipStream_t s);

// The activation functions of the gated non-linearity (SSC_ACT_* of ssc.h).
#ifdef __HIPCC__
__device__ __forceinline__ float act_fn(int kind, float u) {
  switch (kind) {
    case SSC_ACT_RELU: return u > 0.f ? u : 0.f;
    // v_rcp_f32 (one unit in the last place) instead of a correctly rounded division: a
    // fifth of the instructions, and the sigmoid is most of what a gated column costs
    case SSC_ACT_SIGMOID: return __builtin_amdgcn_rcpf(1.f + __expf(-u));
    case SSC_ACT_TANH: return tanhf(u);
    default: return u;
  }
}
#endif

}  // namespace ssc

#endif
