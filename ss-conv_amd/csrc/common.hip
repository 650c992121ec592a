// Error reporting, fill kernels and the popcount scan shared by the rulebook,
// voxel-unique and pair re-ordering paths.
#include "ssc_common.h"

#include <string.h>

namespace ssc {

static thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

__global__ void fill_i32_kernel(int32_t *__restrict__ p, int64_t n, int32_t v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += step) p[i] = v;
}

int fill_i32(int32_t *p, int64_t n, int32_t v, hipStream_t s) {
  if (n <= 0) return SSC_OK;
  int blocks = (int)(ceil_div(n, 256) < 8192 ? ceil_div(n, 256) : 8192);
  hipLaunchKernelGGL(fill_i32_kernel, dim3(blocks), dim3(256), 0, s, p, n, v);
  SSC_LAUNCH_CHECK("fill_i32");
  return SSC_OK;
}

int fill_f32(float *p, int64_t n, float v, hipStream_t s) {
  int32_t bits;
  memcpy(&bits, &v, sizeof(bits));
  return fill_i32(reinterpret_cast<int32_t *>(p), n, bits, s);
}

size_t bit_table_bytes(int64_t n_bits) {
  int64_t w = bit_words(n_bits);
  int64_t nb = ceil_div(w, kScanBlockWords);
  return align_up(w * 4) * 2 + align_up((nb + 1) * 4) + align_up(4 * sizeof(int32_t));
}

BitTable bit_table_carve(Carver &c, int64_t n_bits) {
  BitTable t;
  t.n_words = bit_words(n_bits);
  t.n_scan_blocks = ceil_div(t.n_words, kScanBlockWords);
  t.bits = c.take<uint32_t>(t.n_words);
  t.prefix = c.take<int32_t>(t.n_words);
  t.blocksum = c.take<int32_t>(t.n_scan_blocks + 1);
  t.total = c.take<int32_t>(4);  // [1]: flag word, [2], [3]: for the table's user
  return t;
}

// bits[] = 0, total[0..3] = 0 and (when asked for) blocksum[] = 0 and a counter for every
// word, per_word[] = 0, in one launch.
__global__ void __launch_bounds__(256)
    bit_clear_kernel(uint32_t *__restrict__ bits, int64_t n_words, int32_t *__restrict__ total,
                     int32_t *__restrict__ blocksum, int64_t n_blocksum,
                     int32_t *__restrict__ per_word) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < 4) total[i] = 0;
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (int64_t j = i; j < n_blocksum; j += step) blocksum[j] = 0;
  if (per_word != nullptr)
    for (int64_t j = i; j < n_words; j += step) per_word[j] = 0;
  for (; i < n_words; i += step) bits[i] = 0u;
}

int bit_table_clear(const BitTable &t, hipStream_t s, bool blocksum_too, int32_t *per_word) {
  const int64_t want = ceil_div(t.n_words > 0 ? t.n_words : 1, 256);
  const int blocks = (int)(want < 8192 ? want : 8192);
  hipLaunchKernelGGL(bit_clear_kernel, dim3(blocks), dim3(256), 0, s, t.bits, t.n_words, t.total,
                     t.blocksum, blocksum_too ? t.n_scan_blocks : (int64_t)0, per_word);
  SSC_LAUNCH_CHECK("bit_clear");
  return SSC_OK;
}

// Pass 1: popcount sum of each block of kScanBlockWords words.
__global__ void __launch_bounds__(kScanThreads)
    popc_blocksum_kernel(const uint32_t *__restrict__ bits, int64_t n_words,
                         int32_t *__restrict__ blocksum) {
  __shared__ int lds[kScanThreads / 64 + 1];
  popc_blocksum_block(bits, n_words, blockIdx.x, blocksum, lds);
}

// Pass 2 (popc_prefix_block, ssc_common.h): exclusive prefix per word.
__global__ void __launch_bounds__(kScanThreads)
    popc_prefix_kernel(const uint32_t *__restrict__ bits, int64_t n_words,
                       const int32_t *__restrict__ blocksum, int32_t *__restrict__ prefix,
                       int32_t *__restrict__ total, int32_t *__restrict__ mirror, int ticket) {
  popc_prefix_block(bits, n_words, blocksum, prefix, total, mirror, blockIdx.x == gridDim.x - 1,
                    ticket);
}

int bit_table_scan_prefix(const BitTable &t, hipStream_t s, int32_t *mirror, int ticket) {
  hipLaunchKernelGGL(popc_prefix_kernel, dim3((unsigned)t.n_scan_blocks), dim3(kScanThreads), 0, s,
                     t.bits, t.n_words, t.blocksum, t.prefix, t.total, mirror, ticket);
  SSC_LAUNCH_CHECK("popc_prefix");
  return SSC_OK;
}

int bit_table_scan(const BitTable &t, hipStream_t s, int32_t *mirror, int ticket) {
  if (t.n_words <= 0) return fill_i32(t.total, 1, 0, s);
  hipLaunchKernelGGL(popc_blocksum_kernel, dim3((unsigned)t.n_scan_blocks), dim3(kScanThreads), 0,
                     s, t.bits, t.n_words, t.blocksum);
  SSC_LAUNCH_CHECK("popc_blocksum");
  return bit_table_scan_prefix(t, s, mirror, ticket);
}

// The pinned block and the event of the calling host thread.
struct ReadBack {
  char *pinned = nullptr;
  hipEvent_t done = nullptr;
  bool pending = false;
  int ticket = 0;       // last ticket handed out (read_back_mirror_ticket)
  int spin_ticket = 0;  // the wait in progress ends when this ticket shows up (0: on the event)
};
static thread_local ReadBack g_read_back;

static int read_back_init(ReadBack &r) {
  // (pinned memory from hipHostMalloc is mapped into the device's address space at the same
  // address and coherent with the host at event boundaries)
  if (r.pinned == nullptr)
    SSC_HIP(hipHostMalloc((void **)&r.pinned, kReadBackBytes,
                          hipHostMallocPortable | hipHostMallocMapped | hipHostMallocCoherent));
  if (r.done == nullptr) SSC_HIP(hipEventCreateWithFlags(&r.done, hipEventDisableTiming));
  return SSC_OK;
}

int read_back_mirror(int32_t **mirror) {
  ReadBack &r = g_read_back;
  int rc = read_back_init(r);
  if (rc != SSC_OK) return rc;
  void *dev = nullptr;
  SSC_HIP(hipHostGetDevicePointer(&dev, r.pinned, 0));
  *mirror = static_cast<int32_t *>(dev);
  return SSC_OK;
}

int read_back_mirror_queued(hipStream_t s, int ticket) {
  ReadBack &r = g_read_back;
  SSC_CHECK(r.done != nullptr, SSC_ERUNTIME, "read_back_mirror was not called on this thread");
  SSC_HIP(hipEventRecord(r.done, s));
  r.pending = true;
  r.spin_ticket = ticket;
  return SSC_OK;
}

int read_back_mirror_ticket() {
  ReadBack &r = g_read_back;
  r.ticket = r.ticket >= 0x3FFFFFFF ? 1 : r.ticket + 1;  // never 0
  if (r.pinned != nullptr) reinterpret_cast<volatile int32_t *>(r.pinned)[kMirrorTicket] = 0;
  return r.ticket;
}

int read_back_begin(const void *src_dev, size_t bytes, hipStream_t s) {
  ReadBack &r = g_read_back;
  SSC_CHECK(bytes <= kReadBackBytes, SSC_EINVAL, "read-back of %zu bytes exceeds the pinned block",
            bytes);
  int rc = read_back_init(r);
  if (rc != SSC_OK) return rc;
  if (bytes > 0) SSC_HIP(hipMemcpyAsync(r.pinned, src_dev, bytes, hipMemcpyDeviceToHost, s));
  SSC_HIP(hipEventRecord(r.done, s));
  r.pending = true;
  return SSC_OK;
}

int read_back_end(const void **view) {
  ReadBack &r = g_read_back;
  SSC_CHECK(r.pending, SSC_ERUNTIME, "no read-back was started on this thread");
  r.pending = false;
  if (r.spin_ticket != 0) {
    // The kernel that knows the results stores them in the pinned block and then, with a
    // release at system scope, the ticket: the host sees both while the kernel -- which has
    // other work to do -- still runs.  Should the store not show (it does on this
    // hardware), the event behind the kernel ends the wait.
    const volatile int32_t *m = reinterpret_cast<const volatile int32_t *>(r.pinned);
    const int want = r.spin_ticket;
    r.spin_ticket = 0;
    for (unsigned spins = 1;; ++spins) {
      if (m[kMirrorTicket] == want) break;
      if ((spins & 1023u) == 0) {
        const hipError_t e = hipEventQuery(r.done);
        if (e == hipSuccess) break;
        if (e != hipErrorNotReady)
          return ::ssc::fail(SSC_EHIP, "hipEventQuery failed: %s", hipGetErrorString(e));
      }
    }
    __atomic_thread_fence(__ATOMIC_ACQUIRE);
    *view = r.pinned;
    return SSC_OK;
  }
  SSC_HIP(hipEventSynchronize(r.done));
  *view = r.pinned;
  return SSC_OK;
}

int read_back_view(const void **view, const void *src_dev, size_t bytes, hipStream_t s) {
  int rc = read_back_begin(src_dev, bytes, s);
  if (rc != SSC_OK) return rc;
  return read_back_end(view);
}

int read_back(void *dst_host, const void *src_dev, size_t bytes, hipStream_t s) {
  const void *view;
  int rc = read_back_view(&view, src_dev, bytes, s);
  if (rc == SSC_OK) memcpy(dst_host, view, bytes);
  return rc;
}

}  // namespace ssc

extern "C" {
int ssc_version(void) { return 103; }
const char *ssc_last_error(void) { return ssc::g_error; }
}
