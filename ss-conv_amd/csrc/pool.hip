// Rulebook max / average pooling and segment (global) pooling.
//
// Rulebook pooling is output stationary: the pair lists are first transposed
// into an [n_out, K] table of input rows (-1 = no pair), then every output row
// is produced once, visiting its inputs in ascending offset order -- the order
// in which the reference's per-offset launches touch it.  Input rows are read
// once, output rows written once, no atomics on features.
#include "ssc_common.h"

// Products and sums below are rounded separately, as the scalar statements of the
// reference are: no fused multiply-add contraction in this file.
#pragma clang fp contract(off)

#include <math.h>

#include <mutex>

namespace ssc {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));

// table[key row * K + k] = the other row of the pair; key_plane 1 keys by output rows
// (forward), 0 by input rows (backward).
__global__ void __launch_bounds__(256)
    pair_table_kernel(const int32_t *__restrict__ pairs, int64_t pair_stride,
                      const int32_t *__restrict__ pair_num, int K, int key_plane,
                      int32_t *__restrict__ table) {
  int k = blockIdx.y;
  int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= pair_num[k]) return;
  const int32_t *p = pairs + (int64_t)k * 2 * pair_stride;
  int64_t key = p[key_plane * pair_stride + j];
  table[key * K + k] = p[(1 - key_plane) * pair_stride + j];
}

__global__ void __launch_bounds__(256)
    pair_count_kernel(const int32_t *__restrict__ pairs, int64_t pair_stride,
                      const int32_t *__restrict__ pair_num, int32_t *__restrict__ rf) {
  int k = blockIdx.y;
  int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= pair_num[k]) return;
  atomicAdd(&rf[pairs[((int64_t)k * 2 + 1) * pair_stride + j]], 1);  // integer: exact
}

// Element access for float and half rows.  Half arithmetic follows the reference's at::Half
// operators (every statement of its kernels computes in float and rounds the result to
// half): values travel as floats here and rnd<IO> rounds after every operation; for float it
// is the identity.
template <typename IO>
__device__ __forceinline__ float rnd(float v) {
  return (float)(IO)v;
}
template <typename IO, int VEC>
__device__ __forceinline__ void load_row(const IO *p, float (&x)[VEC]) {
  if constexpr (VEC == 4 && sizeof(IO) == 4) {
    const float4v q = *reinterpret_cast<const float4v *>(p);
    x[0] = q.x; x[1] = q.y; x[2] = q.z; x[3] = q.w;
  } else if constexpr (VEC == 4) {
    const half4v q = *reinterpret_cast<const half4v *>(p);
    x[0] = (float)q.x; x[1] = (float)q.y; x[2] = (float)q.z; x[3] = (float)q.w;
  } else {
    x[0] = (float)p[0];
  }
}
template <typename IO, int VEC>
__device__ __forceinline__ void store_row(IO *p, const float (&x)[VEC]) {
  if constexpr (VEC == 4 && sizeof(IO) == 4) {
    *reinterpret_cast<float4v *>(p) = float4v{x[0], x[1], x[2], x[3]};
  } else if constexpr (VEC == 4) {
    *reinterpret_cast<half4v *>(p) = half4v{(_Float16)x[0], (_Float16)x[1], (_Float16)x[2], (_Float16)x[3]};
  } else {
    p[0] = (IO)x[0];
  }
}

// MODE 0: max with zero start (out = max(0, inputs));  MODE 1: sum of in / (IO)rf.
// VEC = 4 when C % 4 == 0 (16-byte accesses for float, 8-byte for half), else 1.
template <typename IO, int MODE, int VEC>
__global__ void __launch_bounds__(256)
    pool_kernel(const IO *__restrict__ in, int C, const int32_t *__restrict__ table, int K,
                const int32_t *__restrict__ rf, IO *__restrict__ out, int64_t n_out) {
  const int cv = C / VEC;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n_out * cv) return;
  int64_t o = idx / cv;
  int c = (int)(idx - o * cv) * VEC;
  float acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
  float div = 1.f;
  if (MODE == 1) div = rnd<IO>((float)rf[o]);
  const int32_t *t = table + o * K;
  for (int k = 0; k < K; ++k) {
    int64_t i = t[k];
    if (i < 0) continue;
    float x[VEC];
    load_row<IO, VEC>(in + i * C + c, x);
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      if (MODE == 0) {
        if (acc[v] < x[v]) acc[v] = x[v];
      } else {
        acc[v] = rnd<IO>(acc[v] + rnd<IO>(x[v] / div));
      }
    }
  }
  store_row<IO, VEC>(out + o * C + c, acc);
}

// Segment pooling: grid (segment, channel block of 64); 16 row lanes x 64
// channels per block; partial results combined in a fixed order.
constexpr int kSegRows = 16;

template <bool IS_MAX>
__global__ void __launch_bounds__(kSegRows * 64)
    segment_pool_kernel(const float *__restrict__ feats, const int32_t *__restrict__ offsets,
                        float *__restrict__ out, int32_t *__restrict__ out_idx, int C) {
  __shared__ float sval[kSegRows][64];
  __shared__ int sidx[kSegRows][64];
  const int seg = blockIdx.x;
  const int cl = threadIdx.x & 63;
  const int rl = threadIdx.x >> 6;
  const int c = blockIdx.y * 64 + cl;
  const int a = offsets[seg], b = offsets[seg + 1];
  float v = IS_MAX ? -INFINITY : 0.f;
  int arg = -1;
  if (c < C) {
    auto take = [&](float x, int i) {
      if (IS_MAX) {
        if (x > v) { v = x; arg = i; }
      } else {
        v += x;
      }
    };
    // eight rows per trip: the loads are independent and in flight together, the
    // rows are then folded in ascending order, as a one-row-per-trip loop would
    constexpr int U = 8;
    int i = a + rl;
    for (; i + (U - 1) * kSegRows < b; i += U * kSegRows) {
      float x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = feats[(int64_t)(i + u * kSegRows) * C + c];
#pragma unroll
      for (int u = 0; u < U; ++u) take(x[u], i + u * kSegRows);
    }
    for (; i < b; i += kSegRows) take(feats[(int64_t)i * C + c], i);
  }
  sval[rl][cl] = v;
  sidx[rl][cl] = arg;
  __syncthreads();
  if (rl == 0 && c < C) {
#pragma unroll
    for (int r = 1; r < kSegRows; ++r) {
      float x = sval[r][cl];
      if (IS_MAX) {
        int xi = sidx[r][cl];
        // first occurrence wins: larger value, or equal value at a lower row
        if (x > v || (x == v && xi >= 0 && (arg < 0 || xi < arg))) { v = x; arg = xi; }
      } else {
        v += x;
      }
    }
    if (IS_MAX) {
      out[(int64_t)seg * C + c] = v;
      out_idx[(int64_t)seg * C + c] = arg;
    } else {
      out[(int64_t)seg * C + c] = v / (float)(b - a);
    }
  }
}

// Backward of rulebook pooling, input stationary: every input row visits its pairs in
// ascending offset order, the order of the reference's per-offset launches
// (src/pool/indice_maxpool_cuda_functor.cu:426-455: din[i] += dout[o] where in[i] == out[o];
// src/pool/indice_avgpool_cuda_functor.cu: din[i] += dout[o] / (float)rf[o]).
// table is [n_in, K] of output rows.  MODE 0 max, 1 average.
template <typename IO, int MODE, int VEC>
__global__ void __launch_bounds__(256)
    pool_bwd_kernel(const IO *__restrict__ in, const IO *__restrict__ out,
                    const IO *__restrict__ dout, int C, const int32_t *__restrict__ table,
                    int K, const int32_t *__restrict__ rf, IO *__restrict__ din, int64_t n_in) {
  // VEC = 4 when C % 4 == 0, else 1; per column the arithmetic and its order are those of
  // the one-column form
  const int cv = C / VEC;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n_in * cv) return;
  int64_t i = idx / cv;
  int c = (int)(idx - i * cv) * VEC;
  const int32_t *t = table + i * K;
  float acc[VEC], x[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    acc[v] = 0.f;
    x[v] = 0.f;
  }
  if (MODE == 0) load_row<IO, VEC>(in + i * C + c, x);
  for (int k = 0; k < K; ++k) {
    int64_t o = t[k];
    if (o < 0) continue;
    float g[VEC], y[VEC];
    load_row<IO, VEC>(dout + o * C + c, g);
    if (MODE == 0) load_row<IO, VEC>(out + o * C + c, y);
    const float div = MODE == 1 ? rnd<IO>((float)rf[o]) : 1.f;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      if (MODE == 0) {
        if (x[v] == y[v]) acc[v] = rnd<IO>(acc[v] + g[v]);
      } else {
        acc[v] = rnd<IO>(acc[v] + rnd<IO>(g[v] / div));
      }
    }
  }
  store_row<IO, VEC>(din + i * C + c, acc);
}

// Backward of the segment pools (src/pool/global_avgpool_cuda_kernel.cu:44-62,
// global_maxpool_cuda_kernel.cu:45-60): average spreads dout / len over the segment's
// rows; max routes dout to the arg-max row.  din must be zero for the max variant.
template <int VEC>
__global__ void __launch_bounds__(256)
    segment_avg_bwd_kernel(const float *__restrict__ dout, const int32_t *__restrict__ offsets,
                           int n_seg, int C, float *__restrict__ din, int64_t n_rows) {
  // VEC = 4 when C % 4 == 0: one segment search and one 16-byte store per four columns
  const int cv = C / VEC;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n_rows * cv) return;
  int64_t r = idx / cv;
  int c = (int)(idx - r * cv) * VEC;
  int lo = 0, hi = n_seg;  // the segment s with offsets[s] <= r < offsets[s+1]
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (offsets[mid] <= r) lo = mid;
    else hi = mid;
  }
  const bool inside = r >= offsets[0] && r < offsets[n_seg];
  const float len = inside ? (float)(offsets[lo + 1] - offsets[lo]) : 1.f;
  if (VEC == 4) {
    float4v v = {0.f, 0.f, 0.f, 0.f};
    if (inside) {
      const float4v g = *reinterpret_cast<const float4v *>(dout + (int64_t)lo * C + c);
      v = float4v{g.x / len, g.y / len, g.z / len, g.w / len};
    }
    *reinterpret_cast<float4v *>(din + r * C + c) = v;
  } else {
    din[r * C + c] = inside ? dout[(int64_t)lo * C + c] / len : 0.f;
  }
}

__global__ void __launch_bounds__(256)
    segment_max_bwd_kernel(const float *__restrict__ dout, const int32_t *__restrict__ arg,
                           int64_t n, int C, float *__restrict__ din) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  int a = arg[idx];
  if (a >= 0) din[(int64_t)a * C + (idx % C)] = dout[idx];
}

static int pool_common(const void *features, int channels, const int32_t *pairs,
                       int64_t pair_stride, const int32_t *pair_num, int K, void *out,
                       int64_t n_out, void *ws, size_t ws_bytes, hipStream_t s,
                       int32_t **table_out) {
  SSC_CHECK(K >= 1 && K <= SSC_MAX_KERNEL_VOLUME, SSC_ERUNTIME, "kernel volume %d out of range", K);
  SSC_CHECK(channels >= 1 && n_out >= 0 && pair_stride >= 0, SSC_EINVAL, "bad sizes");
  if (n_out == 0) return SSC_OK;
  SSC_CHECK(features && pairs && pair_num && out && ws, SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(ws_bytes >= align_up((size_t)n_out * K * 4), SSC_EWORKSPACE,
            "pool workspace too small");
  int32_t *table = static_cast<int32_t *>(ws);
  int rc = fill_i32(table, n_out * K, -1, s);
  if (rc != SSC_OK) return rc;
  if (pair_stride > 0) {
    hipLaunchKernelGGL(pair_table_kernel, dim3((unsigned)ceil_div(pair_stride, 256), (unsigned)K),
                       dim3(256), 0, s, pairs, pair_stride, pair_num, K, 1, table);
    SSC_LAUNCH_CHECK("pair_table");
  }
  *table_out = table;
  return SSC_OK;
}

// ---- the pair table in library-owned memory ------------------------------------------------
// ssc_pool_max_static_f32 keeps its [n_out, K] pair table in this array instead of a
// caller-provided workspace, so the call allocates nothing.  Every GPU the library runs on
// holds its own copy of the array (SSC_POOL_STATIC_ENTRIES * 4 bytes, until the process
// ends) at its own address; host code never uses the symbol `scratch` itself, only the
// address hipGetSymbolAddress reports for the current device.
static __device__ __align__(256) int32_t scratch[SSC_POOL_STATIC_ENTRIES];

constexpr int kMaxDevices = 64;
static int32_t *g_scratch_of_device[kMaxDevices] = {};
static std::mutex g_scratch_mutex;

// The device address of `scratch` on the current device (looked up once per device).
static int static_table(int32_t **table) {
  int dev = -1;
  SSC_HIP(hipGetDevice(&dev));
  SSC_CHECK(dev >= 0 && dev < kMaxDevices, SSC_ERUNTIME, "device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_of_device[dev] == nullptr) {
    void *ptr = nullptr;
    SSC_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    SSC_CHECK(ptr != nullptr, SSC_EHIP, "hipGetSymbolAddress returned a null address");
    g_scratch_of_device[dev] = static_cast<int32_t *>(ptr);
  }
  *table = g_scratch_of_device[dev];
  return SSC_OK;
}

}  // namespace ssc

using namespace ssc;

extern "C" {

int ssc_pool_max_static_f32(const float *features, int32_t channels, const int32_t *pairs,
                            int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                            float *out, int64_t n_out, ssc_stream_t stream) {
  const int K = kernel_volume;
  SSC_CHECK(K >= 1 && K <= SSC_MAX_KERNEL_VOLUME, SSC_ERUNTIME, "kernel volume %d out of range", K);
  SSC_CHECK(channels >= 1 && n_out >= 0 && pair_stride >= 0, SSC_EINVAL, "bad sizes");
  SSC_CHECK(n_out * K <= (int64_t)SSC_POOL_STATIC_ENTRIES, SSC_EINVAL,
            "n_out * kernel_volume = %lld exceeds the %lld entries of the library's pair table: "
            "use ssc_pool_max_f32 with a workspace",
            (long long)(n_out * K), (long long)SSC_POOL_STATIC_ENTRIES);
  int32_t *table = nullptr;
  int rc = static_table(&table);  // (also for n_out == 0: a first call sets the address up)
  if (rc != SSC_OK) return rc;
  // the table keeps the previous call's entries: pool_common clears what this call uses
  return ssc_pool_max_f32(features, channels, pairs, pair_stride, pair_num, K, out, n_out, table,
                          (size_t)SSC_POOL_STATIC_ENTRIES * sizeof(int32_t), stream);
}

size_t ssc_pool_workspace_bytes(int64_t n_out, int32_t kernel_volume) {
  if (n_out < 0 || kernel_volume < 1) return 0;
  return align_up((size_t)(n_out > 0 ? n_out : 1) * kernel_volume * 4);
}

}  // extern "C"

// mode 0 max, 1 average
template <typename IO>
static int pool_fwd(int mode, const IO *features, int channels, const int32_t *pairs,
                    int64_t pair_stride, const int32_t *pair_num, int K, const int32_t *summaryrf,
                    IO *out, int64_t n_out, void *ws, size_t ws_bytes, hipStream_t s) {
  SSC_CHECK(mode == 0 || n_out == 0 || summaryrf != nullptr, SSC_EINVAL, "summaryrf is NULL");
  int32_t *table = nullptr;
  int rc = pool_common(features, channels, pairs, pair_stride, pair_num, K, out, n_out, ws,
                       ws_bytes, s, &table);
  if (rc != SSC_OK || n_out == 0) return rc;
  const int vec = (channels & 3) == 0 ? 4 : 1;
  const int64_t n = n_out * (channels / vec);
  const dim3 grid((unsigned)ceil_div(n, 256));
#define SSC_POOL_FWD(M, V)                                                                     \
  hipLaunchKernelGGL((pool_kernel<IO, M, V>), grid, dim3(256), 0, s, features, channels, table, \
                     K, summaryrf, out, n_out)
  if (mode == 0) {
    if (vec == 4) SSC_POOL_FWD(0, 4); else SSC_POOL_FWD(0, 1);
  } else {
    if (vec == 4) SSC_POOL_FWD(1, 4); else SSC_POOL_FWD(1, 1);
  }
#undef SSC_POOL_FWD
  SSC_LAUNCH_CHECK("pool");
  return SSC_OK;
}

extern "C" {

int ssc_pool_max_f32(const float *features, int32_t channels, const int32_t *pairs,
                     int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                     float *out, int64_t n_out, void *workspace, size_t workspace_bytes,
                     ssc_stream_t stream) {
  return pool_fwd<float>(0, features, channels, pairs, pair_stride, pair_num, kernel_volume,
                         nullptr, out, n_out, workspace, workspace_bytes, (hipStream_t)stream);
}

int ssc_pool_avg_f32(const float *features, int32_t channels, const int32_t *pairs,
                     int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                     const int32_t *summaryrf, float *out, int64_t n_out, void *workspace,
                     size_t workspace_bytes, ssc_stream_t stream) {
  return pool_fwd<float>(1, features, channels, pairs, pair_stride, pair_num, kernel_volume,
                         summaryrf, out, n_out, workspace, workspace_bytes, (hipStream_t)stream);
}

int ssc_pool_max_f16(const void *features, int32_t channels, const int32_t *pairs,
                     int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                     void *out, int64_t n_out, void *workspace, size_t workspace_bytes,
                     ssc_stream_t stream) {
  return pool_fwd<_Float16>(0, static_cast<const _Float16 *>(features), channels, pairs,
                            pair_stride, pair_num, kernel_volume, nullptr,
                            static_cast<_Float16 *>(out), n_out, workspace, workspace_bytes,
                            (hipStream_t)stream);
}

int ssc_pool_avg_f16(const void *features, int32_t channels, const int32_t *pairs,
                     int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                     const int32_t *summaryrf, void *out, int64_t n_out, void *workspace,
                     size_t workspace_bytes, ssc_stream_t stream) {
  return pool_fwd<_Float16>(1, static_cast<const _Float16 *>(features), channels, pairs,
                            pair_stride, pair_num, kernel_volume, summaryrf,
                            static_cast<_Float16 *>(out), n_out, workspace, workspace_bytes,
                            (hipStream_t)stream);
}

int ssc_summary_rf(const int32_t *pairs, int64_t pair_stride, const int32_t *pair_num,
                   int32_t kernel_volume, int32_t *rf, int64_t n_out, void *workspace,
                   size_t workspace_bytes, ssc_stream_t stream) {
  (void)workspace;
  (void)workspace_bytes;
  hipStream_t s = (hipStream_t)stream;
  SSC_CHECK(kernel_volume >= 1 && kernel_volume <= SSC_MAX_KERNEL_VOLUME, SSC_ERUNTIME,
            "kernel volume out of range");
  if (n_out == 0) return SSC_OK;
  SSC_CHECK(pairs && pair_num && rf, SSC_EINVAL, "NULL pointer argument");
  int rc = fill_i32(rf, n_out, 0, s);
  if (rc != SSC_OK) return rc;
  if (pair_stride > 0) {
    hipLaunchKernelGGL(pair_count_kernel,
                       dim3((unsigned)ceil_div(pair_stride, 256), (unsigned)kernel_volume),
                       dim3(256), 0, s, pairs, pair_stride, pair_num, rf);
    SSC_LAUNCH_CHECK("pair_count");
  }
  return SSC_OK;
}

int ssc_segment_avg_f32(const float *feats, const int32_t *offsets, float *out,
                        int32_t n_segments, int32_t channels, ssc_stream_t stream) {
  SSC_CHECK(n_segments >= 0 && channels >= 1, SSC_EINVAL, "bad sizes");
  if (n_segments == 0) return SSC_OK;
  SSC_CHECK(feats && offsets && out, SSC_EINVAL, "NULL pointer argument");
  hipLaunchKernelGGL(segment_pool_kernel<false>,
                     dim3((unsigned)n_segments, (unsigned)ceil_div(channels, 64)),
                     dim3(kSegRows * 64), 0, (hipStream_t)stream, feats, offsets, out,
                     (int32_t *)nullptr, channels);
  SSC_LAUNCH_CHECK("segment_avg");
  return SSC_OK;
}

int ssc_segment_max_f32(const float *feats, const int32_t *offsets, float *out, int32_t *out_idx,
                        int32_t n_segments, int32_t channels, ssc_stream_t stream) {
  SSC_CHECK(n_segments >= 0 && channels >= 1, SSC_EINVAL, "bad sizes");
  if (n_segments == 0) return SSC_OK;
  SSC_CHECK(feats && offsets && out && out_idx, SSC_EINVAL, "NULL pointer argument");
  hipLaunchKernelGGL(segment_pool_kernel<true>,
                     dim3((unsigned)n_segments, (unsigned)ceil_div(channels, 64)),
                     dim3(kSegRows * 64), 0, (hipStream_t)stream, feats, offsets, out, out_idx,
                     channels);
  SSC_LAUNCH_CHECK("segment_max");
  return SSC_OK;
}

}  // extern "C"

template <typename IO>
static int pool_bwd(int mode, const IO *features, const IO *out_features, const IO *out_grad,
                    int channels, const int32_t *pairs, int64_t pair_stride,
                    const int32_t *pair_num, int K, const int32_t *summaryrf, IO *in_grad,
                    int64_t n_in, void *ws, size_t ws_bytes, hipStream_t s) {
  SSC_CHECK(K >= 1 && K <= SSC_MAX_KERNEL_VOLUME, SSC_ERUNTIME, "kernel volume %d out of range", K);
  SSC_CHECK(channels >= 1 && n_in >= 0 && pair_stride >= 0, SSC_EINVAL, "bad sizes");
  if (n_in == 0) return SSC_OK;
  SSC_CHECK(in_grad && ws, SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(pair_stride == 0 || (out_grad && pairs && pair_num), SSC_EINVAL,
            "NULL pointer argument");
  SSC_CHECK(mode == 1 || pair_stride == 0 || (features && out_features), SSC_EINVAL,
            "NULL pointer argument");
  SSC_CHECK(mode == 0 || pair_stride == 0 || summaryrf, SSC_EINVAL, "summaryrf is NULL");
  SSC_CHECK(ws_bytes >= align_up((size_t)n_in * K * 4), SSC_EWORKSPACE,
            "pool backward workspace too small");
  int32_t *table = static_cast<int32_t *>(ws);
  int rc = fill_i32(table, n_in * K, -1, s);
  if (rc != SSC_OK) return rc;
  if (pair_stride > 0) {
    hipLaunchKernelGGL(pair_table_kernel, dim3((unsigned)ceil_div(pair_stride, 256), (unsigned)K),
                       dim3(256), 0, s, pairs, pair_stride, pair_num, K, 0, table);
    SSC_LAUNCH_CHECK("pair_table");
  }
  const int vec = (channels & 3) == 0 ? 4 : 1;
  const int64_t n = n_in * (channels / vec);
  const dim3 grid((unsigned)ceil_div(n, 256));
#define SSC_POOL_BWD(M, V)                                                                      \
  hipLaunchKernelGGL((pool_bwd_kernel<IO, M, V>), grid, dim3(256), 0, s, features, out_features, \
                     out_grad, channels, table, K, summaryrf, in_grad, n_in)
  if (mode == 0) {
    if (vec == 4) SSC_POOL_BWD(0, 4); else SSC_POOL_BWD(0, 1);
  } else {
    if (vec == 4) SSC_POOL_BWD(1, 4); else SSC_POOL_BWD(1, 1);
  }
#undef SSC_POOL_BWD
  SSC_LAUNCH_CHECK("pool_bwd");
  return SSC_OK;
}

extern "C" {

int ssc_pool_max_bwd_f32(const float *features, const float *out_features, const float *out_grad,
                         int32_t channels, const int32_t *pairs, int64_t pair_stride,
                         const int32_t *pair_num, int32_t kernel_volume, float *in_grad,
                         int64_t n_in, void *workspace, size_t workspace_bytes,
                         ssc_stream_t stream) {
  return pool_bwd<float>(0, features, out_features, out_grad, channels, pairs, pair_stride,
                         pair_num, kernel_volume, nullptr, in_grad, n_in, workspace,
                         workspace_bytes, (hipStream_t)stream);
}

int ssc_pool_max_bwd_f16(const void *features, const void *out_features, const void *out_grad,
                         int32_t channels, const int32_t *pairs, int64_t pair_stride,
                         const int32_t *pair_num, int32_t kernel_volume, void *in_grad,
                         int64_t n_in, void *workspace, size_t workspace_bytes,
                         ssc_stream_t stream) {
  typedef const _Float16 *H;
  return pool_bwd<_Float16>(0, (H)features, (H)out_features, (H)out_grad, channels, pairs,
                            pair_stride, pair_num, kernel_volume, nullptr,
                            static_cast<_Float16 *>(in_grad), n_in, workspace, workspace_bytes,
                            (hipStream_t)stream);
}

int ssc_pool_avg_bwd_f32(const float *out_grad, int32_t channels, const int32_t *pairs,
                         int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                         const int32_t *summaryrf, float *in_grad, int64_t n_in, void *workspace,
                         size_t workspace_bytes, ssc_stream_t stream) {
  return pool_bwd<float>(1, nullptr, nullptr, out_grad, channels, pairs, pair_stride, pair_num,
                         kernel_volume, summaryrf, in_grad, n_in, workspace, workspace_bytes,
                         (hipStream_t)stream);
}

int ssc_pool_avg_bwd_f16(const void *out_grad, int32_t channels, const int32_t *pairs,
                         int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                         const int32_t *summaryrf, void *in_grad, int64_t n_in, void *workspace,
                         size_t workspace_bytes, ssc_stream_t stream) {
  return pool_bwd<_Float16>(1, nullptr, nullptr, static_cast<const _Float16 *>(out_grad), channels,
                            pairs, pair_stride, pair_num, kernel_volume, summaryrf,
                            static_cast<_Float16 *>(in_grad), n_in, workspace, workspace_bytes,
                            (hipStream_t)stream);
}

int ssc_segment_avg_bwd_f32(const float *out_grad, const int32_t *offsets, float *in_grad,
                            int64_t n_rows, int32_t n_segments, int32_t channels,
                            ssc_stream_t stream) {
  SSC_CHECK(n_segments >= 0 && channels >= 1 && n_rows >= 0, SSC_EINVAL, "bad sizes");
  if (n_rows == 0) return SSC_OK;
  SSC_CHECK(in_grad != nullptr, SSC_EINVAL, "in_grad is NULL");
  if (n_segments == 0) return fill_f32(in_grad, n_rows * channels, 0.f, (hipStream_t)stream);
  SSC_CHECK(out_grad && offsets, SSC_EINVAL, "NULL pointer argument");
  if ((channels & 3) == 0)
    hipLaunchKernelGGL(segment_avg_bwd_kernel<4>,
                       dim3((unsigned)ceil_div(n_rows * (channels / 4), 256)), dim3(256), 0,
                       (hipStream_t)stream, out_grad, offsets, (int)n_segments, (int)channels,
                       in_grad, n_rows);
  else
    hipLaunchKernelGGL(segment_avg_bwd_kernel<1>,
                       dim3((unsigned)ceil_div(n_rows * channels, 256)), dim3(256), 0,
                       (hipStream_t)stream, out_grad, offsets, (int)n_segments, (int)channels,
                       in_grad, n_rows);
  SSC_LAUNCH_CHECK("segment_avg_bwd");
  return SSC_OK;
}

int ssc_segment_max_bwd_f32(const float *out_grad, const int32_t *out_idx, float *in_grad,
                            int64_t n_rows, int32_t n_segments, int32_t channels,
                            ssc_stream_t stream) {
  SSC_CHECK(n_segments >= 0 && channels >= 1 && n_rows >= 0, SSC_EINVAL, "bad sizes");
  if (n_rows == 0) return SSC_OK;
  SSC_CHECK(in_grad != nullptr, SSC_EINVAL, "in_grad is NULL");
  int rc = fill_f32(in_grad, n_rows * channels, 0.f, (hipStream_t)stream);
  if (rc != SSC_OK || n_segments == 0) return rc;
  SSC_CHECK(out_grad && out_idx, SSC_EINVAL, "NULL pointer argument");
  const int64_t n = (int64_t)n_segments * channels;
  hipLaunchKernelGGL(segment_max_bwd_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0,
                     (hipStream_t)stream, out_grad, out_idx, n, (int)channels, in_grad);
  SSC_LAUNCH_CHECK("segment_max_bwd");
  return SSC_OK;
}
}
