// Sparse convolution forward as an output-stationary implicit GEMM on fp32 MFMA.
//
// Outputs are cut into tiles of T consecutive rows.  A workgroup owns one tile
// and CN output columns; its accumulators [T, CN] live in LDS for the whole
// kernel.  For every kernel offset k the pairs that land in the tile form one
// contiguous segment of the rulebook (pairs of an offset are ascending in
// output row), so they are packed 16 at a time into the M side of
// v_mfma_f32_16x16x4_f32: the gathered input rows are staged in LDS, the
// matching 16x16 weight fragments stay in registers, and the product is added
// to the LDS accumulators at the pairs' output rows.  Only occupied
// (row, offset) slots cost MFMA work, and because each wave owns a fixed set
// of columns and walks the offsets in ascending order the result is
// bit-reproducible without atomics.
#include "ssc_common.h"

namespace ssc {

typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kKC = 64;       // input channels per chunk = 16 MFMA steps of 4
constexpr int kStage = 64;    // pairs staged per barrier = 4 row blocks of 16
constexpr int kAStride = 68;  // floats per staged row (64 + 4: 16-byte aligned, bank spread)
constexpr int kMinTile = 64;

// ---- weight packing ---------------------------------------------------------------------
// packed[((k*NCB + ncb)*NCH + cc)*1024 + lane*16 + c] =
//     W[k][cc*64 + (lane/16)*16 + c][ncb*16 + lane%16]           (0 outside Cin/Cout)
// i.e. the B fragment of MFMA step c of chunk cc for column block ncb, laid
// out so that one wave reads it as four coalesced 16-byte loads per lane.
__global__ void __launch_bounds__(256)
    pack_filters_kernel(const float *__restrict__ w, int64_t fs_k, int64_t fs_ci, int64_t fs_co,
                        int K, int cin, int cout, int ncb, int nch, float *__restrict__ packed) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)K * ncb * nch * 1024;
  if (idx >= total) return;
  int c = idx & 15;
  int lane = (idx >> 4) & 63;
  int64_t r = idx >> 10;
  int cc = r % nch;
  r /= nch;
  int cb = r % ncb;
  int k = (int)(r / ncb);
  int ci = cc * kKC + (lane >> 4) * 16 + c;
  int co = cb * 16 + (lane & 15);
  float v = 0.f;
  if (ci < cin && co < cout) v = w[k * fs_k + ci * fs_ci + co * fs_co];
  packed[idx] = v;
}

// ---- pair order -------------------------------------------------------------------------
// flag[0] |= 1 when some offset's scatter rows are not strictly ascending.
__global__ void __launch_bounds__(256)
    check_sorted_kernel(const int32_t *__restrict__ pairs, int64_t pair_stride, int plane_s,
                        const int32_t *__restrict__ pair_num, int32_t *__restrict__ flag) {
  int k = blockIdx.y;
  int n = pair_num[k];
  const int32_t *s = pairs + ((int64_t)k * 2 + plane_s) * pair_stride;
  int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j + 1 < n && s[j] >= s[j + 1]) atomicOr(flag, 1);
}

// Re-ordering of unsorted pair lists (rare: inputs not in ascending key order).
// Scatter rows are unique inside an offset, so their rank in a per-offset bit
// table over [0, n_out) is their sorted position.  Every kernel returns at once
// when flag[0] == 0.
__global__ void __launch_bounds__(256)
    resort_clear_kernel(const int32_t *__restrict__ flag, uint32_t *__restrict__ bits, int64_t n) {
  if (flag[0] == 0) return;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += step) bits[i] = 0u;
}

__global__ void __launch_bounds__(256)
    resort_mark_kernel(const int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                       int64_t pair_stride, int plane_s, const int32_t *__restrict__ pair_num,
                       uint32_t *__restrict__ bits, int64_t words_per_k) {
  if (flag[0] == 0) return;
  int k = blockIdx.y;
  int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= pair_num[k]) return;
  uint32_t o = (uint32_t)pairs[((int64_t)k * 2 + plane_s) * pair_stride + j];
  atomicOr(&bits[(int64_t)k * words_per_k + (o >> 5)], 1u << (o & 31u));
}

__global__ void __launch_bounds__(kScanThreads)
    resort_scan_kernel(const int32_t *__restrict__ flag, const uint32_t *__restrict__ bits,
                       int32_t *__restrict__ prefix, int64_t words_per_k) {
  if (flag[0] == 0) return;
  __shared__ int lds[kScanThreads / 64 + 1];
  const uint32_t *b = bits + (int64_t)blockIdx.x * words_per_k;
  int32_t *p = prefix + (int64_t)blockIdx.x * words_per_k;
  int carry = 0;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int64_t base = 0; base < words_per_k; base += kScanThreads) {
    int64_t i = base + threadIdx.x;
    int v = i < words_per_k ? __popc(b[i]) : 0;
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
    if (i < words_per_k) p[i] = carry + wave_off + incl - v;
    carry += tot;
  }
}

__global__ void __launch_bounds__(256)
    resort_scatter_kernel(const int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                          int64_t pair_stride, int plane_s, const int32_t *__restrict__ pair_num,
                          const uint32_t *__restrict__ bits, const int32_t *__restrict__ prefix,
                          int64_t words_per_k, int32_t *__restrict__ sorted) {
  if (flag[0] == 0) return;
  int k = blockIdx.y;
  int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= pair_num[k]) return;
  const int32_t *ps = pairs + ((int64_t)k * 2 + plane_s) * pair_stride;
  const int32_t *pg = pairs + ((int64_t)k * 2 + (1 - plane_s)) * pair_stride;
  uint32_t o = (uint32_t)ps[j];
  int pos = bit_rank(bits + (int64_t)k * words_per_k, prefix + (int64_t)k * words_per_k, o);
  sorted[((int64_t)k * 2 + plane_s) * pair_stride + pos] = (int32_t)o;
  sorted[((int64_t)k * 2 + (1 - plane_s)) * pair_stride + pos] = pg[j];
}

// segs[t*K + k] = first pair of offset k whose scatter row is >= t*T  (t = 0..n_tiles).
__global__ void __launch_bounds__(256)
    tile_segments_kernel(const int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                         const int32_t *__restrict__ sorted, int64_t pair_stride, int plane_s,
                         const int32_t *__restrict__ pair_num, int K, int64_t n_tiles, int T,
                         int32_t *__restrict__ segs) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (n_tiles + 1) * K) return;
  int64_t t = idx / K;
  int k = (int)(idx - t * K);
  const int32_t *src = flag[0] ? sorted : pairs;
  const int32_t *s = src + ((int64_t)k * 2 + plane_s) * pair_stride;
  int64_t target = t * (int64_t)T;
  int lo = 0, hi = pair_num[k];
  while (lo < hi) {
    int mid = (lo + hi) >> 1;
    if (s[mid] < target) lo = mid + 1;
    else hi = mid;
  }
  segs[idx] = lo;
}

// ---- the convolution --------------------------------------------------------------------
// grid = (n_tiles, ceil(ncb / NWAVES)); block = NWAVES waves; wave w owns column
// block  blockIdx.y*NWAVES + w  (16 columns).
// Dynamic LDS: acc[T][CN] | abuf[kStage][kAStride] | orow[kStage]
template <int NWAVES>
__global__ void __launch_bounds__(NWAVES * 64)
    conv_fwd_kernel(const float *__restrict__ features, int cin, const float *__restrict__ packed,
                    const int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                    const int32_t *__restrict__ sorted, int64_t pair_stride, int plane_g,
                    const int32_t *__restrict__ segs, int K, int nch, int ncb,
                    float *__restrict__ out, int64_t n_out, int cout, int T) {
  constexpr int CN = NWAVES * 16;
  constexpr int NT = NWAVES * 64;
  extern __shared__ __align__(16) float lds[];
  float *acc = lds;
  float *abuf = acc + (size_t)T * CN;
  int *orow = reinterpret_cast<int *>(abuf + kStage * kAStride);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 4;   // MFMA k-group
  const int l16 = lane & 15;
  const int64_t tile = blockIdx.x;
  const int64_t row0 = tile * (int64_t)T;
  const int cb = blockIdx.y * NWAVES + wave;  // column block of this wave
  const bool wave_live = cb < ncb;
  const int32_t *src = flag[0] ? sorted : pairs;
  const bool vec4 = (cin & 3) == 0;

  for (int i = tid; i < T * CN; i += NT) acc[i] = 0.f;

  for (int k = 0; k < K; ++k) {
    const int s0 = segs[tile * K + k];
    const int s1 = segs[(tile + 1) * K + k];
    const int n = s1 - s0;
    if (n <= 0) continue;
    const int32_t *pg = src + ((int64_t)k * 2 + plane_g) * pair_stride + s0;
    const int32_t *ps = src + ((int64_t)k * 2 + (1 - plane_g)) * pair_stride + s0;
    for (int cc = 0; cc < nch; ++cc) {
      // weight fragments of (k, chunk cc, column block cb): 16 MFMA steps
      float4v b[4];
      if (wave_live) {
        const float4v *bp = reinterpret_cast<const float4v *>(
            packed + (((int64_t)k * ncb + cb) * nch + cc) * 1024 + lane * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q) b[q] = bp[q];
      }
      for (int m0 = 0; m0 < n; m0 += kStage) {
        __syncthreads();  // previous stage fully consumed (and acc zeroed on first pass)
        // stage: gather up to 64 input rows x 64 channels
        for (int e = tid; e < kStage * 16; e += NT) {
          int p = e >> 4, f4 = e & 15;
          int ch = cc * kKC + f4 * 4;
          float4v v = {0.f, 0.f, 0.f, 0.f};
          if (m0 + p < n) {
            int64_t row = pg[m0 + p];
            const float *fp = features + row * cin + ch;
            if (vec4) {
              if (ch < cin) v = *reinterpret_cast<const float4v *>(fp);
            } else {
              if (ch + 0 < cin) v.x = fp[0];
              if (ch + 1 < cin) v.y = fp[1];
              if (ch + 2 < cin) v.z = fp[2];
              if (ch + 3 < cin) v.w = fp[3];
            }
          }
          *reinterpret_cast<float4v *>(abuf + p * kAStride + f4 * 4) = v;
        }
        if (tid < kStage) orow[tid] = (m0 + tid < n) ? (int)(ps[m0 + tid] - row0) : -1;
        __syncthreads();
        if (wave_live) {
          const int nblk = min(4, (n - m0 + 15) >> 4);
          for (int m = 0; m < nblk; ++m) {
            const float4v *ap =
                reinterpret_cast<const float4v *>(abuf + (m * 16 + l16) * kAStride + g * 16);
            float4v a[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) a[q] = ap[q];
            float4v d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              d = __builtin_amdgcn_mfma_f32_16x16x4f32(a[q].x, b[q].x, d, 0, 0, 0);
              d = __builtin_amdgcn_mfma_f32_16x16x4f32(a[q].y, b[q].y, d, 0, 0, 0);
              d = __builtin_amdgcn_mfma_f32_16x16x4f32(a[q].z, b[q].z, d, 0, 0, 0);
              d = __builtin_amdgcn_mfma_f32_16x16x4f32(a[q].w, b[q].w, d, 0, 0, 0);
            }
            // d[r] = D[row 4g + r][col l16]
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              int ol = orow[m * 16 + 4 * g + r];
              if (ol >= 0) acc[ol * CN + wave * 16 + l16] += d[r];
            }
          }
        }
      }
    }
  }
  __syncthreads();
  // write the tile
  const int col0 = blockIdx.y * CN;
  if ((cout & 3) == 0) {
    for (int e = tid; e < T * (CN / 4); e += NT) {
      int r = e / (CN / 4), c4 = e % (CN / 4);
      int64_t grow = row0 + r;
      int col = col0 + c4 * 4;
      if (grow < n_out && col < cout)
        *reinterpret_cast<float4v *>(out + grow * cout + col) =
            *reinterpret_cast<const float4v *>(acc + r * CN + c4 * 4);
    }
  } else {
    for (int e = tid; e < T * CN; e += NT) {
      int r = e / CN, c = e % CN;
      int64_t grow = row0 + r;
      if (grow < n_out && col0 + c < cout) out[grow * cout + col0 + c] = acc[e];
    }
  }
}

struct ConvPlan {
  int ncb, nch, T;
  int64_t n_tiles, words_per_k;
  size_t lds_bytes;
};

static int pick_tile(int cn) {
  // Two workgroups per CU (160 KB LDS): accumulators + staging must stay under 80 KB.
  size_t budget = 80 * 1024 - (size_t)kStage * kAStride * 4 - kStage * 4 - 512;
  int t = (int)(budget / ((size_t)cn * 4));
  t = t / 16 * 16;
  if (t > 1024) t = 1024;
  if (t < kMinTile) t = kMinTile;
  return t;
}

static ConvPlan make_plan(int64_t n_out, int c_in, int c_out) {
  ConvPlan p;
  p.ncb = (int)ceil_div(c_out, 16);
  p.nch = (int)ceil_div(c_in, kKC);
  p.T = pick_tile(64);
  p.n_tiles = ceil_div(n_out > 0 ? n_out : 1, p.T);
  p.words_per_k = ceil_div(n_out > 0 ? n_out : 1, 32);
  p.lds_bytes = ((size_t)p.T * 64 + (size_t)kStage * kAStride) * 4 + kStage * 4;
  return p;
}

struct ConvWs {
  float *packed;
  int32_t *flag;
  int32_t *segs;
  int32_t *sorted;
  uint32_t *bits;
  int32_t *prefix;
};

static size_t conv_ws_bytes(int64_t n_out, int K, int c_in, int c_out, int64_t pair_stride) {
  ConvPlan p = make_plan(n_out, c_in, c_out);
  int64_t tiles_max = ceil_div(n_out > 0 ? n_out : 1, kMinTile);
  return align_up((size_t)K * p.ncb * p.nch * 1024 * 4) + align_up(4) +
         align_up((size_t)(tiles_max + 1) * K * 4) + align_up((size_t)K * 2 * pair_stride * 4) +
         2 * align_up((size_t)K * p.words_per_k * 4);
}

static ConvWs conv_ws_carve(void *ws, const ConvPlan &p, int64_t n_out, int K,
                            int64_t pair_stride) {
  Carver c(ws);
  ConvWs w;
  int64_t tiles_max = ceil_div(n_out > 0 ? n_out : 1, kMinTile);
  w.packed = c.take<float>((size_t)K * p.ncb * p.nch * 1024);
  w.flag = c.take<int32_t>(1);
  w.segs = c.take<int32_t>((size_t)(tiles_max + 1) * K);
  w.sorted = c.take<int32_t>((size_t)K * 2 * pair_stride);
  w.bits = c.take<uint32_t>((size_t)K * p.words_per_k);
  w.prefix = c.take<int32_t>((size_t)K * p.words_per_k);
  return w;
}

// Optional timing of the convolution kernel alone: a ring of event pairs recorded
// on the caller's stream right around the launch of conv_fwd_kernel.
constexpr int kProfileRing = 512;
static bool g_profile_on = false;
static int g_profile_count = 0;
static hipEvent_t g_profile_ev[kProfileRing][2];
static bool g_profile_init = false;

}  // namespace ssc

using namespace ssc;

extern "C" {

int ssc_profile_conv(int32_t enable) {
  if (enable && !g_profile_init) {
    for (int i = 0; i < kProfileRing; ++i) {
      SSC_HIP(hipEventCreate(&g_profile_ev[i][0]));
      SSC_HIP(hipEventCreate(&g_profile_ev[i][1]));
    }
    g_profile_init = true;
  }
  g_profile_on = enable != 0;
  g_profile_count = 0;
  return SSC_OK;
}

int ssc_profile_conv_read(float *ms, int32_t capacity, int32_t *count) {
  SSC_CHECK(ms != nullptr && count != nullptr, SSC_EINVAL, "NULL pointer argument");
  int n = g_profile_count < kProfileRing ? g_profile_count : kProfileRing;
  if (n > capacity) n = capacity;
  for (int i = 0; i < n; ++i) {
    SSC_HIP(hipEventSynchronize(g_profile_ev[i][1]));
    SSC_HIP(hipEventElapsedTime(&ms[i], g_profile_ev[i][0], g_profile_ev[i][1]));
  }
  *count = n;
  return SSC_OK;
}

size_t ssc_conv_workspace_bytes(int64_t n_out, int32_t kernel_volume, int32_t c_in, int32_t c_out,
                                int64_t pair_stride) {
  if (n_out < 0 || kernel_volume < 1 || c_in < 1 || c_out < 1 || pair_stride < 0) return 0;
  return conv_ws_bytes(n_out, kernel_volume, c_in, c_out, pair_stride);
}

int ssc_conv_fwd_f32(const float *features, int64_t n_in, int32_t c_in, const float *filters,
                     int64_t fs_k, int64_t fs_ci, int64_t fs_co, int32_t c_out,
                     const int32_t *pairs, int64_t pair_stride, const int32_t *pair_num,
                     int32_t kernel_volume, int32_t inverse, int32_t subm, float *out,
                     int64_t n_out, void *workspace, size_t workspace_bytes,
                     ssc_stream_t stream) {
  (void)subm;
  const int K = kernel_volume;
  SSC_CHECK(K >= 1 && K <= SSC_MAX_KERNEL_VOLUME, SSC_ERUNTIME, "kernel volume %d out of range", K);
  SSC_CHECK(c_in >= 1 && c_out >= 1, SSC_EINVAL, "channel counts must be positive");
  SSC_CHECK(n_in >= 0 && n_out >= 0 && pair_stride >= 0, SSC_EINVAL, "negative size");
  SSC_CHECK(n_out < ((int64_t)1 << 31) && n_in < ((int64_t)1 << 31), SSC_EINVAL,
            "row counts must fit 31 bits");
  if (n_out == 0) return SSC_OK;
  SSC_CHECK(out != nullptr, SSC_EINVAL, "out is NULL");
  hipStream_t s = (hipStream_t)stream;
  if (pair_stride == 0 || n_in == 0) return fill_f32(out, n_out * c_out, 0.f, s);
  SSC_CHECK(features && filters && pairs && pair_num && workspace, SSC_EINVAL,
            "NULL pointer argument");
  size_t need = conv_ws_bytes(n_out, K, c_in, c_out, pair_stride);
  SSC_CHECK(workspace_bytes >= need, SSC_EWORKSPACE, "conv workspace too small: %zu < %zu",
            workspace_bytes, need);

  ConvPlan p = make_plan(n_out, c_in, c_out);
  ConvWs w = conv_ws_carve(workspace, p, n_out, K, pair_stride);
  const int plane_g = inverse ? 1 : 0;
  const int plane_s = 1 - plane_g;
  int rc;

  int64_t packed_n = (int64_t)K * p.ncb * p.nch * 1024;
  hipLaunchKernelGGL(pack_filters_kernel, dim3((unsigned)ceil_div(packed_n, 256)), dim3(256), 0, s,
                     filters, fs_k, fs_ci, fs_co, K, c_in, c_out, p.ncb, p.nch, w.packed);
  SSC_LAUNCH_CHECK("pack_filters");

  if ((rc = fill_i32(w.flag, 1, 0, s)) != SSC_OK) return rc;
  dim3 pair_grid((unsigned)ceil_div(pair_stride, 256), (unsigned)K);
  hipLaunchKernelGGL(check_sorted_kernel, pair_grid, dim3(256), 0, s, pairs, pair_stride, plane_s,
                     pair_num, w.flag);
  SSC_LAUNCH_CHECK("check_sorted");
  int64_t nbits_words = (int64_t)K * p.words_per_k;
  unsigned clear_blocks = (unsigned)(ceil_div(nbits_words, 256) < 4096 ? ceil_div(nbits_words, 256) : 4096);
  hipLaunchKernelGGL(resort_clear_kernel, dim3(clear_blocks), dim3(256), 0, s, w.flag, w.bits,
                     nbits_words);
  hipLaunchKernelGGL(resort_mark_kernel, pair_grid, dim3(256), 0, s, w.flag, pairs, pair_stride,
                     plane_s, pair_num, w.bits, p.words_per_k);
  hipLaunchKernelGGL(resort_scan_kernel, dim3(K), dim3(kScanThreads), 0, s, w.flag, w.bits,
                     w.prefix, p.words_per_k);
  hipLaunchKernelGGL(resort_scatter_kernel, pair_grid, dim3(256), 0, s, w.flag, pairs,
                     pair_stride, plane_s, pair_num, w.bits, w.prefix, p.words_per_k, w.sorted);
  SSC_LAUNCH_CHECK("resort");

  int64_t nseg = (p.n_tiles + 1) * K;
  hipLaunchKernelGGL(tile_segments_kernel, dim3((unsigned)ceil_div(nseg, 256)), dim3(256), 0, s,
                     w.flag, pairs, w.sorted, pair_stride, plane_s, pair_num, K, p.n_tiles, p.T,
                     w.segs);
  SSC_LAUNCH_CHECK("tile_segments");

  static bool attr_set = false;
  if (!attr_set) {
    SSC_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(conv_fwd_kernel<4>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    attr_set = true;
  }
  dim3 grid((unsigned)p.n_tiles, (unsigned)ceil_div(p.ncb, 4));
  const bool prof = g_profile_on;
  const int slot = g_profile_count % kProfileRing;
  if (prof) SSC_HIP(hipEventRecord(g_profile_ev[slot][0], s));
  hipLaunchKernelGGL(conv_fwd_kernel<4>, grid, dim3(256), p.lds_bytes, s, features, c_in, w.packed,
                     w.flag, pairs, w.sorted, pair_stride, plane_g, w.segs, K, p.nch, p.ncb, out,
                     n_out, c_out, p.T);
  SSC_LAUNCH_CHECK("conv_fwd");
  if (prof) {
    SSC_HIP(hipEventRecord(g_profile_ev[slot][1], s));
    ++g_profile_count;
  }
  return SSC_OK;
}
}
