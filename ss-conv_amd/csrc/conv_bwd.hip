// Filter gradient of the sparse convolution:
//   dW[k][ci][co] = sum over the pairs (i, o) of offset k of feat[i][ci] * dout[o][co]
// (reference: src/conv/indice_conv.h:344-426, the torch::mm_out(filterGradSub, ...)
// of every offset).  The input gradient needs no kernel of its own: it is the forward
// convolution of dout with the pairs swapped and the filters transposed.
//
// Per offset this is a tall-skinny product [Cin x P_k] * [P_k x Cout] on fp32 MFMA.
// A workgroup owns one offset, one 64 x 64 tile of (ci, co) and one contiguous range
// of the offset's pairs; it gathers 64 pairs at a time into LDS, rows as they lie in
// memory.  Which pair sits in which k slot of an MFMA does not matter for the sum, and
// neither does which channel a lane stands for, as long as the result is stored
// accordingly: lane l of channel block j stands for channel 4l + j, so one 16-byte LDS
// read of a gathered row hands a lane its operands for all four channel blocks, and
// two such reads (features, output gradient) feed 16 MFMAs.  Every wave keeps the
// whole 64 x 64 tile (16 independent accumulators) over a quarter of the pairs; the
// four waves' tiles are added in wave order at the end, and the ranges of pairs by a
// second kernel in ascending order: the result does not depend on timing, no atomics.
#include "ssc_common.h"

#include <type_traits>

namespace ssc {

typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kBwChunk = 64;    // pairs per LDS stage
constexpr int kBwStride = 68;   // floats per channel row in LDS (64 pairs + 4)
constexpr int kBwTile = 64;     // channels per tile side

// Rows of float or half-precision elements; the products and sums are fp32 either way
// (half rows are widened when they are staged in LDS).
typedef int int2v __attribute__((ext_vector_type(2)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4v widen4(const float4v &v) { return v; }
__device__ __forceinline__ float4v widen4(const int2v &v) {
  return __builtin_convertvector(__builtin_bit_cast(half4v, v), float4v);
}
__device__ __forceinline__ float4v load4(const float *p) {
  return *reinterpret_cast<const float4v *>(p);
}
__device__ __forceinline__ float4v load4(const _Float16 *p) {
  return widen4(*reinterpret_cast<const int2v *>(p));
}
// four channels at byte offset `off` of a buffer, as loaded
__device__ __forceinline__ float4v buf_quad(__amdgpu_buffer_rsrc_t r, unsigned off, const float *) {
  return __builtin_bit_cast(float4v, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0));
}
__device__ __forceinline__ int2v buf_quad(__amdgpu_buffer_rsrc_t r, unsigned off,
                                          const _Float16 *) {
  return __builtin_bit_cast(int2v, __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0));
}

// Four channels of row `row`, zero outside the matrix.
template <typename IO>
__device__ __forceinline__ float4v load_quad(const IO *__restrict__ m, int64_t row, int ch,
                                             int width) {
  float4v v = {0.f, 0.f, 0.f, 0.f};
  if (row < 0) return v;
  const IO *p = m + row * width + ch;
  if ((width & 3) == 0) {
    if (ch < width) v = load4(p);
  } else {
    if (ch + 0 < width) v.x = (float)p[0];
    if (ch + 1 < width) v.y = (float)p[1];
    if (ch + 2 < width) v.z = (float)p[2];
    if (ch + 3 < width) v.w = (float)p[3];
  }
  return v;
}

// grid: x = range of pairs, y = offset k, z = tile (ci tile major).  256 threads, four
// workgroups per CU (one wave of each per SIMD: 128 registers a wave).
// BUF: rows are multiples of four channels and both matrices are below 4 GiB, so the gathers
// are range-checked buffer loads at 32-bit byte offsets (a row beyond the range's pairs
// gets an offset outside the buffer and reads zeros): no 64-bit address arithmetic and
// no branches around the loads.
template <typename IO, bool BUF>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4)))
    conv_bwd_filter_kernel(const IO *__restrict__ feats, int cin, unsigned feat_bytes,
                           const IO *__restrict__ dout, int cout, unsigned dout_bytes,
                           const int32_t *__restrict__ pairs, int64_t pair_stride,
                           const int32_t *__restrict__ pair_num, int plane_in, int n_split,
                           int n_co_tiles, float *__restrict__ partial) {
  __shared__ __align__(16) float ft[kBwChunk * kBwStride];  // features, [pair][ci]
  __shared__ __align__(16) float dt[kBwChunk * kBwStride];  // output gradient, [pair][co]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, g = lane >> 4;
  const int s = blockIdx.x, k = blockIdx.y, K = gridDim.y;
  const int ci0 = (blockIdx.z / n_co_tiles) * kBwTile;
  const int co0 = (blockIdx.z % n_co_tiles) * kBwTile;
  const int n = pair_num[k];
  // ranges are multiples of the chunk, so that every workgroup starts on a chunk boundary
  int len = (n + n_split - 1) / n_split;
  len = (len + kBwChunk - 1) / kBwChunk * kBwChunk;
  const int p_begin = min(s * len, n), p_end = min(p_begin + len, n);
  const int32_t *rows_in = pairs + ((int64_t)k * 2 + plane_in) * pair_stride;
  const int32_t *rows_out = pairs + ((int64_t)k * 2 + (1 - plane_in)) * pair_stride;

  // staging: 16 threads per gathered row (256 contiguous bytes), pairs (tid >> 4) + 16j
  const int sp = tid >> 4, sq = (tid & 15) * 4;
  constexpr unsigned kEB = sizeof(IO);
  // rows in flight: as loaded from a buffer, or widened already by the pointer path
  typedef std::conditional_t<BUF, decltype(buf_quad(__amdgpu_buffer_rsrc_t(), 0u, (const IO *)nullptr)),
                             float4v> Held;
  Held rf[4], rd[4];
  const __amdgpu_buffer_rsrc_t rs_f =
      __builtin_amdgcn_make_buffer_rsrc((void *)feats, 0, (int)feat_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_d =
      __builtin_amdgcn_make_buffer_rsrc((void *)dout, 0, (int)dout_bytes, 0x00020000);
  // a quad of channels beyond the matrix width reads zeros as well
  const unsigned col_f = ci0 + sq < cin ? (unsigned)(ci0 + sq) * kEB : 0xFFFFF000u;
  const unsigned col_d = co0 + sq < cout ? (unsigned)(co0 + sq) * kEB : 0xFFFFF000u;
  // row numbers of the chunk after the one being fetched: the gathers never wait for
  // their own index loads
  int idx_i[4], idx_o[4];
  auto fetch_idx = [&](int p0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int p = p0 + sp + 16 * j;
      idx_i[j] = p < p_end ? rows_in[p] : -1;
      idx_o[j] = p < p_end ? rows_out[p] : -1;
    }
  };
  auto fetch = [&](int p0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int p = p0 + sp + 16 * j;
      if constexpr (BUF) {
        const unsigned ri = idx_i[j] >= 0 ? (unsigned)idx_i[j] * ((unsigned)cin * kEB) : 0xFFFFF000u;
        const unsigned ro = idx_o[j] >= 0 ? (unsigned)idx_o[j] * ((unsigned)cout * kEB) : 0xFFFFF000u;
        // saturating: an offset that is already outside stays outside
        const unsigned of = ri > 0xFFFFF000u - col_f ? 0xFFFFF000u : ri + col_f;
        const unsigned od = ro > 0xFFFFF000u - col_d ? 0xFFFFF000u : ro + col_d;
        rf[j] = buf_quad(rs_f, of, feats);
        rd[j] = buf_quad(rs_d, od, dout);
      } else {
        (void)p;
        rf[j] = load_quad(feats, idx_i[j], ci0 + sq, cin);
        rd[j] = load_quad(dout, idx_o[j], co0 + sq, cout);
      }
    }
    fetch_idx(p0 + kBwChunk);
  };
  auto stage = [&]() {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      *reinterpret_cast<float4v *>(ft + (sp + 16 * j) * kBwStride + sq) = widen4(rf[j]);
      *reinterpret_cast<float4v *>(dt + (sp + 16 * j) * kBwStride + sq) = widen4(rd[j]);
    }
  };

  // acc[jm][jn]: D[ci0 + 4*(4g + r) + jm][co0 + 4*l16 + jn] in component r
  float4v acc[4][4];
#pragma unroll
  for (int jm = 0; jm < 4; ++jm)
#pragma unroll
    for (int jn = 0; jn < 4; ++jn) acc[jm][jn] = float4v{0.f, 0.f, 0.f, 0.f};
  // k slot g of this wave's MFMA step tt is pair 4 * (wave + 4 * tt) + g of the chunk
  const float *a_row = ft + (4 * wave + g) * kBwStride + 4 * l16;
  const float *b_row = dt + (4 * wave + g) * kBwStride + 4 * l16;

  if (p_begin < p_end) {
    fetch_idx(p_begin);
    fetch(p_begin);
  }
  for (int p0 = p_begin; p0 < p_end; p0 += kBwChunk) {
    stage();
    __syncthreads();
    if (p0 + kBwChunk < p_end) fetch(p0 + kBwChunk);  // in flight during the MFMAs
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
      const float4v a = *reinterpret_cast<const float4v *>(a_row + tt * 16 * kBwStride);
      const float4v b = *reinterpret_cast<const float4v *>(b_row + tt * 16 * kBwStride);
#pragma unroll
      for (int jm = 0; jm < 4; ++jm)
#pragma unroll
        for (int jn = 0; jn < 4; ++jn)
          acc[jm][jn] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[jm], b[jn], acc[jm][jn], 0, 0, 0);
    }
    __syncthreads();
  }
  // Add the four waves' tiles in wave order through LDS (tile[ci][co], 64 x 64 floats in
  // the staging memory), then write the tile out.
  float *tile = ft;
  static_assert(2 * kBwChunk * kBwStride >= kBwTile * kBwTile, "the tile fits the staging memory");
  for (int w = 0; w < 4; ++w) {
    if (wave == w) {
#pragma unroll
      for (int jm = 0; jm < 4; ++jm)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          // the four column blocks of a lane are four neighbouring columns
          float4v *t = reinterpret_cast<float4v *>(tile + (4 * (4 * g + r) + jm) * kBwTile + 4 * l16);
          const float4v v = {acc[jm][0][r], acc[jm][1][r], acc[jm][2][r], acc[jm][3][r]};
          *t = w == 0 ? v : *t + v;
        }
    }
    __syncthreads();
  }
  float *dst = partial + ((int64_t)s * K + k) * cin * cout;
  for (int e = tid; e < kBwTile * kBwTile; e += 256) {
    const int ci = ci0 + e / kBwTile, co = co0 + e % kBwTile;
    if (ci < cin && co < cout) dst[(int64_t)ci * cout + co] = tile[e];
  }
}

// out[e] = partial[0][e] + partial[1][e] + ... in that order; out may have any strides.
template <typename IO>
__global__ void __launch_bounds__(256)
    conv_bwd_reduce_kernel(const float *__restrict__ partial, int n_split, int K, int cin, int cout,
                           IO *__restrict__ out, int64_t os_k, int64_t os_ci, int64_t os_co) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t per = (int64_t)K * cin * cout;
  if (e >= per) return;
  float v = partial[e];
  for (int s = 1; s < n_split; ++s) v += partial[(int64_t)s * per + e];
  const int co = (int)(e % cout);
  const int64_t r = e / cout;
  const int ci = (int)(r % cin);
  const int k = (int)(r / cin);
  out[k * os_k + ci * os_ci + co * os_co] = (IO)v;
}

static int bwd_split(int K, int c_in, int c_out, int64_t pair_stride) {
  // as many workgroups as the chip holds at once (4 per CU on 256 CUs) when the tiles
  // alone are fewer, but ranges of at least 8 chunks
  const int64_t tiles = ceil_div(c_in, kBwTile) * ceil_div(c_out, kBwTile) * K;
  int64_t s = 1024 / tiles;
  const int64_t max_s = ceil_div(pair_stride > 0 ? pair_stride : 1, 8 * kBwChunk);
  if (s > max_s) s = max_s;
  if (s < 1) s = 1;
  return (int)s;
}

}  // namespace ssc

using namespace ssc;

extern "C" {

size_t ssc_conv_bwd_filter_workspace_bytes(int32_t kernel_volume, int32_t c_in, int32_t c_out,
                                           int64_t pair_stride) {
  if (kernel_volume < 1 || c_in < 1 || c_out < 1 || pair_stride < 0) return 0;
  const int s = bwd_split(kernel_volume, c_in, c_out, pair_stride);
  return align_up((size_t)s * kernel_volume * c_in * c_out * sizeof(float));
}

}  // extern "C"

template <typename IO>
static int conv_bwd_filter(const IO *features, int64_t n_in, int32_t c_in, const IO *out_grad,
                           int64_t n_out, int32_t c_out, const int32_t *pairs,
                           int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                           int32_t inverse, IO *filters_grad, int64_t gs_k, int64_t gs_ci,
                           int64_t gs_co, void *workspace, size_t workspace_bytes,
                           ssc_stream_t stream) {
  const int K = kernel_volume;
  SSC_CHECK(K >= 1 && K <= SSC_MAX_KERNEL_VOLUME, SSC_ERUNTIME, "kernel volume %d out of range", K);
  SSC_CHECK(c_in >= 1 && c_out >= 1, SSC_EINVAL, "channel counts must be positive");
  SSC_CHECK(n_in >= 0 && n_out >= 0 && pair_stride >= 0, SSC_EINVAL, "negative size");
  SSC_CHECK(filters_grad != nullptr, SSC_EINVAL, "filters_grad is NULL");
  hipStream_t s = (hipStream_t)stream;
  const int64_t per = (int64_t)K * c_in * c_out;
  if (pair_stride == 0 || n_in == 0 || n_out == 0) {
    // no pairs: the gradient is zero (the reduce kernel of one zeroed range writes it)
    SSC_CHECK(workspace != nullptr && workspace_bytes >= (size_t)per * sizeof(float),
              SSC_EWORKSPACE, "conv backward workspace too small");
    int rc = fill_f32(static_cast<float *>(workspace), per, 0.f, s);
    if (rc != SSC_OK) return rc;
    hipLaunchKernelGGL(conv_bwd_reduce_kernel<IO>, dim3((unsigned)ceil_div(per, 256)), dim3(256), 0, s,
                       static_cast<const float *>(workspace), 1, K, c_in, c_out, filters_grad, gs_k,
                       gs_ci, gs_co);
    SSC_LAUNCH_CHECK("conv_bwd_reduce");
    return SSC_OK;
  }
  SSC_CHECK(features && out_grad && pairs && pair_num && workspace, SSC_EINVAL,
            "NULL pointer argument");
  const size_t need = ssc_conv_bwd_filter_workspace_bytes(K, c_in, c_out, pair_stride);
  SSC_CHECK(workspace_bytes >= need, SSC_EWORKSPACE,
            "conv backward workspace too small: %zu < %zu", workspace_bytes, need);
  const int n_split = bwd_split(K, c_in, c_out, pair_stride);
  const int n_ci_tiles = (int)ceil_div(c_in, kBwTile), n_co_tiles = (int)ceil_div(c_out, kBwTile);
  SSC_CHECK((int64_t)n_ci_tiles * n_co_tiles <= 65535, SSC_ERUNTIME, "too many channel tiles");
  float *partial = static_cast<float *>(workspace);
  // features are gathered through the plane the forward pass gathered them through
  const int plane_in = inverse ? 1 : 0;
  const dim3 grid((unsigned)n_split, (unsigned)K, (unsigned)(n_ci_tiles * n_co_tiles));
  const uint64_t feat_bytes = (uint64_t)n_in * c_in * sizeof(IO);
  const uint64_t dout_bytes = (uint64_t)n_out * c_out * sizeof(IO);
  // the largest byte offset must stay below the marker that stands for "outside"
  const bool buf = (c_in & 3) == 0 && (c_out & 3) == 0 && feat_bytes <= 0xFFFFF000u &&
                   dout_bytes <= 0xFFFFF000u;
  if (buf)
    hipLaunchKernelGGL((conv_bwd_filter_kernel<IO, true>), grid, dim3(256), 0, s, features, c_in,
                       (unsigned)feat_bytes, out_grad, c_out, (unsigned)dout_bytes, pairs,
                       pair_stride, pair_num, plane_in, n_split, n_co_tiles, partial);
  else
    hipLaunchKernelGGL((conv_bwd_filter_kernel<IO, false>), grid, dim3(256), 0, s, features, c_in, 0u,
                       out_grad, c_out, 0u, pairs, pair_stride, pair_num, plane_in, n_split,
                       n_co_tiles, partial);
  SSC_LAUNCH_CHECK("conv_bwd_filter");
  hipLaunchKernelGGL(conv_bwd_reduce_kernel<IO>, dim3((unsigned)ceil_div(per, 256)), dim3(256), 0, s,
                     partial, n_split, K, c_in, c_out, filters_grad, gs_k, gs_ci, gs_co);
  SSC_LAUNCH_CHECK("conv_bwd_reduce");
  return SSC_OK;
}

extern "C" {

int ssc_conv_bwd_filter_f32(const float *features, int64_t n_in, int32_t c_in,
                            const float *out_grad, int64_t n_out, int32_t c_out,
                            const int32_t *pairs, int64_t pair_stride, const int32_t *pair_num,
                            int32_t kernel_volume, int32_t inverse, float *filters_grad,
                            int64_t gs_k, int64_t gs_ci, int64_t gs_co, void *workspace,
                            size_t workspace_bytes, ssc_stream_t stream) {
  return conv_bwd_filter<float>(features, n_in, c_in, out_grad, n_out, c_out, pairs, pair_stride,
                                pair_num, kernel_volume, inverse, filters_grad, gs_k, gs_ci, gs_co,
                                workspace, workspace_bytes, stream);
}

int ssc_conv_bwd_filter_f16(const void *features, int64_t n_in, int32_t c_in,
                            const void *out_grad, int64_t n_out, int32_t c_out,
                            const int32_t *pairs, int64_t pair_stride, const int32_t *pair_num,
                            int32_t kernel_volume, int32_t inverse, void *filters_grad,
                            int64_t gs_k, int64_t gs_ci, int64_t gs_co, void *workspace,
                            size_t workspace_bytes, ssc_stream_t stream) {
  return conv_bwd_filter<_Float16>(
      static_cast<const _Float16 *>(features), n_in, c_in, static_cast<const _Float16 *>(out_grad),
      n_out, c_out, pairs, pair_stride, pair_num, kernel_volume, inverse,
      static_cast<_Float16 *>(filters_grad), gs_k, gs_ci, gs_co, workspace, workspace_bytes, stream);
}
}
