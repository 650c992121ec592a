// Filter gradient of the sparse convolution:
//   dW[k][ci][co] = sum over the pairs (i, o) of offset k of feat[i][ci] * dout[o][co]
// (reference: src/conv/indice_conv.h:344-426, the torch::mm_out(filterGradSub, ...)
// of every offset).  The input gradient needs no kernel of its own: it is the forward
// convolution of dout with the pairs swapped and the filters transposed.
//
// Per offset this is a tall-skinny product [Cin x P_k] * [P_k x Cout] on fp32 MFMA.
// A workgroup owns one offset, one 64 x 64 tile of (ci, co) and one contiguous range
// of the offset's pairs; it gathers 64 pairs at a time into LDS -- transposed, channel
// major, so that a lane reads the four pairs of four MFMAs with one 16-byte read --
// and keeps its 64 x 64 tile in registers (wave w owns rows 16w .. 16w+15).  Ranges
// are reduced by a second kernel in ascending order, so the result does not depend on
// timing: no atomics.
#include "ssc_common.h"

namespace ssc {

typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kBwChunk = 64;    // pairs per LDS stage
constexpr int kBwStride = 68;   // floats per channel row in LDS (64 pairs + 4)
constexpr int kBwTile = 64;     // channels per tile side

// One 16-byte piece (4 channels) of row `row`, zero outside the matrix.
__device__ __forceinline__ float4v load_quad(const float *__restrict__ m, int64_t row, int ch,
                                             int width) {
  float4v v = {0.f, 0.f, 0.f, 0.f};
  if (row < 0) return v;
  const float *p = m + row * width + ch;
  if ((width & 3) == 0) {
    if (ch < width) v = *reinterpret_cast<const float4v *>(p);
  } else {
    if (ch + 0 < width) v.x = p[0];
    if (ch + 1 < width) v.y = p[1];
    if (ch + 2 < width) v.z = p[2];
    if (ch + 3 < width) v.w = p[3];
  }
  return v;
}

// grid: x = range of pairs, y = offset k, z = tile (ci tile major).  256 threads.
__global__ void __launch_bounds__(256)
    conv_bwd_filter_kernel(const float *__restrict__ feats, int cin,
                           const float *__restrict__ dout, int cout,
                           const int32_t *__restrict__ pairs, int64_t pair_stride,
                           const int32_t *__restrict__ pair_num, int plane_in, int n_split,
                           int n_co_tiles, float *__restrict__ partial) {
  __shared__ __align__(16) float ft[kBwTile * kBwStride];  // features, [ci][pair]
  __shared__ __align__(16) float dt[kBwTile * kBwStride];  // output gradient, [co][pair]
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

  // staging: thread -> pair tid & 63, channel quads (tid >> 6) + 4j
  const int sp = tid & 63, sq = tid >> 6;
  float4v rf[4], rd[4];
  auto fetch = [&](int p0) {
    const int p = p0 + sp;
    const int64_t ri = p < p_end ? rows_in[p] : -1;
    const int64_t ro = p < p_end ? rows_out[p] : -1;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      rf[j] = load_quad(feats, ri, ci0 + (sq + 4 * j) * 4, cin);
      rd[j] = load_quad(dout, ro, co0 + (sq + 4 * j) * 4, cout);
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int ch = (sq + 4 * j) * 4;
      ft[(ch + 0) * kBwStride + sp] = rf[j].x;
      ft[(ch + 1) * kBwStride + sp] = rf[j].y;
      ft[(ch + 2) * kBwStride + sp] = rf[j].z;
      ft[(ch + 3) * kBwStride + sp] = rf[j].w;
      dt[(ch + 0) * kBwStride + sp] = rd[j].x;
      dt[(ch + 1) * kBwStride + sp] = rd[j].y;
      dt[(ch + 2) * kBwStride + sp] = rd[j].z;
      dt[(ch + 3) * kBwStride + sp] = rd[j].w;
    }
  };

  float4v acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = float4v{0.f, 0.f, 0.f, 0.f};
  const float *a_row = ft + (wave * 16 + l16) * kBwStride + g * 4;
  const float *b_row = dt + l16 * kBwStride + g * 4;

  if (p_begin < p_end) fetch(p_begin);
  for (int p0 = p_begin; p0 < p_end; p0 += kBwChunk) {
    stage();
    __syncthreads();
    if (p0 + kBwChunk < p_end) fetch(p0 + kBwChunk);  // in flight during the MFMAs
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      // lane (l16, g) holds the pairs 16q + 4g .. +3 of its channel row: MFMA t of this
      // group multiplies pair 16q + 4g + t on both operands
      const float4v a = *reinterpret_cast<const float4v *>(a_row + q * 16);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float4v b = *reinterpret_cast<const float4v *>(b_row + j * 16 * kBwStride + q * 16);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, acc[j], 0, 0, 0);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, acc[j], 0, 0, 0);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, acc[j], 0, 0, 0);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, acc[j], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  // acc[j] = D[ci = 16*wave + 4g + r][co = 16j + l16], r = component
  float *dst = partial + ((int64_t)s * K + k) * cin * cout;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int co = co0 + j * 16 + l16;
    if (co >= cout) continue;
    const int ci = ci0 + wave * 16 + g * 4;
    if (ci + 0 < cin) dst[(int64_t)(ci + 0) * cout + co] = acc[j].x;
    if (ci + 1 < cin) dst[(int64_t)(ci + 1) * cout + co] = acc[j].y;
    if (ci + 2 < cin) dst[(int64_t)(ci + 2) * cout + co] = acc[j].z;
    if (ci + 3 < cin) dst[(int64_t)(ci + 3) * cout + co] = acc[j].w;
  }
}

// out[e] = partial[0][e] + partial[1][e] + ... in that order; out may have any strides.
__global__ void __launch_bounds__(256)
    conv_bwd_reduce_kernel(const float *__restrict__ partial, int n_split, int K, int cin, int cout,
                           float *__restrict__ out, int64_t os_k, int64_t os_ci, int64_t os_co) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t per = (int64_t)K * cin * cout;
  if (e >= per) return;
  float v = partial[e];
  for (int s = 1; s < n_split; ++s) v += partial[(int64_t)s * per + e];
  const int co = (int)(e % cout);
  const int64_t r = e / cout;
  const int ci = (int)(r % cin);
  const int k = (int)(r / cin);
  out[k * os_k + ci * os_ci + co * os_co] = v;
}

static int bwd_split(int K, int c_in, int c_out, int64_t pair_stride) {
  // enough workgroups to fill the chip a few times over, but ranges of at least 8 chunks
  const int64_t tiles = ceil_div(c_in, kBwTile) * ceil_div(c_out, kBwTile) * K;
  int64_t s = ceil_div(1024, tiles);
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

int ssc_conv_bwd_filter_f32(const float *features, int64_t n_in, int32_t c_in,
                            const float *out_grad, int64_t n_out, int32_t c_out,
                            const int32_t *pairs, int64_t pair_stride, const int32_t *pair_num,
                            int32_t kernel_volume, int32_t inverse, float *filters_grad,
                            int64_t gs_k, int64_t gs_ci, int64_t gs_co, void *workspace,
                            size_t workspace_bytes, ssc_stream_t stream) {
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
    hipLaunchKernelGGL(conv_bwd_reduce_kernel, dim3((unsigned)ceil_div(per, 256)), dim3(256), 0, s,
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
  hipLaunchKernelGGL(conv_bwd_filter_kernel,
                     dim3((unsigned)n_split, (unsigned)K, (unsigned)(n_ci_tiles * n_co_tiles)),
                     dim3(256), 0, s, features, c_in, out_grad, c_out, pairs, pair_stride, pair_num,
                     plane_in, n_split, n_co_tiles, partial);
  SSC_LAUNCH_CHECK("conv_bwd_filter");
  hipLaunchKernelGGL(conv_bwd_reduce_kernel, dim3((unsigned)ceil_div(per, 256)), dim3(256), 0, s,
                     partial, n_split, K, c_in, c_out, filters_grad, gs_k, gs_ci, gs_co);
  SSC_LAUNCH_CHECK("conv_bwd_reduce");
  return SSC_OK;
}
}
