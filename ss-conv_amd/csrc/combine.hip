// Steerable kernel synthesis: dense kernel = sum_beta weight * basis, written
// straight into the contiguous [K, Cin, Cout] layout the convolution consumes.
// One thread per output element; the per-channel descriptor tables replace the
// reference's loop over irrep pairs, its einsum, both concatenations and the
// permute.  The sum over beta runs in ascending order.
#include "ssc_common.h"

namespace ssc {

__global__ void __launch_bounds__(256)
    combine_kernel(const float *__restrict__ weight, const float *__restrict__ basis,
                   const int32_t *__restrict__ chan_out, const int32_t *__restrict__ chan_in,
                   const int32_t *__restrict__ blocks, int n_j, int K, int cin, int cout,
                   float *__restrict__ out) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)K * cin * cout;
  if (idx >= total) return;
  int co = (int)(idx % cout);
  int64_t r = idx / cout;
  int ci = (int)(r % cin);
  int k = (int)(r / cin);
  int i = chan_out[co * 3], u = chan_out[co * 3 + 1], a = chan_out[co * 3 + 2];
  int j = chan_in[ci * 3], v = chan_in[ci * 3 + 1], b = chan_in[ci * 3 + 2];
  const int32_t *blk = blocks + (i * n_j + j) * 6;
  int w_off = blk[0], b_off = blk[1], n_beta = blk[2], m_in = blk[3], d_out = blk[4],
      d_in = blk[5];
  const float *w = weight + w_off + (u * m_in + v) * n_beta;
  const float *bs = basis + b_off + ((int64_t)a * d_in + b) * K + k;
  int64_t beta_stride = (int64_t)d_out * d_in * K;
  float acc = 0.f;
  for (int t = 0; t < n_beta; ++t) acc += w[t] * bs[t * beta_stride];
  out[idx] = acc;
}

}  // namespace ssc

extern "C" int ssc_kernel_combine_f32(const float *weight, const float *basis,
                                      const int32_t *chan_out, const int32_t *chan_in,
                                      const int32_t *blocks, int32_t n_irreps_in,
                                      int32_t kernel_volume, int32_t c_in, int32_t c_out,
                                      float *out, ssc_stream_t stream) {
  SSC_CHECK(weight && basis && chan_out && chan_in && blocks && out, SSC_EINVAL,
            "NULL pointer argument");
  SSC_CHECK(n_irreps_in >= 1 && kernel_volume >= 1 && c_in >= 1 && c_out >= 1, SSC_EINVAL,
            "sizes must be positive");
  int64_t total = (int64_t)kernel_volume * c_in * c_out;
  hipLaunchKernelGGL(ssc::combine_kernel, dim3((unsigned)ssc::ceil_div(total, 256)), dim3(256), 0,
                     (hipStream_t)stream, weight, basis, chan_out, chan_in, blocks, n_irreps_in,
                     kernel_volume, c_in, c_out, out);
  SSC_LAUNCH_CHECK("combine");
  return SSC_OK;
}
