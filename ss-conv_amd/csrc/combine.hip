// Steerable kernel synthesis: dense kernel = sum_beta weight * basis, written
// straight into the contiguous [K, Cin, Cout] layout the convolution consumes.
// One thread per output element; the per-channel descriptor tables replace the
// reference's loop over irrep pairs, its einsum, both concatenations and the
// permute.  The sum over beta runs in ascending order.
#include "combine_element.h"
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
  const float acc = combine_element(weight, basis, chan_out, chan_in, blocks, n_j, K, k, ci, co);
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
