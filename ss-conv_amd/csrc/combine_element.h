// One element of the synthesised dense kernel (shared by combine.hip and the fused
// synthesis + packing kernel of conv.hip).
#ifndef SSC_COMBINE_ELEMENT_H_
#define SSC_COMBINE_ELEMENT_H_

#include "ssc_common.h"

namespace ssc {

// dense[k][ci][co] = sum over beta (ascending) of weight * basis; the per-channel descriptor
// tables replace the reference's loop over irrep pairs, its einsum, both concatenations and
// the permute (ss_conv/utils/kernel.py:267-299).
__device__ __forceinline__ float combine_element(const float *__restrict__ weight,
                                                 const float *__restrict__ basis,
                                                 const int32_t *__restrict__ chan_out,
                                                 const int32_t *__restrict__ chan_in,
                                                 const int32_t *__restrict__ blocks, int n_j, int K,
                                                 int k, int ci, int co) {
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
  return acc;
}

}  // namespace ssc

#endif
