// The one-column-group form of the convolution kernel (conv_kernel.h, TAIL), every instance
// the float path of conv.hip can ask for: a translation unit of its own, so that the two
// halves of the kernel's instances compile side by side.
#include "conv_kernel.h"

namespace ssc {

template <int GATHER, int NS, bool EPI>
int launch_conv_tail(const ConvPlan &p, const ConvWs &w, const float *features, int64_t n_in,
                     int c_in, int K, float *out, int c_out, int col_base,
                     const ConvEpilogue &epi, hipStream_t s) {
  return launch_conv<float, GATHER, 4, NS, EPI, true>(p, w, features, n_in, c_in, K, out, c_out,
                                                      col_base, epi, s);
}

#define SSC_TAIL_INSTANCE(G, S)                                                                   \
  template int launch_conv_tail<G, S, false>(const ConvPlan &, const ConvWs &, const float *,    \
                                             int64_t, int, int, float *, int, int,               \
                                             const ConvEpilogue &, hipStream_t);                 \
  template int launch_conv_tail<G, S, true>(const ConvPlan &, const ConvWs &, const float *,     \
                                            int64_t, int, int, float *, int, int,                \
                                            const ConvEpilogue &, hipStream_t);
// the steps per chunk conv.hip's make_plan can choose, for either checked gather; whole
// chunks for the unchecked one
#define SSC_TAIL_BY_STEPS(G)                                                                    \
  SSC_TAIL_INSTANCE(G, 1) SSC_TAIL_INSTANCE(G, 2) SSC_TAIL_INSTANCE(G, 3) SSC_TAIL_INSTANCE(G, 4) \
  SSC_TAIL_INSTANCE(G, 6) SSC_TAIL_INSTANCE(G, 8) SSC_TAIL_INSTANCE(G, 10)                        \
  SSC_TAIL_INSTANCE(G, 12) SSC_TAIL_INSTANCE(G, 13) SSC_TAIL_INSTANCE(G, 14)                      \
  SSC_TAIL_INSTANCE(G, 15) SSC_TAIL_INSTANCE(G, 16)
SSC_TAIL_BY_STEPS(0)
SSC_TAIL_BY_STEPS(2)
SSC_TAIL_INSTANCE(1, 16)
#undef SSC_TAIL_BY_STEPS
#undef SSC_TAIL_INSTANCE

}  // namespace ssc
