// Definition of launch_conv_f32 (conv_kernel.h) and the list of its instances: every
// combination of gather mode and steps per chunk that conv.hip's make_plan can choose, for
// one (EPI, FORM) pair per translation unit.
#pragma once
#include "conv_kernel.h"

namespace ssc {

template <int GATHER, int NS, bool EPI, int FORM>
int launch_conv_f32(const ConvPlan &p, const ConvWs &w, const float *features, int64_t n_in,
                    int c_in, int K, float *out, int c_out, int col_base, int xcol,
                    const ConvEpilogue &epi, hipStream_t s) {
  return launch_conv<float, GATHER, 4, NS, EPI, FORM>(p, w, features, n_in, c_in, K, out, c_out,
                                                      col_base, xcol, epi, s);
}

}  // namespace ssc

#define SSC_CONV_INSTANCE(G, S, EPI, FORM)                                                      \
  template int ssc::launch_conv_f32<G, S, EPI, FORM>(const ssc::ConvPlan &, const ssc::ConvWs &, \
                                                     const float *, int64_t, int, int, float *,  \
                                                     int, int, int, const ssc::ConvEpilogue &,   \
                                                     hipStream_t);
// checked gathers: every number of steps; the unchecked one: whole chunks
#define SSC_CONV_BY_STEPS(G, EPI, FORM)                                                         \
  SSC_CONV_INSTANCE(G, 1, EPI, FORM) SSC_CONV_INSTANCE(G, 2, EPI, FORM)                         \
  SSC_CONV_INSTANCE(G, 3, EPI, FORM) SSC_CONV_INSTANCE(G, 4, EPI, FORM)                         \
  SSC_CONV_INSTANCE(G, 6, EPI, FORM) SSC_CONV_INSTANCE(G, 8, EPI, FORM)                         \
  SSC_CONV_INSTANCE(G, 10, EPI, FORM) SSC_CONV_INSTANCE(G, 12, EPI, FORM)                       \
  SSC_CONV_INSTANCE(G, 13, EPI, FORM) SSC_CONV_INSTANCE(G, 14, EPI, FORM)                       \
  SSC_CONV_INSTANCE(G, 15, EPI, FORM) SSC_CONV_INSTANCE(G, 16, EPI, FORM)
#define SSC_CONV_INSTANCES(EPI, FORM)                                                           \
  SSC_CONV_BY_STEPS(0, EPI, FORM) SSC_CONV_BY_STEPS(2, EPI, FORM) SSC_CONV_INSTANCE(1, 16, EPI, FORM)
