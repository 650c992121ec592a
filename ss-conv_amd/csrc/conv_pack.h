// The packed order of the convolution's filters (see "weight packing" in conv.hip) and the
// job "synthesise the steerable kernel and pack it", which a layer's rulebook can take along
// in its first launch.
#ifndef SSC_CONV_PACK_H_
#define SSC_CONV_PACK_H_

#include "combine_element.h"
#include "ssc_common.h"

namespace ssc {

constexpr int kPackKC = 64;  // input channels per chunk of half filters (kKC of conv_kernel.h)

struct PackArgs {
  const void *w;  // filters, addressed as w[k*fs_k + ci*fs_ci + co*fs_co]
  int64_t fs_k, fs_ci, fs_co;
  int K, cin, cout, ncb, nch;
  void *packed_out;
  int ns;  // MFMA steps per chunk (float filters; half filters always use whole chunks)
};

// Offset k, input channel ci and output channel co of element idx of the packed filters
// (ci >= cin or co >= cout: a padding element).
template <typename IO>
__device__ __forceinline__ void pack_decode(const PackArgs &a, int64_t idx, int &k, int &ci,
                                            int &co) {
  const int cin = a.cin, ncb = a.ncb, nch = a.nch;
  int64_t r = idx >> 10;
  int cc = r % nch;
  r /= nch;
  int cb = r % ncb;
  k = (int)(r / ncb);
  int lane;
  if constexpr (sizeof(IO) == 2) {
    const int j = idx & 7, q = (idx >> 9) & 1;
    lane = (idx >> 3) & 63;
    ci = cc * kPackKC + 32 * q + (lane >> 4) * 8 + j;
  } else {
    const int full = a.ns >> 2, rem = a.ns & 3;
    const int f = (int)(idx & 1023);  // float inside the fragment
    int cl = -1;  // channel inside the chunk, -1 for a slot without one
    lane = (f >> 2) & 63;
    if (f < full * 256) {
      cl = (f >> 8) * 16 + (lane >> 4) * 4 + (f & 3);
    } else if (f - full * 256 < 64 * rem) {  // the partly used quarter, rem floats per lane
      const int t = f - full * 256;
      lane = t / rem;
      cl = full * 16 + (t - lane * rem) * 4 + (lane >> 4);
    }
    ci = cl < 0 ? cin : cc * (4 * a.ns) + cl;
  }
  co = cb * 16 + (lane & 15);
}

// Element idx of the packed filters.
template <typename IO>
__device__ __forceinline__ void pack_filter_element(const PackArgs &a, int64_t idx) {
  const IO *__restrict__ w = static_cast<const IO *>(a.w);
  int k, ci, co;
  pack_decode<IO>(a, idx, k, ci, co);
  IO v = (IO)0.f;
  if (ci < a.cin && co < a.cout) v = w[k * a.fs_k + ci * a.fs_ci + co * a.fs_co];
  static_cast<IO *>(a.packed_out)[idx] = v;
}


// Synthesis and packing of one layer's filters: every element of the packed filters is
// computed (combine_element), stored at its place and, when it is a real element, in the
// dense [K, Cin, Cout] array as well.
struct CombineJob {
  PackArgs pk;
  const float *weight, *basis;
  const int32_t *chan_out, *chan_in, *blocks;
  int n_j;
  float *dense;
};
static inline int64_t combine_job_elements(const CombineJob &j) {
  return (int64_t)j.pk.K * j.pk.ncb * j.pk.nch * 1024;
}
__device__ __forceinline__ void combine_pack_element(const CombineJob &j, int64_t idx) {
  int k, ci, co;
  pack_decode<float>(j.pk, idx, k, ci, co);
  float v = 0.f;
  if (ci < j.pk.cin && co < j.pk.cout) {
    v = combine_element(j.weight, j.basis, j.chan_out, j.chan_in, j.blocks, j.n_j, j.pk.K, k, ci,
                        co);
    j.dense[((int64_t)k * j.pk.cin + ci) * j.pk.cout + co] = v;
  }
  static_cast<float *>(j.pk.packed_out)[idx] = v;
}
int launch_combine_pack(const CombineJob &job, hipStream_t s);

}  // namespace ssc

#endif
