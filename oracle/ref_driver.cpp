// ref_driver.cpp -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// extern "C" entry points into the *reference's own* CPU code, compiled from
// the sources where they lie under /root/reference (see oracle/Makefile).  The
// resulting oracle/_ref/libssc_ref.so is used by the tests to pin the C
// restatement in ssc_oracle.c; nothing in the product loads it.
//
//   rulebook:   getIndicePairsConv / getIndicePairsDeConv / getIndicePairsSubM
//                                                         (src/conv/geometry.h:140-189, 190-237, 241-288)
//   max pool:   SparseMaxPoolForwardFunctor<tv::CPU>      (src/pool/indice_maxpool_cpp_functor.cpp:16-35)
//   conv parts: SparseGatherFunctor / SparseScatterAddFunctor<tv::CPU>
//                                                         (src/conv/reordering_cpp_functor.cpp:15-44)
#include "geometry.h"
#include "indice_maxpool_functor.h"
#include "reordering_functor.h"

extern "C" {

int ref_rulebook_conv(const int *indices, int n_in, int batch, const int *ks, const int *st,
                      const int *pd, const int *dl, const int *out_shape, int *out_indices,
                      int *grid, int *pairs, int *pair_num) {
  int K = ks[0] * ks[1] * ks[2];
  int vol = out_shape[0] * out_shape[1] * out_shape[2];
  tv::TensorView<const int> t_in(indices, {n_in, 4});
  tv::TensorView<int> t_out(out_indices, {n_in * K, 4});
  tv::TensorView<int> t_grid(grid, {batch * vol});
  tv::TensorView<int> t_pairs(pairs, {K, 2, n_in});
  tv::TensorView<int> t_num(pair_num, {K});
  return getIndicePairsConv<int, int, 3>(t_in, t_out, t_grid, t_pairs, t_num, ks, st, pd, dl,
                                         out_shape);
}

int ref_rulebook_deconv(const int *indices, int n_in, int batch, const int *ks, const int *st,
                        const int *pd, const int *dl, const int *out_shape, int *out_indices,
                        int *grid, int *pairs, int *pair_num) {
  int K = ks[0] * ks[1] * ks[2];
  int vol = out_shape[0] * out_shape[1] * out_shape[2];
  tv::TensorView<const int> t_in(indices, {n_in, 4});
  tv::TensorView<int> t_out(out_indices, {n_in * K, 4});
  tv::TensorView<int> t_grid(grid, {batch * vol});
  tv::TensorView<int> t_pairs(pairs, {K, 2, n_in});
  tv::TensorView<int> t_num(pair_num, {K});
  return getIndicePairsDeConv<int, int, 3>(t_in, t_out, t_grid, t_pairs, t_num, ks, st, pd, dl,
                                           out_shape);
}

int ref_rulebook_subm(const int *indices, int n_in, int batch, const int *ks, const int *st,
                      const int *pd, const int *dl, const int *out_shape, int *grid, int *pairs,
                      int *pair_num) {
  int K = ks[0] * ks[1] * ks[2];
  int vol = out_shape[0] * out_shape[1] * out_shape[2];
  tv::TensorView<const int> t_in(indices, {n_in, 4});
  tv::TensorView<int> t_grid(grid, {batch * vol});
  tv::TensorView<int> t_pairs(pairs, {K, 2, n_in});
  tv::TensorView<int> t_num(pair_num, {K});
  return getIndicePairsSubM<int, int, 3>(t_in, t_grid, t_pairs, t_num, ks, st, pd, dl, out_shape);
}

// pairs_k points at one offset's [2, stride] block (plane 0 inputs, plane 1 outputs).
void ref_maxpool_offset(float *out, int n_out, const float *in, int n_in, int c,
                        const int *pairs_k, int stride, int n) {
  functor::SparseMaxPoolForwardFunctor<tv::CPU, float, int> f;
  f(tv::CPU(), tv::TensorView<float>(out, {n_out, c}), tv::TensorView<const float>(in, {n_in, c}),
    tv::TensorView<const int>(pairs_k, {2, stride}), n);
}

void ref_gather_rows(float *buffer, int n_buf, const float *features, int n_feat, int c,
                     const int *rows, int n) {
  functor::SparseGatherFunctor<tv::CPU, float, int> f;
  f(tv::CPU(), tv::TensorView<float>(buffer, {n_buf, c}),
    tv::TensorView<const float>(features, {n_feat, c}), tv::TensorView<const int>(rows, {n}), n);
}

void ref_scatter_add_rows(float *out, int n_out, const float *buffer, int n_buf, int c,
                          const int *rows, int n) {
  functor::SparseScatterAddFunctor<tv::CPU, float, int> f;
  f(tv::CPU(), tv::TensorView<float>(out, {n_out, c}),
    tv::TensorView<const float>(buffer, {n_buf, c}), tv::TensorView<const int>(rows, {n}), n,
    true);
}
}
