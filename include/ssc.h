/*
 * ssc.h -- C ABI of the MI355X (gfx950) sparse steerable convolution hot path.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void*; NULL = the null stream) and returns 0 on success or a
 * negative SSC_E* code; ssc_last_error() then holds a readable message for the
 * calling thread.  No entry point allocates device memory: the caller supplies
 * outputs and, where stated, a workspace whose size the matching
 * *_workspace_bytes() function reports.  Kernels are enqueued on `stream` and
 * the call returns without synchronising unless its comment says otherwise.
 * Results are reproducible run to run: no floating-point atomics are used and
 * every accumulation order is fixed.
 *
 * All index tensors are int32, all feature tensors fp32, row-major and
 * contiguous unless strides are passed explicitly.
 *
 * Each declaration cites the interface of the reference implementation
 * (paths relative to SS_Conv_lib/) that it stands in for.
 */
#ifndef SSC_H_
#define SSC_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SSC_OK 0
#define SSC_EINVAL (-1)    /* bad argument (reference: std::invalid_argument / TV_ASSERT_INVALID_ARG) */
#define SSC_ERUNTIME (-2)  /* runtime check failed (reference: std::runtime_error / TV_ASSERT_RT_ERR) */
#define SSC_EWORKSPACE (-3)/* workspace too small */
#define SSC_EHIP (-4)      /* a HIP call failed */

#define SSC_MAX_KERNEL_VOLUME 256 /* src/conv/indice_conv.h:44 */

typedef void *ssc_stream_t; /* hipStream_t */

/* Library version (major*10000 + minor*100 + patch). */
int ssc_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char *ssc_last_error(void);

/* Geometry of one sparse convolution / pooling window.
 * Mirrors the argument list of get_indice_pairs_3d
 * (src/ss_conv_ops.cu:31, src/conv/indice_conv.h:21-27). */
typedef struct ssc_geometry {
  int32_t batch_size;
  int32_t out_shape[3];
  int32_t ksize[3];
  int32_t stride[3];
  int32_t padding[3];
  int32_t dilation[3];
  int32_t subm;      /* 1: submanifold (stride forced to 1, padding to ksize/2; indice_conv.h:70-74) */
  int32_t transpose; /* 1: transposed convolution, out = in*stride - padding + k*dilation with
                        out_shape from get_deconv_output_size (geometry.h:82-138, 190-237);
                        ignored when subm is set, as in the reference (indice_conv.h:76-101) */
} ssc_geometry;

/* ------------------------------------------------------------------------
 * Rulebook ("indice pairs").  Replaces getIndicePair<3>
 * (src/conv/indice_conv.h:21-131; GPU kernels src/conv/indice_cuda_functor.cu:23-66,
 * 113-149; CPU algorithm src/conv/geometry.h:18-80,140-189,241-288).
 *
 * Two calls because the number of active outputs is data dependent:
 *   ssc_rulebook_count: marks every reachable output voxel, ranks them and
 *     writes the count to *n_out_host.  SYNCHRONISES `stream` (the reference
 *     learns the same number from torch::_unique, indice_conv.h:120).
 *   ssc_rulebook_emit: writes out_indices[n_out,4] (b,x,y,z) in ascending
 *     order of the flat key ((b*X+x)*Y+y)*Z+z (the order of the reference's GPU
 *     path), pairs[K,2,n_in] (plane 0 input rows, plane 1 output rows, -1
 *     padded) and pair_num[K].  Within one offset the pairs are in ascending
 *     input-row order (the order of the reference's CPU path); the GPU path of
 *     the reference leaves that order to an atomic race.
 * With subm=1 out_indices is not written (outputs are the inputs) and n_out=n_in.
 * The same workspace must be passed, untouched, to both calls.
 * Limits: K = prod(ksize) <= 256; batch_size*prod(out_shape) < 2^31.
 * ---------------------------------------------------------------------- */
size_t ssc_rulebook_workspace_bytes(const ssc_geometry *g, int64_t n_in);

int ssc_rulebook_count(const int32_t *indices /* [n_in,4] device */, int64_t n_in,
                       const ssc_geometry *g, void *workspace, size_t workspace_bytes,
                       int32_t *n_out_host /* host */, ssc_stream_t stream);

/* The same, and *in_order_host = 1 when the input rows come in strictly ascending
 * (b, x, y, z) order (0 otherwise; repeated rows count as disorder).  For such inputs the
 * pairs ssc_rulebook_emit writes ascend, offset by offset, in the output rows as well as
 * in the input rows, which ssc_conv_fwd_f32 can be told (SSC_CONV_PAIRS_CANONICAL); for
 * other inputs only the input rows of an offset ascend.  No counterpart in the reference:
 * it saves the convolution's own order check. */
int ssc_rulebook_count_ordered(const int32_t *indices, int64_t n_in, const ssc_geometry *g,
                               void *workspace, size_t workspace_bytes,
                               int32_t *n_out_host /* host */, int32_t *in_order_host /* host */,
                               ssc_stream_t stream);

int ssc_rulebook_emit(const int32_t *indices, int64_t n_in, const ssc_geometry *g,
                      void *workspace, size_t workspace_bytes,
                      int32_t *out_indices /* [n_out,4] device; may be NULL when subm */,
                      int32_t *pairs /* [K,2,n_in] device */,
                      int32_t *pair_num /* [K] device */, ssc_stream_t stream);

/* The same rulebook with the host's wait moved behind the work that does not depend on the
 * number of outputs (the reference blocks in torch::_unique with the GPU idle,
 * src/conv/indice_conv.h:120):
 *   ssc_rulebook_begin enqueues marking and ranking (the totals land in pinned host memory),
 *     and then pairs[K,2,n_in] and pair_num[K], whose sizes are known beforehand.  With
 *     out_indices it also writes the output rows; the buffer must then hold
 *     ssc_rulebook_out_bound() rows (min(n_in * K, batch_size * prod(out_shape)): room for
 *     any outcome), of which the first n_out are written.  It returns without waiting.
 *   ssc_rulebook_finish, called on the same host thread, waits for the totals only (work
 *     enqueued after ssc_rulebook_begin keeps running) and reports n_out and the input order
 *     as ssc_rulebook_count_ordered does.
 *   ssc_rulebook_rows then writes out_indices[n_out,4] for a caller that did not pass
 *     out_indices to ssc_rulebook_begin (nothing for subm).
 * One rulebook may be between begin and finish per host thread.
 * A row of `indices` whose batch index lies outside [0, batch_size) -- for subm: whose cell
 * lies outside the grid -- is left out of the rulebook and ssc_rulebook_finish (like
 * ssc_rulebook_count) returns SSC_EINVAL; the reference reads and writes outside its grid
 * buffer for such a row (src/conv/indice_cuda_functor.cu:60-61). */
size_t ssc_rulebook_out_bound(const ssc_geometry *g, int64_t n_in);
/* clean_table (may be NULL): device memory of at least ssc_rulebook_clean_table_bytes() bytes
 * that is ALL ZERO when the call's kernels start and that they leave all zero again.  A
 * caller that keeps such a buffer per stream (zeroed once, at least as large as the largest
 * size asked for so far) saves every regular stride-1 rulebook the launch that clears its
 * tables; the size is 0 for geometries that have no use for it.  Calls that share the buffer
 * must not overlap in time, and after a call that failed it must be zeroed again. */
size_t ssc_rulebook_clean_table_bytes(const ssc_geometry *g, int64_t n_in);
int ssc_rulebook_begin(const int32_t *indices, int64_t n_in, const ssc_geometry *g,
                       void *workspace, size_t workspace_bytes,
                       int32_t *pairs /* [K,2,n_in] device */, int32_t *pair_num /* [K] device */,
                       int32_t *out_indices /* [out_capacity,4] device, or NULL */,
                       int64_t out_capacity, void *clean_table, size_t clean_table_bytes,
                       ssc_stream_t stream);
int ssc_rulebook_finish(const ssc_geometry *g, int64_t n_in, int32_t *n_out_host /* host */,
                        int32_t *in_order_host /* host */);
int ssc_rulebook_rows(const ssc_geometry *g, int64_t n_in, void *workspace,
                      size_t workspace_bytes, int32_t *out_indices /* [n_out,4] device */,
                      ssc_stream_t stream);

/* Rulebook and convolution plan of one layer that has no rulebook yet, in one pair of calls --
 * what a layer's forward does between get_indice_pairs and indice_conv
 * (ss_conv/sp_ops/conv.py:131-150, src/conv/indice_conv.h:21-131 then 247-343):
 *   ssc_rulebook_conv_begin is ssc_rulebook_begin, and for a regular convolution (any
 *     stride and dilation; its rulebook counts, on its way, the outputs and the pairs of
 *     every word of its table of cells, for tables of up to 2^25 cells) it also deals the
 *     output rows to the convolution kernel's workgroups, in a launch the rulebook makes
 *     anyway, into the head of `scratch` (ssc_conv_plan_scratch_bytes of
 *     ssc_rulebook_out_bound() rows; may be NULL) -- for a strided layer, whose plan depends
 *     on whether the outputs will outnumber the inputs, once for either case;
 *   ssc_rulebook_conv_finish is ssc_rulebook_finish followed by ssc_conv_plan_build for the
 *     forward direction over the new pairs (pair_stride = n_in), into `plan` and `scratch`
 *     sized for any number of rows from n_out up to the bound; where the rulebook dealt the
 *     rows and the input rows came in key order, the plan needs two to four launches
 *     instead of six or seven.
 * Same host thread for both; one layer between them at a time.  The plan is the one
 * ssc_conv_run_* expects; compared with ssc_conv_plan_build's the ranges begin at other
 * rows, so results agree up to the order of the float sums.
 * `filters` (may be NULL): the arguments of ssc_kernel_combine_packed_f32 for the layer's
 * own filters (c_in and c_out are the call's).  The synthesis depends on nothing the
 * rulebook computes, so it is enqueued inside the rulebook's first launch (more blocks of the
 * kernel that marks the rows' cells; a launch of its own when there are no rows): `out` and
 * `packed` are ready for whatever the stream runs after this call. */
typedef struct ssc_combine_job {
  const float *weight, *basis;
  const int32_t *chan_out, *chan_in, *blocks;
  int32_t n_irreps_in, kernel_volume;
  float *out;   /* [K,c_in,c_out] */
  void *packed; /* ssc_conv_packed_bytes(kernel_volume, c_in, c_out) */
  size_t packed_bytes;
} ssc_combine_job;
int ssc_rulebook_conv_begin(const int32_t *indices, int64_t n_in, const ssc_geometry *g,
                            void *workspace, size_t workspace_bytes,
                            int32_t *pairs /* [K,2,n_in] */, int32_t *pair_num /* [K] */,
                            int32_t *out_indices /* [out_capacity,4] or NULL */,
                            int64_t out_capacity, void *clean_table, size_t clean_table_bytes,
                            int32_t c_in, int32_t c_out, int32_t elem_bytes, void *scratch,
                            size_t scratch_bytes, const ssc_combine_job *filters,
                            ssc_stream_t stream);
int ssc_rulebook_conv_finish(const ssc_geometry *g, int64_t n_in, int32_t *n_out_host /* host */,
                             int32_t *in_order_host /* host */, const int32_t *pairs,
                             const int32_t *pair_num, int32_t c_in, int32_t c_out,
                             int32_t elem_bytes, void *plan, size_t plan_bytes, void *scratch,
                             size_t scratch_bytes, ssc_stream_t stream);

/* ------------------------------------------------------------------------
 * Sparse convolution forward.  Replaces indiceConv<float>
 * (src/conv/indice_conv.h:247-343; bound as indice_conv_fp32,
 * src/ss_conv_ops_api.cpp:21) together with the gather / scatter-add kernels
 * it launches (src/conv/reordering_cuda_functor.cu:23-272):
 *   out[o,:] = sum_k sum_{(i,o) in pairs[k]} features[i,:] * filters[k]
 * as one output-stationary implicit GEMM on fp32 MFMA, offsets accumulated in
 * ascending k.  `filters` is addressed as filters[k*fs_k + ci*fs_ci + co*fs_co]
 * (element strides), so both a contiguous [K,Cin,Cout] kernel and the
 * reference's permuted view of [Cout,Cin,K] (ss_conv/convolution.py:56) work.
 * `inverse` swaps the roles of the two pair planes (indice_conv.h:307,330).
 * `subm`: bit 0 is the reference's flag, accepted for signature parity (the centre
 * offset is treated like any other offset).  Bit 1 (SSC_CONV_PAIRS_CANONICAL) is the
 * caller's promise that, for every offset, the rows that are accumulated into (the
 * output rows; the input rows when `inverse`) ascend strictly -- true of the input rows of
 * every rulebook ssc_rulebook_emit writes, and of the output rows when
 * ssc_rulebook_count_ordered reported ordered input: the order check and the kernels that
 * would re-order the pairs are then not launched.  Without the bit any order is accepted.
 * pair_num stays on the device: no host synchronisation.
 * Every row of out[n_out,Cout] is written (zeros where no pair lands).
 * ---------------------------------------------------------------------- */
#define SSC_CONV_PAIRS_CANONICAL 2

size_t ssc_conv_workspace_bytes(int64_t n_out, int32_t kernel_volume, int32_t c_in,
                                int32_t c_out, int64_t pair_stride);

int ssc_conv_fwd_f32(const float *features /* [n_in,c_in] */, int64_t n_in, int32_t c_in,
                     const float *filters, int64_t fs_k, int64_t fs_ci, int64_t fs_co,
                     int32_t c_out, const int32_t *pairs /* [K,2,pair_stride] */,
                     int64_t pair_stride, const int32_t *pair_num /* [K] device */,
                     int32_t kernel_volume, int32_t inverse, int32_t subm,
                     float *out /* [n_out,c_out] */, int64_t n_out, void *workspace,
                     size_t workspace_bytes, ssc_stream_t stream);

/* Half-precision storage: features, filters and out hold IEEE binary16 elements.  Replaces
 * indiceConv<at::Half> (bound as indice_conv_half, src/ss_conv_ops.cu:74-78,
 * src/ss_conv_ops_api.cpp:23).  Same arguments and workspace as ssc_conv_fwd_f32 (strides
 * in elements).  The arithmetic is that of the fp32 call -- the rows are widened on their
 * way into LDS, products and sums run on fp32 MFMA -- and each output element is rounded
 * to half once (nearest even), where the reference rounds after every offset's GEMM and
 * again in every scatter-add (src/conv/reordering_cuda_functor.cu:158-210). */
int ssc_conv_fwd_f16(const void *features /* [n_in,c_in] half */, int64_t n_in, int32_t c_in,
                     const void *filters /* half */, int64_t fs_k, int64_t fs_ci, int64_t fs_co,
                     int32_t c_out, const int32_t *pairs /* [K,2,pair_stride] */,
                     int64_t pair_stride, const int32_t *pair_num /* [K] device */,
                     int32_t kernel_volume, int32_t inverse, int32_t subm,
                     void *out /* [n_out,c_out] half */, int64_t n_out, void *workspace,
                     size_t workspace_bytes, ssc_stream_t stream);

/* The same convolution in three steps whose results have different lifetimes, for callers
 * that run several convolutions over one rulebook (the reference caches the rulebook under
 * an indice_key, ss_conv/sp_ops/conv.py:124-136, and rebuilds everything else per call;
 * its backward pass walks the same pairs again, src/conv/indice_conv.h:344-426):
 *   ssc_conv_plan_build: the row-block schedule of the kernel (what ssc_conv_fwd_* derives
 *     from the pairs on every call).  The plan stays valid while pairs, pair_num, n_out,
 *     kernel_volume, c_in, c_out, elem_bytes (4: float, 2: half), `inverse` and the number
 *     of feature rows n_in stay the same; `scratch` is needed during the call only.
 *     flags: SSC_CONV_PAIRS_CANONICAL as for ssc_conv_fwd_f32.
 *   ssc_conv_pack_filters_*: the filters in the kernel's fragment order; valid while the
 *     filter values stay the same.
 *   ssc_conv_run_*: the MFMA kernel alone.  Results are bit-identical to ssc_conv_fwd_*.
 * Pairs with one scatter row twice inside an offset are not supported by either form (a
 * rulebook never has them). */
/* Both sizes grow with n_out (and never shrink for a smaller one): buffers sized for an
 * upper bound of n_out serve a plan over any number of rows up to that bound. */
size_t ssc_conv_plan_bytes(int64_t n_out, int32_t kernel_volume, int32_t c_in, int32_t c_out,
                           int64_t pair_stride);
size_t ssc_conv_plan_scratch_bytes(int64_t n_out, int32_t kernel_volume, int32_t c_in,
                                   int32_t c_out, int64_t pair_stride);
size_t ssc_conv_packed_bytes(int32_t kernel_volume, int32_t c_in, int32_t c_out);
int ssc_conv_plan_build(const int32_t *pairs /* [K,2,pair_stride] */, int64_t pair_stride,
                        const int32_t *pair_num /* [K] device */, int32_t kernel_volume,
                        int32_t inverse, int32_t flags, int64_t n_in, int64_t n_out, int32_t c_in,
                        int32_t c_out, int32_t elem_bytes, void *plan, size_t plan_bytes,
                        void *scratch, size_t scratch_bytes, ssc_stream_t stream);
/* How a workgroup's range of `rows` output rows is cut into tiles for a layer of these
 * channel counts (host arithmetic only, no GPU needed; no counterpart in the reference): the
 * range gets *n_tiles tiles, all of *height rows but the last, which has the rest -- more
 * than none and at most *window rows, the height of the accumulator window. */
int ssc_conv_tile_cut(int32_t rows, int32_t c_in, int32_t c_out, int32_t *n_tiles,
                      int32_t *height, int32_t *window);
int ssc_conv_pack_filters_f32(const float *filters, int64_t fs_k, int64_t fs_ci, int64_t fs_co,
                              int32_t kernel_volume, int32_t c_in, int32_t c_out, void *packed,
                              size_t packed_bytes, ssc_stream_t stream);
int ssc_conv_pack_filters_f16(const void *filters, int64_t fs_k, int64_t fs_ci, int64_t fs_co,
                              int32_t kernel_volume, int32_t c_in, int32_t c_out, void *packed,
                              size_t packed_bytes, ssc_stream_t stream);
int ssc_conv_run_f32(const float *features /* [n_in,c_in] */, int64_t n_in, int32_t c_in,
                     const void *packed, size_t packed_bytes, const void *plan, size_t plan_bytes,
                     int64_t pair_stride, int32_t kernel_volume, int32_t c_out,
                     float *out /* [n_out,c_out] */, int64_t n_out, ssc_stream_t stream);
int ssc_conv_run_f16(const void *features /* [n_in,c_in] half */, int64_t n_in, int32_t c_in,
                     const void *packed, size_t packed_bytes, const void *plan, size_t plan_bytes,
                     int64_t pair_stride, int32_t kernel_volume, int32_t c_out,
                     void *out /* [n_out,c_out] half */, int64_t n_out, ssc_stream_t stream);

/* The convolution of ssc_conv_run_f32 with an evaluation-mode batch normalisation and the
 * gated non-linearity applied to every output row before it is stored -- replaces the
 * sequence conv -> bn -> activation of an evaluation-mode block
 * (Common_utils/ss_conv_modules.py:105-117: Convolution.forward, then BatchNorm.forward with
 * running statistics, ss_conv/batchnorm.py:49-136, then Activation._gate,
 * ss_conv/activation.py:55-100) without writing the convolution's own output.
 *
 * The packed filters have c_cols columns (a multiple of 4) in an order of the caller's
 * choice; the tables describe each of them (device memory, c_cols entries):
 *   z = (x - shift[c]) * scale[c] + add[c]          (what ssc_bn_prepare_f32 returns)
 *   mode[c] 0: y = z    1: y = act_scalar(z + pre_bias[c])
 *           2: y = z * act_gate(z_g + pre_bias[g]), g = gate[c]
 *           3: the column is not stored (gates, padding)
 *   y is stored at out[row, dest[c]]; out has c_dest columns.
 * The kernel works on blocks of 64 columns (c / 64).  The gates of a block are one run of at
 * most 16 of its columns, gate_run[2b] the first and gate_run[2b+1] their number for block
 * b (ceil(c_cols / 64) blocks): act_gate is evaluated once per gate and row, and a column of
 * mode 2 must name a gate of its own block's run.  A column whose gate or dest breaks these
 * rules is not stored.
 * Plan and packed filters are those of ssc_conv_plan_build / ssc_conv_pack_filters_f32 for
 * c_out = c_cols.  Refuses a rulebook without pairs (SSC_EINVAL). */
typedef struct ssc_conv_epilogue {
  const float *shift, *scale, *add, *pre_bias;
  const int32_t *mode, *gate, *dest;
  const int32_t *gate_run;
  int32_t act_scalar, act_gate; /* SSC_ACT_* */
  int32_t c_dest;
} ssc_conv_epilogue;

int ssc_conv_run_epilogue_f32(const float *features /* [n_in,c_in] */, int64_t n_in, int32_t c_in,
                              const void *packed, size_t packed_bytes, const void *plan,
                              size_t plan_bytes, int64_t pair_stride, int32_t kernel_volume,
                              int32_t c_cols, const ssc_conv_epilogue *epilogue,
                              float *out /* [n_out,c_dest] */, int64_t n_out,
                              ssc_stream_t stream);
/* The same on half-precision rows (features, packed filters of ssc_conv_pack_filters_f16,
 * plan built with elem_bytes 2, out: half): the sums and the epilogue's arithmetic in fp32,
 * the tables float32 as above, one rounding per stored element. */
int ssc_conv_run_epilogue_f16(const void *features /* [n_in,c_in] half */, int64_t n_in,
                              int32_t c_in, const void *packed, size_t packed_bytes,
                              const void *plan, size_t plan_bytes, int64_t pair_stride,
                              int32_t kernel_volume, int32_t c_cols,
                              const ssc_conv_epilogue *epilogue,
                              void *out /* [n_out,c_dest] half */, int64_t n_out,
                              ssc_stream_t stream);

/* ----------------------------------------------------------------------
 * Gradients of the sparse convolution -- replaces indice_conv_backward_fp32
 * (src/ss_conv_ops_api.cpp:22, src/conv/indice_conv.h:344-426).
 *
 * Input gradient: no entry point of its own.  It is ssc_conv_fwd_f32 applied to
 * out_grad with `inverse` flipped, c_in and c_out exchanged and the filter strides
 * fs_ci and fs_co exchanged (input_grad[i] = sum_k out_grad[o] * W[k]^T over the same
 * pairs).
 *
 * ssc_conv_bwd_filter_f32: filters_grad[k][ci][co] = sum over the pairs (i, o) of
 *   offset k of features[i][ci] * out_grad[o][co], written with the element strides
 *   gs_k, gs_ci, gs_co (every element is written; no atomics; the summation order is
 *   fixed, so two runs give identical bits).  `inverse` is the flag of the forward
 *   call.
 * ---------------------------------------------------------------------- */
size_t ssc_conv_bwd_filter_workspace_bytes(int32_t kernel_volume, int32_t c_in, int32_t c_out,
                                           int64_t pair_stride);
int ssc_conv_bwd_filter_f32(const float *features /* [n_in,c_in] */, int64_t n_in, int32_t c_in,
                            const float *out_grad /* [n_out,c_out] */, int64_t n_out,
                            int32_t c_out, const int32_t *pairs /* [K,2,pair_stride] */,
                            int64_t pair_stride, const int32_t *pair_num /* [K] */,
                            int32_t kernel_volume, int32_t inverse, float *filters_grad,
                            int64_t gs_k, int64_t gs_ci, int64_t gs_co, void *workspace,
                            size_t workspace_bytes, ssc_stream_t stream);

/* Half-precision storage (features, out_grad and filters_grad hold IEEE binary16):
 * replaces the filter half of indiceConvBackward<at::Half> (bound as
 * indice_conv_backward_half, src/ss_conv_ops.cu:79-83, src/ss_conv_ops_api.cpp:24).
 * Products and sums in fp32, one rounding per element of filters_grad; same workspace. */
int ssc_conv_bwd_filter_f16(const void *features /* [n_in,c_in] half */, int64_t n_in,
                            int32_t c_in, const void *out_grad /* [n_out,c_out] half */,
                            int64_t n_out, int32_t c_out,
                            const int32_t *pairs /* [K,2,pair_stride] */, int64_t pair_stride,
                            const int32_t *pair_num /* [K] */, int32_t kernel_volume,
                            int32_t inverse, void *filters_grad /* half */, int64_t gs_k,
                            int64_t gs_ci, int64_t gs_co, void *workspace,
                            size_t workspace_bytes, ssc_stream_t stream);

/* Timing of the convolution kernel alone (no counterpart in the reference, whose
 * timers are commented out, src/conv/indice_conv.h:295,319-341).  While enabled,
 * every enable-th convolution call (enable = 1: every call; the events themselves cost a
 * few microseconds of stream time per timed call) records a pair of HIP events on its
 * stream right around the launch of the MFMA kernel (ring of 512 timed calls).
 * ssc_profile_conv_read waits for the recorded calls and returns their
 * durations in milliseconds, oldest first; enabling again clears the ring. */
int ssc_profile_conv(int32_t enable);
/* Measurement knob, no counterpart in the reference; flags (default 1):
 *   1  lets the convolution kernel give every XCD one column block of its own when the
 *      packed filters are larger than an L2 (0: never);
 *   2  no launch of its own for a last group of 16 output columns that would be alone in
 *      its block of 64 (Cout = 72, 136).  This flag changes the sizes ssc_conv_plan_bytes
 *      and its like return: set it before any plan is sized or built and do not mix plans
 *      across a change.  Results agree up to the order of the float sums of that group.
 *   4  the ranges of output rows per column block rounded down to a multiple of 8 (leaves
 *      CUs without a workgroup where the column blocks do not divide them that way; the
 *      default gives every CU one).  Changes the same sizes; results agree up to the order
 *      of the float sums (see 16).
 *   8  no five-group form: float layers of more than 192 input channels whose last group
 *      of 16 output columns would be alone in its block of 64 (Cout = 200, 72 + 64 n)
 *      otherwise run one launch per block of 64 columns, the last of which takes the lone
 *      group along.  Changes the same sizes; results agree up to the order of the float
 *      sums of that group.
 *  16  no second work split: plans of long kernels (an estimated thousand stages or more
 *      per workgroup) otherwise deal the output rows to the workgroups twice, the second
 *      time by the row-block counts the first split came to.  Results agree up to the
 *      order of the float sums (an output row's products are added offset by offset within
 *      a row-block group and chunk by chunk over the groups; which offsets share a group
 *      follows the tiles); every plan by itself is bit-reproducible.
 *  32  the second work split for every plan, whatever its size (for tests).
 *  64  one range of output rows to a workgroup for every plan: plans of middle size (an
 *      estimated 250 row-block groups per workgroup or more, and no second split) otherwise
 *      cut the rows into two ranges per workgroup and give a workgroup two of them by the
 *      groups they came to, many with few.  Changes the sizes; results as for 16.
 * 128  two ranges to a workgroup for every plan (for tests).
 * 256  no kernel of its own for float layers of at most 8 input channels (the first layer of
 *      a network on raw point features), which otherwise compute every output row in
 *      registers from a table of its input rows instead of on the matrix pipeline.  Changes
 *      the sizes; results agree up to the order of the float sums.
 * 512  the schedule filled by a launch of its own for every plan: plans with one range to a
 *      workgroup and a single work split otherwise have it filled range by range by the
 *      launch that counts the ranges' row blocks.  Results are bit-identical (only where in
 *      its buffers a range's part of the schedule lies differs). */
int ssc_conv_tuning(int32_t flags);
/* Tell the library that the caller queues index work (ssc_rulebook_*, ssc_conv_plan_build) on
 * a stream of its own, where it runs while a convolution on another stream holds every CU
 * with nearly all of its LDS (the convolution kernel leaves about 4 KB of a CU's 160 KB):
 * with on != 0 those calls pick kernels that fit into what is left (smaller blocks, two
 * launches for the schedule instead of one) and so run beside the convolution instead of
 * behind it.  Results are the same bit for bit.  A setting of the calling host thread;
 * returns its previous value (default 0). */
int ssc_index_beside_conv(int32_t on);
int ssc_profile_conv_read(float *ms /* host */, int32_t capacity, int32_t *count /* host */);

/* ------------------------------------------------------------------------
 * Steerable kernel synthesis.  Replaces SE3Kernel.combination
 * (ss_conv/utils/kernel.py:267-299: one einsum "uvb,bijxyz->uivjxyz" per pair
 * of irreps, two torch.cat) fused with the permute of
 * ss_conv/convolution.py:56: writes the dense kernel directly as contiguous
 * out[K,c_in,c_out].
 *   chan_out[c_out,3] : (irrep index i, multiplicity index u, component a)
 *   chan_in [c_in ,3] : (irrep index j, multiplicity index v, component b)
 *   blocks[n_i*n_j,6] : (weight offset, basis offset, n_beta, m_in, d_out, d_in),
 *                       n_beta = 0 for an absent block (zeros, kernel.py:287-291)
 *   basis             : all kernel_i_j buffers [n_beta,d_out,d_in,K] concatenated
 * ---------------------------------------------------------------------- */
int ssc_kernel_combine_f32(const float *weight, const float *basis,
                           const int32_t *chan_out, const int32_t *chan_in,
                           const int32_t *blocks, int32_t n_irreps_in,
                           int32_t kernel_volume, int32_t c_in, int32_t c_out,
                           float *out /* [K,c_in,c_out] */, ssc_stream_t stream);

/* The same synthesis with the filters also written in the convolution kernel's packed order
 * (what ssc_conv_pack_filters_f32 makes of `out` read as [K, Cin, Cout]; `packed` of
 * ssc_conv_packed_bytes(kernel_volume, c_in, c_out) bytes): a layer that synthesises its
 * kernel on every training forward (ss_conv/convolution.py:56) saves the packing launch. */
int ssc_kernel_combine_packed_f32(const float *weight, const float *basis,
                                  const int32_t *chan_out, const int32_t *chan_in,
                                  const int32_t *blocks, int32_t n_irreps_in,
                                  int32_t kernel_volume, int32_t c_in, int32_t c_out,
                                  float *out /* [K, c_in, c_out] */, void *packed,
                                  size_t packed_bytes, ssc_stream_t stream);

/* ------------------------------------------------------------------------
 * Rulebook pooling.  Replace indiceMaxPool<float> (src/pool/indice_maxpool.h:15-50,
 * kernels src/pool/indice_maxpool_cuda_functor.cu:22-156), indiceAvgPool<float>
 * (src/pool/indice_avgpool.h:17-52, kernels src/pool/indice_avgpool_cuda_functor.cu:21-171)
 * and indiceSummaryRF (src/ss_conv_ops.cu:116-145, src/pool/indiceSummaryRF.cu:21-36).
 *   max: out[o,c] = max(0, max_{(i,o)} features[i,c])      (output starts at 0, indice_maxpool.h:24)
 *   avg: out[o,c] = sum_{k ascending} features[i_k,c] / (float)summaryrf[o]
 *   rf : rf[o]    = number of pairs that target o
 * One output-stationary launch over all offsets instead of one launch per offset.
 * ---------------------------------------------------------------------- */
size_t ssc_pool_workspace_bytes(int64_t n_out, int32_t kernel_volume);

int ssc_pool_max_f32(const float *features, int32_t channels, const int32_t *pairs,
                     int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                     float *out, int64_t n_out, void *workspace, size_t workspace_bytes,
                     ssc_stream_t stream);

/* ssc_pool_max_f32 for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops with a fixed memory budget, harnesses that forbid hipMalloc).  No
 * counterpart in the reference, whose every pooling call allocates its output and
 * temporaries through torch (src/pool/indice_maxpool.h:24).  Same result, bit for bit; the
 * pair table lives in an array inside the library (SSC_POOL_STATIC_ENTRIES int32 per GPU,
 * held until the process ends) instead of a workspace, so the call -- the look-up of that
 * array's address on the first call per device aside, which a caller under graph capture
 * makes beforehand with n_out = 0 -- only enqueues kernels.  n_out * kernel_volume must
 * not exceed SSC_POOL_STATIC_ENTRIES (SSC_EINVAL otherwise).  All calls on one GPU share the
 * array: calls that overlap in time on one GPU (different streams, different host threads)
 * race; calls on one stream do not. */
#define SSC_POOL_STATIC_ENTRIES (4 << 20) /* 16 MiB */
int ssc_pool_max_static_f32(const float *features, int32_t channels, const int32_t *pairs,
                            int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                            float *out, int64_t n_out, ssc_stream_t stream);

int ssc_pool_avg_f32(const float *features, int32_t channels, const int32_t *pairs,
                     int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                     const int32_t *summaryrf /* [n_out] */, float *out, int64_t n_out,
                     void *workspace, size_t workspace_bytes, ssc_stream_t stream);

int ssc_summary_rf(const int32_t *pairs, int64_t pair_stride, const int32_t *pair_num,
                   int32_t kernel_volume, int32_t *rf /* [n_out] */, int64_t n_out,
                   void *workspace, size_t workspace_bytes, ssc_stream_t stream);

/* Half-precision rulebook pooling -- replaces indice_maxpool_half / indice_avgpool_half
 * (src/ss_conv_ops_api.cpp:29,34: indiceMaxPool<at::Half>, indiceAvgPool<at::Half>) and, further
 * down, their backward passes (src/ss_conv_ops_api.cpp:30,35).  features, out (and the
 * gradients) are IEEE half rows.  Arithmetic as at::Half's operators do it in the reference's
 * kernels: every operation computes in float and rounds to half, so the average is
 * out = half(out + half(in / half(rf))) over the offsets in ascending order; the maximum
 * is exact in any type.  Workspace as for the float entries. */
int ssc_pool_max_f16(const void *features, int32_t channels, const int32_t *pairs,
                     int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                     void *out, int64_t n_out, void *workspace, size_t workspace_bytes,
                     ssc_stream_t stream);
int ssc_pool_avg_f16(const void *features, int32_t channels, const int32_t *pairs,
                     int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                     const int32_t *summaryrf, void *out, int64_t n_out, void *workspace,
                     size_t workspace_bytes, ssc_stream_t stream);

/* Backward of rulebook pooling -- replaces indice_maxpool_backward_fp32 /
 * indice_avgpool_backward_fp32 (src/ss_conv_ops_api.cpp, src/pool/indice_maxpool.h:52-86,
 * src/pool/indice_avgpool.h:54-90).  in_grad [n_in, channels] is written completely:
 *   max: in_grad[i] = sum over the pairs (i, o), offsets ascending, of out_grad[o] where
 *        features[i] == out_features[o] (element-wise);
 *   avg: in_grad[i] = sum over the pairs of out_grad[o] / (float)summaryrf[o].
 * Workspace: ssc_pool_workspace_bytes(n_in, kernel_volume). */
int ssc_pool_max_bwd_f32(const float *features, const float *out_features, const float *out_grad,
                         int32_t channels, const int32_t *pairs, int64_t pair_stride,
                         const int32_t *pair_num, int32_t kernel_volume, float *in_grad,
                         int64_t n_in, void *workspace, size_t workspace_bytes,
                         ssc_stream_t stream);
int ssc_pool_avg_bwd_f32(const float *out_grad, int32_t channels, const int32_t *pairs,
                         int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                         const int32_t *summaryrf, float *in_grad, int64_t n_in, void *workspace,
                         size_t workspace_bytes, ssc_stream_t stream);
/* The same for half rows (indice_maxpool_backward_half / indice_avgpool_backward_half,
 * src/ss_conv_ops_api.cpp:30,35): in_grad = half(in_grad + out_grad) where the input equals
 * the pooled value, half(in_grad + half(out_grad / half(rf))) for the average. */
int ssc_pool_max_bwd_f16(const void *features, const void *out_features, const void *out_grad,
                         int32_t channels, const int32_t *pairs, int64_t pair_stride,
                         const int32_t *pair_num, int32_t kernel_volume, void *in_grad,
                         int64_t n_in, void *workspace, size_t workspace_bytes,
                         ssc_stream_t stream);
int ssc_pool_avg_bwd_f16(const void *out_grad, int32_t channels, const int32_t *pairs,
                         int64_t pair_stride, const int32_t *pair_num, int32_t kernel_volume,
                         const int32_t *summaryrf, void *in_grad, int64_t n_in, void *workspace,
                         size_t workspace_bytes, ssc_stream_t stream);


/* ------------------------------------------------------------------------
 * Segment ("global") pooling over row ranges offsets[s]..offsets[s+1].
 * Replace global_avgpool_fp / global_maxpool_fp (src/pool/global_avgpool.cpp:13-20,
 * src/pool/global_avgpool_cuda_kernel.cu:16-42, src/pool/global_maxpool_cuda_kernel.cu:16-43).
 *   avg: sum of the segment's rows divided by its length (empty segment: 0/0 = NaN)
 *   max: maximum and the row index of its first occurrence (empty: -inf, -1)
 * ---------------------------------------------------------------------- */
int ssc_segment_avg_f32(const float *feats /* [sum_n,c] */, const int32_t *offsets /* [b+1] */,
                        float *out /* [b,c] */, int32_t n_segments, int32_t channels,
                        ssc_stream_t stream);

int ssc_segment_max_f32(const float *feats, const int32_t *offsets, float *out,
                        int32_t *out_idx /* [b,c] */, int32_t n_segments, int32_t channels,
                        ssc_stream_t stream);

/* Backward of the segment pools -- replaces global_avgpool_bp / global_maxpool_bp
 * (src/pool/global_avgpool_cuda_kernel.cu:44-62, global_maxpool_cuda_kernel.cu:45-60).
 * in_grad [n_rows, channels] is written completely (rows outside every segment get 0). */
int ssc_segment_avg_bwd_f32(const float *out_grad /* [n_segments,channels] */,
                            const int32_t *offsets, float *in_grad, int64_t n_rows,
                            int32_t n_segments, int32_t channels, ssc_stream_t stream);
int ssc_segment_max_bwd_f32(const float *out_grad, const int32_t *out_idx /* arg-max rows */,
                            float *in_grad, int64_t n_rows, int32_t n_segments, int32_t channels,
                            ssc_stream_t stream);

/* ------------------------------------------------------------------------
 * Point <-> voxel.
 * ssc_voxel_coords: voxel index of each point, (int)((p + half) / unit) in fp32
 *   with IEEE division and truncation (ss_conv/sp_ops/voxelize.py:85-86).
 * ssc_unique_*: sorted unique rows of an int32 [n,4] (b,x,y,z) table with the
 *   inverse map and counts; stands in for torch.unique(dim=0, return_inverse,
 *   return_counts) at voxelize.py:88.  count SYNCHRONISES `stream`.
 *   Coordinates must satisfy 0 <= b < dims[0], 0 <= x < dims[1], ... (a row that does
 *   not is left out and the counting call returns SSC_EINVAL) and prod(dims) < 2^31.
 * ssc_voxel_map: replaces voxel2point_map (src/voxelize/voxel2point.cpp:12-18,
 *   src/voxelize/voxel2point_cuda_kernel.cu:16-42).  out_maps must be
 *   pre-initialised as the reference's caller does (functional.py:344-349).
 *   Modes 3/4 list the points of a voxel in ascending point order (the
 *   reference leaves the order to an atomic race).
 * ssc_voxel_reduce_f32: replaces voxelize_fp (src/voxelize/voxelize_cuda_kernel.h:18-40):
 *   out[v,c] = sum_i mult * feats[map[v,i],c], mult = 1/count in mode 4 else 1.
 *   Every row of out is written.
 * ssc_three_nn / ssc_three_interp_f32: replace three_nn / three_interpolate_fp
 *   (src/voxelize/interpolation.cpp, src/voxelize/interpolate_cuda_kernel.cu:8-121).
 *   Rows are (b,x,y,z) floats; a known row counts only for queries with the
 *   same b; ties keep the lower index; dist2 holds squared distances.
 * ---------------------------------------------------------------------- */
int ssc_voxel_coords(const float *points /* [n,3] */, const int64_t *batch_ids /* [n] */,
                     int64_t n, const float half_extent[3], const float unit[3],
                     int32_t *coords /* [n,4] */, ssc_stream_t stream);

size_t ssc_unique_workspace_bytes(const int32_t dims[4], int64_t n);

int ssc_unique_count(const int32_t *coords /* [n,4] */, int64_t n, const int32_t dims[4],
                     void *workspace, size_t workspace_bytes, int32_t *n_unique_host,
                     ssc_stream_t stream);

int ssc_unique_emit(const int32_t *coords, int64_t n, const int32_t dims[4], void *workspace,
                    size_t workspace_bytes, int64_t n_unique, int32_t *unique /* [m,4] */,
                    int32_t *inverse /* [n] */, int32_t *counts /* [m]; may be NULL */,
                    ssc_stream_t stream);

/* The same result with one wait of the host instead of two or three
 * (ss_conv/sp_ops/voxelize.py:88-93: torch.unique(dim=0, return_inverse, return_counts)
 * followed by the largest count): inverse[n] and counts have sizes known beforehand when
 * counts is given room for n entries (entries beyond the number of distinct rows stay 0),
 * so ssc_unique_build fills both, then SYNCHRONISES `stream` for
 * totals_host[0] = number of distinct rows and totals_host[1] = largest count;
 * ssc_unique_rows then writes unique[m,4] from the same, untouched workspace. */
int ssc_unique_build(const int32_t *coords /* [n,4] */, int64_t n, const int32_t dims[4],
                     void *workspace, size_t workspace_bytes, int32_t *inverse /* [n] */,
                     int32_t *counts /* [n] */, int32_t *totals_host /* [2] host */,
                     ssc_stream_t stream);

int ssc_unique_rows(const int32_t dims[4], int64_t n, void *workspace, size_t workspace_bytes,
                    int32_t *unique /* [m,4] */, ssc_stream_t stream);

/* Point filter and batch partition of Point2Voxel.forward
 * (ss_conv/sp_ops/voxelize.py:40-83: drop the points outside the grid, give every batch
 * element left without points one zero point, order by batch id), for batch ids that
 * are non-decreasing and lie in [0, SSC_P2V_MAX_IDS): a stream compaction instead of
 * torch.unique / boolean indexing / torch.sort.
 * ssc_p2v_scan marks the surviving points and counts them per id; it SYNCHRONISES
 *   `stream` and fills three host arrays: hist_all[id] = points with that id,
 *   hist_valid[id] = survivors with that id, flags = {an id is out of range, ids
 *   decrease somewhere}.  With a flag set the caller must take another path.
 * ssc_p2v_compact (same workspace, untouched in between) writes the m = sum(hist_valid)
 *   + #{id: hist_all > 0, hist_valid == 0} rows of the result: points [m,3], features
 *   [m,channels], ids [m], and the voxel coordinates (b, vx, vy, vz) of every row as
 *   ssc_voxel_coords computes them; out_dest [n] (may be NULL) receives the output row of
 *   every input row, -1 for a dropped one (what a caller needs to send gradients of the
 *   output features back to the input features). */
#define SSC_P2V_MAX_IDS 4096
size_t ssc_p2v_workspace_bytes(int64_t n);
int ssc_p2v_scan(const float *points /* [n,3] */, const int64_t *batch_ids /* [n] */, int64_t n,
                 const float half_extent[3], void *workspace, size_t workspace_bytes,
                 int32_t *hist_all_host /* [SSC_P2V_MAX_IDS] */,
                 int32_t *hist_valid_host /* [SSC_P2V_MAX_IDS] */, int32_t *flags_host /* [2] */,
                 ssc_stream_t stream);
int ssc_p2v_compact(const float *points, const float *feats /* [n,channels] */,
                    const int64_t *batch_ids, int64_t n, int32_t channels,
                    const float half_extent[3], const float unit[3], void *workspace,
                    size_t workspace_bytes, float *out_points /* [m,3] */,
                    float *out_feats /* [m,channels] */, int64_t *out_ids /* [m] */,
                    int32_t *out_coords /* [m,4] */, int32_t *out_dest /* [n] or NULL */,
                    ssc_stream_t stream);

/* Point2Voxel.forward (ss_conv/sp_ops/voxelize.py:29-99) as one call, for batch ids that are
 * non-decreasing and lie in [0, n_ids): point filter and batch partition (as ssc_p2v_scan /
 * ssc_p2v_compact), voxel index of every row, sorted unique voxels (torch.unique(dim=0),
 * voxelize.py:88), the voxel of every row, and the per-voxel feature reduction (voxelize_fp,
 * src/voxelize/voxelize_cuda_kernel.h:18-40: mode 1 first point, 2 last point, 3 sum,
 * 4 mean; points of a voxel are added in ascending point order).  All kernels are queued
 * with the data-dependent sizes kept on the device and every output sized for n rows
 * (there are never more rows or voxels than points); the call SYNCHRONISES once, for
 *   totals_host = {rows m, voxels v, flags, batch ids left without points,
 *                  ids present, ids present that kept points, largest id present, 0}
 * and the histograms hist_all_host[n_ids] / hist_valid_host[n_ids] (points and surviving
 * points per id), while its last kernels still run.  The first m rows of out_points [n,3],
 * out_ids [n], inverse [n] (voxel of each row) and the first v rows of out_indices [n,4],
 * out_feats [n,channels], counts [n] (points per voxel), sel [n] (modes 1 and 2: the row a
 * voxel took its features from; may be NULL otherwise) are valid; dest [n] is the output row
 * of every input row (-1: dropped).  flags != 0 (bit 0: an id outside [0, n_ids), bit 1:
 * ids decrease, bit 2: a voxel outside the grid): the outputs must be discarded and another
 * path taken.  The unique-rows table spans n_ids * prod(limit + 1) cells (< 2^31).
 * ssc_p2v_voxelize_bwd_f32: gradient of the features, feats_grad [n,channels] written
 * completely (voxelize_bp, src/voxelize/voxelize_cuda_kernel.h:44-58, through dest /
 * inverse instead of the point lists). */
size_t ssc_p2v_voxelize_workspace_bytes(int64_t n, int32_t n_ids, const int32_t limit[3]);
int ssc_p2v_voxelize_f32(const float *points /* [n,3] */, const float *feats /* [n,channels] */,
                         const int64_t *batch_ids /* [n] */, int64_t n, int32_t channels,
                         const float half_extent[3], const float unit[3], const int32_t limit[3],
                         int32_t n_ids, int32_t mode, void *workspace, size_t workspace_bytes,
                         float *out_points, int64_t *out_ids, int32_t *out_indices,
                         float *out_feats, int32_t *inverse, int32_t *counts, int32_t *dest,
                         int32_t *sel, int32_t *hist_all_host /* [n_ids] host */,
                         int32_t *hist_valid_host /* [n_ids] host */,
                         int32_t *totals_host /* [8] host */, ssc_stream_t stream);
int ssc_p2v_voxelize_bwd_f32(const float *out_grad /* [v,channels] */, int32_t channels,
                             const int32_t *dest /* [n] */, const int32_t *inverse,
                             const int32_t *counts, const int32_t *sel, int32_t mode, int64_t n,
                             float *feats_grad /* [n,channels] */, ssc_stream_t stream);

int ssc_voxel_map(const int32_t *inverse /* [n] */, const int32_t *ids /* [n] */,
                  int32_t *out_maps /* [m,max_active+1] */, int32_t n_point, int32_t n_voxel,
                  int32_t max_active, int32_t mode, ssc_stream_t stream);

int ssc_voxel_reduce_f32(const float *feats /* [n,c] */, float *out /* [m,c] */,
                         const int32_t *maps /* [m,max_active+1] */, int32_t mode,
                         int32_t n_voxel, int32_t max_active, int32_t channels,
                         ssc_stream_t stream);

int ssc_three_nn(int32_t n, int32_t m, const float *unknown /* [n,4] */,
                 const float *known /* [m,4] */, float *dist2 /* [n,3] */,
                 int32_t *idx /* [n,3] */, ssc_stream_t stream);

/* The same search with a small workspace for the batch range of every 256 known rows:
 * blocks of queries then skip the known rows of other batch elements without loading
 * them (known rows grouped by batch element, as Voxel2Point passes them, are scanned
 * once per batch element instead of once per block).  Results are identical. */
size_t ssc_three_nn_workspace_bytes(int32_t m);
int ssc_three_nn_ws(int32_t n, int32_t m, const float *unknown, const float *known, float *dist2,
                    int32_t *idx, void *workspace, size_t workspace_bytes, ssc_stream_t stream);

/* The same search when the known rows are voxel centres: known[j] is the centre of voxel
 * voxel_indices[j] = (b, x, y, z) of a grid of dims[3] cells per batch element, i.e.
 * known[j] = (b, origin + (xyz + 0.5) * unit) up to rounding (what Voxel2Point computes,
 * ss_conv/sp_ops/voxelize.py:131-140).  The neighbours are looked up around the query's own
 * cell through an occupancy bit table instead of among all m rows; distances, indices and
 * ties are those of ssc_three_nn.  The voxel rows must be distinct.  A query far from every
 * voxel is scanned against all rows; many such queries, a query with a batch value outside
 * 0 .. batch_size-1 or a voxel row outside the grid make the call fall back to the plain
 * scan by itself. */
size_t ssc_three_nn_grid_workspace_bytes(int32_t n, int32_t m, int32_t batch_size,
                                         const int32_t dims[3]);
int ssc_three_nn_grid(int32_t n, int32_t m, const float *unknown /* [n,4] */,
                      const float *known /* [m,4] */, const int32_t *voxel_indices /* [m,4] */,
                      int32_t batch_size, const int32_t dims[3], const float origin[3],
                      const float unit[3], float *dist2 /* [n,3] */, int32_t *idx /* [n,3] */,
                      void *workspace, size_t workspace_bytes, ssc_stream_t stream);

/* Voxel2Point.forward with points (ss_conv/sp_ops/voxelize.py:131-160) as one call: the
 * voxel centres ((index * unit - 0.5 extent) + 0.5 unit, as the reference rounds them), the
 * three nearest centres of every point among the voxels of its batch element (the search of
 * ssc_three_nn_grid: same indices and ties as ssc_three_nn), the inverse-distance weights
 * 1 / (sqrt(d2) + 1e-8) normalised to sum 1, and the interpolation of ssc_three_interp_f32.
 * points [n,3] with batch_ids [n] (int64); voxel_indices [m,4] (b, x, y, z), distinct, m >= 1;
 * dims: cells per axis of the search grid (at least the largest index + 1).  Returns
 * out [n,channels] and, for the backward pass (ssc_three_interp_bwd_f32), idx [n,3] and
 * weight [n,3]. */
size_t ssc_v2p_workspace_bytes(int32_t n, int32_t m, int32_t batch_size, const int32_t dims[3]);
int ssc_v2p_interpolate_f32(const float *points, const int64_t *batch_ids, int32_t n,
                            const int32_t *voxel_indices, const float *voxel_feats, int32_t m,
                            int32_t channels, int32_t batch_size, const int32_t dims[3],
                            const float unit[3], const float extent[3], float *out, int32_t *idx,
                            float *weight, void *workspace, size_t workspace_bytes,
                            ssc_stream_t stream);

int ssc_three_interp_f32(int32_t c, int32_t m, int32_t n, const float *feats /* [m,c] */,
                         const int32_t *idx /* [n,3] */, const float *weight /* [n,3] */,
                         float *out /* [n,c] */, ssc_stream_t stream);

/* Backward of the two operators above -- replace voxelize_bp
 * (src/voxelize/voxelize_cuda_kernel.h:44-58) and three_interpolate_bp
 * (src/voxelize/interpolate_cuda_kernel.cu:104-121).  Both write their gradient
 * completely.  The interpolation gradient accumulates with float atomics (several
 * queries share a row), as the reference does: its last bits depend on the order. */
int ssc_voxel_reduce_bwd_f32(const float *out_grad /* [m,c] */, float *feats_grad /* [n,c] */,
                             const int32_t *maps, int32_t mode, int32_t n_voxel,
                             int32_t max_active, int32_t channels, int64_t n_point,
                             ssc_stream_t stream);
int ssc_three_interp_bwd_f32(int32_t c, int32_t n, int32_t m, const float *out_grad /* [n,c] */,
                             const int32_t *idx, const float *weight,
                             float *points_grad /* [m,c] */, ssc_stream_t stream);

/* ------------------------------------------------------------------------
 * SE(3) batch normalisation and gated non-linearity over feature rows [n, c_in].
 * Replace the torch code of BatchNorm.forward (ss_conv/batchnorm.py:49-136) and
 * Activation._gate (ss_conv/activation.py:55-100) and their autograd.
 *
 * Channel layout, described once per layer by int32 tables on the device:
 *   field_of[c]     field (block of 2l+1 columns) of input column c
 *   scalar_idx[c]   ordinal of column c among the scalar (l = 0) columns, -1 otherwise
 *   field_first[f], field_dim[f]   first column and number of columns of field f
 *   out_mode[j]     for output column j < c_out: 0 copy, 1 scalar activation,
 *                   2 multiplied by the activation of its gate (NULL: all 0)
 *   gate_col[j]     input column of the gate of output column j (read when mode 2)
 *   gated_first[c], gated_dim[c]   for a gate column c >= c_out: the output columns
 *                   it gates (dim 0 or NULL: none)
 *
 * ssc_bn_prepare_f32 turns statistics into per-column constants:
 *   training != 0: shift = column mean for scalar columns (0 elsewhere); norm of a
 *     field = mean over rows of the sum of its (x - shift)^2; running_mean /
 *     running_var move by `momentum` towards them (batchnorm.py:73-100)
 *   training == 0: shift and norm are the running statistics
 *   scale[c] = weight[field] / sqrt(norm[field] + eps)   (weight NULL: 1)
 *   add[c]   = bias[scalar_idx[c]] for scalar columns    (bias NULL: 0)
 *   field_rstd[f] = 1 / sqrt(norm[f] + eps)
 * ssc_bnact_fwd_f32: z = (x - shift) * scale + add (a NULL vector is the identity);
 *   y[:, j] = z_j | act_scalar(z_j + pre_bias[j]) | z_j * act_gate(z_g + pre_bias[g]).
 * ssc_bnact_bwd_sums_f32: with dz = dL/dz of every input column (the activation's
 *   chain rule applied to dy), sums[c] = sum over rows of dz, sums[c_in + c] = sum
 *   over rows of dz * (x - shift): what the parameter gradients and the gradient
 *   through the batch statistics need.
 * ssc_bnact_bwd_f32: dx = scale * (dz - dz_mean) - coef * (x - shift)
 *   (dz_mean / coef NULL: 0; the caller derives them from the sums).
 * Sums are accumulated per block of rows and added in block order: reproducible.
 * ---------------------------------------------------------------------- */
#define SSC_ACT_NONE 0
#define SSC_ACT_RELU 1
#define SSC_ACT_SIGMOID 2
#define SSC_ACT_TANH 3

size_t ssc_bn_workspace_bytes(int64_t n, int32_t c);

int ssc_bn_prepare_f32(const float *x /* [n,c] */, int64_t n, int32_t c, const int32_t *field_of,
                       const int32_t *scalar_idx, const int32_t *field_first,
                       const int32_t *field_dim, int32_t n_fields, int32_t training, float eps,
                       float momentum, const float *weight /* [n_fields] or NULL */,
                       const float *bias /* [n_scalar] or NULL */,
                       float *running_mean /* [n_scalar], in/out */,
                       float *running_var /* [n_fields], in/out */, float *shift /* [c] */,
                       float *scale /* [c] */, float *add /* [c] */,
                       float *field_rstd /* [n_fields] */, void *workspace,
                       size_t workspace_bytes, ssc_stream_t stream);

int ssc_bnact_fwd_f32(const float *x /* [n,c_in] */, int64_t n, int32_t c_in, const float *shift,
                      const float *scale, const float *add, const float *pre_bias /* [c_in] */,
                      const int32_t *out_mode /* [c_out] */, const int32_t *gate_col /* [c_out] */,
                      int32_t act_scalar, int32_t act_gate, float *y /* [n,c_out] */,
                      int32_t c_out, ssc_stream_t stream);

int ssc_bnact_bwd_sums_f32(const float *x, const float *dy /* [n,c_out] */, int64_t n,
                           int32_t c_in, int32_t c_out, const float *shift, const float *scale,
                           const float *add, const float *pre_bias, const int32_t *out_mode,
                           const int32_t *gate_col, const int32_t *gated_first /* [c_in] */,
                           const int32_t *gated_dim /* [c_in] */, int32_t act_scalar,
                           int32_t act_gate, float *sums /* [2*c_in] */, void *workspace,
                           size_t workspace_bytes /* ssc_bn_workspace_bytes(n, c_in) */,
                           ssc_stream_t stream);

int ssc_bnact_bwd_f32(const float *x, const float *dy, int64_t n, int32_t c_in, int32_t c_out,
                      const float *shift, const float *scale, const float *add,
                      const float *pre_bias, const int32_t *out_mode, const int32_t *gate_col,
                      const int32_t *gated_first, const int32_t *gated_dim, int32_t act_scalar,
                      int32_t act_gate, const float *dz_mean /* [c_in] or NULL */,
                      const float *coef /* [c_in] or NULL */, float *dx /* [n,c_in] */,
                      ssc_stream_t stream);

/* ------------------------------------------------------------------------
 * One factor per row and field: y[r][c] = x[r][c] * scale[r][field_of[c]].  Replaces the
 * expand / cat / multiply of the per-field dropout (ss_conv/dropout.py:29-46: a field's
 * 2l+1 components share one Bernoulli draw); the draws themselves stay with the caller,
 * so the random stream is the reference's.  The backward pass is the same call on the
 * output gradient.  x and y may be the same buffer.
 * ---------------------------------------------------------------------- */
int ssc_field_scale_f32(const float *x /* [n,c] */, int64_t n, int32_t c,
                        const float *scale /* [n,n_fields] */, int32_t n_fields,
                        const int32_t *field_of /* [c] */, float *y /* [n,c] */,
                        ssc_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SSC_H_ */
