/*
 * ssc_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar, single-thread C restatement of the reference's algorithms for the
 * sparse steerable convolution hot path.  It exists only to check the HIP
 * kernels (tests, the smoke run, and the bench's CPU-baseline leg); the
 * product never links, imports or calls it.
 *
 * Citations are relative to the reference's SS_Conv_lib/ directory.
 * Pinning status of each function is listed in oracle/README.md.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ND 3

/* Candidate outputs of one input voxel, src/conv/geometry.h:18-80.
 * For each dimension the reachable output range is [lo, hi] with
 *   lo = (in - (k-1)*d - 1 + s + p) / s,  hi = (in + p) / s     (C division)
 * and candidates are visited from hi downwards, last dimension fastest.
 * out receives rows of (x, y, z, offset); the return value is the number of
 * candidates that fall inside out_shape.  The offset of a candidate is
 *   sum_dim  m_dim * ((in - out*s + p) / d),  m = (k1*k2, k2, 1). */
static int orc_valid_out_pos(const int *in, const int *ks, const int *st, const int *pd,
                             const int *dl, const int *out_shape, int *out) {
  int lo[ND], hi[ND], cnt[ND];
  for (int a = 0; a < ND; ++a) {
    lo[a] = (in[a] - (ks[a] - 1) * dl[a] - 1 + st[a] + pd[a]) / st[a];
    hi[a] = (in[a] + pd[a]) / st[a];
    cnt[a] = (hi[a] - lo[a]) / dl[a] + 1;
  }
  int n = 0;
  for (int cx = 0; cx < cnt[0]; ++cx)
    for (int cy = 0; cy < cnt[1]; ++cy)
      for (int cz = 0; cz < cnt[2]; ++cz) {
        int c[ND] = {cx, cy, cz};
        int ok = 1, off = 0, m = 1;
        int pos[ND];
        for (int a = ND - 1; a >= 0; --a) {
          pos[a] = hi[a] - c[a] * dl[a];
          if (pos[a] < 0 || pos[a] > out_shape[a] - 1) ok = 0;
          off += m * (in[a] - pos[a] * st[a] + pd[a]) / dl[a];
          m *= ks[a];
        }
        if (ok) {
          out[n * 4 + 0] = pos[0];
          out[n * 4 + 1] = pos[1];
          out[n * 4 + 2] = pos[2];
          out[n * 4 + 3] = off;
          ++n;
        }
      }
  return n;
}

/* getValidOutPosTranspose, src/conv/geometry.h:82-138: the outputs a transposed
 * convolution reaches from `in` are in*s - p + k*d per dimension, visited from the
 * largest downwards, last dimension fastest; the offset of a candidate is its kernel
 * index sum_dim m_dim * ((out - lo) / d), m = (k1*k2, k2, 1). */
static int orc_valid_out_pos_transpose(const int *in, const int *ks, const int *st,
                                       const int *pd, const int *dl, const int *out_shape,
                                       int *out) {
  int lo[ND], hi[ND], cnt[ND];
  for (int a = 0; a < ND; ++a) {
    lo[a] = in[a] * st[a] - pd[a];
    hi[a] = lo[a] + (ks[a] - 1) * dl[a];
    cnt[a] = (hi[a] - lo[a]) / dl[a] + 1;
  }
  int n = 0;
  for (int cx = 0; cx < cnt[0]; ++cx)
    for (int cy = 0; cy < cnt[1]; ++cy)
      for (int cz = 0; cz < cnt[2]; ++cz) {
        int c[ND] = {cx, cy, cz};
        int ok = 1, off = 0, m = 1;
        int pos[ND];
        for (int a = ND - 1; a >= 0; --a) {
          pos[a] = hi[a] - c[a] * dl[a];
          if (pos[a] < 0 || pos[a] > out_shape[a] - 1) ok = 0;
          off += m * (pos[a] - lo[a]) / dl[a];
          m *= ks[a];
        }
        if (ok) {
          out[n * 4 + 0] = pos[0];
          out[n * 4 + 1] = pos[1];
          out[n * 4 + 2] = pos[2];
          out[n * 4 + 3] = off;
          ++n;
        }
      }
  return n;
}

static int64_t orc_flat(const int *pos, const int *shape) {
  /* utils/tensorview.h:457-468 (rowArrayIdx) */
  return ((int64_t)pos[0] * shape[1] + pos[1]) * shape[2] + pos[2];
}

/* Regular sparse conv rulebook, CPU semantics of src/conv/geometry.h:140-189:
 * inputs visited in row order, outputs numbered in first-touch order, pairs of
 * an offset appended in input-row order.
 *   indices[n_in,4] (b,x,y,z); out_indices[cap,4]; pairs[K,2,n_in] pre-filled
 *   with -1 by the caller (indice_conv.h:49); pair_num[K] pre-zeroed.
 * Returns the number of active outputs, or -1 when memory runs out. */
typedef int (*orc_candidates)(const int *, const int *, const int *, const int *, const int *,
                              const int *, int *);
static int orc_rulebook_with(orc_candidates candidates, const int *indices, int n_in, int batch,
                             const int *ks, const int *st, const int *pd, const int *dl,
                             const int *out_shape, int *out_indices, int *pairs, int *pair_num);

int orc_rulebook_conv(const int *indices, int n_in, int batch, const int *ks, const int *st,
                      const int *pd, const int *dl, const int *out_shape, int *out_indices,
                      int *pairs, int *pair_num) {
  return orc_rulebook_with(orc_valid_out_pos, indices, n_in, batch, ks, st, pd, dl, out_shape,
                           out_indices, pairs, pair_num);
}

/* Transposed convolution rulebook, src/conv/geometry.h:190-237: the loop of the regular
 * rulebook over the candidates of getValidOutPosTranspose. */
int orc_rulebook_deconv(const int *indices, int n_in, int batch, const int *ks, const int *st,
                        const int *pd, const int *dl, const int *out_shape, int *out_indices,
                        int *pairs, int *pair_num) {
  return orc_rulebook_with(orc_valid_out_pos_transpose, indices, n_in, batch, ks, st, pd, dl,
                           out_shape, out_indices, pairs, pair_num);
}

static int orc_rulebook_with(orc_candidates candidates, const int *indices, int n_in, int batch,
                             const int *ks, const int *st, const int *pd, const int *dl,
                             const int *out_shape, int *out_indices, int *pairs, int *pair_num) {
  int64_t vol = (int64_t)out_shape[0] * out_shape[1] * out_shape[2];
  int K = ks[0] * ks[1] * ks[2];
  int *grid = (int *)malloc(sizeof(int) * (size_t)(vol * batch));
  int *cand = (int *)malloc(sizeof(int) * (size_t)K * 4);
  if (!grid || !cand) { free(grid); free(cand); return -1; }
  for (int64_t i = 0; i < vol * batch; ++i) grid[i] = -1;
  int n_out = 0;
  for (int j = 0; j < n_in; ++j) {
    int b = indices[j * 4];
    int nc = candidates(indices + j * 4 + 1, ks, st, pd, dl, out_shape, cand);
    for (int c = 0; c < nc; ++c) {
      const int *p = cand + c * 4;
      int off = p[3];
      int64_t cell = orc_flat(p, out_shape) + vol * b;
      if (grid[cell] == -1) {
        out_indices[n_out * 4 + 0] = b;
        out_indices[n_out * 4 + 1] = p[0];
        out_indices[n_out * 4 + 2] = p[1];
        out_indices[n_out * 4 + 3] = p[2];
        grid[cell] = n_out++;
      }
      int slot = pair_num[off]++;
      pairs[((int64_t)off * 2 + 0) * n_in + slot] = j;
      pairs[((int64_t)off * 2 + 1) * n_in + slot] = grid[cell];
    }
  }
  free(grid);
  free(cand);
  return n_out;
}

/* Submanifold rulebook, src/conv/geometry.h:241-288: outputs are the inputs;
 * a pair exists where the candidate position holds an active input. */
int orc_rulebook_subm(const int *indices, int n_in, int batch, const int *ks, const int *st,
                      const int *pd, const int *dl, const int *out_shape, int *pairs,
                      int *pair_num) {
  int64_t vol = (int64_t)out_shape[0] * out_shape[1] * out_shape[2];
  int K = ks[0] * ks[1] * ks[2];
  int *grid = (int *)malloc(sizeof(int) * (size_t)(vol * batch));
  int *cand = (int *)malloc(sizeof(int) * (size_t)K * 4);
  if (!grid || !cand) { free(grid); free(cand); return -1; }
  for (int64_t i = 0; i < vol * batch; ++i) grid[i] = -1;
  for (int j = 0; j < n_in; ++j)
    grid[orc_flat(indices + j * 4 + 1, out_shape) + vol * indices[j * 4]] = j;
  for (int j = 0; j < n_in; ++j) {
    int nc = orc_valid_out_pos(indices + j * 4 + 1, ks, st, pd, dl, out_shape, cand);
    for (int c = 0; c < nc; ++c) {
      const int *p = cand + c * 4;
      int64_t cell = orc_flat(p, out_shape) + vol * indices[j * 4];
      if (grid[cell] > -1) {
        int slot = pair_num[p[3]]++;
        pairs[((int64_t)p[3] * 2 + 0) * n_in + slot] = j;
        pairs[((int64_t)p[3] * 2 + 1) * n_in + slot] = grid[cell];
      }
    }
  }
  free(grid);
  free(cand);
  return n_in;
}

/* Row gather and scatter-add of the CPU conv path,
 * src/conv/reordering_cpp_functor.cpp:15-44. */
void orc_gather_rows(float *buffer, const float *features, const int *rows, int n, int c) {
  for (int i = 0; i < n; ++i)
    memcpy(buffer + (size_t)i * c, features + (size_t)rows[i] * c, sizeof(float) * (size_t)c);
}

void orc_scatter_add_rows(float *out, const float *buffer, const int *rows, int n, int c) {
  for (int i = 0; i < n; ++i) {
    float *o = out + (size_t)rows[i] * c;
    const float *b = buffer + (size_t)i * c;
    for (int j = 0; j < c; ++j) o[j] += b[j];
  }
}

/* Plain fp32 row-major GEMM c[m,n] = a[m,k] * b[k,n], the torch::mm_out of
 * src/conv/indice_conv.h:320 (fp32 accumulation, k ascending). */
void orc_mm_f32(float *c, const float *a, const float *b, int m, int k, int n) {
  for (int i = 0; i < m; ++i) {
    float *ci = c + (size_t)i * n;
    for (int j = 0; j < n; ++j) ci[j] = 0.f;
    for (int p = 0; p < k; ++p) {
      float av = a[(size_t)i * k + p];
      const float *bp = b + (size_t)p * n;
      for (int j = 0; j < n; ++j) ci[j] += av * bp[j];
    }
  }
}

/* Max pool over one offset's pairs, src/pool/indice_maxpool_cpp_functor.cpp:16-35.
 * The caller zero-fills out first (src/pool/indice_maxpool.h:24). */
void orc_maxpool_offset(float *out, const float *in, const int *rows_in, const int *rows_out,
                        int n, int c) {
  for (int r = 0; r < n; ++r) {
    const float *x = in + (size_t)rows_in[r] * c;
    float *y = out + (size_t)rows_out[r] * c;
    for (int j = 0; j < c; ++j)
      if (y[j] < x[j]) y[j] = x[j];
  }
}

/* Avg pool over one offset's pairs: the reference has no CPU body
 * (src/pool/indice_avgpool.h:34-39 returns zeros); this follows the CUDA kernel
 * text src/pool/indice_avgpool_cuda_functor.cu:159-161:
 *   out = out + in / (float)rf[out_row]. */
void orc_avgpool_offset(float *out, const float *in, const int *rows_in, const int *rows_out,
                        int n, int c, const int *rf) {
  for (int r = 0; r < n; ++r) {
    const float *x = in + (size_t)rows_in[r] * c;
    float *y = out + (size_t)rows_out[r] * c;
    float d = (float)rf[rows_out[r]];
    for (int j = 0; j < c; ++j) y[j] = y[j] + x[j] / d;
  }
}

/* Receptive-field count, src/pool/indiceSummaryRF.cu:21-36. */
void orc_summary_rf_offset(int *rf, const int *rows_out, int n) {
  for (int r = 0; r < n; ++r) rf[rows_out[r]] += 1;
}

/* Segment mean, src/pool/global_avgpool_cuda_kernel.cu:16-34: serial fp32 sum
 * from 1e-50f (== 0.0f in fp32) in row order, divided by the length. */
void orc_segment_avg(const float *feats, const int *offsets, float *out, int nseg, int c) {
  for (int s = 0; s < nseg; ++s) {
    int a = offsets[s], b = offsets[s + 1];
    for (int j = 0; j < c; ++j) {
      float acc = (float)1e-50;
      for (int i = a; i < b; ++i) acc += feats[(size_t)i * c + j];
      out[(size_t)s * c + j] = acc / (float)(b - a);
    }
  }
}

/* Segment max + argmax, src/pool/global_maxpool_cuda_kernel.cu:16-35: start at
 * (float)-1e50 == -inf, strict '>' so the first maximum wins. */
void orc_segment_max(const float *feats, const int *offsets, float *out, int *out_idx, int nseg,
                     int c) {
  for (int s = 0; s < nseg; ++s) {
    int a = offsets[s], b = offsets[s + 1];
    for (int j = 0; j < c; ++j) {
      int arg = -1;
      float best = (float)-1e50;
      for (int i = a; i < b; ++i)
        if (feats[(size_t)i * c + j] > best) {
          arg = i;
          best = feats[(size_t)i * c + j];
        }
      out_idx[(size_t)s * c + j] = arg;
      out[(size_t)s * c + j] = best;
    }
  }
}

/* Point list of each voxel, src/voxelize/voxel2point_cuda_kernel.cu:16-37.
 * Points are visited in ascending row order, which fixes the list order the
 * reference leaves to an atomic race (modes 3/4); mode 1 keeps the smallest
 * id, mode 2 the largest.  maps must be pre-initialised by the caller as in
 * ss_conv/sp_ops/functional.py:344-349. */
void orc_voxel_map(const int *inverse, const int *ids, int *maps, int n_point, int max_active,
                   int mode) {
  for (int r = 0; r < n_point; ++r) {
    int *out = maps + (size_t)inverse[r] * (max_active + 1);
    int id = ids[r];
    if (mode == 1) { if (id < out[1]) out[1] = id; out[0] = 1; }
    if (mode == 2) { if (id > out[1]) out[1] = id; out[0] = 1; }
    if (mode == 3 || mode == 4) { int cnt = out[0]++; out[cnt + 1] = id; }
  }
}

/* Per-voxel feature reduction, src/voxelize/voxelize_cuda_kernel.h:18-32:
 * out[v,c] += mult * feats[p,c] in list order, mult = 1/count when averaging. */
void orc_voxel_reduce(const float *feats, float *out, const int *maps, int mode, int n_voxel,
                      int max_active, int c) {
  for (int v = 0; v < n_voxel; ++v) {
    const int *r = maps + (size_t)v * (max_active + 1);
    int na = r[0];
    float mult = (mode == 4 && na > 0) ? (float)1 / (float)na : (float)1;
    float *o = out + (size_t)v * c;
    for (int i = 1; i <= na; ++i) {
      const float *x = feats + (size_t)r[i] * c;
      for (int j = 0; j < c; ++j) {
        float t = mult * x[j];
        o[j] = o[j] + t;
      }
    }
  }
}

/* Brute-force 3 nearest neighbours within the same batch id,
 * src/voxelize/interpolate_cuda_kernel.cu:8-55: fp32 squared distance in the
 * kernel's expression order, double accumulators starting at 1e40, strict '<'
 * (the lowest index wins a tie), indices start at 0. */
void orc_three_nn(int n, int m, const float *unknown, const float *known, float *dist2,
                  int *idx) {
  for (int q = 0; q < n; ++q) {
    float ub = unknown[q * 4], ux = unknown[q * 4 + 1], uy = unknown[q * 4 + 2],
          uz = unknown[q * 4 + 3];
    double b1 = 1e40, b2 = 1e40, b3 = 1e40;
    int i1 = 0, i2 = 0, i3 = 0;
    for (int k = 0; k < m; ++k) {
      if (known[k * 4] != ub) continue;
      float x = known[k * 4 + 1], y = known[k * 4 + 2], z = known[k * 4 + 3];
      float dx = ux - x, dy = uy - y, dz = uz - z;
      float xx = dx * dx, yy = dy * dy, zz = dz * dz;
      float d = (xx + yy) + zz;
      if (d < b1) { b3 = b2; i3 = i2; b2 = b1; i2 = i1; b1 = d; i1 = k; }
      else if (d < b2) { b3 = b2; i3 = i2; b2 = d; i2 = k; }
      else if (d < b3) { b3 = d; i3 = k; }
    }
    dist2[q * 3] = (float)b1; dist2[q * 3 + 1] = (float)b2; dist2[q * 3 + 2] = (float)b3;
    idx[q * 3] = i1; idx[q * 3 + 1] = i2; idx[q * 3 + 2] = i3;
  }
}

/* Weighted sum of three rows, src/voxelize/interpolate_cuda_kernel.cu:79-101. */
void orc_three_interp(int c, int m, int n, const float *feats, const int *idx,
                      const float *weight, float *out) {
  (void)m;
  for (int q = 0; q < n; ++q)
    for (int j = 0; j < c; ++j) {
      float a = weight[q * 3] * feats[(size_t)idx[q * 3] * c + j];
      float b = weight[q * 3 + 1] * feats[(size_t)idx[q * 3 + 1] * c + j];
      float d = weight[q * 3 + 2] * feats[(size_t)idx[q * 3 + 2] * c + j];
      out[(size_t)q * c + j] = (a + b) + d;
    }
}
