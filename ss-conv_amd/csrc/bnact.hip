// SE(3) batch normalisation and gated non-linearity over feature rows [N, C], as
// bandwidth-bound kernels: the statistics take two reads of the features, the
// fused normalise + gate pass one read and one write.
//
// Channel layout (the layout of the reference layers, ss_conv/batchnorm.py:49-136 and
// ss_conv/activation.py:55-100): C_in columns = the fields of Rs (2l+1 columns each)
// followed by one gate scalar per non-scalar field; the output keeps the first C_out
// columns.  Tables describe it once per layer:
//   field_of[c]     field of input column c            scalar_idx[c]  ordinal of c among
//   field_first[f]  first column of field f                           the scalar columns,
//   field_dim[f]    columns of field f                                -1 for the others
//   out_mode[j]     0 copy, 1 scalar activation, 2 multiplied by its gate
//   gate_col[j]     input column of the gate of output column j (mode 2)
//   gated_first[c], gated_dim[c]   for a gate column c: the output columns it gates
//
// Threads run along the columns (coalesced rows), so what belongs to a column sits in
// registers; a block covers a slab of rows and writes one partial sum per column, and
// the partials are added in block order: the same result on every run.
#include "ssc_common.h"

namespace ssc {

constexpr int kBnThreads = 256;
constexpr int kBnMaxBlocks = 1024;      // row slabs of the kernels that leave partial sums
constexpr int kBnMaxApplyBlocks = 4096; // row slabs of the backward apply kernel (no partial sums)
constexpr int kBnMaxBwdChannels = 1536;  // column tables of the backward kernels: 48 KB of LDS

struct BnShape {
  int tx, ty;             // threads along columns / rows (tx * ty == kBnThreads)
  int rows_per_block;
  int blocks;
};

// `c` counts the units a thread handles: columns, or groups of four columns.
static BnShape bn_shape(int64_t n, int c, int max_tx = kBnThreads,
                        int max_blocks = kBnMaxBlocks) {
  BnShape s;
  s.tx = 16;
  while (s.tx < c && s.tx < max_tx) s.tx <<= 1;
  s.ty = kBnThreads / s.tx;
  int64_t rpb = ceil_div(n > 0 ? n : 1, max_blocks);
  rpb = ceil_div(rpb, s.ty) * s.ty;  // whole trips of the row lanes
  if (rpb < 4 * s.ty) rpb = 4 * s.ty;
  s.rows_per_block = (int)rpb;
  s.blocks = (int)ceil_div(n > 0 ? n : 1, rpb);
  return s;
}

// derivative of act_fn at u
__device__ __forceinline__ float act_grad(int kind, float u) {
  switch (kind) {
    case SSC_ACT_RELU: return u > 0.f ? 1.f : 0.f;
    case SSC_ACT_SIGMOID: {
      float s = __builtin_amdgcn_rcpf(1.f + __expf(-u));
      return s * (1.f - s);
    }
    case SSC_ACT_TANH: {
      float t = tanhf(u);
      return 1.f - t * t;
    }
    default: return 1.f;
  }
}

// Sum over the row lanes of a block, in lane order; valid in row lane 0.
__device__ __forceinline__ float reduce_rows(float v, float *red, int tx, int ty, int TX, int TY) {
  red[ty * TX + tx] = v;
  __syncthreads();
  float s = 0.f;
  if (ty == 0)
    for (int i = 0; i < TY; ++i) s += red[i * TX + tx];
  __syncthreads();
  return s;
}

// Kernels that stream the rows come in two widths: V = 4 (a thread owns four
// consecutive columns and moves 16 bytes per access; needs column counts divisible by
// four) and V = 1.
template <int V> struct Vec;
template <> struct Vec<1> {
  float v[1];
  __device__ __forceinline__ void load(const float *p) { v[0] = p[0]; }
  __device__ __forceinline__ void store(float *p) const { p[0] = v[0]; }
};
template <> struct Vec<4> {
  float v[4];
  __device__ __forceinline__ void load(const float *p) {
    float4 t = *reinterpret_cast<const float4 *>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  __device__ __forceinline__ void store(float *p) const {
    *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};

// Statistics of the rows of block b, column by column.
// SQUARE == 0: partial[b*C + c] = sum of x[r,c] and partial_sq[b*C + c] = sum of x[r,c]^2.
// SQUARE == 1: partial_sq[b*C + c] = sum of (x[r,c] - shift[c])^2, for the groups of V
// columns that hold a scalar column (scalar_idx[c] >= 0) only: the other columns are not
// centred (their shift is 0), so the first pass already has their sum of squares, and
// this pass neither reads nor writes them.
template <int SQUARE, int V>
__global__ void __launch_bounds__(kBnThreads)
    bn_partial_kernel(const float *__restrict__ x, int64_t n, int C, int TX, int rows_per_block,
                      const float *__restrict__ shift, const int32_t *__restrict__ scalar_idx,
                      float *__restrict__ partial, float *__restrict__ partial_sq) {
  __shared__ float red[kBnThreads];
  const int TY = kBnThreads / TX;
  const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
  const int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
  for (int c0 = 0; c0 < C; c0 += TX * V) {
    const int c = c0 + tx * V;
    constexpr int U = 4;  // rows in flight per thread
    float acc[U][V], accq[U][V];
    float sh[V];
    bool wanted = c < C;
    if (SQUARE) {
      bool any = false;
#pragma unroll
      for (int i = 0; i < V; ++i) any = any || (c + i < C && scalar_idx[c + i] >= 0);
      wanted = any;
    }
#pragma unroll
    for (int i = 0; i < V; ++i) {
#pragma unroll
      for (int u = 0; u < U; ++u) acc[u][i] = accq[u][i] = 0.f;
      sh[i] = (SQUARE && c + i < C) ? shift[c + i] : 0.f;
    }
    if (wanted) {
      int64_t r = r0 + ty;
      for (; r + (U - 1) * TY < r1; r += U * TY) {
        Vec<V> a[U];
#pragma unroll
        for (int u = 0; u < U; ++u) a[u].load(x + (r + u * TY) * C + c);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int i = 0; i < V; ++i) {
            const float v = a[u].v[i] - sh[i];
            if (!SQUARE) acc[u][i] += v;
            accq[u][i] += v * v;
          }
      }
      for (; r < r1; r += TY) {  // at most U - 1 rows are left
        Vec<V> a;
        a.load(x + r * C + c);
#pragma unroll
        for (int i = 0; i < V; ++i) {
          const float v = a.v[i] - sh[i];
          if (!SQUARE) acc[0][i] += v;
          accq[0][i] += v * v;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < V; ++i) {
      if (!SQUARE) {
        float s = reduce_rows((acc[0][i] + acc[1][i]) + (acc[2][i] + acc[3][i]), red, tx, ty, TX, TY);
        if (ty == 0 && c + i < C) partial[(int64_t)blockIdx.x * C + c + i] = s;
      }
      float q = reduce_rows((accq[0][i] + accq[1][i]) + (accq[2][i] + accq[3][i]), red, tx, ty, TX, TY);
      if (ty == 0 && wanted && c + i < C) partial_sq[(int64_t)blockIdx.x * C + c + i] = q;
    }
  }
}

// out[c] = inv_n * sum over blocks of partial[b*C + c]; with scalar_idx, 0 for the
// columns that are not scalars.  kColsumCols columns x 64 slices of the blocks per
// workgroup (few columns each, for enough workgroups: the sums are a chain of dependent
// loads); a column's slices are added in slice order.
constexpr int kColsumCols = 4;
__global__ void __launch_bounds__(256)
    bn_colsum_kernel(const float *__restrict__ partial, int nb, int C, double inv_n,
                     const int32_t *__restrict__ scalar_idx, float *__restrict__ out) {
  constexpr int kSlices = 256 / kColsumCols;
  __shared__ double red[kSlices][kColsumCols];
  const int cx = threadIdx.x % kColsumCols, part = threadIdx.x / kColsumCols;
  const int c = blockIdx.x * kColsumCols + cx;
  double s = 0.0;
  if (c < C && (scalar_idx == nullptr || scalar_idx[c] >= 0))
    for (int b = part; b < nb; b += kSlices) s += partial[(int64_t)b * C + c];
  red[part][cx] = s;
  __syncthreads();
  if (part == 0 && c < C) {
    double t = 0.0;
    for (int i = 0; i < kSlices; ++i) t += red[i][cx];
    out[c] = (float)(t * inv_n);
  }
}

// One block.  From the column mean squares (training) or the running statistics
// (evaluation): per-column shift / scale / add, per-field 1/sqrt(norm + eps), and the
// running statistics' update (reference: batchnorm.py:73-112).
__global__ void __launch_bounds__(256)
    bn_finalize_kernel(int C, int training, float eps, float momentum,
                       const int32_t *__restrict__ field_of,
                       const int32_t *__restrict__ scalar_idx,
                       const int32_t *__restrict__ field_first,
                       const int32_t *__restrict__ field_dim, int n_fields,
                       const float *__restrict__ weight, const float *__restrict__ bias,
                       float *__restrict__ running_mean, float *__restrict__ running_var,
                       float *__restrict__ shift, float *__restrict__ scale,
                       float *__restrict__ add, float *__restrict__ field_rstd,
                       const float *__restrict__ col_msq /* [C], training only */) {
  if (training) {
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
      const int si = scalar_idx[c];
      if (si >= 0) running_mean[si] = (1.f - momentum) * running_mean[si] + momentum * shift[c];
    }
  } else {
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
      const int si = scalar_idx[c];
      shift[c] = si >= 0 ? running_mean[si] : 0.f;
    }
  }
  __syncthreads();
  for (int f = threadIdx.x; f < n_fields; f += blockDim.x) {
    float norm;
    if (training) {
      norm = 0.f;
      for (int j = 0; j < field_dim[f]; ++j) norm += col_msq[field_first[f] + j];
      running_var[f] = (1.f - momentum) * running_var[f] + momentum * norm;
    } else {
      norm = running_var[f];
    }
    field_rstd[f] = 1.f / sqrtf(norm + eps);
  }
  __syncthreads();
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    const int f = field_of[c];
    scale[c] = field_rstd[f] * (weight ? weight[f] : 1.f);
    const int si = scalar_idx[c];
    add[c] = (bias && si >= 0) ? bias[si] : 0.f;
  }
}

// Per-column constants of the normalisation (identity when the pointers are null).
struct ColAffine {
  const float *shift, *scale, *add, *pre_bias;
  __device__ __forceinline__ float z(float x, int c) const {
    float v = x;
    if (shift) v -= shift[c];
    if (scale) v *= scale[c];
    if (add) v += add[c];
    return v;
  }
  __device__ __forceinline__ float pb(int c) const { return pre_bias ? pre_bias[c] : 0.f; }
};

// y[r, j] = activation of the normalised x[r, j] (see out_mode above)
template <int V>
__global__ void __launch_bounds__(kBnThreads)
    bnact_fwd_kernel(const float *__restrict__ x, int64_t n, int c_in, int c_out, int TX,
                     int rows_per_block, ColAffine aff, const int32_t *__restrict__ out_mode,
                     const int32_t *__restrict__ gate_col, int act_s, int act_g,
                     float *__restrict__ y) {
  const int TY = kBnThreads / TX;
  const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
  const int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
  for (int j = tx * V; j < c_out; j += TX * V) {
    int mode[V], g[V];
    float sh[V], sc[V], ad[V], pbj[V], gsh[V], gsc[V], gad[V];
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const int c = j + i < c_out ? j + i : j;  // V == 4 only with c_out % 4 == 0
      mode[i] = out_mode ? out_mode[c] : 0;
      g[i] = mode[i] == 2 ? gate_col[c] : c;
      sh[i] = aff.shift ? aff.shift[c] : 0.f;
      sc[i] = aff.scale ? aff.scale[c] : 1.f;
      ad[i] = aff.add ? aff.add[c] : 0.f;
      pbj[i] = aff.pb(c);
      gsh[i] = aff.shift ? aff.shift[g[i]] : 0.f;
      gsc[i] = aff.scale ? aff.scale[g[i]] : 1.f;
      gad[i] = (aff.add ? aff.add[g[i]] : 0.f) + aff.pb(g[i]);
    }
    // the next row's loads are in flight while the current row is worked on
    Vec<V> a, an;
    float xg[V], xgn[V];
    auto load_row = [&](int64_t r, Vec<V> &dst, float (&dg)[V]) {
      const float *xr = x + r * c_in;
      dst.load(xr + j);
#pragma unroll
      // the columns of a field share their gate: neighbouring lanes read the same word
      for (int i = 0; i < V; ++i) dg[i] = xr[g[i]];
    };
    int64_t r = r0 + ty;
    if (r < r1) load_row(r, a, xg);
    for (; r < r1; r += TY) {
      load_row(r + TY < r1 ? r + TY : r, an, xgn);  // the last trip reloads its own row
      Vec<V> o;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        float v = (a.v[i] - sh[i]) * sc[i] + ad[i];
        if (mode[i] == 1) {
          v = act_fn(act_s, v + pbj[i]);
        } else if (mode[i] == 2) {
          float gv = (xg[i] - gsh[i]) * gsc[i] + gad[i];
          v *= act_fn(act_g, gv);
        }
        o.v[i] = v;
      }
      o.store(y + r * c_out + j);
      a = an;
#pragma unroll
      for (int i = 0; i < V; ++i) xg[i] = xgn[i];
    }
  }
}

// Per-column constants and tables of the backward kernels, staged in LDS once per block:
// the row loops then read nothing but rows from memory.
struct ColTables {
  float *shift, *scale, *add, *pre;      // [c_in]
  int *mode, *gate, *gfirst, *gdim;      // [c_in] (mode/gate: output columns only)
  __device__ __forceinline__ float z(float x, int c) const {
    return (x - shift[c]) * scale[c] + add[c];
  }
};

__device__ __forceinline__ ColTables stage_tables(float *lds, int c_in, int c_out,
                                                  const ColAffine &aff,
                                                  const int32_t *__restrict__ out_mode,
                                                  const int32_t *__restrict__ gate_col,
                                                  const int32_t *__restrict__ gated_first,
                                                  const int32_t *__restrict__ gated_dim) {
  ColTables t;
  t.shift = lds;
  t.scale = lds + c_in;
  t.add = lds + 2 * c_in;
  t.pre = lds + 3 * c_in;
  t.mode = reinterpret_cast<int *>(lds + 4 * c_in);
  t.gate = t.mode + c_in;
  t.gfirst = t.mode + 2 * c_in;
  t.gdim = t.mode + 3 * c_in;
  for (int c = threadIdx.x; c < c_in; c += blockDim.x) {
    t.shift[c] = aff.shift ? aff.shift[c] : 0.f;
    t.scale[c] = aff.scale ? aff.scale[c] : 1.f;
    t.add[c] = aff.add ? aff.add[c] : 0.f;
    t.pre[c] = aff.pre_bias ? aff.pre_bias[c] : 0.f;
    t.mode[c] = (out_mode && c < c_out) ? out_mode[c] : 0;
    t.gate[c] = (out_mode && c < c_out && out_mode[c] == 2) ? gate_col[c] : c;
    t.gfirst[c] = gated_dim ? gated_first[c] : 0;
    t.gdim[c] = (gated_dim && c >= c_out) ? gated_dim[c] : 0;
  }
  __syncthreads();
  return t;
}

// Gradient reaching the normalised value of input column c at row r (xr, dr: the row
// of x and of dy; xc = xr[c]).
__device__ __forceinline__ float bnact_dz(const float *__restrict__ xr,
                                          const float *__restrict__ dr, float xc, int c, int c_out,
                                          const ColTables &t, int act_s, int act_g) {
  if (c < c_out) {
    const int mode = t.mode[c];
    float d = dr[c];
    if (mode == 1) {
      d *= act_grad(act_s, t.z(xc, c) + t.pre[c]);
    } else if (mode == 2) {
      const int g = t.gate[c];
      d *= act_fn(act_g, t.z(xr[g], g) + t.pre[g]);
    }
    return d;
  }
  const int dim = t.gdim[c];
  if (dim <= 0) return 0.f;
  const int first = t.gfirst[c];
  float acc = 0.f;
  for (int j = first; j < first + dim; ++j) acc += dr[j] * t.z(xr[j], j);
  return acc * act_grad(act_g, t.z(xc, c) + t.pre[c]);
}

// What a thread keeps in registers for its group of V output columns.
template <int V> struct GroupConst {
  int mode[V], g[V];
  float sh[V], sc[V], ad[V], pre[V], gsh[V], gsc[V], gadp[V];
  __device__ __forceinline__ void init(const ColTables &t, int c0) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const int c = c0 + i;
      mode[i] = t.mode[c];
      g[i] = t.gate[c];
      sh[i] = t.shift[c];
      sc[i] = t.scale[c];
      ad[i] = t.add[c];
      pre[i] = t.pre[c];
      gsh[i] = t.shift[g[i]];
      gsc[i] = t.scale[g[i]];
      gadp[i] = t.add[g[i]] + t.pre[g[i]];
    }
  }
  // dz of column i of the group: x and dy of the column, xg the row's value in the
  // column of the gate
  __device__ __forceinline__ float dz(int i, float x, float dy, float xg, int act_s,
                                      int act_g) const {
    if (mode[i] == 1) return dy * act_grad(act_s, (x - sh[i]) * sc[i] + ad[i] + pre[i]);
    if (mode[i] == 2) return dy * act_fn(act_g, (xg - gsh[i]) * gsc[i] + gadp[i]);
    return dy;
  }
};

// One row's worth of a group's inputs: the group's columns of x and dy and the values in
// its gates' columns.  Loaded one row ahead of its use, so that a wave always has the next
// row's loads in flight while it works on the current one.
template <int V> struct GroupRow {
  Vec<V> x, dy;
  float xg[V];
  __device__ __forceinline__ void load(const float *__restrict__ xr, const float *__restrict__ dr,
                                       int c0, const GroupConst<V> &gc) {
    x.load(xr + c0);
    dy.load(dr + c0);
#pragma unroll
    for (int i = 0; i < V; ++i) xg[i] = xr[gc.g[i]];
  }
};

// A gate column's inputs for one row: its own value and, for a field of up to kMaxDim
// columns, the field's x and dy.  Loaded one row ahead like GroupRow.
constexpr int kGateMaxDim = 9;  // fields up to l = 4; wider fields take the plain loop
struct GateRow {
  float xc, xs[kGateMaxDim], ds[kGateMaxDim];
  __device__ __forceinline__ void load(const float *__restrict__ xr, const float *__restrict__ dr,
                                       int c, int first, int dim) {
    xc = xr[c];
#pragma unroll
    for (int j = 0; j < kGateMaxDim; ++j) {
      xs[j] = j < dim ? xr[first + j] : 0.f;
      ds[j] = j < dim ? dr[first + j] : 0.f;
    }
  }
  // dz of the gate column (see bnact_dz)
  __device__ __forceinline__ float dz(const ColTables &t, int c, int first, int dim,
                                      int act_g) const {
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < kGateMaxDim; ++j)
      if (j < dim) acc += ds[j] * t.z(xs[j], first + j);
    return acc * act_grad(act_g, t.z(xc, c) + t.pre[c]);
  }
};

// Work items of the backward kernels: the output columns in groups of V, then the gate
// columns one by one (a gate's gradient sums over its whole field, about as much work
// as a group of plain columns).
// The groups are padded to a multiple of TX items (TX <= 64 threads take one item each per
// pass), so that a pass is all groups or all gate columns: the two kinds run different
// code, and lanes of one wave that disagreed would execute both.
struct BwdItem {
  int c;       // first column
  int width;   // V for a group, 1 for a gate column, 0 for padding and beyond the last item
  bool group;  // a group of output columns (not a gate column)
};
__host__ __device__ __forceinline__ int bwd_groups_padded(int c_out, int V, int TX) {
  return (c_out / V + TX - 1) / TX * TX;
}
template <int V>
__device__ __forceinline__ BwdItem bwd_item(int it, int c_in, int c_out, int TX) {
  const int nvec = c_out / V, nvp = bwd_groups_padded(c_out, V, TX);
  BwdItem w;
  w.group = it < nvec;
  if (it < nvp) {
    w.c = it * V;
    w.width = w.group ? V : 0;
  } else {
    w.c = c_out + (it - nvp);
    w.width = w.c < c_in ? 1 : 0;
  }
  return w;
}
// thread shape of the backward kernels: at most one wave of items per row of threads
static BnShape bwd_shape(int64_t n, int c_out, int V, int max_blocks = kBnMaxBlocks) {
  return bn_shape(n, c_out / V, 64, max_blocks);
}

// partial[b*2C + c] = sum of dz over the rows of block b, partial[b*2C + C + c] = sum of
// dz * (x - shift)
template <int V>
__global__ void __launch_bounds__(kBnThreads)
    bnact_bwd_partial_kernel(const float *__restrict__ x, const float *__restrict__ dy, int64_t n,
                             int c_in, int c_out, int TX, int rows_per_block, ColAffine aff,
                             const int32_t *__restrict__ out_mode,
                             const int32_t *__restrict__ gate_col,
                             const int32_t *__restrict__ gated_first,
                             const int32_t *__restrict__ gated_dim, int act_s, int act_g,
                             float *__restrict__ partial) {
  __shared__ float red[kBnThreads];
  extern __shared__ float lds[];
  const ColTables t =
      stage_tables(lds, c_in, c_out, aff, out_mode, gate_col, gated_first, gated_dim);
  const int TY = kBnThreads / TX;
  const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
  const int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
  const int n_items = bwd_groups_padded(c_out, V, TX) + (c_in - c_out);
  for (int it0 = 0; it0 < n_items; it0 += TX) {
    const BwdItem w = bwd_item<V>(it0 + tx, c_in, c_out, TX);
    float sb[V], sa[V], sh[V];
#pragma unroll
    for (int i = 0; i < V; ++i) {
      sb[i] = sa[i] = 0.f;
      sh[i] = i < w.width ? t.shift[w.c + i] : 0.f;
    }
    if (w.group) {
      GroupConst<V> gc;
      gc.init(t, w.c);
      GroupRow<V> cur, nxt;
      int64_t r = r0 + ty;
      if (r < r1) cur.load(x + r * c_in, dy + r * c_out, w.c, gc);
      for (; r < r1; r += TY) {
        const int64_t rn = r + TY < r1 ? r + TY : r;  // the last trip reloads its own row
        nxt.load(x + rn * c_in, dy + rn * c_out, w.c, gc);
#pragma unroll
        for (int i = 0; i < V; ++i) {
          float d = gc.dz(i, cur.x.v[i], cur.dy.v[i], cur.xg[i], act_s, act_g);
          sb[i] += d;
          sa[i] += d * (cur.x.v[i] - sh[i]);
        }
        cur = nxt;
      }
    } else if (w.width == 1) {
      const int dim = t.gdim[w.c], first = t.gfirst[w.c];
      if (dim > 0 && dim <= kGateMaxDim) {
        GateRow cur, nxt;
        int64_t r = r0 + ty;
        if (r < r1) cur.load(x + r * c_in, dy + r * c_out, w.c, first, dim);
        for (; r < r1; r += TY) {
          const int64_t rn = r + TY < r1 ? r + TY : r;
          nxt.load(x + rn * c_in, dy + rn * c_out, w.c, first, dim);
          float d = cur.dz(t, w.c, first, dim, act_g);
          sb[0] += d;
          sa[0] += d * (cur.xc - sh[0]);
          cur = nxt;
        }
      } else {
        for (int64_t r = r0 + ty; r < r1; r += TY) {
          const float *xr = x + r * c_in;
          const float xc = xr[w.c];
          float d = bnact_dz(xr, dy + r * c_out, xc, w.c, c_out, t, act_s, act_g);
          sb[0] += d;
          sa[0] += d * (xc - sh[0]);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < V; ++i) {
      float tb = reduce_rows(sb[i], red, tx, ty, TX, TY);
      float ta = reduce_rows(sa[i], red, tx, ty, TX, TY);
      if (ty == 0 && i < w.width) {
        partial[(int64_t)blockIdx.x * 2 * c_in + w.c + i] = tb;
        partial[(int64_t)blockIdx.x * 2 * c_in + c_in + w.c + i] = ta;
      }
    }
  }
}

// dx[r,c] = scale[c] * (dz - dz_mean[c]) - coef[c] * (x[r,c] - shift[c])
template <int V>
__global__ void __launch_bounds__(kBnThreads)
    bnact_bwd_kernel(const float *__restrict__ x, const float *__restrict__ dy, int64_t n, int c_in,
                     int c_out, int TX, int rows_per_block, ColAffine aff,
                     const int32_t *__restrict__ out_mode, const int32_t *__restrict__ gate_col,
                     const int32_t *__restrict__ gated_first,
                     const int32_t *__restrict__ gated_dim, int act_s, int act_g,
                     const float *__restrict__ dz_mean, const float *__restrict__ coef,
                     float *__restrict__ dx) {
  extern __shared__ float lds[];
  const ColTables t =
      stage_tables(lds, c_in, c_out, aff, out_mode, gate_col, gated_first, gated_dim);
  const int TY = kBnThreads / TX;
  const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
  const int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
  const int n_items = bwd_groups_padded(c_out, V, TX) + (c_in - c_out);
  for (int it = tx; it < n_items; it += TX) {
    const BwdItem w = bwd_item<V>(it, c_in, c_out, TX);
    float sh[V], sc[V], dm[V], cf[V];
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const int k = i < w.width ? w.c + i : w.c;
      sh[i] = t.shift[k];
      sc[i] = t.scale[k];
      dm[i] = dz_mean ? dz_mean[k] : 0.f;
      cf[i] = coef ? coef[k] : 0.f;
    }
    if (w.group) {
      GroupConst<V> gc;
      gc.init(t, w.c);
      GroupRow<V> cur, nxt;
      int64_t r = r0 + ty;
      if (r < r1) cur.load(x + r * c_in, dy + r * c_out, w.c, gc);
      for (; r < r1; r += TY) {
        const int64_t rn = r + TY < r1 ? r + TY : r;  // the last trip reloads its own row
        nxt.load(x + rn * c_in, dy + rn * c_out, w.c, gc);
        Vec<V> o;
#pragma unroll
        for (int i = 0; i < V; ++i) {
          float d = gc.dz(i, cur.x.v[i], cur.dy.v[i], cur.xg[i], act_s, act_g);
          o.v[i] = sc[i] * (d - dm[i]) - cf[i] * (cur.x.v[i] - sh[i]);
        }
        o.store(dx + r * c_in + w.c);
        cur = nxt;
      }
    } else if (w.width == 1) {
      const int dim = t.gdim[w.c], first = t.gfirst[w.c];
      if (dim > 0 && dim <= kGateMaxDim) {
        GateRow cur, nxt;
        int64_t r = r0 + ty;
        if (r < r1) cur.load(x + r * c_in, dy + r * c_out, w.c, first, dim);
        for (; r < r1; r += TY) {
          const int64_t rn = r + TY < r1 ? r + TY : r;
          nxt.load(x + rn * c_in, dy + rn * c_out, w.c, first, dim);
          float d = cur.dz(t, w.c, first, dim, act_g);
          dx[r * c_in + w.c] = sc[0] * (d - dm[0]) - cf[0] * (cur.xc - sh[0]);
          cur = nxt;
        }
      } else {
        for (int64_t r = r0 + ty; r < r1; r += TY) {
          const float *xr = x + r * c_in;
          const float xc = xr[w.c];
          float d = bnact_dz(xr, dy + r * c_out, xc, w.c, c_out, t, act_s, act_g);
          dx[r * c_in + w.c] = sc[0] * (d - dm[0]) - cf[0] * (xc - sh[0]);
        }
      }
    }
  }
}

// Both backward kernels in the form used when a row fits one pass: TX threads per row,
// thread tx owns the group of V output columns tx*V .. (c_out/V groups) AND the gate
// column c_out + tx (c_in - c_out gates), TX >= both counts.  A gate column's gradient is
// act'(gate) * sum_j dy[j] * z[j] over its field's columns; the threads that own those
// columns have x[j] and dy[j] in registers anyway, so they leave the products in LDS and
// the gate's thread adds them up in ascending column order -- the sum, and its rounding,
// of the plain loop (bnact_dz), without reading the field's columns again.
//   APPLY = false: partial[b*2C + c] = sum of dz over the block's rows,
//                  partial[b*2C + C + c] = sum of dz * (x - shift)
//   APPLY = true:  dx[r,c] = scale[c] * (dz - dz_mean[c]) - coef[c] * (x[r,c] - shift[c])
template <int V, bool APPLY>
__global__ void __launch_bounds__(kBnThreads)
    bnact_bwd_row_kernel(const float *__restrict__ x, const float *__restrict__ dy, int64_t n,
                         int c_in, int c_out, int TX, int rows_per_block, ColAffine aff,
                         const int32_t *__restrict__ out_mode,
                         const int32_t *__restrict__ gate_col,
                         const int32_t *__restrict__ gated_first,
                         const int32_t *__restrict__ gated_dim, int act_s, int act_g,
                         const float *__restrict__ dz_mean, const float *__restrict__ coef,
                         float *__restrict__ dx, float *__restrict__ partial) {
  __shared__ float red[kBnThreads];
  extern __shared__ float lds[];
  const ColTables t =
      stage_tables(lds, c_in, c_out, aff, out_mode, gate_col, gated_first, gated_dim);
  const int TY = kBnThreads / TX;
  float *prod = lds + 8 * c_in;  // [2][TY][c_out]: dy * z of the row's output columns
  const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
  const int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
  const bool has_group = tx < c_out / V;
  const int c0 = has_group ? tx * V : 0;
  const int cg = c_out + tx;  // this thread's gate column
  const bool own_gate_col = cg < c_in;
  const int cgs = own_gate_col ? cg : 0;
  // a gate without a field (dim 0) has dz = 0, as in bnact_dz
  const int gfirst = own_gate_col ? t.gfirst[cgs] : 0, gdim = own_gate_col ? t.gdim[cgs] : 0;
  const float g_sh = t.shift[cgs], g_sc = t.scale[cgs], g_adp = t.add[cgs] + t.pre[cgs];
  GroupConst<V> gc;
  gc.init(t, c0);
  float sh[V], sc[V], dm[V], cf[V], sb[V], sa[V];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    sh[i] = t.shift[c0 + i];
    sc[i] = t.scale[c0 + i];
    dm[i] = (APPLY && dz_mean) ? dz_mean[c0 + i] : 0.f;
    cf[i] = (APPLY && coef) ? coef[c0 + i] : 0.f;
    sb[i] = sa[i] = 0.f;
  }
  const float g_dm = (APPLY && dz_mean) ? dz_mean[cgs] : 0.f;
  const float g_cf = (APPLY && coef) ? coef[cgs] : 0.f;
  float sbg = 0.f, sag = 0.f;
  // rows are taken TY at a time by the whole block (the trip count is the same for every
  // thread: there is a barrier in the loop); a thread's row may lie beyond the slab
  GroupRow<V> cur, nxt;
  float xg_cur = 0.f, xg_nxt = 0.f;
  auto load_row = [&](int64_t r, GroupRow<V> &row, float &xgate) {
    if (has_group) row.load(x + r * c_in, dy + r * c_out, c0, gc);
    if (own_gate_col) xgate = x[r * c_in + cg];
  };
  if (r0 + ty < r1) load_row(r0 + ty, cur, xg_cur);
  int par = 0;
  for (int64_t rb = r0; rb < r1; rb += TY) {
    const int64_t r = rb + ty;
    const bool live = r < r1;
    const int64_t rn = r + TY < r1 ? r + TY : (live ? r : r1 - 1);  // a row that exists
    load_row(rn, nxt, xg_nxt);
    float *prow = prod + ((size_t)par * TY + ty) * c_out;
    if (has_group && live) {
      Vec<V> o;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float xv = cur.x.v[i], dv = cur.dy.v[i];
        prow[c0 + i] = dv * ((xv - sh[i]) * sc[i] + gc.ad[i]);
        const float d = gc.dz(i, xv, dv, cur.xg[i], act_s, act_g);
        if (APPLY) {
          o.v[i] = sc[i] * (d - dm[i]) - cf[i] * (xv - sh[i]);
        } else {
          sb[i] += d;
          sa[i] += d * (xv - sh[i]);
        }
      }
      if (APPLY) o.store(dx + r * c_in + c0);
    }
    __syncthreads();
    if (own_gate_col && live) {
      float acc = 0.f;
      for (int j = 0; j < gdim; ++j) acc += prow[gfirst + j];
      const float d = gdim > 0 ? acc * act_grad(act_g, (xg_cur - g_sh) * g_sc + g_adp) : 0.f;
      if (APPLY) {
        dx[r * c_in + cg] = g_sc * (d - g_dm) - g_cf * (xg_cur - g_sh);
      } else {
        sbg += d;
        sag += d * (xg_cur - g_sh);
      }
    }
    cur = nxt;
    xg_cur = xg_nxt;
    par ^= 1;
  }
  if (!APPLY) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const float tb = reduce_rows(sb[i], red, tx, ty, TX, TY);
      const float ta = reduce_rows(sa[i], red, tx, ty, TX, TY);
      if (ty == 0 && has_group) {
        partial[(int64_t)blockIdx.x * 2 * c_in + c0 + i] = tb;
        partial[(int64_t)blockIdx.x * 2 * c_in + c_in + c0 + i] = ta;
      }
    }
    const float tb = reduce_rows(sbg, red, tx, ty, TX, TY);
    const float ta = reduce_rows(sag, red, tx, ty, TX, TY);
    if (ty == 0 && own_gate_col) {
      partial[(int64_t)blockIdx.x * 2 * c_in + cg] = tb;
      partial[(int64_t)blockIdx.x * 2 * c_in + c_in + cg] = ta;
    }
  }
}

// Thread shape of bnact_bwd_row_kernel, or tx = 0 when a row does not fit one pass.
static BnShape bwd_row_shape(int64_t n, int c_in, int c_out, int V, int max_blocks) {
  const int items = c_out / V > c_in - c_out ? c_out / V : c_in - c_out;
  BnShape s;
  s.tx = 0;
  if (items > kBnThreads) return s;
  return bn_shape(n, items, kBnThreads, max_blocks);
}
static size_t bwd_row_lds(int c_in, int c_out, int tx) {
  return ((size_t)c_in * 8 + 2 * (size_t)(kBnThreads / tx) * c_out) * sizeof(float);
}

// bytes of LDS for the staged column tables
static size_t bn_tables_lds(int c_in) { return (size_t)c_in * 8 * sizeof(float); }

// Partial sums of at most kBnMaxBlocks row slabs (whatever the thread layout), two per
// column, plus one vector of column values.
static size_t bn_ws_bytes(int64_t n, int c) {
  int64_t blocks = n < kBnMaxBlocks ? (n > 0 ? n : 1) : kBnMaxBlocks;
  return align_up((size_t)blocks * 2 * c * sizeof(float)) + align_up((size_t)c * sizeof(float));
}

static bool act_ok(int a) { return a >= SSC_ACT_NONE && a <= SSC_ACT_TANH; }


// y[r][c] = x[r][c] * scale[r][field_of[c]]: one factor per row and field, shared by the
// field's 2l+1 components (the per-field dropout masks, ss_conv/dropout.py:25-46).
// One thread per 4 columns (V = 4) or per column.
typedef float float4v __attribute__((ext_vector_type(4)));
template <int V>
__global__ void __launch_bounds__(256)
    field_scale_kernel(const float *__restrict__ x, int64_t n, int c, const float *__restrict__ scale,
                       int n_fields, const int32_t *__restrict__ field_of, float *__restrict__ y) {
  const int cv = c / V;
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n * cv) return;
  const int64_t r = e / cv;
  const int col = (int)(e - r * cv) * V;
  const float *s = scale + r * n_fields;
  if (V == 4) {
    float4v v = *reinterpret_cast<const float4v *>(x + r * c + col);
    v.x *= s[field_of[col]];
    v.y *= s[field_of[col + 1]];
    v.z *= s[field_of[col + 2]];
    v.w *= s[field_of[col + 3]];
    *reinterpret_cast<float4v *>(y + r * c + col) = v;
  } else {
    y[r * c + col] = x[r * c + col] * s[field_of[col]];
  }
}

}  // namespace ssc

using namespace ssc;

extern "C" {

size_t ssc_bn_workspace_bytes(int64_t n, int32_t c) {
  if (n < 0 || c < 1) return 0;
  return bn_ws_bytes(n, c);
}

int ssc_bn_prepare_f32(const float *x, int64_t n, int32_t c, const int32_t *field_of,
                       const int32_t *scalar_idx, const int32_t *field_first,
                       const int32_t *field_dim, int32_t n_fields, int32_t training, float eps,
                       float momentum, const float *weight, const float *bias,
                       float *running_mean, float *running_var, float *shift, float *scale,
                       float *add, float *field_rstd, void *workspace, size_t workspace_bytes,
                       ssc_stream_t stream) {
  SSC_CHECK(n >= 0 && c >= 1 && n_fields >= 1, SSC_EINVAL, "negative or empty size");
  SSC_CHECK(field_of && scalar_idx && field_first && field_dim && running_var && shift && scale &&
                add && field_rstd && workspace,
            SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(!training || n > 0, SSC_EINVAL, "batch statistics of an empty batch");
  SSC_CHECK(!training || x != nullptr, SSC_EINVAL, "x is NULL");
  size_t need = bn_ws_bytes(n, c);
  SSC_CHECK(workspace_bytes >= need, SSC_EWORKSPACE, "batch-norm workspace too small: %zu < %zu",
            workspace_bytes, need);
  hipStream_t s = (hipStream_t)stream;
  const int V = (c & 3) == 0 ? 4 : 1;
  BnShape sh = bn_shape(n, c / V);
  Carver cv(workspace);
  float *partial = cv.take<float>((size_t)sh.blocks * 2 * c);
  float *partial_sq = partial + (size_t)sh.blocks * c;
  float *col_msq = cv.take<float>((size_t)c);
  const double inv_n = n > 0 ? 1.0 / (double)n : 0.0;
  if (training) {
    // sums and sums of squares in one pass over the rows; the column means (of the scalar
    // columns; 0 elsewhere) go to shift[]; a second pass over the scalar columns replaces
    // their sums of squares by centred ones
    if (V == 4)
      hipLaunchKernelGGL((bn_partial_kernel<0, 4>), dim3(sh.blocks), dim3(kBnThreads), 0, s, x, n,
                         c, sh.tx, sh.rows_per_block, (const float *)nullptr, scalar_idx, partial,
                         partial_sq);
    else
      hipLaunchKernelGGL((bn_partial_kernel<0, 1>), dim3(sh.blocks), dim3(kBnThreads), 0, s, x, n,
                         c, sh.tx, sh.rows_per_block, (const float *)nullptr, scalar_idx, partial,
                         partial_sq);
    hipLaunchKernelGGL(bn_colsum_kernel, dim3((unsigned)ceil_div(c, kColsumCols)), dim3(256), 0, s, partial,
                       sh.blocks, c, inv_n, scalar_idx, shift);
    if (V == 4)
      hipLaunchKernelGGL((bn_partial_kernel<1, 4>), dim3(sh.blocks), dim3(kBnThreads), 0, s, x, n,
                         c, sh.tx, sh.rows_per_block, shift, scalar_idx, partial, partial_sq);
    else
      hipLaunchKernelGGL((bn_partial_kernel<1, 1>), dim3(sh.blocks), dim3(kBnThreads), 0, s, x, n,
                         c, sh.tx, sh.rows_per_block, shift, scalar_idx, partial, partial_sq);
    hipLaunchKernelGGL(bn_colsum_kernel, dim3((unsigned)ceil_div(c, kColsumCols)), dim3(256), 0, s,
                       partial_sq, sh.blocks, c, inv_n, (const int32_t *)nullptr, col_msq);
  }
  hipLaunchKernelGGL(bn_finalize_kernel, dim3(1), dim3(256), 0, s, c, training, eps, momentum,
                     field_of, scalar_idx, field_first, field_dim,
                     n_fields, weight, bias, running_mean, running_var, shift, scale, add,
                     field_rstd, col_msq);
  SSC_LAUNCH_CHECK("bn_prepare");
  return SSC_OK;
}

int ssc_bnact_fwd_f32(const float *x, int64_t n, int32_t c_in, const float *shift,
                      const float *scale, const float *add, const float *pre_bias,
                      const int32_t *out_mode, const int32_t *gate_col, int32_t act_scalar,
                      int32_t act_gate, float *y, int32_t c_out, ssc_stream_t stream) {
  SSC_CHECK(n >= 0 && c_in >= 1 && c_out >= 1 && c_out <= c_in, SSC_EINVAL,
            "bad shape: n %lld, c_in %d, c_out %d", (long long)n, c_in, c_out);
  SSC_CHECK(act_ok(act_scalar) && act_ok(act_gate), SSC_EINVAL, "unknown activation code");
  if (n == 0) return SSC_OK;
  SSC_CHECK(x && y, SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(out_mode == nullptr || gate_col != nullptr, SSC_EINVAL, "gate_col is NULL");
  const int V = ((c_in | c_out) & 3) == 0 ? 4 : 1;
  BnShape sh = bn_shape(n, c_out / V);
  ColAffine aff = {shift, scale, add, pre_bias};
  if (V == 4)
    hipLaunchKernelGGL(bnact_fwd_kernel<4>, dim3(sh.blocks), dim3(kBnThreads), 0,
                       (hipStream_t)stream, x, n, c_in, c_out, sh.tx, sh.rows_per_block, aff,
                       out_mode, gate_col, act_scalar, act_gate, y);
  else
    hipLaunchKernelGGL(bnact_fwd_kernel<1>, dim3(sh.blocks), dim3(kBnThreads), 0,
                       (hipStream_t)stream, x, n, c_in, c_out, sh.tx, sh.rows_per_block, aff,
                       out_mode, gate_col, act_scalar, act_gate, y);
  SSC_LAUNCH_CHECK("bnact_fwd");
  return SSC_OK;
}

int ssc_bnact_bwd_sums_f32(const float *x, const float *dy, int64_t n, int32_t c_in, int32_t c_out,
                           const float *shift, const float *scale, const float *add,
                           const float *pre_bias, const int32_t *out_mode,
                           const int32_t *gate_col, const int32_t *gated_first,
                           const int32_t *gated_dim, int32_t act_scalar, int32_t act_gate,
                           float *sums, void *workspace, size_t workspace_bytes,
                           ssc_stream_t stream) {
  SSC_CHECK(n >= 0 && c_in >= 1 && c_out >= 1 && c_out <= c_in, SSC_EINVAL,
            "bad shape: n %lld, c_in %d, c_out %d", (long long)n, c_in, c_out);
  SSC_CHECK(act_ok(act_scalar) && act_ok(act_gate), SSC_EINVAL, "unknown activation code");
  SSC_CHECK(c_in <= kBnMaxBwdChannels, SSC_EINVAL, "at most %d channels in the backward pass",
            kBnMaxBwdChannels);
  SSC_CHECK(sums && workspace, SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(n == 0 || (x && dy), SSC_EINVAL, "NULL pointer argument");
  size_t need = bn_ws_bytes(n, c_in);
  SSC_CHECK(workspace_bytes >= need, SSC_EWORKSPACE, "batch-norm workspace too small: %zu < %zu",
            workspace_bytes, need);
  hipStream_t s = (hipStream_t)stream;
  if (n == 0) return fill_f32(sums, 2 * (int64_t)c_in, 0.f, s);
  const int V = ((c_in | c_out) & 3) == 0 ? 4 : 1;
  BnShape sh = bwd_shape(n, c_out, V);
  float *partial = static_cast<float *>(workspace);
  ColAffine aff = {shift, scale, add, pre_bias};
  const BnShape rs = bwd_row_shape(n, c_in, c_out, V, kBnMaxBlocks);
  if (rs.tx > 0 && bwd_row_lds(c_in, c_out, rs.tx) <= 64 * 1024) {
    // a row fits one pass: gate gradients from the products the group threads leave in LDS
    const size_t lds_bytes = bwd_row_lds(c_in, c_out, rs.tx);
    if (V == 4)
      hipLaunchKernelGGL((bnact_bwd_row_kernel<4, false>), dim3(rs.blocks), dim3(kBnThreads),
                         lds_bytes, s, x, dy, n, c_in, c_out, rs.tx, rs.rows_per_block, aff,
                         out_mode, gate_col, gated_first, gated_dim, act_scalar, act_gate,
                         (const float *)nullptr, (const float *)nullptr, (float *)nullptr, partial);
    else
      hipLaunchKernelGGL((bnact_bwd_row_kernel<1, false>), dim3(rs.blocks), dim3(kBnThreads),
                         lds_bytes, s, x, dy, n, c_in, c_out, rs.tx, rs.rows_per_block, aff,
                         out_mode, gate_col, gated_first, gated_dim, act_scalar, act_gate,
                         (const float *)nullptr, (const float *)nullptr, (float *)nullptr, partial);
    sh = rs;
  } else if (V == 4)
    hipLaunchKernelGGL(bnact_bwd_partial_kernel<4>, dim3(sh.blocks), dim3(kBnThreads),
                       bn_tables_lds(c_in), s, x, dy,
                       n, c_in, c_out, sh.tx, sh.rows_per_block, aff, out_mode, gate_col,
                       gated_first, gated_dim, act_scalar, act_gate, partial);
  else
    hipLaunchKernelGGL(bnact_bwd_partial_kernel<1>, dim3(sh.blocks), dim3(kBnThreads),
                       bn_tables_lds(c_in), s, x, dy,
                       n, c_in, c_out, sh.tx, sh.rows_per_block, aff, out_mode, gate_col,
                       gated_first, gated_dim, act_scalar, act_gate, partial);
  hipLaunchKernelGGL(bn_colsum_kernel, dim3((unsigned)ceil_div(2 * c_in, kColsumCols)), dim3(256), 0, s,
                     partial, sh.blocks, 2 * c_in, 1.0, (const int32_t *)nullptr, sums);
  SSC_LAUNCH_CHECK("bnact_bwd_sums");
  return SSC_OK;
}

int ssc_bnact_bwd_f32(const float *x, const float *dy, int64_t n, int32_t c_in, int32_t c_out,
                      const float *shift, const float *scale, const float *add,
                      const float *pre_bias, const int32_t *out_mode, const int32_t *gate_col,
                      const int32_t *gated_first, const int32_t *gated_dim, int32_t act_scalar,
                      int32_t act_gate, const float *dz_mean, const float *coef, float *dx,
                      ssc_stream_t stream) {
  SSC_CHECK(n >= 0 && c_in >= 1 && c_out >= 1 && c_out <= c_in, SSC_EINVAL,
            "bad shape: n %lld, c_in %d, c_out %d", (long long)n, c_in, c_out);
  SSC_CHECK(act_ok(act_scalar) && act_ok(act_gate), SSC_EINVAL, "unknown activation code");
  SSC_CHECK(c_in <= kBnMaxBwdChannels, SSC_EINVAL, "at most %d channels in the backward pass",
            kBnMaxBwdChannels);
  if (n == 0) return SSC_OK;
  SSC_CHECK(x && dy && dx, SSC_EINVAL, "NULL pointer argument");
  const int V = ((c_in | c_out) & 3) == 0 ? 4 : 1;
  BnShape sh = bwd_shape(n, c_out, V, kBnMaxApplyBlocks);
  ColAffine aff = {shift, scale, add, pre_bias};
  const BnShape rs = bwd_row_shape(n, c_in, c_out, V, kBnMaxApplyBlocks);
  if (rs.tx > 0 && bwd_row_lds(c_in, c_out, rs.tx) <= 64 * 1024) {
    const size_t lds_bytes = bwd_row_lds(c_in, c_out, rs.tx);
    if (V == 4)
      hipLaunchKernelGGL((bnact_bwd_row_kernel<4, true>), dim3(rs.blocks), dim3(kBnThreads),
                         lds_bytes, (hipStream_t)stream, x, dy, n, c_in, c_out, rs.tx,
                         rs.rows_per_block, aff, out_mode, gate_col, gated_first, gated_dim,
                         act_scalar, act_gate, dz_mean, coef, dx, (float *)nullptr);
    else
      hipLaunchKernelGGL((bnact_bwd_row_kernel<1, true>), dim3(rs.blocks), dim3(kBnThreads),
                         lds_bytes, (hipStream_t)stream, x, dy, n, c_in, c_out, rs.tx,
                         rs.rows_per_block, aff, out_mode, gate_col, gated_first, gated_dim,
                         act_scalar, act_gate, dz_mean, coef, dx, (float *)nullptr);
  } else if (V == 4)
    hipLaunchKernelGGL(bnact_bwd_kernel<4>, dim3(sh.blocks), dim3(kBnThreads),
                       bn_tables_lds(c_in), (hipStream_t)stream, x, dy, n, c_in, c_out, sh.tx, sh.rows_per_block, aff,
                       out_mode, gate_col, gated_first, gated_dim, act_scalar, act_gate, dz_mean,
                       coef, dx);
  else
    hipLaunchKernelGGL(bnact_bwd_kernel<1>, dim3(sh.blocks), dim3(kBnThreads),
                       bn_tables_lds(c_in), (hipStream_t)stream, x, dy, n, c_in, c_out, sh.tx, sh.rows_per_block, aff,
                       out_mode, gate_col, gated_first, gated_dim, act_scalar, act_gate, dz_mean,
                       coef, dx);
  SSC_LAUNCH_CHECK("bnact_bwd");
  return SSC_OK;
}

int ssc_field_scale_f32(const float *x, int64_t n, int32_t c, const float *scale, int32_t n_fields,
                        const int32_t *field_of, float *y, ssc_stream_t stream) {
  SSC_CHECK(n >= 0 && c >= 1 && n_fields >= 1, SSC_EINVAL, "bad shape: n %lld, c %d, fields %d",
            (long long)n, c, n_fields);
  if (n == 0) return SSC_OK;
  SSC_CHECK(x && scale && field_of && y, SSC_EINVAL, "NULL pointer argument");
  const int V = (c & 3) == 0 ? 4 : 1;
  const int64_t items = n * (c / V);
  SSC_CHECK(ceil_div(items, 256) < ((int64_t)1 << 31), SSC_EINVAL, "tensor too large");
  const dim3 grid((unsigned)ceil_div(items, 256));
  if (V == 4)
    hipLaunchKernelGGL(field_scale_kernel<4>, grid, dim3(256), 0, (hipStream_t)stream, x, n, c,
                       scale, n_fields, field_of, y);
  else
    hipLaunchKernelGGL(field_scale_kernel<1>, grid, dim3(256), 0, (hipStream_t)stream, x, n, c,
                       scale, n_fields, field_of, y);
  SSC_LAUNCH_CHECK("field_scale");
  return SSC_OK;
}
}
