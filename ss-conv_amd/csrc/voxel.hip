// Point <-> voxel kernels: voxel coordinates of points, per-voxel point lists,
// per-voxel feature reduction, 3-nearest-neighbour search and interpolation.
#include "ssc_common.h"

#include <type_traits>

// Products and sums below are rounded separately, as the scalar statements of the
// reference are: no fused multiply-add contraction in this file.  (Plain operators
// only: the __fmul_rn / __fadd_rn wrappers are compiled before this pragma and
// would still be fused.)
#pragma clang fp contract(off)

#include <math.h>
#include <string.h>

namespace ssc {

typedef float float4v __attribute__((ext_vector_type(4)));

// (int)((p + half) / unit) per axis: fp32 add, IEEE fp32 divide, truncation.
__global__ void __launch_bounds__(256)
    voxel_coords_kernel(const float *__restrict__ pts, const int64_t *__restrict__ ids, int64_t n,
                        float hx, float hy, float hz, float ux, float uy, float uz,
                        int32_t *__restrict__ coords) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float x = pts[i * 3], y = pts[i * 3 + 1], z = pts[i * 3 + 2];
  int vx = (int)((x + hx) / ux);
  int vy = (int)((y + hy) / uy);
  int vz = (int)((z + hz) / uz);
  reinterpret_cast<int4 *>(coords)[i] = make_int4((int)ids[i], vx, vy, vz);
}

// Point lists.  Modes 3/4: slot by atomic counter (any order), then each list is
// sorted by id so the result does not depend on the race.
__global__ void __launch_bounds__(256)
    voxel_map_kernel(const int32_t *__restrict__ inverse, const int32_t *__restrict__ ids,
                     int32_t *__restrict__ maps, int n_point, int max_active, int mode) {
  int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= n_point) return;
  int32_t *out = maps + (int64_t)inverse[r] * (max_active + 1);
  int id = ids[r];
  if (mode == 1) {
    atomicMin(&out[1], id);
    out[0] = 1;
  } else if (mode == 2) {
    atomicMax(&out[1], id);
    out[0] = 1;
  } else {
    int slot = atomicAdd(&out[0], 1);
    if (slot < max_active) out[slot + 1] = id;
  }
}

__global__ void __launch_bounds__(256)
    voxel_map_sort_kernel(int32_t *__restrict__ maps, int n_voxel, int max_active) {
  int v = blockIdx.x * blockDim.x + threadIdx.x;
  if (v >= n_voxel) return;
  int32_t *row = maps + (int64_t)v * (max_active + 1);
  int n = row[0];
  if (n > max_active) n = max_active;
  for (int i = 2; i <= n; ++i) {  // insertion sort of row[1..n]
    int key = row[i];
    int j = i - 1;
    while (j >= 1 && row[j] > key) {
      row[j + 1] = row[j];
      --j;
    }
    row[j + 1] = key;
  }
}

// out[v,c] = sum over the voxel's list of mult * feats[p,c]; the product is
// rounded before the add, as an atomicAdd of a product is.
__global__ void __launch_bounds__(256)
    voxel_reduce_kernel(const float *__restrict__ feats, float *__restrict__ out,
                        const int32_t *__restrict__ maps, int mode, int64_t n_voxel,
                        int max_active, int C) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n_voxel * C) return;
  int64_t v = idx / C;
  int c = (int)(idx - v * C);
  const int32_t *r = maps + v * (max_active + 1);
  int na = r[0];
  float mult = (mode == 4 && na > 0) ? 1.f / (float)na : 1.f;
  float acc = 0.f;
  for (int i = 1; i <= na; ++i) {
    float t = mult * feats[(int64_t)r[i] * C + c];
    acc = acc + t;
  }
  out[idx] = acc;
}

// Brute-force 3-NN: known rows streamed through LDS in tiles.
// A known row only counts for queries of the same batch element, so a tile none of
// whose rows falls into the batch range of the block's queries is skipped after its
// load; with rows grouped by batch element (the usual case) a block then scans its
// own element's rows only.  The scan order, and with it the tie rule, is unchanged.
// With tile_range (the batch range of every tile, from nn_tile_range_kernel) a tile
// outside the block's range is not even loaded.
constexpr int kNnTile = 256;

// tile_range[2t], tile_range[2t+1] = smallest and largest batch value of known rows
// t*256 .. t*256+255.  One block per tile.
__global__ void __launch_bounds__(kNnTile)
    nn_tile_range_kernel(int m, const float *__restrict__ known, float *__restrict__ tile_range) {
  __shared__ float red[2][kNnTile / 64];
  const int kk = blockIdx.x * kNnTile + threadIdx.x;
  float lo = INFINITY, hi = -INFINITY;
  if (kk < m) lo = hi = known[(int64_t)kk * 4];
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    lo = fminf(lo, __shfl_xor(lo, d, 64));
    hi = fmaxf(hi, __shfl_xor(hi, d, 64));
  }
  if ((threadIdx.x & 63) == 0) {
    red[0][threadIdx.x >> 6] = lo;
    red[1][threadIdx.x >> 6] = hi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kNnTile / 64; ++w) {
      lo = fminf(lo, red[0][w]);
      hi = fmaxf(hi, red[1][w]);
    }
    tile_range[2 * blockIdx.x] = lo;
    tile_range[2 * blockIdx.x + 1] = hi;
  }
}

// Eight lanes per query, each scanning every eighth row of a tile; their three best are
// merged at the end.  Scanning in row order and replacing on strictly smaller distance
// keeps the three smallest (distance, row) pairs in lexicographic order, so the merge
// compares (distance, row) and the result is the sequential scan's, ties included.
constexpr int kNnLanes = 8;

struct Best3 {
  float b1, b2, b3;
  int i1, i2, i3;
  __device__ __forceinline__ void insert(float d, int k) {  // (d, k) after every kept pair it ties
    if (d < b1 || (d == b1 && k < i1)) {
      b3 = b2; i3 = i2; b2 = b1; i2 = i1; b1 = d; i1 = k;
    } else if (d < b2 || (d == b2 && k < i2)) {
      b3 = b2; i3 = i2; b2 = d; i2 = k;
    } else if (d < b3 || (d == b3 && k < i3)) {
      b3 = d; i3 = k;
    }
  }
};

// weight[j] = r_j / ((r_0 + r_1) + r_2) with r_j = 1 / (sqrt(d_j) + 1e-8)
// (ss_conv/sp_ops/voxelize.py:156-159), for kernels that know a query's three distances.
__device__ __forceinline__ void nn_weights(float d1, float d2, float d3, float *__restrict__ w) {
  const float r0 = 1.0f / (sqrtf(d1) + 1e-8f);
  const float r1 = 1.0f / (sqrtf(d2) + 1e-8f);
  const float r2 = 1.0f / (sqrtf(d3) + 1e-8f);
  const float norm = (r0 + r1) + r2;
  w[0] = r0 / norm;
  w[1] = r1 / norm;
  w[2] = r2 / norm;
}

// weight (optional): the interpolation weights of the queries written, beside dist2 / idx.
__global__ void __launch_bounds__(kNnTile)
    three_nn_kernel(int n, int m, const float *__restrict__ unknown,
                    const float *__restrict__ known, const float *__restrict__ tile_range,
                    float *__restrict__ dist2, int32_t *__restrict__ idx,
                    const int32_t *__restrict__ only_if, int only_above,
                    float *__restrict__ weight = nullptr) {
  // (a condition on a device-side counter, the same for every thread of the grid)
  if (only_if && only_if[0] <= only_above) return;
  __shared__ float4v tile[kNnTile];
  __shared__ float red[2][kNnTile / 64];
  const int q = blockIdx.x * (kNnTile / kNnLanes) + threadIdx.x / kNnLanes;
  const int sub = threadIdx.x % kNnLanes;
  float4v u = {0.f, 0.f, 0.f, 0.f};
  if (q < n) u = reinterpret_cast<const float4v *>(unknown)[q];
  // batch range of the block's queries
  float lo = q < n ? u.x : INFINITY, hi = q < n ? u.x : -INFINITY;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    lo = fminf(lo, __shfl_xor(lo, d, 64));
    hi = fmaxf(hi, __shfl_xor(hi, d, 64));
  }
  if ((threadIdx.x & 63) == 0) {
    red[0][threadIdx.x >> 6] = lo;
    red[1][threadIdx.x >> 6] = hi;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kNnTile / 64; ++w) {
    lo = fminf(lo, red[0][w]);
    hi = fmaxf(hi, red[1][w]);
  }
  Best3 best = {INFINITY, INFINITY, INFINITY, 0, 0, 0};
  for (int base = 0; base < m; base += kNnTile) {
    if (tile_range) {  // the same for the whole block
      const int t = base / kNnTile;
      if (tile_range[2 * t] > hi || tile_range[2 * t + 1] < lo) continue;
    }
    int kk = base + threadIdx.x;
    __syncthreads();
    bool hit = false;
    if (kk < m) {
      float4v p = reinterpret_cast<const float4v *>(known)[kk];
      tile[threadIdx.x] = p;
      hit = p.x >= lo && p.x <= hi;
    }
    if (!__syncthreads_or(hit)) continue;
    int cnt = min(kNnTile, m - base);
    for (int t = sub; t < cnt; t += kNnLanes) {
      float4v p = tile[t];
      if (p.x != u.x) continue;
      float dx = u.y - p.y, dy = u.z - p.z, dz = u.w - p.w;
      float xx = dx * dx, yy = dy * dy, zz = dz * dz;
      float d = (xx + yy) + zz;
      int k = base + t;
      // rows come in ascending order within a lane: strictly smaller replaces
      if (d < best.b1) {
        best.b3 = best.b2; best.i3 = best.i2; best.b2 = best.b1; best.i2 = best.i1;
        best.b1 = d; best.i1 = k;
      } else if (d < best.b2) {
        best.b3 = best.b2; best.i3 = best.i2; best.b2 = d; best.i2 = k;
      } else if (d < best.b3) {
        best.b3 = d; best.i3 = k;
      }
    }
  }
  // merge the lanes of a query (a slot that was never filled is (inf, 0) in every lane)
#pragma unroll
  for (int d = 1; d < kNnLanes; d <<= 1) {
    const float o1 = __shfl_xor(best.b1, d, 64), o2 = __shfl_xor(best.b2, d, 64),
                o3 = __shfl_xor(best.b3, d, 64);
    const int j1 = __shfl_xor(best.i1, d, 64), j2 = __shfl_xor(best.i2, d, 64),
              j3 = __shfl_xor(best.i3, d, 64);
    if (o1 < INFINITY) best.insert(o1, j1);
    if (o2 < INFINITY) best.insert(o2, j2);
    if (o3 < INFINITY) best.insert(o3, j3);
  }
  if (q < n && sub == 0) {
    dist2[q * 3] = best.b1; dist2[q * 3 + 1] = best.b2; dist2[q * 3 + 2] = best.b3;
    idx[q * 3] = best.i1; idx[q * 3 + 1] = best.i2; idx[q * 3 + 2] = best.i3;
    if (weight != nullptr) nn_weights(best.b1, best.b2, best.b3, weight + q * 3);
  }
}

// out[q,c] = (w0*f0 + w1*f1) + w2*f2, threads along c for coalesced rows.
__global__ void __launch_bounds__(256)
    three_interp_kernel(int C, int n, const float *__restrict__ feats,
                        const int32_t *__restrict__ idx, const float *__restrict__ weight,
                        float *__restrict__ out) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (int64_t)n * C) return;
  int64_t q = e / C;
  int c = (int)(e - q * C);
  float a = weight[q * 3] * feats[(int64_t)idx[q * 3] * C + c];
  float b = weight[q * 3 + 1] * feats[(int64_t)idx[q * 3 + 1] * C + c];
  float d = weight[q * 3 + 2] * feats[(int64_t)idx[q * 3 + 2] * C + c];
  out[e] = (a + b) + d;
}

}  // namespace ssc

using namespace ssc;

extern "C" {

int ssc_voxel_coords(const float *points, const int64_t *batch_ids, int64_t n,
                     const float half_extent[3], const float unit[3], int32_t *coords,
                     ssc_stream_t stream) {
  SSC_CHECK(n >= 0, SSC_EINVAL, "n is negative");
  if (n == 0) return SSC_OK;
  SSC_CHECK(points && batch_ids && half_extent && unit && coords, SSC_EINVAL,
            "NULL pointer argument");
  hipLaunchKernelGGL(voxel_coords_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0,
                     (hipStream_t)stream, points, batch_ids, n, half_extent[0], half_extent[1],
                     half_extent[2], unit[0], unit[1], unit[2], coords);
  SSC_LAUNCH_CHECK("voxel_coords");
  return SSC_OK;
}

int ssc_voxel_map(const int32_t *inverse, const int32_t *ids, int32_t *out_maps, int32_t n_point,
                  int32_t n_voxel, int32_t max_active, int32_t mode, ssc_stream_t stream) {
  SSC_CHECK(mode >= 1 && mode <= 4, SSC_EINVAL, "mode must be 1..4");
  SSC_CHECK(n_point >= 0 && n_voxel >= 0 && max_active >= 1, SSC_EINVAL, "bad sizes");
  if (n_point == 0) return SSC_OK;
  SSC_CHECK(inverse && ids && out_maps, SSC_EINVAL, "NULL pointer argument");
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(voxel_map_kernel, dim3((unsigned)ceil_div(n_point, 256)), dim3(256), 0, s,
                     inverse, ids, out_maps, n_point, max_active, mode);
  SSC_LAUNCH_CHECK("voxel_map");
  if (mode >= 3 && n_voxel > 0) {
    hipLaunchKernelGGL(voxel_map_sort_kernel, dim3((unsigned)ceil_div(n_voxel, 256)), dim3(256), 0,
                       s, out_maps, n_voxel, max_active);
    SSC_LAUNCH_CHECK("voxel_map_sort");
  }
  return SSC_OK;
}

int ssc_voxel_reduce_f32(const float *feats, float *out, const int32_t *maps, int32_t mode,
                         int32_t n_voxel, int32_t max_active, int32_t channels,
                         ssc_stream_t stream) {
  SSC_CHECK(n_voxel >= 0 && max_active >= 1 && channels >= 1, SSC_EINVAL, "bad sizes");
  if (n_voxel == 0) return SSC_OK;
  SSC_CHECK(feats && out && maps, SSC_EINVAL, "NULL pointer argument");
  int64_t n = (int64_t)n_voxel * channels;
  hipLaunchKernelGGL(voxel_reduce_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0,
                     (hipStream_t)stream, feats, out, maps, mode, (int64_t)n_voxel, max_active,
                     channels);
  SSC_LAUNCH_CHECK("voxel_reduce");
  return SSC_OK;
}

int ssc_three_nn(int32_t n, int32_t m, const float *unknown, const float *known, float *dist2,
                 int32_t *idx, ssc_stream_t stream) {
  SSC_CHECK(n >= 0 && m >= 0, SSC_EINVAL, "bad sizes");
  if (n == 0) return SSC_OK;
  SSC_CHECK(unknown && dist2 && idx && (m == 0 || known), SSC_EINVAL, "NULL pointer argument");
  hipLaunchKernelGGL(three_nn_kernel, dim3((unsigned)ceil_div(n, kNnTile / kNnLanes)), dim3(kNnTile), 0,
                     (hipStream_t)stream, n, m, unknown, known, (const float *)nullptr, dist2, idx,
                     (const int32_t *)nullptr, 0);
  SSC_LAUNCH_CHECK("three_nn");
  return SSC_OK;
}

size_t ssc_three_nn_workspace_bytes(int32_t m) {
  if (m < 0) return 0;
  return align_up((size_t)ceil_div(m > 0 ? m : 1, kNnTile) * 2 * sizeof(float));
}

int ssc_three_nn_ws(int32_t n, int32_t m, const float *unknown, const float *known, float *dist2,
                    int32_t *idx, void *workspace, size_t workspace_bytes, ssc_stream_t stream) {
  SSC_CHECK(n >= 0 && m >= 0, SSC_EINVAL, "bad sizes");
  if (n == 0) return SSC_OK;
  SSC_CHECK(unknown && dist2 && idx && (m == 0 || known), SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(workspace != nullptr && workspace_bytes >= ssc_three_nn_workspace_bytes(m),
            SSC_EWORKSPACE, "three_nn workspace too small");
  float *tile_range = static_cast<float *>(workspace);
  if (m > 0) {
    hipLaunchKernelGGL(nn_tile_range_kernel, dim3((unsigned)ceil_div(m, kNnTile)), dim3(kNnTile), 0,
                       (hipStream_t)stream, m, known, tile_range);
    SSC_LAUNCH_CHECK("nn_tile_range");
  }
  hipLaunchKernelGGL(three_nn_kernel, dim3((unsigned)ceil_div(n, kNnTile / kNnLanes)), dim3(kNnTile), 0,
                     (hipStream_t)stream, n, m, unknown, known, tile_range, dist2, idx,
                     (const int32_t *)nullptr, 0);
  SSC_LAUNCH_CHECK("three_nn");
  return SSC_OK;
}

}  // extern "C"

// ---- 3-NN among voxel centres by grid search ----------------------------------------------
// When the known rows are the centres of voxels whose integer coordinates are at hand, a
// query's neighbours are found around its own cell instead of among all rows: a bit table
// over the cells says which are occupied, the rank of a set bit gives the voxel's row
// (through rank2row, so the rows need not be in key order), and cells are visited in shells
// of growing Chebyshev distance r.  After shell r every cell not yet visited differs from
// the query's cell by more than r in some axis, so its centre is at least `bound` away
// (the distance to the nearest unvisited layer of centres); once the third best distance
// is below that bound the result is final.  Distances are computed from the same operands
// by the same expression as the plain scan and candidates are ranked by (distance, row):
// the result is the plain scan's, ties included.  A query that does not settle within
// kGridNnMaxShell shells (a far-away point, a nearly empty cloud) is put on a list and
// scanned against all rows by a wave of a second kernel; when more than an eighth of the
// queries end up there the plain scan, launched behind with the list's length as its
// condition, redoes the call instead.  The voxel rows must be distinct; a voxel row outside
// the grid, or a query whose batch value is not one of 0 .. batch-1, sends the call to the
// plain scan as well.
namespace ssc {

constexpr int kGridNnMaxShell = 4;

struct GridNn {
  int batch, dim[3];
  float origin[3], unit[3];
};

// The grid as Voxel2Point states it: centre of a voxel = (index * unit - half_extent) +
// half_unit, the three roundings of the reference's expression (voxelize.py:139).
struct V2pGrid {
  float unit[3], half_extent[3], half_unit[3];
};
__device__ __forceinline__ float v2p_centre(int index, const V2pGrid &g, int a) {
  return ((float)index * g.unit[a] - g.half_extent[a]) + g.half_unit[a];
}

__device__ __forceinline__ bool nng_inside(const int4 &r, const GridNn &g) {
  return r.x >= 0 && r.x < g.batch && r.y >= 0 && r.y < g.dim[0] && r.z >= 0 && r.z < g.dim[1] &&
         r.w >= 0 && r.w < g.dim[2];
}

// disorder[0] is set when the rows do not come in strictly ascending key order (for rows in
// that order the rank of a cell is its row).
__global__ void __launch_bounds__(256)
    nng_mark_kernel(const int32_t *__restrict__ coords, int m, GridNn g,
                    uint32_t *__restrict__ bits, int32_t *__restrict__ unsettled,
                    int32_t *__restrict__ disorder) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= m) return;
  const int4 r = reinterpret_cast<const int4 *>(coords)[j];
  if (!nng_inside(r, g)) {  // a voxel the table cannot hold: only the plain scan sees it
    atomicOr(unsettled, 1 << 30);
    return;
  }
  const uint32_t key = (uint32_t)(((r.x * g.dim[0] + r.y) * g.dim[1] + r.z) * g.dim[2] + r.w);
  if (j + 1 < m) {
    const int4 q = reinterpret_cast<const int4 *>(coords)[j + 1];
    const uint32_t next =
        (uint32_t)(((q.x * g.dim[0] + q.y) * g.dim[1] + q.z) * g.dim[2] + q.w);
    if (!nng_inside(q, g) || next <= key) atomicOr(disorder, 1);
  }
  atomicOr(&bits[key >> 5], 1u << (key & 31u));
}

__global__ void __launch_bounds__(256)
    nng_rank2row_kernel(const int32_t *__restrict__ coords, int m, GridNn g,
                        const uint32_t *__restrict__ bits, const int32_t *__restrict__ prefix,
                        int32_t *__restrict__ rank2row, const int32_t *__restrict__ skip_if_ordered) {
  // (rows in key order, and a search that ranks its candidates by cell: nobody reads the map)
  if (skip_if_ordered != nullptr && skip_if_ordered[0] == 0) return;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= m) return;
  const int4 r = reinterpret_cast<const int4 *>(coords)[j];
  if (!nng_inside(r, g)) return;
  const uint32_t key = (uint32_t)(((r.x * g.dim[0] + r.y) * g.dim[1] + r.z) * g.dim[2] + r.w);
  rank2row[bit_rank(bits, prefix, key)] = j;
}

// Eight lanes per query share the columns (x, y) of a shell; their candidates are merged
// after every shell (an all-to-all exchange, so each lane knows the query's three best and
// takes the same decision).  A query that has not settled after the last shell is appended
// to `list`; `counter` counts them (and is forced far above n by nng_mark_kernel or by a
// query with an impossible batch value, which sends the whole call to the plain scan).
constexpr int kGridNnLanes = 8;
constexpr int kGridNnAll = 1 << 30;  // counter value that means "redo every query"

__device__ __forceinline__ void nng_merge_lanes(Best3 &b) {
#pragma unroll
  for (int d = 1; d < kGridNnLanes; d <<= 1) {
    const float o1 = __shfl_xor(b.b1, d, 64), o2 = __shfl_xor(b.b2, d, 64),
                o3 = __shfl_xor(b.b3, d, 64);
    const int j1 = __shfl_xor(b.i1, d, 64), j2 = __shfl_xor(b.i2, d, 64),
              j3 = __shfl_xor(b.i3, d, 64);
    if (o1 < INFINITY) b.insert(o1, j1);
    if (o2 < INFINITY) b.insert(o2, j2);
    if (o3 < INFINITY) b.insert(o3, j3);
  }
}

// CENTRES (Voxel2Point's own call): the known points are the centres of the voxels as vg
// states them, so a candidate's distance comes from its cell -- the same three roundings that
// wrote known[] -- and nothing is loaded for it but the table word that holds its bit; with
// the voxel rows in key order (disorder[0] == 0) a cell's rank is its row, so candidates are
// ranked by (distance, cell) and only a query's three winners are looked up; otherwise a
// candidate's row comes from rank2row as in the other form.  weight (optional) as for
// three_nn_kernel.
template <bool CENTRES>
__global__ void __launch_bounds__(256)
    three_nn_grid_kernel(int n, int m, const float *__restrict__ unknown,
                         const float *__restrict__ known, GridNn g,
                         const uint32_t *__restrict__ bits, const int32_t *__restrict__ prefix,
                         const int32_t *__restrict__ rank2row, float *__restrict__ dist2,
                         int32_t *__restrict__ idx, int32_t *__restrict__ counter,
                         int32_t *__restrict__ list, V2pGrid vg,
                         const int32_t *__restrict__ disorder, float *__restrict__ weight) {
  const bool by_cell = CENTRES && disorder[0] == 0;
  const int q = blockIdx.x * (256 / kGridNnLanes) + threadIdx.x / kGridNnLanes;
  const int sub = threadIdx.x % kGridNnLanes;
  const bool live = q < n;  // dead groups run along (the shuffles want every lane)
  float4v u = {-1.f, 0.f, 0.f, 0.f};
  if (live) u = reinterpret_cast<const float4v *>(unknown)[q];
  const Best3 none = {INFINITY, INFINITY, INFINITY, 0, 0, 0};
  Best3 acc = none;  // the query's three best so far, the same in its eight lanes
  const float pos[3] = {u.y, u.z, u.w};
  const int b = (int)u.x;
  const bool batch_ok = (float)b == u.x && b >= 0 && b < g.batch;
  bool settled = !live;
  if (live && !batch_ok) {
    if (sub == 0) atomicOr(counter, kGridNnAll);
    settled = true;
  }
  int c[3] = {0, 0, 0};
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    const int v = (int)floorf((pos[a] - g.origin[a]) / g.unit[a]);
    c[a] = v < 0 ? 0 : (v >= g.dim[a] ? g.dim[a] - 1 : v);
  }
  for (int r = 0; r <= kGridNnMaxShell; ++r) {
    if (__all(settled)) break;  // (every query of the wave: the same decision in all lanes)
    Best3 cur = none;
    if (!settled) {
      const int x0 = max(c[0] - r, 0), x1 = min(c[0] + r, g.dim[0] - 1);
      const int y0 = max(c[1] - r, 0), y1 = min(c[1] + r, g.dim[1] - 1);
      const int z0 = max(c[2] - r, 0), z1 = min(c[2] + r, g.dim[2] - 1);
      const int ny = y1 - y0 + 1, ncol = (x1 - x0 + 1) * ny;
      for (int col = sub; col < ncol; col += kGridNnLanes) {
        const int x = x0 + col / ny, y = y0 + col % ny;
        // cells of the shell only: in the interior of the box just the two end cells in z
        const bool face = abs(x - c[0]) == r || abs(y - c[1]) == r;
        const uint32_t base = (uint32_t)(((b * g.dim[0] + x) * g.dim[1] + y) * g.dim[2]);
        float xx = 0.f, yy = 0.f;  // (CENTRES) the column's share of the distance
        if constexpr (CENTRES) {
          const float dx = u.y - v2p_centre(x, vg, 0), dy = u.z - v2p_centre(y, vg, 1);
          xx = dx * dx;
          yy = dy * dy;
        }
        // The column's cells of the shell are neighbours along z: one or two words of the
        // table (2 r + 1 <= 9 cells).  Their set bits are taken from a mask, so the empty
        // cells -- nearly all of them -- cost nothing.  (Loading the words of four of a
        // lane's columns before looking at any: 43 against 46 us on clouds of 65 k points,
        // 63 against 57 on 131 k.)
        const uint32_t k0 = base + (uint32_t)z0, k1 = base + (uint32_t)z1;
        for (uint32_t wi = k0 >> 5; wi <= (k1 >> 5); ++wi) {
          const uint32_t w = bits[wi];
          if (w == 0u) continue;
          const uint32_t lo_bit = wi == (k0 >> 5) ? (k0 & 31u) : 0u;
          const uint32_t hi_bit = wi == (k1 >> 5) ? (k1 & 31u) : 31u;
          uint32_t cand = w & (0xFFFFFFFFu << lo_bit) & (0xFFFFFFFFu >> (31u - hi_bit));
          if (!face) {  // only the column's two end cells belong to the shell
            uint32_t ends = 0u;
            const int za = c[2] - r, zb = c[2] + r;
            if (za >= z0 && ((base + (uint32_t)za) >> 5) == wi)
              ends |= 1u << ((base + (uint32_t)za) & 31u);
            if (zb <= z1 && ((base + (uint32_t)zb) >> 5) == wi)
              ends |= 1u << ((base + (uint32_t)zb) & 31u);
            cand &= ends;
          }
          if (cand == 0u) continue;
          const int wp = by_cell ? 0 : prefix[wi];
          while (cand != 0u) {
            const uint32_t bit = (uint32_t)__ffs((int)cand) - 1u;
            cand &= cand - 1u;
            const uint32_t key = (wi << 5) + bit;
            if constexpr (CENTRES) {
              const float dz = u.w - v2p_centre((int)(key - base), vg, 2);
              const float zz = dz * dz;
              const int id = by_cell ? (int)key : rank2row[wp + __popc(w & ((1u << bit) - 1u))];
              cur.insert((xx + yy) + zz, id);
            } else {
              const int row = rank2row[wp + __popc(w & ((1u << bit) - 1u))];
              const float4v p = reinterpret_cast<const float4v *>(known)[row];
              if (p.x == u.x) {
                const float dx = u.y - p.y, dy = u.z - p.z, dz = u.w - p.w;
                const float x2 = dx * dx, y2 = dy * dy, z2 = dz * dz;
                cur.insert((x2 + y2) + z2, row);
              }
            }
          }
        }
      }
    }
    nng_merge_lanes(cur);
    if (!settled) {
      if (cur.b1 < INFINITY) acc.insert(cur.b1, cur.i1);
      if (cur.b2 < INFINITY) acc.insert(cur.b2, cur.i2);
      if (cur.b3 < INFINITY) acc.insert(cur.b3, cur.i3);
      // distance to the nearest layer of centres that has not been visited
      float bound = INFINITY;
#pragma unroll
      for (int a = 0; a < 3; ++a) {
        if (c[a] - r - 1 >= 0)
          bound = fminf(bound, pos[a] - (g.origin[a] + ((float)(c[a] - r) - 0.5f) * g.unit[a]));
        if (c[a] + r + 1 <= g.dim[a] - 1)
          bound = fminf(bound, (g.origin[a] + ((float)(c[a] + r) + 1.5f) * g.unit[a]) - pos[a]);
      }
      if (bound == INFINITY) {
        settled = true;  // the whole grid of this batch element has been visited
      } else if (bound > 0.f && acc.b3 < bound * bound * 0.9999f) {
        settled = true;
      } else if (r == kGridNnMaxShell && sub == 0) {
        const int at = atomicAdd(counter, 1);
        if (at >= 0 && at < n) list[at] = q;
      }
    }
  }
  if (live && sub == 0) {
    if (by_cell) {  // the winners' rows: the ranks of their cells
      if (acc.b1 < INFINITY) acc.i1 = bit_rank(bits, prefix, (uint32_t)acc.i1);
      if (acc.b2 < INFINITY) acc.i2 = bit_rank(bits, prefix, (uint32_t)acc.i2);
      if (acc.b3 < INFINITY) acc.i3 = bit_rank(bits, prefix, (uint32_t)acc.i3);
    }
    dist2[q * 3] = acc.b1; dist2[q * 3 + 1] = acc.b2; dist2[q * 3 + 2] = acc.b3;
    idx[q * 3] = acc.i1; idx[q * 3 + 1] = acc.i2; idx[q * 3 + 2] = acc.i3;
    if (weight != nullptr) nn_weights(acc.b1, acc.b2, acc.b3, weight + q * 3);
  }
}

// The queries the grid search left open, one workgroup each: all rows, 256 at a time with
// four loads in flight per thread, then the threads' candidates merged through LDS.
// (Nothing to do when the counter says that the plain scan redoes the call.)
__global__ void __launch_bounds__(256)
    three_nn_list_kernel(int n, int m, const float *__restrict__ unknown,
                         const float *__restrict__ known, const int32_t *__restrict__ counter,
                         const int32_t *__restrict__ list, int redo_above,
                         float *__restrict__ dist2, int32_t *__restrict__ idx,
                         float *__restrict__ weight) {
  __shared__ float sd[4][3];
  __shared__ int si[4][3];
  const int count = counter[0];
  if (count <= 0 || count > redo_above) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int e = blockIdx.x; e < count; e += gridDim.x) {
    const int q = list[e];
    const float4v u = reinterpret_cast<const float4v *>(unknown)[q];
    Best3 best = {INFINITY, INFINITY, INFINITY, 0, 0, 0};
    auto consider = [&](const float4v &p, int row) {
      if (p.x != u.x) return;
      const float dx = u.y - p.y, dy = u.z - p.z, dz = u.w - p.w;
      const float xx = dx * dx, yy = dy * dy, zz = dz * dz;
      best.insert((xx + yy) + zz, row);
    };
    int row = threadIdx.x;
    for (; row + 3 * 256 < m; row += 4 * 256) {
      float4v p[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) p[k] = reinterpret_cast<const float4v *>(known)[row + k * 256];
#pragma unroll
      for (int k = 0; k < 4; ++k) consider(p[k], row + k * 256);
    }
    for (; row < m; row += 256) consider(reinterpret_cast<const float4v *>(known)[row], row);
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float o1 = __shfl_xor(best.b1, d, 64), o2 = __shfl_xor(best.b2, d, 64),
                  o3 = __shfl_xor(best.b3, d, 64);
      const int j1 = __shfl_xor(best.i1, d, 64), j2 = __shfl_xor(best.i2, d, 64),
                j3 = __shfl_xor(best.i3, d, 64);
      if (o1 < INFINITY) best.insert(o1, j1);
      if (o2 < INFINITY) best.insert(o2, j2);
      if (o3 < INFINITY) best.insert(o3, j3);
    }
    if (lane == 0) {
      sd[wave][0] = best.b1; sd[wave][1] = best.b2; sd[wave][2] = best.b3;
      si[wave][0] = best.i1; si[wave][1] = best.i2; si[wave][2] = best.i3;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int w = 1; w < 4; ++w)
        for (int k = 0; k < 3; ++k)
          if (sd[w][k] < INFINITY) best.insert(sd[w][k], si[w][k]);
      dist2[q * 3] = best.b1; dist2[q * 3 + 1] = best.b2; dist2[q * 3 + 2] = best.b3;
      idx[q * 3] = best.i1; idx[q * 3 + 1] = best.i2; idx[q * 3 + 2] = best.i3;
      if (weight != nullptr) nn_weights(best.b1, best.b2, best.b3, weight + q * 3);
    }
    __syncthreads();
  }
}

static int64_t nng_cells(int32_t batch, const int32_t *dims) {
  if (batch < 1 || !dims || dims[0] < 1 || dims[1] < 1 || dims[2] < 1) return -1;
  const int64_t cells = (int64_t)batch * dims[0] * dims[1] * dims[2];
  return cells < ((int64_t)1 << 31) ? cells : -1;
}

}  // namespace ssc

extern "C" {

size_t ssc_three_nn_grid_workspace_bytes(int32_t n, int32_t m, int32_t batch_size,
                                         const int32_t dims[3]) {
  const int64_t cells = nng_cells(batch_size, dims);
  if (cells < 0 || m < 0 || n < 0) return 0;
  return bit_table_bytes(cells) + align_up((size_t)(m > 0 ? m : 1) * sizeof(int32_t)) +
         align_up((size_t)(n > 0 ? n : 1) * sizeof(int32_t));
}

// The grid search, queued.  vg (optional): the known points are the voxels' centres as vg
// states them (three_nn_grid_kernel<true>); weight (optional): the interpolation weights are
// written with the result; table_cleared: the caller has zeroed the table and its totals.
static int nn_grid_enqueue(int32_t n, int32_t m, const float *unknown, const float *known,
                           const int32_t *voxel_indices, int32_t batch_size,
                           const int32_t dims[3], const float origin[3], const float unit[3],
                           float *dist2, int32_t *idx, void *workspace, hipStream_t s,
                           const V2pGrid *vg, float *weight, bool table_cleared) {
  const int64_t cells = nng_cells(batch_size, dims);
  GridNn g;
  g.batch = batch_size;
  for (int a = 0; a < 3; ++a) {
    g.dim[a] = dims[a];
    g.origin[a] = origin[a];
    g.unit[a] = unit[a];
  }
  Carver c(workspace);
  BitTable t = bit_table_carve(c, cells);
  int32_t *rank2row = c.take<int32_t>((size_t)(m > 0 ? m : 1));
  int32_t *list = c.take<int32_t>((size_t)n);
  // t.total[1] and [2] are cleared with the table and not used by the scan: the counter of
  // the queries left open, and the flag "voxel rows not in key order"
  int32_t *counter = t.total + 1, *disorder = t.total + 2;
  int rc;
  if (!table_cleared && (rc = bit_table_clear(t, s)) != SSC_OK) return rc;
  if (m > 0) {
    hipLaunchKernelGGL(nng_mark_kernel, dim3((unsigned)ceil_div(m, 256)), dim3(256), 0, s,
                       voxel_indices, m, g, t.bits, counter, disorder);
    SSC_LAUNCH_CHECK("nng_mark");
  }
  if ((rc = bit_table_scan(t, s)) != SSC_OK) return rc;
  if (m > 0) {
    hipLaunchKernelGGL(nng_rank2row_kernel, dim3((unsigned)ceil_div(m, 256)), dim3(256), 0, s,
                       voxel_indices, m, g, t.bits, t.prefix, rank2row,
                       vg != nullptr ? disorder : (const int32_t *)nullptr);
    SSC_LAUNCH_CHECK("nng_rank2row");
  }
  const dim3 grid((unsigned)ceil_div(n, 256 / kGridNnLanes));
  if (vg != nullptr) {
    hipLaunchKernelGGL(three_nn_grid_kernel<true>, grid, dim3(256), 0, s, n, m, unknown, known, g,
                       t.bits, t.prefix, rank2row, dist2, idx, counter, list, *vg, disorder,
                       weight);
  } else {
    hipLaunchKernelGGL(three_nn_grid_kernel<false>, grid, dim3(256), 0, s, n, m, unknown, known,
                       g, t.bits, t.prefix, rank2row, dist2, idx, counter, list, V2pGrid{},
                       disorder, weight);
  }
  SSC_LAUNCH_CHECK("three_nn_grid");
  const int redo_above = n / 8;
  hipLaunchKernelGGL(three_nn_list_kernel, dim3(512), dim3(256), 0, s, n, m, unknown, known,
                     counter, list, redo_above, dist2, idx, weight);
  SSC_LAUNCH_CHECK("three_nn_list");
  hipLaunchKernelGGL(three_nn_kernel, dim3((unsigned)ceil_div(n, kNnTile / kNnLanes)), dim3(kNnTile),
                     0, s, n, m, unknown, known, (const float *)nullptr, dist2, idx,
                     (const int32_t *)counter, redo_above, weight);
  SSC_LAUNCH_CHECK("three_nn");
  return SSC_OK;
}

int ssc_three_nn_grid(int32_t n, int32_t m, const float *unknown, const float *known,
                      const int32_t *voxel_indices, int32_t batch_size, const int32_t dims[3],
                      const float origin[3], const float unit[3], float *dist2, int32_t *idx,
                      void *workspace, size_t workspace_bytes, ssc_stream_t stream) {
  SSC_CHECK(n >= 0 && m >= 0, SSC_EINVAL, "bad sizes");
  const int64_t cells = nng_cells(batch_size, dims);
  SSC_CHECK(cells > 0, SSC_EINVAL, "batch_size * prod(dims) must be positive and below 2^31");
  SSC_CHECK(origin && unit && unit[0] > 0.f && unit[1] > 0.f && unit[2] > 0.f, SSC_EINVAL,
            "voxel extents must be positive");
  if (n == 0) return SSC_OK;
  SSC_CHECK(unknown && dist2 && idx && (m == 0 || (known && voxel_indices)), SSC_EINVAL,
            "NULL pointer argument");
  SSC_CHECK(workspace != nullptr &&
                workspace_bytes >= ssc_three_nn_grid_workspace_bytes(n, m, batch_size, dims),
            SSC_EWORKSPACE, "three_nn_grid workspace too small");
  return nn_grid_enqueue(n, m, unknown, known, voxel_indices, batch_size, dims, origin, unit,
                         dist2, idx, workspace, (hipStream_t)stream, nullptr, nullptr, false);
}

}  // extern "C"

// ---- Voxel2Point as one call ----------------------------------------------------------------
// What Voxel2Point.forward does with a dozen tensor operations around the search and the
// interpolation (ss_conv/sp_ops/voxelize.py:131-160), as kernels of one call.
namespace ssc {

// unknown[i] = (batch id, x, y, z) of point i; known[j] = (b, centre of voxel j) (v2p_centre).
// The blocks behind those of the points and voxels zero the search's table and its totals
// (what bit_table_clear would do in a launch of its own).
__global__ void __launch_bounds__(256)
    v2p_prepare_kernel(const float *__restrict__ pts, const int64_t *__restrict__ ids, int n,
                       const int32_t *__restrict__ vox, int m, V2pGrid g,
                       float *__restrict__ unknown, float *__restrict__ known, int row_blocks,
                       uint32_t *__restrict__ bits, int64_t n_words, int32_t *__restrict__ total) {
  if ((int)blockIdx.x >= row_blocks) {
    const int64_t step = (int64_t)(gridDim.x - row_blocks) * blockDim.x;
    int64_t w = (int64_t)(blockIdx.x - row_blocks) * blockDim.x + threadIdx.x;
    if (w < 4) total[w] = 0;
    for (; w < n_words; w += step) bits[w] = 0u;
    return;
  }
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    const float4v u = {(float)ids[i], pts[(int64_t)i * 3], pts[(int64_t)i * 3 + 1],
                       pts[(int64_t)i * 3 + 2]};
    reinterpret_cast<float4v *>(unknown)[i] = u;
  }
  if (i < m) {
    const int4 r = reinterpret_cast<const int4 *>(vox)[i];
    float4v k;
    k.x = (float)r.x;
    k.y = v2p_centre(r.y, g, 0);
    k.z = v2p_centre(r.z, g, 1);
    k.w = v2p_centre(r.w, g, 2);
    reinterpret_cast<float4v *>(known)[i] = k;
  }
}

}  // namespace ssc

extern "C" {

size_t ssc_v2p_workspace_bytes(int32_t n, int32_t m, int32_t batch_size, const int32_t dims[3]) {
  const size_t search = ssc_three_nn_grid_workspace_bytes(n, m, batch_size, dims);
  if (search == 0) return 0;
  return search + align_up((size_t)(n > 0 ? n : 1) * 16) + align_up((size_t)(m > 0 ? m : 1) * 16) +
         align_up((size_t)(n > 0 ? n : 1) * 12);
}

int ssc_v2p_interpolate_f32(const float *points, const int64_t *batch_ids, int32_t n,
                            const int32_t *voxel_indices, const float *voxel_feats, int32_t m,
                            int32_t channels, int32_t batch_size, const int32_t dims[3],
                            const float unit[3], const float extent[3], float *out, int32_t *idx,
                            float *weight, void *workspace, size_t workspace_bytes,
                            ssc_stream_t stream) {
  SSC_CHECK(n >= 0 && m >= 1 && channels >= 1, SSC_EINVAL, "bad sizes");
  SSC_CHECK(unit && extent && dims, SSC_EINVAL, "NULL pointer argument");
  if (n == 0) return SSC_OK;
  SSC_CHECK(points && batch_ids && voxel_indices && voxel_feats && out && idx && weight &&
                workspace,
            SSC_EINVAL, "NULL pointer argument");
  const size_t search = ssc_three_nn_grid_workspace_bytes(n, m, batch_size, dims);
  SSC_CHECK(search > 0 && workspace_bytes >= ssc_v2p_workspace_bytes(n, m, batch_size, dims),
            SSC_EWORKSPACE, "v2p workspace too small");
  hipStream_t s = (hipStream_t)stream;
  Carver c(workspace);
  char *search_ws = c.take<char>(search);
  float *unknown = c.take<float>((size_t)n * 4);
  float *known = c.take<float>((size_t)m * 4);
  float *dist2 = c.take<float>((size_t)n * 3);
  V2pGrid g;
  float origin[3];
  for (int a = 0; a < 3; ++a) {
    g.unit[a] = unit[a];
    g.half_extent[a] = 0.5f * extent[a];
    g.half_unit[a] = 0.5f * unit[a];
    origin[a] = -0.5f * extent[a];
  }
  // (the table of the search, as nn_grid_enqueue will carve it from the same bytes)
  Carver cs(search_ws);
  const BitTable t = bit_table_carve(cs, nng_cells(batch_size, dims));
  const int row_blocks = (int)ceil_div(n > m ? n : m, 256);
  int64_t clear_blocks = ceil_div(t.n_words, 256 * 4);
  if (clear_blocks > 2048) clear_blocks = 2048;
  if (clear_blocks < 1) clear_blocks = 1;
  hipLaunchKernelGGL(v2p_prepare_kernel, dim3((unsigned)(row_blocks + clear_blocks)), dim3(256), 0,
                     s, points, batch_ids, n, voxel_indices, m, g, unknown, known, row_blocks,
                     t.bits, t.n_words, t.total);
  SSC_LAUNCH_CHECK("v2p_prepare");
  // the search ranks its candidates by the centres of their cells and writes the weights
  int rc = nn_grid_enqueue(n, m, unknown, known, voxel_indices, batch_size, dims, origin, unit,
                           dist2, idx, search_ws, s, &g, weight, true);
  if (rc != SSC_OK) return rc;
  return ssc_three_interp_f32(channels, m, n, voxel_feats, idx, weight, out, stream);
}

int ssc_three_interp_f32(int32_t c, int32_t m, int32_t n, const float *feats, const int32_t *idx,
                         const float *weight, float *out, ssc_stream_t stream) {
  (void)m;
  SSC_CHECK(c >= 1 && n >= 0, SSC_EINVAL, "bad sizes");
  if (n == 0) return SSC_OK;
  SSC_CHECK(feats && idx && weight && out, SSC_EINVAL, "NULL pointer argument");
  int64_t e = (int64_t)n * c;
  hipLaunchKernelGGL(three_interp_kernel, dim3((unsigned)ceil_div(e, 256)), dim3(256), 0,
                     (hipStream_t)stream, c, n, feats, idx, weight, out);
  SSC_LAUNCH_CHECK("three_interp");
  return SSC_OK;
}
}

// ---- point filter and batch partition of Point2Voxel -------------------------------------
// The reference's forward (ss_conv/sp_ops/voxelize.py:40-83) drops the points outside
// the grid, gives every batch element left without points one zero point, and orders
// the survivors by batch id (stable).  For batch ids that are already non-decreasing
// and small non-negative integers -- clouds concatenated one after the other -- that is a
// stream compaction plus a shift per batch element: no sort, no unique.
namespace ssc {

// Pass 1: one wave per 64 points.  inside bit per point (a ballot: no atomics),
// histograms of all ids and of the surviving ids, flags[0] |= 1 for an id outside
// [0, max_ids), flags[1] |= 1 when ids decrease.  The waves of a block add their counts up
// in LDS first (bins for the ids first .. first + 63, `first` the id of the block's first
// point; any other id goes straight to memory) and the block then issues one atomic per
// id it saw: atomics on one address are served one after the other, and with a wave's
// worth of points per atomic a cloud of 16384 points put 256 of them on its counter.
constexpr int kP2vScanThreads = 1024;
__global__ void __launch_bounds__(kP2vScanThreads)
    p2v_scan_kernel(const float *__restrict__ pts, const int64_t *__restrict__ ids, int64_t n,
                    float hx, float hy, float hz, int max_ids, uint32_t *__restrict__ bits,
                    int32_t *__restrict__ hist_all, int32_t *__restrict__ hist_valid,
                    int32_t *__restrict__ flags, int32_t *__restrict__ block_inside = nullptr) {
  __shared__ int s_all[64], s_valid[64];
  __shared__ int s_first, s_inside;
  if (threadIdx.x == 0) s_inside = 0;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int lane = threadIdx.x & 63;
  const bool live = i < n;
  bool inside = false;
  int64_t id = -1;
  if (threadIdx.x < 64) {
    s_all[threadIdx.x] = 0;
    s_valid[threadIdx.x] = 0;
  }
  if (live) {
    const float x = pts[i * 3], y = pts[i * 3 + 1], z = pts[i * 3 + 2];
    inside = !(fabsf(x) > hx) && !(fabsf(y) > hy) && !(fabsf(z) > hz);
    id = ids[i];
    if (id < 0 || id >= max_ids) atomicOr(&flags[0], 1);
    if (i > 0 && ids[i - 1] > id) atomicOr(&flags[1], 1);
  }
  if (threadIdx.x == 0) s_first = (int)(id < 0 ? 0 : (id >= max_ids ? max_ids - 1 : id));
  __syncthreads();
  const int first_id = s_first;
  const unsigned long long in_mask = __ballot(inside);
  if (live && (lane & 31) == 0) bits[i >> 5] = (uint32_t)(in_mask >> (lane & 32));
  // (with block_inside: the block's number of inside points, for a compaction that ranks
  // its points without a scan of the bits)
  if (block_inside != nullptr && lane == 0 && in_mask) atomicAdd(&s_inside, __popcll(in_mask));
  const bool ok_id = live && id >= 0 && id < max_ids;
  unsigned long long todo = __ballot(ok_id);
  while (todo) {  // one trip per distinct id of the wave
    const int first = __ffsll((long long)todo) - 1;
    const int v = __shfl((int)id, first, 64);
    const unsigned long long same = __ballot(ok_id && (int)id == v);
    if (lane == first) {
      const int nv = __popcll(same & in_mask);
      const unsigned bin = (unsigned)(v - first_id);
      if (bin < 64u) {
        atomicAdd(&s_all[bin], __popcll(same));
        if (nv) atomicAdd(&s_valid[bin], nv);
      } else {
        atomicAdd(&hist_all[v], __popcll(same));
        if (nv) atomicAdd(&hist_valid[v], nv);
      }
    }
    todo &= ~same;
  }
  __syncthreads();
  if (threadIdx.x < 64) {
    const int a = s_all[threadIdx.x], b = s_valid[threadIdx.x];
    if (a) atomicAdd(&hist_all[first_id + threadIdx.x], a);
    if (b) atomicAdd(&hist_valid[first_id + threadIdx.x], b);
  }
  if (block_inside != nullptr && threadIdx.x == 0) block_inside[blockIdx.x] = s_inside;
}

// One block of 256 threads: start[e] = survivors with an id below e; shift[e] = ids below e
// that are present but have no survivor (each of them receives one zero point).  Returns
// the number of such ids in *n_empty (thread 255 holds it).
__device__ __forceinline__ void p2v_prefix_block(const int32_t *__restrict__ hist_all,
                                                 const int32_t *__restrict__ hist_valid,
                                                 int32_t *__restrict__ start,
                                                 int32_t *__restrict__ shift, int *s_valid,
                                                 int *s_empty, int *n_empty) {
  constexpr int PER = SSC_P2V_MAX_IDS / 256;
  const int t = threadIdx.x;
  int sv = 0, se = 0;
  for (int j = 0; j < PER; ++j) {
    const int e = t * PER + j;
    sv += hist_valid[e];
    se += (hist_all[e] > 0 && hist_valid[e] == 0) ? 1 : 0;
  }
  s_valid[t] = sv;
  s_empty[t] = se;
  __syncthreads();
  int bv = 0, be = 0;
  for (int u = 0; u < t; ++u) {
    bv += s_valid[u];
    be += s_empty[u];
  }
  for (int j = 0; j < PER; ++j) {
    const int e = t * PER + j;
    start[e] = bv;
    shift[e] = be;
    bv += hist_valid[e];
    be += (hist_all[e] > 0 && hist_valid[e] == 0) ? 1 : 0;
  }
  *n_empty = be;  // of thread 255: all of them
}

__global__ void __launch_bounds__(256)
    p2v_prefix_kernel(const int32_t *__restrict__ hist_all, const int32_t *__restrict__ hist_valid,
                      int32_t *__restrict__ start, int32_t *__restrict__ shift) {
  __shared__ int s_valid[256], s_empty[256];
  int n_empty;
  p2v_prefix_block(hist_all, hist_valid, start, shift, s_valid, s_empty, &n_empty);
}

// Pass 2a: surviving point i goes to row rank(i) + shift[id]; threads n..n+MAX_IDS-1
// write the zero point of an id without survivors.  Also writes the voxel coordinates
// ((int)((p + half) / unit) in fp32, as voxel_coords_kernel does).
__global__ void __launch_bounds__(256)
    p2v_compact_kernel(const float *__restrict__ pts, const int64_t *__restrict__ ids, int64_t n,
                       const uint32_t *__restrict__ bits, const int32_t *__restrict__ prefix,
                       const int32_t *__restrict__ hist_all,
                       const int32_t *__restrict__ hist_valid, const int32_t *__restrict__ start,
                       const int32_t *__restrict__ shift, float hx, float hy, float hz, float ux,
                       float uy, float uz, float *__restrict__ out_pts,
                       int64_t *__restrict__ out_ids, int32_t *__restrict__ coords,
                       int32_t *__restrict__ dest, int32_t *__restrict__ src, int max_ids,
                       uint32_t *__restrict__ vox_bits, int d1, int d2, int d3,
                       int32_t *__restrict__ flags) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  float x = 0.f, y = 0.f, z = 0.f;
  int64_t id;
  int pos;
  if (i < n) {
    id = ids[i];
    // (a caller that runs this kernel without looking at the scan's flags first may hold
    // ids outside the tables: such a point is dropped, the flags tell)
    const bool inside = ((bits[i >> 5] >> (i & 31)) & 1u) && id >= 0 && id < max_ids;
    pos = inside ? bit_rank(bits, prefix, (uint32_t)i) + shift[id] : -1;
    dest[i] = pos;
    if (!inside) return;
    x = pts[i * 3];
    y = pts[i * 3 + 1];
    z = pts[i * 3 + 2];
  } else {
    id = i - n;
    if (id >= max_ids || hist_all[id] == 0 || hist_valid[id] != 0) return;
    pos = start[id] + shift[id];
  }
  if (src != nullptr) src[pos] = i < n ? (int32_t)i : -1;  // input row behind output row pos
  out_pts[(int64_t)pos * 3] = x;
  out_pts[(int64_t)pos * 3 + 1] = y;
  out_pts[(int64_t)pos * 3 + 2] = z;
  out_ids[pos] = id;
  const int vx = (int)((x + hx) / ux);
  const int vy = (int)((y + hy) / uy);
  const int vz = (int)((z + hz) / uz);
  reinterpret_cast<int4 *>(coords)[pos] = make_int4((int)id, vx, vy, vz);
  if (vox_bits != nullptr) {  // mark the voxel in the table of the unique-rows step
    if ((unsigned)vx < (unsigned)d1 && (unsigned)vy < (unsigned)d2 && (unsigned)vz < (unsigned)d3) {
      const uint32_t key = (uint32_t)((((int)id * d1 + vx) * d2 + vy) * d3 + vz);
      atomicOr(&vox_bits[key >> 5], 1u << (key & 31u));
    } else {
      atomicOr(&flags[0], 4);
    }
  }
}

// Pass 2b: feature rows follow their points (dest[i] from pass 2a, -1 = dropped);
// rows n..n+MAX_IDS-1 stand for the zero points.
__global__ void __launch_bounds__(256)
    p2v_feats_kernel(const float *__restrict__ feats, int64_t n, int C,
                     const int32_t *__restrict__ dest, const int32_t *__restrict__ hist_all,
                     const int32_t *__restrict__ hist_valid, const int32_t *__restrict__ start,
                     const int32_t *__restrict__ shift, float *__restrict__ out) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t i = e / C;
  const int c = (int)(e - i * C);
  if (i < n) {
    const int pos = dest[i];
    if (pos >= 0) out[(int64_t)pos * C + c] = feats[e];
  } else {
    const int64_t id = i - n;
    if (id >= SSC_P2V_MAX_IDS || hist_all[id] == 0 || hist_valid[id] != 0) return;
    out[(int64_t)(start[id] + shift[id]) * C + c] = 0.f;
  }
}

struct P2vWs {
  BitTable table;
  int32_t *hist_all, *hist_valid, *flags, *start, *shift, *dest;
};

static size_t p2v_ws_walk(void *base, int64_t n, P2vWs *w) {
  Carver c(base);
  P2vWs t;
  t.table = bit_table_carve(c, n > 0 ? n : 1);
  t.hist_all = c.take<int32_t>(SSC_P2V_MAX_IDS);
  t.hist_valid = c.take<int32_t>(SSC_P2V_MAX_IDS);  // directly behind hist_all
  t.flags = c.take<int32_t>(2);
  t.start = c.take<int32_t>(SSC_P2V_MAX_IDS);
  t.shift = c.take<int32_t>(SSC_P2V_MAX_IDS);
  t.dest = c.take<int32_t>(n > 0 ? n : 1);
  if (w) *w = t;
  return c.used;
}

}  // namespace ssc

extern "C" {

size_t ssc_p2v_workspace_bytes(int64_t n) {
  if (n < 0) return 0;
  // the carve sizes do not depend on the base address
  return ssc::p2v_ws_walk(nullptr, n, nullptr);
}

int ssc_p2v_scan(const float *points, const int64_t *batch_ids, int64_t n,
                 const float half_extent[3], void *workspace, size_t workspace_bytes,
                 int32_t *hist_all_host, int32_t *hist_valid_host, int32_t *flags_host,
                 ssc_stream_t stream) {
  SSC_CHECK(n > 0, SSC_EINVAL, "n must be positive");
  SSC_CHECK(n < ((int64_t)1 << 31), SSC_EINVAL, "n must fit 31 bits");
  SSC_CHECK(points && batch_ids && half_extent && workspace && hist_all_host && hist_valid_host &&
                flags_host,
            SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(workspace_bytes >= ssc_p2v_workspace_bytes(n), SSC_EWORKSPACE,
            "p2v workspace too small");
  hipStream_t s = (hipStream_t)stream;
  P2vWs w;
  p2v_ws_walk(workspace, n, &w);
  int rc;
  // hist_all, hist_valid and flags are cleared with one fill (they are adjacent up to
  // alignment padding, which the fill covers as well)
  const int64_t clear_n = (w.flags + 2) - w.hist_all;
  if ((rc = fill_i32(w.hist_all, clear_n, 0, s)) != SSC_OK) return rc;
  hipLaunchKernelGGL(p2v_scan_kernel, dim3((unsigned)ceil_div(n, kP2vScanThreads)),
                     dim3(kP2vScanThreads), 0, s, points,
                     batch_ids, n, half_extent[0], half_extent[1], half_extent[2],
                     (int)SSC_P2V_MAX_IDS, w.table.bits, w.hist_all, w.hist_valid, w.flags);
  SSC_LAUNCH_CHECK("p2v_scan");
  if ((rc = bit_table_scan(w.table, s)) != SSC_OK) return rc;
  hipLaunchKernelGGL(p2v_prefix_kernel, dim3(1), dim3(256), 0, s, w.hist_all, w.hist_valid,
                     w.start, w.shift);
  SSC_LAUNCH_CHECK("p2v_prefix");
  // the two histograms and the flags sit side by side: one copy brings all three
  static_assert((2 * SSC_P2V_MAX_IDS + 256) * sizeof(int32_t) <= kReadBackBytes, "pinned block");
  const void *view;
  if ((rc = read_back_view(&view, w.hist_all, clear_n * sizeof(int32_t), s)) != SSC_OK) return rc;
  const int32_t *land = (const int32_t *)view;
  memcpy(hist_all_host, land, SSC_P2V_MAX_IDS * sizeof(int32_t));
  memcpy(hist_valid_host, land + (w.hist_valid - w.hist_all), SSC_P2V_MAX_IDS * sizeof(int32_t));
  memcpy(flags_host, land + (w.flags - w.hist_all), 2 * sizeof(int32_t));
  return SSC_OK;
}

int ssc_p2v_compact(const float *points, const float *feats, const int64_t *batch_ids, int64_t n,
                    int32_t channels, const float half_extent[3], const float unit[3],
                    void *workspace, size_t workspace_bytes, float *out_points, float *out_feats,
                    int64_t *out_ids, int32_t *out_coords, int32_t *out_dest,
                    ssc_stream_t stream) {
  SSC_CHECK(n > 0 && channels >= 1, SSC_EINVAL, "bad sizes");
  SSC_CHECK(points && feats && batch_ids && half_extent && unit && workspace && out_points &&
                out_feats && out_ids && out_coords,
            SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(workspace_bytes >= ssc_p2v_workspace_bytes(n), SSC_EWORKSPACE,
            "p2v workspace too small");
  hipStream_t s = (hipStream_t)stream;
  P2vWs w;
  p2v_ws_walk(workspace, n, &w);
  // where every input row went (-1: dropped), for the caller if it asks
  int32_t *dest = out_dest ? out_dest : w.dest;
  const int64_t rows = n + SSC_P2V_MAX_IDS;
  hipLaunchKernelGGL(p2v_compact_kernel, dim3((unsigned)ceil_div(rows, 256)), dim3(256), 0, s,
                     points, batch_ids, n, w.table.bits, w.table.prefix, w.hist_all, w.hist_valid,
                     w.start, w.shift, half_extent[0], half_extent[1], half_extent[2], unit[0],
                     unit[1], unit[2], out_points, out_ids, out_coords, dest, (int32_t *)nullptr,
                     (int)SSC_P2V_MAX_IDS, (uint32_t *)nullptr, 0, 0, 0, (int32_t *)nullptr);
  SSC_LAUNCH_CHECK("p2v_compact");
  hipLaunchKernelGGL(p2v_feats_kernel, dim3((unsigned)ceil_div(rows * channels, 256)), dim3(256), 0,
                     s, feats, n, (int)channels, dest, w.hist_all, w.hist_valid, w.start,
                     w.shift, out_feats);
  SSC_LAUNCH_CHECK("p2v_feats");
  return SSC_OK;
}
}

// ---- Point2Voxel in one call ---------------------------------------------------------------
// Filter, batch partition, unique voxels and the per-voxel feature reduction of
// Point2Voxel.forward (ss_conv/sp_ops/voxelize.py:40-99) queued as one chain of kernels that
// keeps every data-dependent size on the device: outputs are written into buffers with room
// for n rows (there are never more rows or voxels than points), the totals land in pinned
// host memory, and the host waits once, for them, while the last two kernels still run.
// The per-voxel point lists are linked chains (head[voxel], next[row]; built with an atomic
// exchange, so in no particular order); the reduction brings each chain into ascending row
// order through a bit map over row numbers held one word per lane, which makes the sums
// independent of the race -- and leaves no [voxels, largest population] table to size.
namespace ssc {

// Everything the chain needs cleared, in one launch: a[0..n_a) = 0 (histograms and flags),
// vox_bits[0..n_words) = 0, head[0..n_head) = -1, totals[0..8) = 0.
__global__ void __launch_bounds__(256)
    p2vx_clear_kernel(int32_t *__restrict__ a, int64_t n_a, uint32_t *__restrict__ vox_bits,
                      int64_t n_words, int32_t *__restrict__ head, int64_t n_head,
                      int32_t *__restrict__ totals) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  if (i < 8) totals[i] = 0;
  for (int64_t j = i; j < n_a; j += step) a[j] = 0;
  for (int64_t j = i; j < n_head; j += step) head[j] = -1;
  for (int64_t j = i; j < n_words; j += step) vox_bits[j] = 0u;
}

// The compaction of the one-call chain: p2v_compact_kernel without the scans before it.  A
// block takes the kP2vScanThreads points of one block of p2v_scan_kernel (the blocks after
// the points' take the ids, for the zero points of ids left without survivors) and works
// out for itself what the scans would have told it: the inside points before the block (a
// sum over block_inside[], at most n / 1024 numbers), the rank of a point inside the block
// (the popcounts of the block's 32 words of inside bits), and start / shift of every id (a
// scan of the two histograms, n_ids numbers, in LDS).  The last block of points leaves the
// number of inside points in inside_total[0]; block 0 the number of ids left without points
// in extra[0] and the two histograms in mirror_hist (memory the host reads).
constexpr int kP2vIdsPerThread = SSC_P2V_MAX_IDS / kP2vScanThreads;
__global__ void __launch_bounds__(kP2vScanThreads)
    p2vx_compact_kernel(const float *__restrict__ pts, const int64_t *__restrict__ ids, int64_t n,
                        const uint32_t *__restrict__ bits,
                        const int32_t *__restrict__ block_inside, int n_point_blocks,
                        const int32_t *__restrict__ hist_all,
                        const int32_t *__restrict__ hist_valid, float hx, float hy, float hz,
                        float ux, float uy, float uz, float *__restrict__ out_pts,
                        int64_t *__restrict__ out_ids, int32_t *__restrict__ coords,
                        int32_t *__restrict__ dest, int32_t *__restrict__ src, int n_ids,
                        uint32_t *__restrict__ vox_bits, int d1, int d2, int d3,
                        int32_t *__restrict__ flags, int32_t *__restrict__ inside_total,
                        int32_t *__restrict__ extra, int32_t *__restrict__ mirror_hist) {
  static_assert(kP2vIdsPerThread >= 1 && kP2vIdsPerThread * kP2vScanThreads == SSC_P2V_MAX_IDS,
                "ids per thread");
  __shared__ int s_start[SSC_P2V_MAX_IDS], s_shift[SSC_P2V_MAX_IDS];
  __shared__ int s_wave_a[kP2vScanThreads / 64], s_wave_b[kP2vScanThreads / 64];
  __shared__ int s_word[32], s_wprefix[32];
  __shared__ int s_before;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  // start[e] = survivors with an id below e; shift[e] = ids below e that are present but
  // have no survivor: every thread a run of consecutive ids, then a scan over the threads
  int hv[kP2vIdsPerThread], he[kP2vIdsPerThread], sv = 0, se = 0;
#pragma unroll
  for (int j = 0; j < kP2vIdsPerThread; ++j) {
    const int e = t * kP2vIdsPerThread + j;
    const int a = e < n_ids ? hist_all[e] : 0, v = e < n_ids ? hist_valid[e] : 0;
    hv[j] = v;
    he[j] = (a > 0 && v == 0) ? 1 : 0;
    sv += hv[j];
    se += he[j];
    if (blockIdx.x == 0 && e < n_ids) {
      mirror_hist[e] = a;
      mirror_hist[n_ids + e] = v;
    }
  }
  // the inside points of the blocks before this one (blocks of ids: of all blocks)
  int before = 0;
  const int upto = (int)blockIdx.x < n_point_blocks ? (int)blockIdx.x : n_point_blocks;
  for (int b = t; b < upto; b += kP2vScanThreads) before += block_inside[b];
  int iv = sv, ie = se, ib = before;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int ov = __shfl_up(iv, d, 64), oe = __shfl_up(ie, d, 64);
    if (lane >= d) {
      iv += ov;
      ie += oe;
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) ib += __shfl_xor(ib, d, 64);
  if (lane == 63) {
    s_wave_a[wave] = iv;
    s_wave_b[wave] = ie;
  }
  if (t == 0) s_before = 0;
  if (t < 32) {
    const int64_t w = (int64_t)blockIdx.x * (kP2vScanThreads / 32) + t;
    s_word[t] = ((int)blockIdx.x < n_point_blocks && w * 32 < n) ? (int)bits[w] : 0;
  }
  __syncthreads();
  if (lane == 0 && ib) atomicAdd(&s_before, ib);
  int bv = iv - sv, be = ie - se;
  int all_e = 0;
  for (int u = 0; u < kP2vScanThreads / 64; ++u) {
    if (u < wave) {
      bv += s_wave_a[u];
      be += s_wave_b[u];
    }
    all_e += s_wave_b[u];
  }
#pragma unroll
  for (int j = 0; j < kP2vIdsPerThread; ++j) {
    const int e = t * kP2vIdsPerThread + j;
    s_start[e] = bv;
    s_shift[e] = be;
    bv += hv[j];
    be += he[j];
  }
  if (t < 32) {  // (one half of the first wave)
    const int c = __popc((uint32_t)s_word[t]);
    int incl = c;
#pragma unroll
    for (int d = 1; d < 32; d <<= 1) {
      const int o = __shfl_up(incl, d, 64);
      if (t >= d) incl += o;
    }
    s_wprefix[t] = incl - c;
  }
  __syncthreads();
  if (blockIdx.x == 0 && t == 0) extra[0] = all_e;
  if ((int)blockIdx.x == n_point_blocks - 1 && t == 0)
    inside_total[0] = s_before + s_wprefix[31] + __popc((uint32_t)s_word[31]);
  float x = 0.f, y = 0.f, z = 0.f;
  int64_t id;
  int pos;
  const int64_t i = (int64_t)blockIdx.x * kP2vScanThreads + t;
  if ((int)blockIdx.x < n_point_blocks) {
    if (i >= n) return;
    id = ids[i];
    const uint32_t word = (uint32_t)s_word[t >> 5];
    const bool inside = ((word >> (t & 31)) & 1u) && id >= 0 && id < n_ids;
    pos = inside ? s_before + s_wprefix[t >> 5] + __popc(word & ((1u << (t & 31)) - 1u)) +
                       s_shift[inside ? (int)id : 0]
                 : -1;
    dest[i] = pos;
    if (!inside) return;
    x = pts[i * 3];
    y = pts[i * 3 + 1];
    z = pts[i * 3 + 2];
  } else {
    id = (int64_t)((int)blockIdx.x - n_point_blocks) * kP2vScanThreads + t;
    if (id >= n_ids || hist_all[id] == 0 || hist_valid[id] != 0) return;
    pos = s_start[id] + s_shift[id];
  }
  src[pos] = (int)blockIdx.x < n_point_blocks ? (int32_t)i : -1;  // input row behind row pos
  out_pts[(int64_t)pos * 3] = x;
  out_pts[(int64_t)pos * 3 + 1] = y;
  out_pts[(int64_t)pos * 3 + 2] = z;
  out_ids[pos] = id;
  const int vx = (int)((x + hx) / ux);
  const int vy = (int)((y + hy) / uy);
  const int vz = (int)((z + hz) / uz);
  reinterpret_cast<int4 *>(coords)[pos] = make_int4((int)id, vx, vy, vz);
  if ((unsigned)vx < (unsigned)d1 && (unsigned)vy < (unsigned)d2 && (unsigned)vz < (unsigned)d3) {
    const uint32_t key = (uint32_t)((((int)id * d1 + vx) * d2 + vy) * d3 + vz);
    atomicOr(&vox_bits[key >> 5], 1u << (key & 31u));
  } else {
    atomicOr(&flags[0], 4);
  }
}

// First pass of the scan over the voxel table; block 0 also hands the chain's other totals
// to the table's total[] -- [1] surviving points, [2] ids left without points, [3] flags
// (bit 0: an id outside the table, bit 1: ids decrease, bit 2: a voxel outside the grid) --
// from where the scan's second pass copies them, with the number of voxels, to the host.
__global__ void __launch_bounds__(kScanThreads)
    p2vx_vox_blocksum_kernel(const uint32_t *__restrict__ bits, int64_t n_words,
                             int32_t *__restrict__ blocksum,
                             const int32_t *__restrict__ inside_total,
                             const int32_t *__restrict__ extra,
                             const int32_t *__restrict__ flags, int32_t *__restrict__ vox_total) {
  __shared__ int lds[kScanThreads / 64 + 1];
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    vox_total[1] = inside_total[0];
    vox_total[2] = extra[0];
    vox_total[3] = (flags[0] & 5) | ((flags[1] & 1) << 1);
  }
  popc_blocksum_block(bits, n_words, blockIdx.x, blocksum, lds);
}

// Blocks below link_blocks: row pos < rows: inverse[pos] = rank of its voxel, and the row is
// pushed onto that voxel's chain.  The other blocks decode the voxel table into out_indices.
__global__ void __launch_bounds__(256)
    p2vx_link_kernel(const int32_t *__restrict__ coords, const int32_t *__restrict__ n_inside,
                     const int32_t *__restrict__ extra, const uint32_t *__restrict__ vox_bits,
                     const int32_t *__restrict__ vox_prefix, int64_t n_words, int d0, int d1,
                     int d2, int d3, int64_t link_blocks, const int32_t *__restrict__ flags,
                     int32_t *__restrict__ inverse, int32_t *__restrict__ head,
                     int32_t *__restrict__ next, int32_t *__restrict__ out_indices) {
  // With a flag set (ids outside the tables, ids out of order, a voxel outside the grid)
  // the compaction has left rows unwritten and the caller will discard everything: the
  // rows' tables must not be followed.
  if ((flags[0] | flags[1]) != 0) return;
  if ((int64_t)blockIdx.x >= link_blocks) {
    const int64_t step = (int64_t)(gridDim.x - link_blocks) * blockDim.x;
    int64_t w = ((int64_t)blockIdx.x - link_blocks) * blockDim.x + threadIdx.x;
    for (; w < n_words; w += step) emit_rows_of_word(vox_bits, vox_prefix, w, d1, d2, d3, out_indices);
    return;
  }
  const int64_t pos = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (pos >= (int64_t)n_inside[0] + extra[0]) return;
  const int4 r = reinterpret_cast<const int4 *>(coords)[pos];
  if (!((unsigned)r.x < (unsigned)d0 && (unsigned)r.y < (unsigned)d1 &&
        (unsigned)r.z < (unsigned)d2 && (unsigned)r.w < (unsigned)d3)) {
    inverse[pos] = -1;  // (flagged by the kernel that marked the table)
    return;
  }
  const uint32_t key = (uint32_t)(((r.x * d1 + r.y) * d2 + r.z) * d3 + r.w);
  const int rk = bit_rank(vox_bits, vox_prefix, key);
  inverse[pos] = rk;
  next[pos] = atomicExch(&head[rk], (int32_t)pos);
}

// The feature reduction of the one-call chain.  Eight lanes per voxel (eight voxels to a
// wave): the lanes walk the voxel's chain together (count, smallest and largest row, the
// first four rows), then
//   mode 1 / 2: the features of the first / last row,
//   mode 3 / 4: sum over the rows in ascending order of mult * feats, mult = 1 / count in
//               mode 4 (product rounded before the add, as in voxel_reduce_kernel).
// Nearly every voxel holds a point or two: up to four rows are ordered in registers.  A
// voxel with more is left to the whole wave afterwards (p2vx_reduce_long): rows of a window
// of 2048 row numbers are entered into a bit map, lane l holding word l, and read back bit
// by bit; windows follow each other upwards.  Lanes run along the channels.  src[row] is
// the input row behind a row (-1: a zero point).
__device__ __forceinline__ void p2vx_reduce_long(const float *__restrict__ feats, int C,
                                                 const int32_t *__restrict__ src,
                                                 const int32_t *__restrict__ next, int first,
                                                 int lo, int hi, float mult,
                                                 float *__restrict__ o, int lane) {
  for (int c0 = 0; c0 < C; c0 += 256) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    auto add_row = [&](int p) {
      const int sr = __builtin_amdgcn_readfirstlane(src[p]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int c = c0 + lane + 64 * j;
        if (c < C) {
          const float f = sr >= 0 ? feats[(int64_t)sr * C + c] : 0.f;
          const float t = mult * f;
          acc[j] = acc[j] + t;
        }
      }
    };
    for (int base = lo & ~2047; base <= hi; base += 2048) {
      uint32_t mine = 0u;
      for (int p = first; p >= 0; p = __builtin_amdgcn_readfirstlane(next[p])) {
        const int off = p - base;
        if ((unsigned)off < 2048u && (off >> 5) == lane) mine |= 1u << (off & 31);
      }
      unsigned long long lanes = __ballot(mine != 0u);
      while (lanes) {
        const int l = __ffsll((long long)lanes) - 1;
        lanes &= lanes - 1;
        uint32_t w = (uint32_t)__shfl((int)mine, l, 64);
        while (w) {
          const int b = __ffs((int)w) - 1;
          w &= w - 1;
          add_row(base + l * 32 + b);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = c0 + lane + 64 * j;
      if (c < C) o[c] = acc[j];
    }
  }
}

constexpr int kP2vGroup = 8;    // lanes to a voxel
constexpr int kP2vShort = 4;    // rows ordered in registers
// VEC: 4 when the rows hold a multiple of four channels (16-byte loads and stores), else 1.
template <int VEC>
__global__ void __launch_bounds__(256)
    p2vx_reduce_kernel(const float *__restrict__ feats, int C, const int32_t *__restrict__ src,
                       const int32_t *__restrict__ head, const int32_t *__restrict__ next,
                       const int32_t *__restrict__ n_voxel, const int32_t *__restrict__ flags,
                       int mode, float *__restrict__ out, int32_t *__restrict__ counts,
                       int32_t *__restrict__ sel) {
  if ((flags[0] | flags[1]) != 0) return;  // (see p2vx_link_kernel)
  const int lane = threadIdx.x & 63, gl = lane & (kP2vGroup - 1);
  const int64_t v = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * (64 / kP2vGroup) +
                    (lane / kP2vGroup);
  const bool live = v < n_voxel[0];
  const int first = live ? head[v] : -1;
  int n = 0, lo = 0x7FFFFFFF, hi = -1;
  int r[kP2vShort];
#pragma unroll
  for (int q = 0; q < kP2vShort; ++q) r[q] = 0x7FFFFFFF;
  for (int p = first; p >= 0; p = next[p]) {
#pragma unroll
    for (int q = 0; q < kP2vShort; ++q)
      if (n == q) r[q] = p;
    ++n;
    lo = p < lo ? p : lo;
    hi = p > hi ? p : hi;
  }
  if (live && gl == 0) counts[v] = n;
  float *o = out + v * C;
  const bool is_long = live && (mode == 3 || mode == 4) && n > kP2vShort;
  using Vec = typename std::conditional<VEC == 4, float4, float>::type;
  auto load = [&](int sr, int c) -> Vec {
    if constexpr (VEC == 4) {
      return sr >= 0 ? *reinterpret_cast<const float4 *>(feats + (int64_t)sr * C + c)
                     : make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
      return sr >= 0 ? feats[(int64_t)sr * C + c] : 0.f;
    }
  };
  if (live && (mode == 1 || mode == 2)) {
    const int p = mode == 1 ? lo : hi;
    if (gl == 0 && sel != nullptr) sel[v] = p;
    const int sr = n > 0 ? src[p] : -1;
    for (int c = gl * VEC; c < C; c += kP2vGroup * VEC) *reinterpret_cast<Vec *>(o + c) = load(sr, c);
  } else if (live && !is_long) {
    // ascending rows: a sorting network over the (at most) four row numbers, unused places
    // holding the largest integer
    auto order = [](int &a, int &b) {
      const int x = a < b ? a : b, y = a < b ? b : a;
      a = x;
      b = y;
    };
    order(r[0], r[1]);
    order(r[2], r[3]);
    order(r[0], r[2]);
    order(r[1], r[3]);
    order(r[1], r[2]);
    const float mult = (mode == 4 && n > 0) ? 1.f / (float)n : 1.f;
    int sr[kP2vShort];
#pragma unroll
    for (int q = 0; q < kP2vShort; ++q) sr[q] = q < n ? src[r[q]] : -1;
    for (int c = gl * VEC; c < C; c += kP2vGroup * VEC) {
      Vec f[kP2vShort];
#pragma unroll
      for (int q = 0; q < kP2vShort; ++q)
        if (q < n) f[q] = load(sr[q], c);
      float acc[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
#pragma unroll
      for (int q = 0; q < kP2vShort; ++q) {
        if (q < n) {
          const float *fe = reinterpret_cast<const float *>(&f[q]);
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const float t = mult * fe[e];
            acc[e] = acc[e] + t;
          }
        }
      }
      *reinterpret_cast<Vec *>(o + c) = *reinterpret_cast<const Vec *>(acc);
    }
  }
  // voxels with more rows, one after the other, by the whole wave
  unsigned long long todo = __ballot(is_long && gl == 0);
  while (todo) {
    const int l = __ffsll((long long)todo) - 1;
    todo &= todo - 1;
    const int64_t vv = (int64_t)__shfl((int)v, l, 64);  // (fewer than 2^31 voxels)
    const int f1 = __shfl(first, l, 64), n1 = __shfl(n, l, 64);
    const int lo1 = __shfl(lo, l, 64), hi1 = __shfl(hi, l, 64);
    const float mult = mode == 4 ? 1.f / (float)n1 : 1.f;
    p2vx_reduce_long(feats, C, src, next, f1, lo1, hi1, mult, out + vv * C, lane);
  }
}

// d_feats[i, c] of input row i: mult * d_out[voxel of its row] (modes 3 / 4), d_out for the
// row its voxel took its features from (modes 1 / 2), 0 for a dropped row
// (src/voxelize/voxelize_cuda_kernel.h:44-58 through the point lists).
__global__ void __launch_bounds__(256)
    p2vx_bwd_kernel(const float *__restrict__ d_out, int C, const int32_t *__restrict__ dest,
                    const int32_t *__restrict__ inverse, const int32_t *__restrict__ counts,
                    const int32_t *__restrict__ sel, int mode, int64_t n,
                    float *__restrict__ d_feats) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n * C) return;
  const int64_t i = e / C;
  const int c = (int)(e - i * C);
  float g = 0.f;
  const int pos = dest[i];
  if (pos >= 0) {
    const int v = inverse[pos];
    if (v >= 0) {
      if (mode == 1 || mode == 2) {
        if (sel[v] == pos) g = d_out[(int64_t)v * C + c];
      } else {
        const float mult = mode == 4 ? 1.f / (float)counts[v] : 1.f;
        g = mult * d_out[(int64_t)v * C + c];
      }
    }
  }
  d_feats[e] = g;
}

struct P2vxWs {
  BitTable inside;  // over the n points
  BitTable vox;     // over the voxel grid
  int32_t *hist_all, *hist_valid, *flags, *start, *shift;
  int32_t *coords, *head, *next, *src, *totals;
};

static size_t p2vx_ws_walk(void *base, int64_t n, int64_t cells, P2vxWs *w) {
  Carver c(base);
  P2vxWs t;
  const size_t rows = (size_t)(n > 0 ? n : 1);
  t.inside = bit_table_carve(c, (int64_t)rows);
  t.vox = bit_table_carve(c, cells);
  t.hist_all = c.take<int32_t>(SSC_P2V_MAX_IDS);
  t.hist_valid = c.take<int32_t>(SSC_P2V_MAX_IDS);  // directly behind hist_all
  t.flags = c.take<int32_t>(2);                      // directly behind hist_valid
  t.start = c.take<int32_t>(SSC_P2V_MAX_IDS);
  t.shift = c.take<int32_t>(SSC_P2V_MAX_IDS);
  t.coords = c.take<int32_t>(rows * 4);
  t.head = c.take<int32_t>(rows);
  t.next = c.take<int32_t>(rows);
  t.src = c.take<int32_t>(rows);
  t.totals = c.take<int32_t>(8);
  if (w) *w = t;
  return c.used;
}

static int64_t p2vx_cells(int32_t n_ids, const int32_t limit[3]) {
  if (n_ids < 1 || n_ids > SSC_P2V_MAX_IDS) return 0;
  int64_t cells = n_ids;
  for (int a = 0; a < 3; ++a) {
    if (limit[a] < 1) return 0;
    cells *= (int64_t)limit[a] + 1;  // a point on the upper face has index == limit
    if (cells >= ((int64_t)1 << 31)) return 0;
  }
  return cells;
}

}  // namespace ssc

extern "C" {

size_t ssc_p2v_voxelize_workspace_bytes(int64_t n, int32_t n_ids, const int32_t limit[3]) {
  if (n < 0 || limit == nullptr) return 0;
  const int64_t cells = ssc::p2vx_cells(n_ids, limit);
  if (cells == 0) return 0;
  return ssc::p2vx_ws_walk(nullptr, n, cells, nullptr);
}

int ssc_p2v_voxelize_f32(const float *points, const float *feats, const int64_t *batch_ids,
                         int64_t n, int32_t channels, const float half_extent[3],
                         const float unit[3], const int32_t limit[3], int32_t n_ids, int32_t mode,
                         void *workspace, size_t workspace_bytes, float *out_points,
                         int64_t *out_ids, int32_t *out_indices, float *out_feats,
                         int32_t *inverse, int32_t *counts, int32_t *dest, int32_t *sel,
                         int32_t *hist_all_host, int32_t *hist_valid_host, int32_t *totals_host,
                         ssc_stream_t stream) {
  SSC_CHECK(n > 0 && n < ((int64_t)1 << 31) && channels >= 1, SSC_EINVAL, "bad sizes");
  SSC_CHECK(mode >= 1 && mode <= 4, SSC_EINVAL, "mode must be 1, 2, 3 or 4");
  SSC_CHECK(points && feats && batch_ids && half_extent && unit && limit && workspace &&
                out_points && out_ids && out_indices && out_feats && inverse && counts && dest &&
                hist_all_host && hist_valid_host && totals_host,
            SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(mode >= 3 || sel != nullptr, SSC_EINVAL, "sel is NULL (modes 1 and 2 need it)");
  const int64_t cells = p2vx_cells(n_ids, limit);
  SSC_CHECK(cells > 0, SSC_EINVAL,
            "n_ids must lie in [1, %d] and n_ids * prod(limit + 1) below 2^31",
            (int)SSC_P2V_MAX_IDS);
  SSC_CHECK(workspace_bytes >= p2vx_ws_walk(nullptr, n, cells, nullptr), SSC_EWORKSPACE,
            "p2v workspace too small");
  static_assert((16 + 2 * SSC_P2V_MAX_IDS) * sizeof(int32_t) <= kReadBackBytes, "pinned block");
  hipStream_t s = (hipStream_t)stream;
  P2vxWs w;
  p2vx_ws_walk(workspace, n, cells, &w);
  const int d1 = limit[0] + 1, d2 = limit[1] + 1, d3 = limit[2] + 1;
  int rc;
  int32_t *mirror = nullptr;
  if ((rc = read_back_mirror(&mirror)) != SSC_OK) return rc;
  // mirror: [0..3] sizes and flags (the voxel table's scan), [16 ..) the two histograms
  int32_t *extra = w.totals;  // [0]: ids left without points

  const int64_t clear_a = (w.flags + 2) - w.hist_all;
  const int64_t clear_most = w.vox.n_words > n ? w.vox.n_words : n;
  const int64_t clear_blocks = ceil_div(clear_most > clear_a ? clear_most : clear_a, 256);
  hipLaunchKernelGGL(p2vx_clear_kernel, dim3((unsigned)(clear_blocks < 4096 ? clear_blocks : 4096)),
                     dim3(256), 0, s, w.hist_all, clear_a, w.vox.bits, w.vox.n_words, w.head, n,
                     w.totals);
  SSC_LAUNCH_CHECK("p2vx_clear");
  const int64_t point_blocks = ceil_div(n, kP2vScanThreads);
  hipLaunchKernelGGL(p2v_scan_kernel, dim3((unsigned)point_blocks), dim3(kP2vScanThreads), 0, s,
                     points, batch_ids, n, half_extent[0], half_extent[1], half_extent[2],
                     (int)n_ids, w.inside.bits, w.hist_all, w.hist_valid, w.flags,
                     w.inside.prefix /* the blocks' inside counts */);
  SSC_LAUNCH_CHECK("p2v_scan");
  // the compaction ranks its points from the blocks' counts and scans the histograms for
  // itself: no scan of the inside bits, no launch for the per-id tables
  hipLaunchKernelGGL(p2vx_compact_kernel,
                     dim3((unsigned)(point_blocks + ceil_div(n_ids, kP2vScanThreads))),
                     dim3(kP2vScanThreads), 0, s, points, batch_ids, n, w.inside.bits,
                     w.inside.prefix, (int)point_blocks, w.hist_all, w.hist_valid, half_extent[0],
                     half_extent[1], half_extent[2], unit[0], unit[1], unit[2], out_points,
                     out_ids, w.coords, dest, w.src, (int)n_ids, w.vox.bits, d1, d2, d3, w.flags,
                     w.inside.total, extra, mirror + 16);
  SSC_LAUNCH_CHECK("p2vx_compact");
  // the scan of the voxel table; its first pass hands the other totals and the flags to the
  // table's total[], its second pass copies all of them to the host's mirror: [0] voxels,
  // [1] surviving points, [2] ids left without points, [3] flags.  Then the event the host
  // will wait for; the two kernels after it run while the host wakes up
  hipLaunchKernelGGL(p2vx_vox_blocksum_kernel, dim3((unsigned)w.vox.n_scan_blocks),
                     dim3(kScanThreads), 0, s, w.vox.bits, w.vox.n_words, w.vox.blocksum,
                     w.inside.total, extra, w.flags, w.vox.total);
  SSC_LAUNCH_CHECK("p2vx_vox_blocksum");
  const int ticket = read_back_mirror_ticket();
  if ((rc = bit_table_scan_prefix(w.vox, s, mirror, ticket)) != SSC_OK) return rc;
  if ((rc = read_back_mirror_queued(s, ticket)) != SSC_OK) return rc;
  const int64_t link_blocks = ceil_div(n, 256);
  int64_t row_blocks = ceil_div(w.vox.n_words, 256);
  if (row_blocks > 2048) row_blocks = 2048;
  hipLaunchKernelGGL(p2vx_link_kernel, dim3((unsigned)(link_blocks + row_blocks)), dim3(256), 0, s,
                     w.coords, w.inside.total, extra, w.vox.bits, w.vox.prefix, w.vox.n_words,
                     (int)n_ids, d1, d2, d3, link_blocks, w.flags, inverse, w.head, w.next,
                     out_indices);
  SSC_LAUNCH_CHECK("p2vx_link");
  // (16-byte accesses need rows of a multiple of four channels from aligned bases)
  const bool vec4 = (channels & 3) == 0 && (((uintptr_t)feats | (uintptr_t)out_feats) & 15) == 0;
  hipLaunchKernelGGL(vec4 ? p2vx_reduce_kernel<4> : p2vx_reduce_kernel<1>,
                     dim3((unsigned)ceil_div(n, 4 * (64 / kP2vGroup))), dim3(256), 0, s, feats,
                     (int)channels, w.src, w.head, w.next, w.vox.total, w.flags, (int)mode, out_feats,
                     counts, sel);
  SSC_LAUNCH_CHECK("p2vx_reduce");
  const void *view;
  if ((rc = read_back_end(&view)) != SSC_OK) return rc;
  const int32_t *m = static_cast<const int32_t *>(view);
  totals_host[0] = m[1] + m[2];  // rows: survivors + zero points
  totals_host[1] = m[0];         // voxels
  totals_host[2] = m[3];         // flags
  totals_host[3] = m[2];         // ids left without points
  memcpy(hist_all_host, m + 16, (size_t)n_ids * sizeof(int32_t));
  memcpy(hist_valid_host, m + 16 + n_ids, (size_t)n_ids * sizeof(int32_t));
  // what callers ask the histograms first: how many ids there are, how many of them kept
  // points, and the largest one
  int present = 0, alive = 0, largest = -1;
  for (int i = 0; i < n_ids; ++i) {
    if (hist_all_host[i] > 0) {
      ++present;
      largest = i;
      alive += hist_valid_host[i] > 0;
    }
  }
  totals_host[4] = present;
  totals_host[5] = alive;
  totals_host[6] = largest;
  totals_host[7] = 0;
  return SSC_OK;
}

int ssc_p2v_voxelize_bwd_f32(const float *out_grad, int32_t channels, const int32_t *dest,
                             const int32_t *inverse, const int32_t *counts, const int32_t *sel,
                             int32_t mode, int64_t n, float *feats_grad, ssc_stream_t stream) {
  SSC_CHECK(n >= 0 && channels >= 1 && mode >= 1 && mode <= 4, SSC_EINVAL, "bad sizes");
  if (n == 0) return SSC_OK;
  SSC_CHECK(out_grad && dest && inverse && counts && feats_grad, SSC_EINVAL,
            "NULL pointer argument");
  SSC_CHECK(mode >= 3 || sel != nullptr, SSC_EINVAL, "sel is NULL (modes 1 and 2 need it)");
  hipLaunchKernelGGL(p2vx_bwd_kernel, dim3((unsigned)ceil_div(n * channels, 256)), dim3(256), 0,
                     (hipStream_t)stream, out_grad, (int)channels, dest, inverse, counts, sel,
                     (int)mode, n, feats_grad);
  SSC_LAUNCH_CHECK("p2vx_bwd");
  return SSC_OK;
}
}

// ---- backward of the feature reduction and of the interpolation ---------------------------
namespace ssc {

// d_feats[p,c] = mult * d_out[v,c] for every point p in voxel v's list (a point is in at
// most one list, so these are plain stores); src/voxelize/voxelize_cuda_kernel.h:44-58.
__global__ void __launch_bounds__(256)
    voxel_reduce_bwd_kernel(const float *__restrict__ d_out, float *__restrict__ d_feats,
                            const int32_t *__restrict__ maps, int mode, int64_t n_voxel,
                            int max_active, int C) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n_voxel * C) return;
  int64_t v = idx / C;
  int c = (int)(idx - v * C);
  const int32_t *r = maps + v * (max_active + 1);
  int na = r[0];
  float mult = (mode == 4 && na > 0) ? 1.f / (float)na : 1.f;
  float g = mult * d_out[idx];
  for (int i = 1; i <= na; ++i) d_feats[(int64_t)r[i] * C + c] = g;
}

// grad_points[idx[q,j], c] += grad_out[q,c] * weight[q,j]: several queries share a row, so
// this accumulates with float atomics, as src/voxelize/interpolate_cuda_kernel.cu:104-121
// does (the order of the additions, hence the last bits, is not fixed there either).
__global__ void __launch_bounds__(256)
    three_interp_bwd_kernel(int C, int n, const float *__restrict__ grad_out,
                            const int32_t *__restrict__ idx, const float *__restrict__ weight,
                            float *__restrict__ grad_points) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (int64_t)n * C) return;
  int64_t q = e / C;
  int c = (int)(e - q * C);
  float g = grad_out[e];
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    float t = g * weight[q * 3 + j];
    atomicAdd(&grad_points[(int64_t)idx[q * 3 + j] * C + c], t);
  }
}

}  // namespace ssc

extern "C" {

int ssc_voxel_reduce_bwd_f32(const float *out_grad, float *feats_grad, const int32_t *maps,
                             int32_t mode, int32_t n_voxel, int32_t max_active, int32_t channels,
                             int64_t n_point, ssc_stream_t stream) {
  SSC_CHECK(n_voxel >= 0 && max_active >= 1 && channels >= 1 && n_point >= 0, SSC_EINVAL,
            "bad sizes");
  if (n_point == 0) return SSC_OK;
  SSC_CHECK(feats_grad != nullptr, SSC_EINVAL, "feats_grad is NULL");
  hipStream_t s = (hipStream_t)stream;
  int rc = ssc::fill_f32(feats_grad, n_point * channels, 0.f, s);
  if (rc != SSC_OK || n_voxel == 0) return rc;
  SSC_CHECK(out_grad && maps, SSC_EINVAL, "NULL pointer argument");
  int64_t n = (int64_t)n_voxel * channels;
  hipLaunchKernelGGL(ssc::voxel_reduce_bwd_kernel, dim3((unsigned)ssc::ceil_div(n, 256)), dim3(256),
                     0, s, out_grad, feats_grad, maps, mode, (int64_t)n_voxel, max_active, channels);
  SSC_LAUNCH_CHECK("voxel_reduce_bwd");
  return SSC_OK;
}

int ssc_three_interp_bwd_f32(int32_t c, int32_t n, int32_t m, const float *out_grad,
                             const int32_t *idx, const float *weight, float *points_grad,
                             ssc_stream_t stream) {
  SSC_CHECK(c >= 1 && n >= 0 && m >= 0, SSC_EINVAL, "bad sizes");
  if (m == 0) return SSC_OK;
  SSC_CHECK(points_grad != nullptr, SSC_EINVAL, "points_grad is NULL");
  hipStream_t s = (hipStream_t)stream;
  int rc = ssc::fill_f32(points_grad, (int64_t)m * c, 0.f, s);
  if (rc != SSC_OK || n == 0) return rc;
  SSC_CHECK(out_grad && idx && weight, SSC_EINVAL, "NULL pointer argument");
  int64_t e = (int64_t)n * c;
  hipLaunchKernelGGL(ssc::three_interp_bwd_kernel, dim3((unsigned)ssc::ceil_div(e, 256)), dim3(256),
                     0, s, c, n, out_grad, idx, weight, points_grad);
  SSC_LAUNCH_CHECK("three_interp_bwd");
  return SSC_OK;
}
}
