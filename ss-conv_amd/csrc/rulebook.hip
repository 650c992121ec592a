// Rulebook (indice pair) generation and sorted-unique of voxel coordinates.
//
// Both are "number a set of grid cells in ascending flat-key order" problems.
// The set is held as a bit table over the dense key space (1 bit per cell:
// 32x smaller than the reference's int32 grid, L2/MALL resident at the sizes
// this path sees) and a popcount prefix turns membership into the rank of the
// key, i.e. the output row.  No sort, no probing, no result-bearing atomics:
// atomicOr on the bit table is order independent.
#include "conv_pack.h"
#include "ssc_common.h"

namespace ssc {

struct Geom {
  int batch;
  int os[3], ks[3], st[3], pd[3], dl[3];
  int K;
  int subm;
  int tr;  // transposed convolution: out = in * stride - padding + k * dilation
};

static int make_geom(const ssc_geometry *g, Geom *o) {
  SSC_CHECK(g != nullptr, SSC_EINVAL, "geometry is NULL");
  o->batch = g->batch_size;
  o->subm = g->subm != 0;
  o->tr = !o->subm && g->transpose != 0;  // src/conv/indice_conv.h:76-101: subm comes first
  o->K = 1;
  for (int a = 0; a < 3; ++a) {
    o->os[a] = g->out_shape[a];
    o->ks[a] = g->ksize[a];
    o->dl[a] = g->dilation[a];
    if (o->subm) {  // src/conv/indice_conv.h:70-74
      o->st[a] = 1;
      o->pd[a] = g->ksize[a] / 2;
    } else {
      o->st[a] = g->stride[a];
      o->pd[a] = g->padding[a];
    }
    SSC_CHECK(o->ks[a] >= 1 && o->st[a] >= 1 && o->dl[a] >= 1 && o->pd[a] >= 0 && o->os[a] >= 1,
              SSC_EINVAL, "bad geometry in dimension %d", a);
    SSC_CHECK(o->st[a] == 1 || o->dl[a] == 1, SSC_EINVAL,
              "stride > 1 together with dilation > 1 is not supported");
    o->K *= o->ks[a];
  }
  SSC_CHECK(o->K <= SSC_MAX_KERNEL_VOLUME, SSC_ERUNTIME, "kernel volume %d exceeds %d", o->K,
            SSC_MAX_KERNEL_VOLUME);
  SSC_CHECK(o->batch >= 1, SSC_EINVAL, "batch_size must be positive");
  int64_t cells = (int64_t)o->batch * o->os[0] * o->os[1] * o->os[2];
  SSC_CHECK(cells < ((int64_t)1 << 31), SSC_ERUNTIME,
            "batch_size * prod(out_shape) = %lld does not fit 31 bits", (long long)cells);
  return SSC_OK;
}

static inline int64_t geom_cells(const Geom &g) {
  return (int64_t)g.batch * g.os[0] * g.os[1] * g.os[2];
}

// Output position reached from input coordinate `in` through kernel tap `k` in
// one dimension: (in + p - k*d) / s when that is a non-negative multiple of s
// and inside the output extent.  Equivalent to the candidate enumeration of
// src/conv/geometry.h:18-80 (stride>1 with dilation>1 is rejected on the host).
// Transposed (`tr`): in*s - p + k*d when inside the extent (src/conv/geometry.h:82-138).
__device__ __forceinline__ bool tap_to_out(int in, int k, int s, int p, int d, int extent,
                                           int *out, bool tr = false) {
  if (tr) {
    const int t = in * s - p + k * d;
    if (t < 0 || t >= extent) return false;
    *out = t;
    return true;
  }
  int t = in + p - k * d;
  if (t < 0) return false;
  int q = t / s;
  if (q * s != t || q >= extent) return false;
  *out = q;
  return true;
}

__device__ __forceinline__ bool pair_key(const Geom &g, const int32_t *__restrict__ row, int k,
                                         uint32_t *key) {
  int kz = k % g.ks[2];
  int ky = (k / g.ks[2]) % g.ks[1];
  int kx = k / (g.ks[2] * g.ks[1]);
  int ox, oy, oz;
  const bool tr = g.tr != 0;
  if (!tap_to_out(row[1], kx, g.st[0], g.pd[0], g.dl[0], g.os[0], &ox, tr)) return false;
  if (!tap_to_out(row[2], ky, g.st[1], g.pd[1], g.dl[1], g.os[1], &oy, tr)) return false;
  if (!tap_to_out(row[3], kz, g.st[2], g.pd[2], g.dl[2], g.os[2], &oz, tr)) return false;
  *key = (uint32_t)(((row[0] * g.os[0] + ox) * g.os[1] + oy) * g.os[2] + oz);
  return true;
}

// (b, x, y, z) of row a strictly before row b in key order
__device__ __forceinline__ bool row_before(const int4 &a, const int4 &b) {
  if (a.x != b.x) return a.x < b.x;
  if (a.y != b.y) return a.y < b.y;
  if (a.z != b.z) return a.z < b.z;
  return a.w < b.w;
}

// Flag word of a table (total[1]): bit 0 = the rows do not come in strictly ascending key
// order; bit 1 = some row lies outside the grid.  Such a row is skipped by every kernel (its
// key would address memory outside the table), and the host turns the bit into an error.
constexpr int kFlagDisorder = 1;
constexpr int kFlagBadRow = 2;

// A regular convolution reaches only output cells inside the grid whatever the spatial
// coordinates of a row are, so only its batch index must be checked; a submanifold
// rulebook and the unique-rows table use the row's own cell.
__device__ __forceinline__ bool batch_in_range(const int32_t *row, const Geom &g) {
  return (unsigned)row[0] < (unsigned)g.batch;
}
__device__ __forceinline__ bool cell_in_range(const int4 &r, int d0, int d1, int d2, int d3) {
  return (unsigned)r.x < (unsigned)d0 && (unsigned)r.y < (unsigned)d1 &&
         (unsigned)r.z < (unsigned)d2 && (unsigned)r.w < (unsigned)d3;
}
__device__ __forceinline__ bool row_usable(const int32_t *row, const Geom &g) {
  if (!g.subm) return batch_in_range(row, g);
  return cell_in_range(*reinterpret_cast<const int4 *>(row), g.batch, g.os[0], g.os[1], g.os[2]);
}

// The share of grid row `row` of `rows` (of gridDim.x blocks of 256 threads each) in a
// layer's filter job.
__device__ __forceinline__ void combine_job_rows(const CombineJob &job, int64_t job_elements,
                                                 int row, int rows) {
  const int64_t step = (int64_t)rows * gridDim.x * 256;
  for (int64_t idx = ((int64_t)row * gridDim.x + blockIdx.x) * 256 + threadIdx.x;
       idx < job_elements; idx += step)
    combine_pack_element(job, idx);
}

// Regular conv: mark every output cell reachable from an active input, and count
// the pairs of every 64-row chunk (chunk_count is [K, n_chunks]; for a regular
// convolution a pair exists wherever the geometry allows it, so the counts do not
// depend on the table).  One wave per chunk of 64 input rows and x offset, one lane per row.
// disorder[0] |= 1 when some input row does not come strictly before its successor.
// The taps of one (kx, ky) differ in z only, so their output cells are neighbours
// in the key space: their bits are gathered into one mask per 32-bit word, the word
// is read first, and the atomic is issued only when it would change the word
// (most cells are reached from several inputs).
// JOB: the grid rows from ks[0] on synthesise and pack the layer's filters (work that
// depends on nothing here and that the layer would otherwise launch by itself).
// word_pairs (optional, zero on entry): word_pairs[w] += the pairs that land on the cells of
// table word w (integer adds: the sums do not depend on their order), the work measure of a
// convolution's plan (see SplitRequest).
template <bool JOB>
__global__ void __launch_bounds__(256)
    mark_count_kernel(const int32_t *__restrict__ indices, int64_t n_in, Geom g,
                      uint32_t *__restrict__ bits, int32_t *__restrict__ chunk_count,
                      int64_t n_chunks, int32_t *__restrict__ disorder, CombineJob job,
                      int64_t job_elements, int32_t *__restrict__ word_pairs) {
  if constexpr (JOB) {
    if ((int)blockIdx.y >= g.ks[0]) {
      combine_job_rows(job, job_elements, (int)blockIdx.y - g.ks[0], (int)gridDim.y - g.ks[0]);
      return;
    }
  }
  int64_t chunk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (chunk >= n_chunks) return;
  const int lane = threadIdx.x & 63;
  int64_t i = chunk * 64 + lane;
  bool live = i < n_in;
  int32_t row[4] = {0, 0, 0, 0};
  if (live) *reinterpret_cast<int4 *>(row) = reinterpret_cast<const int4 *>(indices)[i];
  if (blockIdx.y == 0 && i + 1 < n_in &&
      !row_before(*reinterpret_cast<int4 *>(row), reinterpret_cast<const int4 *>(indices)[i + 1]))
    atomicOr(disorder, kFlagDisorder);
  if (live && !batch_in_range(row, g)) {
    if (blockIdx.y == 0) atomicOr(disorder, kFlagBadRow);
    live = false;
  }
  // blockIdx.y = kx: the taps of one x offset per wave, for more waves in flight
  const int kx = blockIdx.y;
  int k = kx * g.ks[1] * g.ks[2];
  {
    int ox = 0;
    const bool tr = g.tr != 0;
    const bool okx = live && tap_to_out(row[1], kx, g.st[0], g.pd[0], g.dl[0], g.os[0], &ox, tr);
    // the cells a row reaches through the taps of one (kx, ky) are distinct: every bit of
    // `mask` is one pair
    auto flush = [&](uint32_t word, uint32_t mask) {
      if (mask == 0u) return;
      if ((bits[word] & mask) != mask) atomicOr(&bits[word], mask);
      if (word_pairs != nullptr) atomicAdd(&word_pairs[word], __popc(mask));
    };
    for (int ky = 0; ky < g.ks[1]; ++ky) {
      int oy = 0;
      const bool okxy =
          okx && tap_to_out(row[2], ky, g.st[1], g.pd[1], g.dl[1], g.os[1], &oy, tr);
      const uint32_t base = (uint32_t)(((row[0] * g.os[0] + ox) * g.os[1] + oy) * g.os[2]);
      uint32_t word = 0xFFFFFFFFu, mask = 0u;
      for (int kz = 0; kz < g.ks[2]; ++kz, ++k) {
        int oz = 0;
        const bool ok =
            okxy && tap_to_out(row[3], kz, g.st[2], g.pd[2], g.dl[2], g.os[2], &oz, tr);
        unsigned long long m = __ballot(ok);
        if (lane == 0) chunk_count[(int64_t)k * n_chunks + chunk] = __popcll(m);
        if (ok) {
          const uint32_t key = base + (uint32_t)oz;
          if ((key >> 5) != word) {
            flush(word, mask);
            word = key >> 5;
            mask = 0u;
          }
          mask |= 1u << (key & 31u);
        }
      }
      if (word_pairs == nullptr) {
        flush(word, mask);
        continue;
      }
      // The rows of a wave are neighbours in key order, so the words their taps end in come
      // in runs of equal lanes: the first lane of a run adds the run's pairs with one atomic
      // (a wave's 64 adds to one address would be served one after the other).
      if (mask != 0u && (bits[word] & mask) != mask) atomicOr(&bits[word], mask);
      const int cnt = __popc(mask);
      if (mask == 0u) word = 0xFFFFFFFFu;
      const uint32_t before = __shfl_up(word, 1, 64);
      const bool head = lane == 0 || word != before;
      const unsigned long long heads = __ballot(head);
      int incl = cnt;
#pragma unroll
      for (int dd = 1; dd < 64; dd <<= 1) {
        const int o = __shfl_up(incl, dd, 64);
        if (lane >= dd) incl += o;
      }
      // the run of a first lane ends before the next first lane
      const unsigned long long later = lane < 63 ? heads >> (lane + 1) : 0ull;
      const int last = later != 0ull ? lane + __ffsll((long long)later) - 1 : 63;
      const int run = __shfl(incl, last, 64) - (incl - cnt);
      if (head && run > 0) atomicAdd(&word_pairs[word], run);
    }
  }
}

// ---- marking by dilation -------------------------------------------------------------------
// With stride 1 and dilation 1 the active outputs are the active inputs dilated by the
// kernel's extent: output o is active when some input sits at o - p + k, 0 <= k < ks.  In
// the shifted coordinate u = i + p that reads u - k = o, so an input table over
// u in [0, os + ks - 1) per axis holds every input that can reach the grid.  Marking then
// costs one atomic per input row (instead of one per row and (kx, ky)), and the output table
// is computed word by word from the input table -- no atomics, every word written, so it
// needs no clearing -- by the kernel that also sums the words' popcounts for the scan.
// Rows of the output table must be whole words (os[2] a multiple of 32).
struct DenseIn {
  int U[3];  // extents of the input table per batch element
  int Wz;    // words per z row
};

static inline bool dense_marking_applies(const Geom &g, int64_t n_in, DenseIn *d) {
  if (g.subm || g.tr || (g.os[2] & 31) != 0) return false;
  for (int a = 0; a < 3; ++a)
    if (g.st[a] != 1 || g.dl[a] != 1 || g.ks[a] > 32) return false;
  for (int a = 0; a < 3; ++a) d->U[a] = g.os[a] + g.ks[a] - 1;
  d->Wz = (d->U[2] + 31) / 32;
  const int64_t in_words = (int64_t)g.batch * d->U[0] * d->U[1] * d->Wz;
  // the dilation walks the whole table: not for a few voxels in a huge grid
  return in_words < ((int64_t)1 << 26) && geom_cells(g) / 32 <= 64 * n_in;
}

static inline int64_t dense_in_words(const Geom &g, const DenseIn &d) {
  return (int64_t)g.batch * d.U[0] * d.U[1] * d.Wz;
}

// As mark_count_kernel (same grid, same chunk counts, same flags), but the wave marks the
// cells of its input rows in the input table instead of the output cells they reach.
// JOB: as for mark_count_kernel.
template <bool JOB>
__global__ void __launch_bounds__(256)
    mark_in_count_kernel(const int32_t *__restrict__ indices, int64_t n_in, Geom g, DenseIn d,
                         uint32_t *__restrict__ in_bits, int32_t *__restrict__ chunk_count,
                         int64_t n_chunks, int32_t *__restrict__ flags, CombineJob job,
                         int64_t job_elements) {
  if constexpr (JOB) {
    if ((int)blockIdx.y >= g.ks[0]) {
      combine_job_rows(job, job_elements, (int)blockIdx.y - g.ks[0], (int)gridDim.y - g.ks[0]);
      return;
    }
  }
  int64_t chunk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (chunk >= n_chunks) return;
  const int lane = threadIdx.x & 63;
  int64_t i = chunk * 64 + lane;
  bool live = i < n_in;
  int32_t row[4] = {0, 0, 0, 0};
  if (live) *reinterpret_cast<int4 *>(row) = reinterpret_cast<const int4 *>(indices)[i];
  if (blockIdx.y == 0 && i + 1 < n_in &&
      !row_before(*reinterpret_cast<int4 *>(row), reinterpret_cast<const int4 *>(indices)[i + 1]))
    atomicOr(flags, kFlagDisorder);
  if (live && !batch_in_range(row, g)) {
    if (blockIdx.y == 0) atomicOr(flags, kFlagBadRow);
    live = false;
  }
  if (blockIdx.y == 0 && live) {
    const int ux = row[1] + g.pd[0], uy = row[2] + g.pd[1], uz = row[3] + g.pd[2];
    if ((unsigned)ux < (unsigned)d.U[0] && (unsigned)uy < (unsigned)d.U[1] &&
        (unsigned)uz < (unsigned)d.U[2]) {
      const int64_t w = (((int64_t)row[0] * d.U[0] + ux) * d.U[1] + uy) * d.Wz + (uz >> 5);
      atomicOr(&in_bits[w], 1u << (uz & 31));
    }
  }
  const int kx = blockIdx.y;
  int k = kx * g.ks[1] * g.ks[2];
  int ox = 0;
  const bool okx = live && tap_to_out(row[1], kx, 1, g.pd[0], 1, g.os[0], &ox);
  for (int ky = 0; ky < g.ks[1]; ++ky) {
    int oy = 0;
    const bool okxy = okx && tap_to_out(row[2], ky, 1, g.pd[1], 1, g.os[1], &oy);
    for (int kz = 0; kz < g.ks[2]; ++kz, ++k) {
      int oz = 0;
      const bool ok = okxy && tap_to_out(row[3], kz, 1, g.pd[2], 1, g.os[2], &oz);
      unsigned long long m = __ballot(ok);
      if (lane == 0) chunk_count[(int64_t)k * n_chunks + chunk] = __popcll(m);
    }
  }
}

// Submanifold / unique: mark the cells of the rows themselves.
// JOB: the blocks behind those of the rows work on a layer's filter job (see mark_count_kernel).
template <bool JOB>
__global__ void __launch_bounds__(256)
    mark_rows_kernel(const int32_t *__restrict__ coords, int64_t n, int d0, int d1, int d2, int d3,
                     uint32_t *__restrict__ bits, int32_t *__restrict__ flags, int want_order,
                     CombineJob job, int64_t job_elements) {
  if constexpr (JOB) {
    const int64_t row_blocks = (n + 255) / 256;
    if ((int64_t)blockIdx.x >= row_blocks) {
      const int64_t step = ((int64_t)gridDim.x - row_blocks) * 256;
      for (int64_t idx = ((int64_t)blockIdx.x - row_blocks) * 256 + threadIdx.x;
           idx < job_elements; idx += step)
        combine_pack_element(job, idx);
      return;
    }
  }
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int4 r = reinterpret_cast<const int4 *>(coords)[i];
  if (want_order && i + 1 < n && !row_before(r, reinterpret_cast<const int4 *>(coords)[i + 1]))
    atomicOr(flags, kFlagDisorder);
  if (!cell_in_range(r, d0, d1, d2, d3)) {
    atomicOr(flags, kFlagBadRow);
    return;
  }
  uint32_t key = (uint32_t)(((r.x * d1 + r.y) * d2 + r.z) * d3 + r.w);
  atomicOr(&bits[key >> 5], 1u << (key & 31u));
}

__global__ void __launch_bounds__(256)
    emit_rows_kernel(const uint32_t *__restrict__ bits, const int32_t *__restrict__ prefix,
                     int64_t n_words, int d1, int d2, int d3, int32_t *__restrict__ out) {
  int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (w < n_words) emit_rows_of_word(bits, prefix, w, d1, d2, d3, out);
}

// rank -> input row, for the submanifold rulebook (outputs keep the input numbering).
__global__ void __launch_bounds__(256)
    rank_to_row_kernel(const int32_t *__restrict__ indices, int64_t n_in, Geom g,
                       const uint32_t *__restrict__ bits, const int32_t *__restrict__ prefix,
                       int32_t *__restrict__ rank2row) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_in) return;
  int4 r = reinterpret_cast<const int4 *>(indices)[i];
  if (!cell_in_range(r, g.batch, g.os[0], g.os[1], g.os[2])) return;
  uint32_t key = (uint32_t)(((r.x * g.os[0] + r.y) * g.os[1] + r.z) * g.os[2] + r.w);
  rank2row[bit_rank(bits, prefix, key)] = (int32_t)i;
}

__device__ __forceinline__ bool bit_test(const uint32_t *__restrict__ bits, uint32_t key) {
  return (bits[key >> 5] >> (key & 31u)) & 1u;
}

// Pair counting for the submanifold rulebook (a pair needs its output cell to be
// active): one wave per chunk of 64 input rows, per tap the number of rows of the
// chunk that own a pair.  chunk_count is [K, n_chunks].
__global__ void __launch_bounds__(256)
    count_pairs_kernel(const int32_t *__restrict__ indices, int64_t n_in, Geom g,
                       const uint32_t *__restrict__ bits, int32_t *__restrict__ chunk_count,
                       int64_t n_chunks) {
  int64_t chunk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (chunk >= n_chunks) return;
  int lane = threadIdx.x & 63;
  int64_t i = chunk * 64 + lane;
  bool live = i < n_in;
  int32_t row[4] = {0, 0, 0, 0};
  if (live) *reinterpret_cast<int4 *>(row) = reinterpret_cast<const int4 *>(indices)[i];
  live = live && row_usable(row, g);
  for (int k = 0; k < g.K; ++k) {
    uint32_t key;
    bool ok = live && pair_key(g, row, k, &key);
    if (ok && g.subm) ok = bit_test(bits, key);
    unsigned long long m = __ballot(ok);
    if (lane == 0) chunk_count[(int64_t)k * n_chunks + chunk] = __popcll(m);
  }
}

// Per tap: exclusive scan of the chunk counts in place; the total is pair_num[k].
__device__ __forceinline__ void scan_chunks_of_tap(int32_t *__restrict__ chunk_count,
                                                   int64_t n_chunks, int k,
                                                   int32_t *__restrict__ pair_num, int *lds) {
  int32_t *c = chunk_count + (int64_t)k * n_chunks;
  int carry = 0;
  for (int64_t base = 0; base < n_chunks; base += kScanThreads) {
    int64_t i = base + threadIdx.x;
    int v = i < n_chunks ? c[i] : 0;
    int tot;
    int ex = block_exclusive_scan(v, lds, &tot);
    if (i < n_chunks) c[i] = carry + ex;
    carry += tot;
  }
  if (threadIdx.x == 0) pair_num[k] = carry;
}

__global__ void __launch_bounds__(kScanThreads)
    scan_chunks_kernel(int32_t *__restrict__ chunk_count, int64_t n_chunks,
                       int32_t *__restrict__ pair_num) {
  __shared__ int lds[kScanThreads / 64 + 1];
  scan_chunks_of_tap(chunk_count, n_chunks, blockIdx.x, pair_num, lds);
}

// Two jobs that both need nothing but the marking kernel's results, in one launch: blocks
// below n_scan_blocks run the first pass of the table's popcount scan, the K blocks after
// them scan the chunk counts of one tap each (regular convolutions only: a submanifold
// rulebook counts its pairs after the table is ranked).
// SEED: the blocks of the table also leave, for every word, the output rows and the pairs
// that lie in the words of its scan block before it (seed_rows[]; seed_pairs[], which holds
// the words' own pairs on entry, as mark_count_kernel counted them), and the block's pairs
// (pairsum[]), as the seeded form of dilate_blocksum_kernel does for the dilation path.
template <bool SEED>
__global__ void __launch_bounds__(kScanThreads)
    blocksum_scan_chunks_kernel(const uint32_t *__restrict__ bits, int64_t n_words,
                                int32_t *__restrict__ blocksum, int64_t n_scan_blocks,
                                int32_t *__restrict__ chunk_count, int64_t n_chunks,
                                int32_t *__restrict__ pair_num, int32_t *__restrict__ seed_rows,
                                int32_t *__restrict__ seed_pairs, int32_t *__restrict__ pairsum) {
  __shared__ int lds[kScanThreads / 64 + 1];
  if ((int64_t)blockIdx.x >= n_scan_blocks) {
    scan_chunks_of_tap(chunk_count, n_chunks, (int)(blockIdx.x - n_scan_blocks), pair_num, lds);
    return;
  }
  if constexpr (SEED) {
    // every thread kScanItems consecutive words, as the second pass of the table's scan
    const int64_t w0 = (int64_t)blockIdx.x * kScanBlockWords + (int64_t)threadIdx.x * kScanItems;
    int cr[kScanItems], cp[kScanItems], sr = 0, sp = 0;
#pragma unroll
    for (int i = 0; i < kScanItems; ++i) {
      cr[i] = w0 + i < n_words ? __popc(bits[w0 + i]) : 0;
      cp[i] = w0 + i < n_words ? seed_pairs[w0 + i] : 0;
      sr += cr[i];
      sp += cp[i];
    }
    int tot_r, tot_p;
    int er = block_exclusive_scan(sr, lds, &tot_r);
    int ep = block_exclusive_scan(sp, lds, &tot_p);
#pragma unroll
    for (int i = 0; i < kScanItems; ++i) {
      if (w0 + i < n_words) {
        seed_rows[w0 + i] = er;
        seed_pairs[w0 + i] = ep;
      }
      er += cr[i];
      ep += cp[i];
    }
    if (threadIdx.x == 0) {
      blocksum[blockIdx.x] = tot_r;
      pairsum[blockIdx.x] = tot_p;
    }
  } else {
    popc_blocksum_block(bits, n_words, blockIdx.x, blocksum, lds);
  }
}

// Output table from the input table (see "marking by dilation"), the block sums of its
// popcounts (blocksum[], one store per block), and, in the K blocks after the
// table's, the scan of the chunk counts.  Word (b, x, y, zw) of the output is the OR over
// (kx, ky) of the bits 32 zw + kz .. + 31, for every kz, of input row (b, x + kx, y + ky).
// KS > 0: the kernel's three extents equal KS (loops unrolled, all
// loads of a thread in flight at once); KS = 0: any extents.
// SEED: the kernel also leaves, for every word, the output rows and the pairs that lie in
// the words of its scan block before it (seed_rows[], seed_pairs[]), and the block's pairs
// (pairsum[]): the work measure of the convolution's plan (see SplitRequest).  The pairs
// that land on the outputs of a word are the set input bits over all taps -- the popcounts of
// the same shifted words the OR is taken of.
template <int KS, bool SEED>
__global__ void __launch_bounds__(kScanThreads)
    dilate_blocksum_kernel(const uint32_t *__restrict__ in_bits, Geom g, DenseIn d,
                           uint32_t *__restrict__ bits, int64_t n_words, int64_t n_word_blocks,
                           int32_t *__restrict__ blocksum, int32_t *__restrict__ chunk_count,
                           int64_t n_chunks, int32_t *__restrict__ pair_num,
                           int32_t *__restrict__ seed_rows, int32_t *__restrict__ seed_pairs,
                           int32_t *__restrict__ pairsum) {
  if ((int64_t)blockIdx.x >= n_word_blocks) {
    __shared__ int lds[kScanThreads / 64 + 1];
    scan_chunks_of_tap(chunk_count, n_chunks, (int)(blockIdx.x - n_word_blocks), pair_num, lds);
    return;
  }
  // One block per scan block of kScanBlockWords words, kScanItems words per thread: the
  // block's popcount is one plain store.  (A block per kScanThreads words with an atomic
  // add per wave put 32 atomics on every block sum; device-scope atomics on one address
  // are served one after the other, and that chain, not the loads, was the kernel's time.)
  const int ksx = KS > 0 ? KS : g.ks[0], ksy = KS > 0 ? KS : g.ks[1], ksz = KS > 0 ? KS : g.ks[2];
  const uint32_t zw_n = (uint32_t)g.os[2] >> 5;  // words per output row
  const int64_t xstep = (int64_t)d.U[1] * d.Wz;
  int v = 0;
  // One word of the output table: the OR of its taps' shifted input words; *landing = the
  // pairs that land on its cells.
  auto word_of = [&](int64_t w, int *landing) -> uint32_t {
    uint32_t t = (uint32_t)w;  // (fewer than 2^26 words)
    const int zw = (int)(t % zw_n);
    t /= zw_n;
    const int y = (int)(t % (uint32_t)g.os[1]);
    t /= (uint32_t)g.os[1];
    const int x = (int)(t % (uint32_t)g.os[0]);
    const int b = (int)(t / (uint32_t)g.os[0]);
    const uint32_t *rowp = in_bits + (((int64_t)b * d.U[0] + x) * d.U[1] + y) * d.Wz + zw;
    uint32_t out = 0u;
    int land = 0;
#pragma unroll
    for (int kx = 0; kx < ksx; ++kx) {
#pragma unroll
      for (int ky = 0; ky < ksy; ++ky) {
        const uint32_t *p = rowp + kx * xstep + ky * d.Wz;
        // (with ksz > 1, Wz > os[2] / 32: word zw + 1 exists)
        const uint32_t lo = p[0], hi = ksz > 1 ? p[1] : 0u;
        uint32_t acc = lo;
        if constexpr (SEED) land += __popc(lo);
#pragma unroll
        for (int kz = 1; kz < ksz; ++kz) {
          const uint32_t shifted = (lo >> kz) | (hi << (32 - kz));
          acc |= shifted;
          if constexpr (SEED) land += __popc(shifted);
        }
        out |= acc;
      }
    }
    *landing = land;
    return out;
  };
  if constexpr (SEED) {
    // Every thread takes kScanItems consecutive words, so that the prefixes over the block's
    // words in their order need the threads' sums and nothing else: no table of the words'
    // counts in LDS (a block then fits beside a workgroup that has taken nearly all of a
    // CU's LDS, as the convolution's do).
    __shared__ int lds[kScanThreads / 64 + 1];
    const int64_t w0 = (int64_t)blockIdx.x * kScanBlockWords + (int64_t)threadIdx.x * kScanItems;
    int cr[kScanItems], cp[kScanItems], sr = 0, sp = 0;
    uint32_t ob[kScanItems];
#pragma unroll
    for (int i = 0; i < kScanItems; ++i) {
      ob[i] = 0u;
      cp[i] = 0;
      if (w0 + i < n_words) ob[i] = word_of(w0 + i, &cp[i]);
      cr[i] = __popc(ob[i]);
      sr += cr[i];
      sp += cp[i];
    }
    int tot_r, tot_p;
    int er = block_exclusive_scan(sr, lds, &tot_r);
    int ep = block_exclusive_scan(sp, lds, &tot_p);
#pragma unroll
    for (int i = 0; i < kScanItems; ++i) {
      if (w0 + i < n_words) {
        bits[w0 + i] = ob[i];
        seed_rows[w0 + i] = er;
        seed_pairs[w0 + i] = ep;
      }
      er += cr[i];
      ep += cp[i];
    }
    if (threadIdx.x == 0) {
      blocksum[blockIdx.x] = tot_r;
      pairsum[blockIdx.x] = tot_p;
    }
    return;
  }
#pragma unroll 2
  for (int it = 0; it < kScanItems; ++it) {
    const int64_t w = (int64_t)blockIdx.x * kScanBlockWords + it * kScanThreads + threadIdx.x;
    if (w >= n_words) break;
    int unused;
    const uint32_t out = word_of(w, &unused);
    bits[w] = out;
    v += __popc(out);
  }
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) v += __shfl_xor(v, s, 64);
  __shared__ int wave_sum[kScanThreads / 64];
  if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    int total = 0;
#pragma unroll
    for (int i = 0; i < kScanThreads / 64; ++i) total += wave_sum[i];
    blocksum[blockIdx.x] = total;
  }
}

// Dynamic LDS of the kernels that add up the scan blocks' sums: a long long and an int for
// every scan block and one more (as much as the table needs, not room for kSeedMaxBlocks: a
// block of theirs then fits beside a workgroup that has taken nearly all of a CU's LDS).
static inline size_t seed_lds_bytes(int64_t n_scan_blocks) {
  return (size_t)(n_scan_blocks + 1) * 12 + 8;
}
__device__ __forceinline__ int *seed_lds_rows(long long *dyn, int64_t n_scan_blocks) {
  return reinterpret_cast<int *>(dyn + n_scan_blocks + 1);
}

// The placing of the range boundaries of a SplitRequest, for the group of 16 ranges `group`
// (kScanThreads threads: 16 lanes to a range).  Range w begins at the first cell c (a word
// of the table) with
//   work(c) = pairs below c * tile_rows + rows below c * tile_cost  >=  w / n_rng of the total,
// its first row being the rows below c.  The block first adds up the block sums of rows and
// pairs in LDS (at most kSeedMaxBlocks of each); a range's lanes then find the scan block by
// bisection there and the cell inside it by three rounds of 16 probes.
__device__ __forceinline__ void split_ranges_block(int group, int64_t n_words,
                                                   int64_t n_scan_blocks,
                                                   const int32_t *__restrict__ blocksum,
                                                   const int32_t *__restrict__ pairsum,
                                                   const int32_t *__restrict__ seed_rows,
                                                   const int32_t *__restrict__ seed_pairs,
                                                   const SplitRequest &rq, long long *pairs_base,
                                                   int *rows_base) {
  // (pairs_base, rows_base: n_scan_blocks + 1 entries each in the kernel's dynamic LDS, see
  // seed_lds_bytes)
  __shared__ int lds[kScanThreads / 64 + 1];
  __shared__ long long wave_p[kScanThreads / 64];
  const int nb = (int)n_scan_blocks;  // <= kSeedMaxBlocks
  {
    // exclusive prefixes of the block sums: every thread a run of consecutive blocks
    constexpr int kPer = kSeedMaxBlocks / kScanThreads;
    const int first = threadIdx.x * kPer;
    int r[kPer], sr = 0;
    long long pp[kPer], sp = 0;
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      r[i] = first + i < nb ? blocksum[first + i] : 0;
      pp[i] = first + i < nb ? (long long)pairsum[first + i] : 0;
      sr += r[i];
      sp += pp[i];
    }
    int tot_r;
    int er = block_exclusive_scan(sr, lds, &tot_r);
    // the pairs as 64-bit sums: scan inside the wave, then over the waves
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    long long incl = sp;
#pragma unroll
    for (int dd = 1; dd < 64; dd <<= 1) {
      const long long o = __shfl_up(incl, dd, 64);
      if (lane >= dd) incl += o;
    }
    if (lane == 63) wave_p[wave] = incl;
    __syncthreads();
    long long ep = incl - sp;
    for (int i = 0; i < wave; ++i) ep += wave_p[i];
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      if (first + i <= nb) {
        rows_base[first + i] = er;
        pairs_base[first + i] = ep;
      }
      er += r[i];
      ep += pp[i];
    }
    if (threadIdx.x == kScanThreads - 1 && first + kPer <= nb) {  // nb == kSeedMaxBlocks
      rows_base[nb] = er;
      pairs_base[nb] = ep;
    }
    __syncthreads();
  }
  const long long n_out = rows_base[nb];
  const long long T = rq.tile_rows, cost = rq.tile_cost;
  const long long total_work = pairs_base[nb] * T + n_out * cost;
  auto work_of_block = [&](int b) -> long long { return pairs_base[b] * T + rows_base[b] * cost; };
  auto work_of_cell = [&](long long c) -> long long {
    if (c >= n_words) return total_work;
    const int b = (int)(c >> 11);  // kScanBlockWords = 2048 words to a scan block
    return (pairs_base[b] + seed_pairs[c]) * T + ((long long)rows_base[b] + seed_rows[c]) * cost;
  };
  static_assert(kScanBlockWords == 2048, "the cell search assumes scan blocks of 2048 words");
  const int sub = threadIdx.x & 15;
  const int w = group * (kScanThreads / 16) + (threadIdx.x >> 4);
  const bool mine = w >= 1 && w < rq.n_rng;
  // ceil(total * w / n_rng); ranges without a target (w = 0, w >= n_rng) search for nothing
  long long target = mine ? (total_work * w + rq.n_rng - 1) / rq.n_rng : 0;
  // the scan block: the last one whose work before it is below the target
  int lo_b = 0, hi_b = nb;  // work_of_block(lo_b) < target (or lo_b = 0) ; answer in block lo_b
  while (hi_b - lo_b > 1) {
    const int mid = (lo_b + hi_b) >> 1;
    if (work_of_block(mid) < target) lo_b = mid;
    else hi_b = mid;
  }
  long long lo = (long long)lo_b * kScanBlockWords;  // work(lo) < target <= work(lo + width),
  int width = kScanBlockWords;                       // or the target is not positive
  const int shift = (threadIdx.x & 63) & ~15;
#pragma unroll
  for (int round = 0; round < 3; ++round) {
    const int stride = width >> 4;  // 128, 8, then single cells
    const long long c = stride > 0 ? lo + (long long)stride * (sub + 1) : lo + sub + 1;
    const bool reached = work_of_cell(c) >= target;
    const unsigned hits = (unsigned)((__ballot(reached) >> shift) & 0xFFFFull);
    // (the last probe of the first two rounds is lo + width, which reaches the target)
    const int first = hits ? __ffs(hits) - 1 : 15;
    if (stride > 0) {
      lo += (long long)stride * first;
      width = stride;
    } else {
      lo += first + 1;  // the cell itself
      width = 0;
    }
  }
  // after the rounds of 128 and 8 the third one probed the 8 cells lo + 1 .. lo + 8 (lanes
  // 0..7; lanes 8..15 probe beyond and reach the target as well): lo is the first cell that
  // reaches it
  if (sub == 0) {
    if (mine) {
      long long c = target > 0 ? lo : 0;
      if (c > n_words) c = n_words;
      long long row = c >= n_words ? n_out
                                   : (long long)rows_base[(int)(c >> 11)] + seed_rows[c];
      rq.range_row0[w] = (int32_t)row;
    } else if (w == 0) {
      rq.range_row0[0] = 0;
      rq.range_row0[rq.n_rng] = (int32_t)n_out;
    }
  }
}

// Block `block` of the blocks that serve a SplitRequest (split_request_blocks): the first
// ones place the boundaries of the request itself, the others those of its alternative.
__device__ __forceinline__ void split_request_block(int block, int64_t n_words,
                                                    int64_t n_scan_blocks,
                                                    const int32_t *__restrict__ blocksum,
                                                    const int32_t *__restrict__ pairsum,
                                                    const int32_t *__restrict__ seed_rows,
                                                    const int32_t *__restrict__ seed_pairs,
                                                    const SplitRequest &rq, long long *pairs_base,
                                                    int *rows_base) {
  const int main_blocks = (rq.n_rng + kScanThreads / 16 - 1) / (kScanThreads / 16);
  if (block < main_blocks) {
    split_ranges_block(block, n_words, n_scan_blocks, blocksum, pairsum, seed_rows, seed_pairs, rq,
                       pairs_base, rows_base);
  } else {
    const SplitRequest alt = {rq.n_rng_alt, rq.tile_rows_alt, rq.tile_cost, rq.range_row0_alt,
                              0, 0, nullptr};
    split_ranges_block(block - main_blocks, n_words, n_scan_blocks, blocksum, pairsum, seed_rows,
                       seed_pairs, alt, pairs_base, rows_base);
  }
}

// The second pass of the table's scan (popc_prefix_block) and, in the blocks after the
// table's, the range boundaries of a SplitRequest (split_ranges_block): for rulebooks whose
// pair launch does not take the prefixes in two levels (no room for the output rows at
// hand).  Dynamic LDS: seed_lds_bytes.
__global__ void __launch_bounds__(kScanThreads)
    prefix_split_kernel(const uint32_t *__restrict__ bits, int64_t n_words, int64_t n_scan_blocks,
                        const int32_t *__restrict__ blocksum, int32_t *__restrict__ prefix,
                        int32_t *__restrict__ total, int32_t *__restrict__ mirror,
                        const int32_t *__restrict__ pairsum,
                        const int32_t *__restrict__ seed_rows,
                        const int32_t *__restrict__ seed_pairs, SplitRequest rq, int ticket) {
  if ((int64_t)blockIdx.x < n_scan_blocks) {
    popc_prefix_block(bits, n_words, blocksum, prefix, total, mirror,
                      (int64_t)blockIdx.x == n_scan_blocks - 1, ticket);
    return;
  }
  extern __shared__ long long seed_dyn[];
  split_request_block((int)(blockIdx.x - n_scan_blocks), n_words, n_scan_blocks, blocksum, pairsum,
                      seed_rows, seed_pairs, rq, seed_dyn, seed_lds_rows(seed_dyn, n_scan_blocks));
}

// What the two-level form of write_pairs_kernel needs besides the table: the scan blocks'
// sums (the prefix of a word is then the sum of the blocks before its own plus its prefix
// inside the block, seed_rows[]: no launch for the scan's second pass), a SplitRequest to
// serve on the way (n_rng = 0: none), and where the totals go.
struct TwoLevel {
  const int32_t *blocksum, *pairsum, *seed_rows, *seed_pairs;
  int64_t n_scan_blocks;
  SplitRequest split;
  int split_blocks;
  int32_t *total, *mirror;
  int ticket;
  int clear_total;  // total[] lies in a table kept clean between calls: zero it once read
};

template <int KS, bool TWO>
__global__ void __launch_bounds__(256)
    write_pairs_kernel(const int32_t *__restrict__ indices, int64_t n_in, Geom g,
                       const uint32_t *__restrict__ bits, const int32_t *__restrict__ prefix,
                       const int32_t *__restrict__ rank2row,
                       const int32_t *__restrict__ chunk_prefix, int64_t n_chunks,
                       const int32_t *__restrict__ pair_num, int32_t *__restrict__ pairs,
                       int64_t n_words, int32_t *__restrict__ out_indices,
                       uint32_t *__restrict__ clean, int64_t clean_words, int row_blocks,
                       TwoLevel two) {
  extern __shared__ long long seed_dyn[];  // (TWO: seed_lds_bytes; otherwise none)
  int *const base_s = TWO ? seed_lds_rows(seed_dyn, two.n_scan_blocks) : nullptr;
  if constexpr (TWO) {
    static_assert(kScanThreads == 256, "one block size for the table's scan and this kernel");
    if (blockIdx.y == 0) {
      // the first row of the grid (its blocks start first: the host is waiting for the
      // totals): the range boundaries of the convolution's plan, and one block for the totals
      if ((int)blockIdx.x < two.split_blocks) {
        split_request_block((int)blockIdx.x, n_words, two.n_scan_blocks, two.blocksum, two.pairsum,
                            two.seed_rows, two.seed_pairs, two.split, seed_dyn, base_s);
        return;
      }
      if ((int)blockIdx.x != two.split_blocks) return;
    }
    // sums of the scan blocks before every block (at most kSeedMaxBlocks of them)
    __shared__ int lds[kScanThreads / 64 + 1];
    constexpr int kPer = kSeedMaxBlocks / kScanThreads;
    const int nb = (int)two.n_scan_blocks, first = threadIdx.x * kPer;
    int r[kPer], sr = 0;
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      r[i] = first + i < nb ? two.blocksum[first + i] : 0;
      sr += r[i];
    }
    int tot;
    int er = block_exclusive_scan(sr, lds, &tot);
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      if (first + i <= nb) base_s[first + i] = er;
      er += r[i];
    }
    if (threadIdx.x == kScanThreads - 1 && first + kPer <= nb) base_s[nb] = er;
    __syncthreads();
    if (blockIdx.y == 0) {
      // the totals: the number of outputs and the flags, for later kernels and for the
      // host, which is waiting for the ticket while this launch still runs
      if (threadIdx.x == 0) {
        two.total[0] = tot;
        volatile int32_t *m = two.mirror;
        m[0] = tot;
        m[1] = two.total[1];
        m[2] = two.total[2];
        m[3] = two.total[3];
        __hip_atomic_store(two.mirror + kMirrorTicket, two.ticket, __ATOMIC_RELEASE,
                           __HIP_MEMORY_SCOPE_SYSTEM);
        if (two.clear_total) {
          two.total[0] = 0;
          two.total[1] = 0;
          two.total[2] = 0;
          two.total[3] = 0;
        }
      }
      return;
    }
  }
  const int by = (int)blockIdx.y - (TWO ? 1 : 0);  // (the two-level form's first row is above)
  if (by >= g.ks[0]) {
    // the rows of the grid beyond the kernel's x extent: the output rows, and the words of
    // a table that no kernel reads any more and the next call expects to find zero
    const int64_t step = (int64_t)row_blocks * gridDim.x * blockDim.x;
    const int64_t w0 = ((int64_t)(by - g.ks[0]) * gridDim.x + blockIdx.x) * blockDim.x +
                       threadIdx.x;
    if (out_indices != nullptr) {
      for (int64_t w = w0; w < n_words; w += step) {
        if constexpr (TWO) {
          const uint32_t b = bits[w];
          if (b != 0)
            emit_rows_of_word_at(b, base_s[w >> 11] + two.seed_rows[w], w, g.os[0], g.os[1],
                                 g.os[2], out_indices);
        } else {
          emit_rows_of_word(bits, prefix, w, g.os[0], g.os[1], g.os[2], out_indices);
        }
      }
    }
    for (int64_t w = w0; w < clean_words; w += step) clean[w] = 0u;
    return;
  }
  int64_t chunk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (chunk >= n_chunks) return;
  int lane = threadIdx.x & 63;
  int64_t i = chunk * 64 + lane;
  bool live = i < n_in;
  int32_t row[4] = {0, 0, 0, 0};
  if (live) *reinterpret_cast<int4 *>(row) = reinterpret_cast<const int4 *>(indices)[i];
  const bool usable = live && row_usable(row, g);  // (a row outside the grid owns no pair)
  // The taps of one (kx, ky) differ in z only: their cells are neighbours in the key
  // space, so the table word and its prefix are loaded once per word, not per tap.
  uint32_t word = 0xFFFFFFFFu, wbits = 0u;
  int wprefix = 0;
  // blockIdx.y = kx: the taps of one x offset per wave, for more waves in flight (a wave
  // per (kx, ky) was tried and is no faster, and fetching the table words of all (kx, ky)
  // before any is used is slower, 15.5 against 13.7 us on the benchmark layer: the kernel is
  // bound by its stores)
  const int kx = by;
  int k = kx * g.ks[1] * g.ks[2];
  int ox = 0;
  const bool tr = g.tr != 0;
  const bool okx = usable && tap_to_out(row[1], kx, g.st[0], g.pd[0], g.dl[0], g.os[0], &ox, tr);
  const int ksy = KS > 0 ? KS : g.ks[1], ksz = KS > 0 ? KS : g.ks[2];
#pragma unroll
  for (int ky = 0; ky < ksy; ++ky) {
    int oy = 0;
    const bool okxy = okx && tap_to_out(row[2], ky, g.st[1], g.pd[1], g.dl[1], g.os[1], &oy, tr);
    const uint32_t base = (uint32_t)(((row[0] * g.os[0] + ox) * g.os[1] + oy) * g.os[2]);
#pragma unroll
    for (int kz = 0; kz < ksz; ++kz, ++k) {
      int oz = 0;
      bool ok = okxy && tap_to_out(row[3], kz, g.st[2], g.pd[2], g.dl[2], g.os[2], &oz, tr);
      const uint32_t key = base + (uint32_t)oz;
      if (ok && (key >> 5) != word) {
        word = key >> 5;
        wbits = bits[word];
        if constexpr (TWO) wprefix = base_s[word >> 11] + two.seed_rows[word];
        else wprefix = prefix[word];
      }
      if (ok && g.subm) ok = (wbits >> (key & 31u)) & 1u;
      unsigned long long m = __ballot(ok);
      int32_t *pin = pairs + ((int64_t)k * 2 + 0) * n_in;
      int32_t *pout = pairs + ((int64_t)k * 2 + 1) * n_in;
      if (ok) {
        int slot = chunk_prefix[(int64_t)k * n_chunks + chunk] +
                   __popcll(m & ((1ull << lane) - 1ull));
        int r = wprefix + __popc(wbits & ((1u << (key & 31u)) - 1u));
        if (g.subm) r = rank2row[r];
        pin[slot] = (int32_t)i;
        pout[slot] = r;
      }
      if (live && i >= pair_num[k]) {
        pin[i] = -1;
        pout[i] = -1;
      }
    }
  }
}

// inverse[i] = rank of row i's cell; counts[rank] += 1 (integer atomics: exact).  With
// max_count, max_count[0] = the largest count: the row that raises a cell's count to its
// final value sees that value, so the maximum over all rows of (count seen + 1) is it
// (one atomic per wave).
__global__ void __launch_bounds__(256)
    inverse_counts_kernel(const int32_t *__restrict__ coords, int64_t n, int d0, int d1, int d2,
                          int d3,
                          const uint32_t *__restrict__ bits, const int32_t *__restrict__ prefix,
                          int32_t *__restrict__ inverse, int32_t *__restrict__ counts,
                          int32_t *__restrict__ max_count) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int seen = 0;
  if (i < n) {
    int4 r = reinterpret_cast<const int4 *>(coords)[i];
    if (cell_in_range(r, d0, d1, d2, d3)) {
      uint32_t key = (uint32_t)(((r.x * d1 + r.y) * d2 + r.z) * d3 + r.w);
      int rk = bit_rank(bits, prefix, key);
      inverse[i] = rk;
      if (counts) seen = atomicAdd(&counts[rk], 1) + 1;
    } else {
      inverse[i] = -1;  // a row outside the grid: the call reports it
    }
  }
  if (max_count) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
      const int o = __shfl_xor(seen, d, 64);
      seen = o > seen ? o : seen;
    }
    if ((threadIdx.x & 63) == 0 && seen > 0) atomicMax(max_count, seen);
  }
}

struct RulebookWs {
  BitTable table;
  int32_t *chunk_count;  // [K, n_chunks]
  int32_t *rank2row;     // [n_in] (subm)
  int64_t n_chunks;
  uint32_t *in_bits;     // input table of the dilation path (when it applies)
  DenseIn dense;
  bool use_dense;
  // seed of a convolution's work split (regular convolutions, tables of at most
  // kSeedMaxBlocks scan blocks): rows and pairs before every word inside its scan block,
  // pairs of every block
  bool can_seed;
  int32_t *seed_rows, *seed_pairs, *pairsum;
};

static inline bool seed_applies(const Geom &g) {
  return ceil_div(bit_words(geom_cells(g)), kScanBlockWords) <= kSeedMaxBlocks;
}

static size_t rulebook_ws_bytes(const Geom &g, int64_t n_in) {
  int64_t n_chunks = ceil_div(n_in > 0 ? n_in : 1, 64);
  DenseIn d;
  const size_t dense = dense_marking_applies(g, n_in, &d)
                           ? align_up((size_t)dense_in_words(g, d) * 4)
                           : 0;
  const size_t seed = !g.subm && seed_applies(g)
                          ? 2 * align_up((size_t)bit_words(geom_cells(g)) * 4) +
                                align_up((size_t)(kSeedMaxBlocks + 1) * 4)
                          : 0;
  return bit_table_bytes(geom_cells(g)) + align_up((size_t)g.K * n_chunks * 4) +
         align_up((size_t)(n_in > 0 ? n_in : 1) * 4) + dense + seed;
}

// Bytes of the table a caller may keep between calls (ssc_rulebook_clean_table_bytes): a
// header of 256 bytes that holds the table's totals and flags, then the input table of the
// dilation path.  0 when the geometry does not take that path.
constexpr size_t kCleanHeader = 256;
static size_t rulebook_clean_bytes(const Geom &g, int64_t n_in) {
  DenseIn d;
  if (n_in <= 0 || !dense_marking_applies(g, n_in, &d)) return 0;
  return kCleanHeader + align_up((size_t)dense_in_words(g, d) * 4);
}

static RulebookWs rulebook_ws_carve(void *ws, const Geom &g, int64_t n_in) {
  Carver c(ws);
  RulebookWs w;
  w.table = bit_table_carve(c, geom_cells(g));
  w.n_chunks = ceil_div(n_in > 0 ? n_in : 1, 64);
  w.chunk_count = c.take<int32_t>((size_t)g.K * w.n_chunks);
  w.rank2row = c.take<int32_t>(n_in > 0 ? n_in : 1);
  w.use_dense = dense_marking_applies(g, n_in, &w.dense);
  w.in_bits = w.use_dense ? c.take<uint32_t>((size_t)dense_in_words(g, w.dense)) : nullptr;
  w.can_seed = !g.subm && seed_applies(g);
  w.seed_rows = w.seed_pairs = w.pairsum = nullptr;
  if (w.can_seed) {
    w.seed_rows = c.take<int32_t>((size_t)w.table.n_words);
    w.seed_pairs = c.take<int32_t>((size_t)w.table.n_words);
    w.pairsum = c.take<int32_t>((size_t)kSeedMaxBlocks + 1);
  }
  return w;
}

}  // namespace ssc

using namespace ssc;

// ---- host side of the rulebook ------------------------------------------------------------
static int rulebook_check(const ssc_geometry *g, Geom *gg, const int32_t *indices, int64_t n_in,
                          const void *workspace, size_t workspace_bytes) {
  int rc = make_geom(g, gg);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(n_in >= 0, SSC_EINVAL, "n_in is negative");
  SSC_CHECK(n_in * gg->K < ((int64_t)1 << 40), SSC_EINVAL, "n_in * kernel volume too large");
  if (n_in == 0) return SSC_OK;
  SSC_CHECK(indices != nullptr && workspace != nullptr, SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(workspace_bytes >= rulebook_ws_bytes(*gg, n_in), SSC_EWORKSPACE,
            "rulebook workspace too small: %zu < %zu", workspace_bytes,
            rulebook_ws_bytes(*gg, n_in));
  return SSC_OK;
}

// Enqueue: the scan's second pass, and beside it the range boundaries of a convolution's plan.
static int launch_prefix_split(const RulebookWs &w, const SplitRequest &split, int32_t *mirror,
                               int ticket, hipStream_t s) {
  const int64_t word_blocks = w.table.n_scan_blocks;
  hipLaunchKernelGGL(prefix_split_kernel,
                     dim3((unsigned)(word_blocks + split_request_blocks(split))),
                     dim3(kScanThreads), seed_lds_bytes(word_blocks), s, w.table.bits,
                     w.table.n_words, word_blocks, w.table.blocksum, w.table.prefix, w.table.total,
                     mirror, w.pairsum, w.seed_rows, w.seed_pairs, split, ticket);
  SSC_LAUNCH_CHECK("prefix_split");
  return SSC_OK;
}

// Enqueue: clear the table, mark the output cells (counting the pairs of every chunk on the
// way for a regular convolution), scan.  Afterwards total[0] = number of marked cells,
// total[1] = flags, both also in `mirror` when given.  With pair_num, a regular
// convolution's chunk counts are scanned beside the first pass of the table scan (and
// rulebook_pairs must be told so).
static int rulebook_mark_and_scan(const int32_t *indices, int64_t n_in, const Geom &gg,
                                  const RulebookWs &w, int32_t *pair_num, int32_t *mirror,
                                  hipStream_t s, const SplitRequest *split = nullptr,
                                  bool table_is_clean = false, bool two_level = false,
                                  const CombineJob *job = nullptr, int ticket = 0) {
  int rc;
  if (w.use_dense && pair_num != nullptr) {
    // input table cleared (with the totals) unless the caller keeps one that every call
    // leaves clean, inputs marked, outputs by dilation
    BitTable in = w.table;
    in.bits = w.in_bits;
    in.n_words = dense_in_words(gg, w.dense);
    if (!table_is_clean && (rc = bit_table_clear(in, s, true)) != SSC_OK) return rc;
    const int64_t mark_blocks = ceil_div(w.n_chunks, 4);
    if (job != nullptr) {
      const int64_t n = combine_job_elements(*job);
      const int64_t rows = std::min<int64_t>(ceil_div(ceil_div(n, 256), mark_blocks), 1024);
      hipLaunchKernelGGL(mark_in_count_kernel<true>,
                         dim3((unsigned)mark_blocks, (unsigned)(gg.ks[0] + rows)), dim3(256), 0, s,
                         indices, n_in, gg, w.dense, w.in_bits, w.chunk_count, w.n_chunks,
                         w.table.total + 1, *job, n);
    } else {
      hipLaunchKernelGGL(mark_in_count_kernel<false>,
                         dim3((unsigned)mark_blocks, (unsigned)gg.ks[0]), dim3(256), 0, s, indices,
                         n_in, gg, w.dense, w.in_bits, w.chunk_count, w.n_chunks,
                         w.table.total + 1, CombineJob{}, (int64_t)0);
    }
    SSC_LAUNCH_CHECK("mark_in_count");
    const int64_t word_blocks = w.table.n_scan_blocks;
    const int ks = (gg.ks[0] == gg.ks[1] && gg.ks[1] == gg.ks[2]) ? gg.ks[0] : 0;
    // (two_level: the launch of the pair lists works with the scan blocks' sums and the
    // prefixes inside the blocks, which this kernel's seeded form leaves: no second pass)
    const bool seed = (split != nullptr || two_level) && w.can_seed;
    auto kernel = seed ? (ks == 3   ? dilate_blocksum_kernel<3, true>
                          : ks == 5 ? dilate_blocksum_kernel<5, true>
                                    : dilate_blocksum_kernel<0, true>)
                       : (ks == 3   ? dilate_blocksum_kernel<3, false>
                          : ks == 5 ? dilate_blocksum_kernel<5, false>
                                    : dilate_blocksum_kernel<0, false>);
    hipLaunchKernelGGL(kernel, dim3((unsigned)(word_blocks + gg.K)), dim3(kScanThreads), 0, s,
                       w.in_bits, gg, w.dense, w.table.bits, w.table.n_words, word_blocks,
                       w.table.blocksum, w.chunk_count, w.n_chunks, pair_num, w.seed_rows,
                       w.seed_pairs, w.pairsum);
    SSC_LAUNCH_CHECK("dilate_blocksum");
    if (two_level) return SSC_OK;
    if (!seed || split == nullptr) return bit_table_scan_prefix(w.table, s, mirror, ticket);
    return launch_prefix_split(w, *split, mirror, ticket, s);
  }
  // (a regular convolution off the dilation path -- strided, dilated -- whose plan is to be
  // seeded or whose pair launch takes the prefixes in two levels: the marking kernel counts
  // the pairs of every table word on its way, in seed_pairs[], zeroed with the table)
  const bool seed = !gg.subm && pair_num != nullptr && (split != nullptr || two_level) && w.can_seed;
  if ((rc = bit_table_clear(w.table, s, false, seed ? w.seed_pairs : nullptr)) != SSC_OK) return rc;
  if (gg.subm) {
    if (job != nullptr) {
      const int64_t n = combine_job_elements(*job);
      const int64_t more = std::min<int64_t>(ceil_div(n, 256), 4096);
      hipLaunchKernelGGL(mark_rows_kernel<true>, dim3((unsigned)(ceil_div(n_in, 256) + more)),
                         dim3(256), 0, s, indices, n_in, gg.batch, gg.os[0], gg.os[1], gg.os[2],
                         w.table.bits, w.table.total + 1, 1, *job, n);
    } else {
      hipLaunchKernelGGL(mark_rows_kernel<false>, dim3((unsigned)ceil_div(n_in, 256)), dim3(256), 0,
                         s, indices, n_in, gg.batch, gg.os[0], gg.os[1], gg.os[2], w.table.bits,
                         w.table.total + 1, 1, CombineJob{}, (int64_t)0);
    }
    SSC_LAUNCH_CHECK("mark_rows");
    return bit_table_scan(w.table, s, mirror, ticket);
  }
  {
    const int64_t mark_blocks = ceil_div(w.n_chunks, 4);
    int32_t *word_pairs = seed ? w.seed_pairs : nullptr;
    if (job != nullptr) {
      const int64_t n = combine_job_elements(*job);
      const int64_t rows = std::min<int64_t>(ceil_div(ceil_div(n, 256), mark_blocks), 1024);
      hipLaunchKernelGGL(mark_count_kernel<true>,
                         dim3((unsigned)mark_blocks, (unsigned)(gg.ks[0] + rows)), dim3(256), 0, s,
                         indices, n_in, gg, w.table.bits, w.chunk_count, w.n_chunks,
                         w.table.total + 1, *job, n, word_pairs);
    } else {
      hipLaunchKernelGGL(mark_count_kernel<false>, dim3((unsigned)mark_blocks, (unsigned)gg.ks[0]),
                         dim3(256), 0, s, indices, n_in, gg, w.table.bits, w.chunk_count,
                         w.n_chunks, w.table.total + 1, CombineJob{}, (int64_t)0, word_pairs);
    }
  }
  SSC_LAUNCH_CHECK("mark_count");
  if (pair_num == nullptr) return bit_table_scan(w.table, s, mirror, ticket);
  auto sums_kernel = seed ? blocksum_scan_chunks_kernel<true> : blocksum_scan_chunks_kernel<false>;
  hipLaunchKernelGGL(sums_kernel, dim3((unsigned)(w.table.n_scan_blocks + gg.K)),
                     dim3(kScanThreads), 0, s, w.table.bits, w.table.n_words, w.table.blocksum,
                     w.table.n_scan_blocks, w.chunk_count, w.n_chunks, pair_num, w.seed_rows,
                     w.seed_pairs, w.pairsum);
  SSC_LAUNCH_CHECK("blocksum_scan_chunks");
  if (two_level) return SSC_OK;
  if (!seed || split == nullptr) return bit_table_scan_prefix(w.table, s, mirror, ticket);
  return launch_prefix_split(w, *split, mirror, ticket, s);
}

// Enqueue: the pair lists and, with out_indices, the output rows (one launch for both).
// chunks_scanned: rulebook_mark_and_scan has scanned the chunk counts already.
static int rulebook_pairs(const int32_t *indices, int64_t n_in, const Geom &gg,
                          const RulebookWs &w, int32_t *out_indices, int32_t *pairs,
                          int32_t *pair_num, bool chunks_scanned, hipStream_t s,
                          uint32_t *clean = nullptr, int64_t clean_words = 0,
                          const TwoLevel *two = nullptr) {
  unsigned chunk_blocks = (unsigned)ceil_div(w.n_chunks, 4);
  if (gg.subm) {  // a regular convolution's counts were taken while marking the table
    hipLaunchKernelGGL(rank_to_row_kernel, dim3((unsigned)ceil_div(n_in, 256)), dim3(256), 0, s,
                       indices, n_in, gg, w.table.bits, w.table.prefix, w.rank2row);
    SSC_LAUNCH_CHECK("rank_to_row");
    hipLaunchKernelGGL(count_pairs_kernel, dim3(chunk_blocks), dim3(256), 0, s, indices, n_in, gg,
                       w.table.bits, w.chunk_count, w.n_chunks);
    SSC_LAUNCH_CHECK("count_pairs");
  }
  if (gg.subm || !chunks_scanned) {
    hipLaunchKernelGGL(scan_chunks_kernel, dim3(gg.K), dim3(kScanThreads), 0, s, w.chunk_count,
                       w.n_chunks, pair_num);
    SSC_LAUNCH_CHECK("scan_chunks");
  }
  // rows of the grid beyond the kernel's x extent write out_indices[] (see the kernel)
  int64_t row_blocks = (gg.subm || out_indices == nullptr)
                           ? 0
                           : ceil_div(ceil_div(w.table.n_words, 256), chunk_blocks);
  if (clean != nullptr) {
    const int64_t clean_blocks = ceil_div(ceil_div(clean_words, 256), chunk_blocks);
    if (clean_blocks > row_blocks) row_blocks = clean_blocks;
  }
  if (row_blocks > 4096) row_blocks = 4096;
  const int ks = gg.ks[1] == gg.ks[2] ? gg.ks[1] : 0;
  if (two != nullptr) {  // one more row of the grid: range boundaries and totals
    auto kernel = ks == 3 ? write_pairs_kernel<3, true> : ks == 5 ? write_pairs_kernel<5, true>
                  : ks == 2 ? write_pairs_kernel<2, true> : write_pairs_kernel<0, true>;
    hipLaunchKernelGGL(kernel, dim3(chunk_blocks, (unsigned)(gg.ks[0] + row_blocks + 1)),
                       dim3(256), seed_lds_bytes(two->n_scan_blocks), s, indices, n_in, gg, w.table.bits, w.table.prefix, w.rank2row,
                       w.chunk_count, w.n_chunks, pair_num, pairs, w.table.n_words, out_indices,
                       clean, clean_words, (int)row_blocks, *two);
    SSC_LAUNCH_CHECK("write_pairs");
    return SSC_OK;
  }
  auto kernel = ks == 3 ? write_pairs_kernel<3, false> : ks == 5 ? write_pairs_kernel<5, false>
                : ks == 2 ? write_pairs_kernel<2, false> : write_pairs_kernel<0, false>;
  hipLaunchKernelGGL(kernel, dim3(chunk_blocks, (unsigned)(gg.ks[0] + row_blocks)), dim3(256), 0,
                     s, indices, n_in, gg, w.table.bits, w.table.prefix, w.rank2row, w.chunk_count,
                     w.n_chunks, pair_num, pairs, w.table.n_words,
                     gg.subm ? (int32_t *)nullptr : out_indices, clean, clean_words,
                     (int)row_blocks, TwoLevel{});
  SSC_LAUNCH_CHECK("write_pairs");
  return SSC_OK;
}

// An upper bound of the number of outputs that needs no look at the data.
static int64_t rulebook_out_bound(const Geom &gg, int64_t n_in) {
  if (gg.subm) return n_in;
  const int64_t by_pairs = n_in * gg.K, cells = geom_cells(gg);
  return by_pairs < cells ? by_pairs : cells;
}

// The two totals as the host sees them.
static int rulebook_totals(const int32_t *host, const Geom &gg, int64_t n_in, int32_t *n_out_host,
                           int32_t *in_order_host) {
  SSC_CHECK((host[1] & kFlagBadRow) == 0, SSC_EINVAL,
            "an input row lies outside the grid (batch index not in [0, %d)%s)", gg.batch,
            gg.subm ? ", or a coordinate outside the spatial shape" : "");
  *n_out_host = gg.subm ? (int32_t)n_in : host[0];
  *in_order_host = (host[1] & kFlagDisorder) == 0 ? 1 : 0;
  return SSC_OK;
}

extern "C" {

size_t ssc_rulebook_workspace_bytes(const ssc_geometry *g, int64_t n_in) {
  Geom gg;
  if (make_geom(g, &gg) != SSC_OK) return 0;
  return rulebook_ws_bytes(gg, n_in);
}

int ssc_rulebook_count(const int32_t *indices, int64_t n_in, const ssc_geometry *g,
                       void *workspace, size_t workspace_bytes, int32_t *n_out_host,
                       ssc_stream_t stream) {
  int32_t in_order = 0;
  return ssc_rulebook_count_ordered(indices, n_in, g, workspace, workspace_bytes, n_out_host,
                                    &in_order, stream);
}

int ssc_rulebook_count_ordered(const int32_t *indices, int64_t n_in, const ssc_geometry *g,
                               void *workspace, size_t workspace_bytes, int32_t *n_out_host,
                               int32_t *in_order_host, ssc_stream_t stream) {
  Geom gg;
  int rc = rulebook_check(g, &gg, indices, n_in, workspace, workspace_bytes);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(n_out_host != nullptr && in_order_host != nullptr, SSC_EINVAL,
            "n_out_host or in_order_host is NULL");
  if (n_in == 0) {  // src/conv/indice_cuda_functor.cu:262-263
    *n_out_host = 0;
    *in_order_host = 1;
    return SSC_OK;
  }
  hipStream_t s = (hipStream_t)stream;
  RulebookWs w = rulebook_ws_carve(workspace, gg, n_in);
  if ((rc = rulebook_mark_and_scan(indices, n_in, gg, w, nullptr, nullptr, s)) != SSC_OK) return rc;
  int32_t host[2];
  if ((rc = read_back(host, w.table.total, sizeof(host), s)) != SSC_OK) return rc;
  return rulebook_totals(host, gg, n_in, n_out_host, in_order_host);
}

int ssc_rulebook_emit(const int32_t *indices, int64_t n_in, const ssc_geometry *g,
                      void *workspace, size_t workspace_bytes, int32_t *out_indices,
                      int32_t *pairs, int32_t *pair_num, ssc_stream_t stream) {
  Geom gg;
  int rc = rulebook_check(g, &gg, indices, n_in, workspace, workspace_bytes);
  if (rc != SSC_OK) return rc;
  hipStream_t s = (hipStream_t)stream;
  SSC_CHECK(pair_num != nullptr, SSC_EINVAL, "pair_num is NULL");
  if (n_in == 0) return fill_i32(pair_num, gg.K, 0, s);
  SSC_CHECK(pairs != nullptr, SSC_EINVAL, "pairs is NULL");
  SSC_CHECK(gg.subm || out_indices != nullptr, SSC_EINVAL, "out_indices is NULL");
  RulebookWs w = rulebook_ws_carve(workspace, gg, n_in);
  return rulebook_pairs(indices, n_in, gg, w, out_indices, pairs, pair_num, false, s);
}

size_t ssc_rulebook_out_bound(const ssc_geometry *g, int64_t n_in) {
  Geom gg;
  if (n_in < 0 || make_geom(g, &gg) != SSC_OK) return 0;
  return (size_t)rulebook_out_bound(gg, n_in);
}

size_t ssc_rulebook_clean_table_bytes(const ssc_geometry *g, int64_t n_in) {
  Geom gg;
  if (n_in < 0 || make_geom(g, &gg) != SSC_OK) return 0;
  return rulebook_clean_bytes(gg, n_in);
}

int ssc_rulebook_begin(const int32_t *indices, int64_t n_in, const ssc_geometry *g,
                       void *workspace, size_t workspace_bytes, int32_t *pairs, int32_t *pair_num,
                       int32_t *out_indices, int64_t out_capacity, void *clean_table,
                       size_t clean_table_bytes, ssc_stream_t stream) {
  bool seeded = false;
  return ssc::rulebook_begin_impl(indices, n_in, g, workspace, workspace_bytes, pairs, pair_num,
                                  out_indices, out_capacity, clean_table, clean_table_bytes,
                                  nullptr, &seeded, (hipStream_t)stream, nullptr);
}
}  // extern "C"

int ssc::rulebook_begin_impl(const int32_t *indices, int64_t n_in, const ssc_geometry *g,
                             void *workspace, size_t workspace_bytes, int32_t *pairs,
                             int32_t *pair_num, int32_t *out_indices, int64_t out_capacity,
                             void *clean_table, size_t clean_table_bytes,
                             const SplitRequest *split, bool *seeded, hipStream_t s,
                             const CombineJob *job) {
  Geom gg;
  *seeded = false;
  int rc = rulebook_check(g, &gg, indices, n_in, workspace, workspace_bytes);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(pair_num != nullptr, SSC_EINVAL, "pair_num is NULL");
  SSC_CHECK(n_in == 0 || pairs != nullptr, SSC_EINVAL, "pairs is NULL");
  // the filters' job rides on the first launch that looks at the rows; without rows it runs alone
  if (job != nullptr && n_in == 0) {
    if ((rc = launch_combine_pack(*job, s)) != SSC_OK) return rc;
    job = nullptr;
  }
  if (n_in == 0) return fill_i32(pair_num, gg.K, 0, s);
  SSC_CHECK(out_indices == nullptr || out_capacity >= rulebook_out_bound(gg, n_in), SSC_EINVAL,
            "out_indices holds %lld rows, fewer than the bound of %lld", (long long)out_capacity,
            (long long)rulebook_out_bound(gg, n_in));
  RulebookWs w = rulebook_ws_carve(workspace, gg, n_in);
  // the kernel that finishes the scan leaves the totals in pinned host memory; the pair
  // lists (and the output rows, when the caller brought room for any number of them), whose
  // sizes do not depend on the totals, are computed while the host wakes up
  int32_t *mirror = nullptr;
  if ((rc = read_back_mirror(&mirror)) != SSC_OK) return rc;
  if (split != nullptr &&
      !(w.can_seed && split->n_rng >= 1 && split->n_rng <= kMaxRanges &&
        split->range_row0 != nullptr && split->n_rng_alt >= 0 && split->n_rng_alt <= kMaxRanges &&
        (split->n_rng_alt == 0 || split->range_row0_alt != nullptr)))
    split = nullptr;
  *seeded = split != nullptr;
  // A table the caller keeps between calls: all zero now, and all zero again when the
  // kernels queued here are done (the launch of the pair lists clears it: by then nothing
  // reads it any more).  It holds the input table of the dilation path behind a header with
  // the totals and flags, and saves the launch that would clear them.
  uint32_t *clean = nullptr;
  int64_t clean_words = 0;
  const size_t clean_need = rulebook_clean_bytes(gg, n_in);
  if (clean_table != nullptr && w.use_dense && clean_need > 0 && clean_table_bytes >= clean_need) {
    clean = static_cast<uint32_t *>(clean_table);
    clean_words = (int64_t)(clean_need / 4);
    w.table.total = static_cast<int32_t *>(clean_table);
    w.in_bits = clean + kCleanHeader / 4;
  }
  // With room for the output rows at hand a regular rulebook needs no launch for the scan's
  // second pass: the launch of the pair lists takes the prefixes in two levels, places the
  // range boundaries and hands the totals to the host, which sees them (read_back_end) while
  // that launch still runs.
  const int split_blocks = split ? split_request_blocks(*split) : 0;
  const bool two_level = w.can_seed && out_indices != nullptr &&
                         ceil_div(w.n_chunks, 4) > split_blocks;
  // (the kernel that finishes the scan stores a ticket behind the totals, for the host to
  // spin on: it then sees them a few microseconds before the event behind the kernel says so)
  const int ticket = read_back_mirror_ticket();
  if ((rc = rulebook_mark_and_scan(indices, n_in, gg, w, pair_num, mirror, s, split,
                                   clean != nullptr, two_level, job, ticket)) != SSC_OK)
    return rc;
  if (!two_level) {
    if ((rc = read_back_mirror_queued(s, ticket)) != SSC_OK) return rc;
    return rulebook_pairs(indices, n_in, gg, w, out_indices, pairs, pair_num, true, s, clean,
                          clean_words);
  }
  TwoLevel two = {w.table.blocksum, w.pairsum, w.seed_rows, w.seed_pairs, w.table.n_scan_blocks,
                  split ? *split : SplitRequest{0, 0, 0, nullptr, 0, 0, nullptr}, split_blocks,
                  w.table.total,
                  mirror, ticket, clean != nullptr ? 1 : 0};
  // (the header of a clean table holds the totals: the block that hands them to the host
  // clears it, the other blocks the words behind it)
  if ((rc = rulebook_pairs(indices, n_in, gg, w, out_indices, pairs, pair_num, true, s,
                           clean ? clean + kCleanHeader / 4 : nullptr,
                           clean ? clean_words - (int64_t)(kCleanHeader / 4) : 0, &two)) != SSC_OK)
    return rc;
  return read_back_mirror_queued(s, two.ticket);
}

extern "C" {

int ssc_rulebook_finish(const ssc_geometry *g, int64_t n_in, int32_t *n_out_host,
                        int32_t *in_order_host) {
  Geom gg;
  int rc = make_geom(g, &gg);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(n_out_host != nullptr && in_order_host != nullptr, SSC_EINVAL,
            "n_out_host or in_order_host is NULL");
  if (n_in == 0) {
    *n_out_host = 0;
    *in_order_host = 1;
    return SSC_OK;
  }
  const void *view;
  if ((rc = read_back_end(&view)) != SSC_OK) return rc;
  return rulebook_totals(static_cast<const int32_t *>(view), gg, n_in, n_out_host, in_order_host);
}

int ssc_rulebook_rows(const ssc_geometry *g, int64_t n_in, void *workspace, size_t workspace_bytes,
                      int32_t *out_indices, ssc_stream_t stream) {
  Geom gg;
  int rc = make_geom(g, &gg);
  if (rc != SSC_OK) return rc;
  if (n_in == 0 || gg.subm) return SSC_OK;
  SSC_CHECK(workspace != nullptr && out_indices != nullptr, SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(workspace_bytes >= rulebook_ws_bytes(gg, n_in), SSC_EWORKSPACE,
            "rulebook workspace too small");
  RulebookWs w = rulebook_ws_carve(workspace, gg, n_in);
  hipLaunchKernelGGL(emit_rows_kernel, dim3((unsigned)ceil_div(w.table.n_words, 256)), dim3(256), 0,
                     (hipStream_t)stream, w.table.bits, w.table.prefix, w.table.n_words, gg.os[0],
                     gg.os[1], gg.os[2], out_indices);
  SSC_LAUNCH_CHECK("emit_rows");
  return SSC_OK;
}

size_t ssc_unique_workspace_bytes(const int32_t dims[4], int64_t n) {
  (void)n;
  int64_t cells = (int64_t)dims[0] * dims[1] * dims[2] * dims[3];
  if (cells <= 0 || cells >= ((int64_t)1 << 31)) return 0;
  return bit_table_bytes(cells);
}

static int unique_check(const int32_t dims[4], int64_t n, const void *ws, size_t ws_bytes,
                        int64_t *cells) {
  SSC_CHECK(dims != nullptr, SSC_EINVAL, "dims is NULL");
  for (int a = 0; a < 4; ++a) SSC_CHECK(dims[a] >= 1, SSC_EINVAL, "dims[%d] must be positive", a);
  *cells = (int64_t)dims[0] * dims[1] * dims[2] * dims[3];
  SSC_CHECK(*cells < ((int64_t)1 << 31), SSC_ERUNTIME, "prod(dims) does not fit 31 bits");
  SSC_CHECK(n >= 0, SSC_EINVAL, "n is negative");
  SSC_CHECK(n == 0 || ws != nullptr, SSC_EINVAL, "workspace is NULL");
  SSC_CHECK(n == 0 || ws_bytes >= bit_table_bytes(*cells), SSC_EWORKSPACE,
            "unique workspace too small");
  return SSC_OK;
}

static int unique_bad_row(const int32_t dims[4]) {
  return fail(SSC_EINVAL, "a row lies outside the grid of (%d, %d, %d, %d) cells", dims[0], dims[1],
              dims[2], dims[3]);
}

int ssc_unique_count(const int32_t *coords, int64_t n, const int32_t dims[4], void *workspace,
                     size_t workspace_bytes, int32_t *n_unique_host, ssc_stream_t stream) {
  int64_t cells;
  int rc = unique_check(dims, n, workspace, workspace_bytes, &cells);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(n_unique_host != nullptr, SSC_EINVAL, "n_unique_host is NULL");
  if (n == 0) {
    *n_unique_host = 0;
    return SSC_OK;
  }
  hipStream_t s = (hipStream_t)stream;
  Carver c(workspace);
  BitTable t = bit_table_carve(c, cells);
  if ((rc = bit_table_clear(t, s)) != SSC_OK) return rc;
  hipLaunchKernelGGL(mark_rows_kernel<false>, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s,
                     coords, n, dims[0], dims[1], dims[2], dims[3], t.bits, t.total + 1, 0,
                     CombineJob{}, (int64_t)0);
  SSC_LAUNCH_CHECK("mark_rows");
  if ((rc = bit_table_scan(t, s)) != SSC_OK) return rc;
  int32_t host[2];
  if ((rc = read_back(host, t.total, sizeof(host), s)) != SSC_OK) return rc;
  if (host[1] & kFlagBadRow) return unique_bad_row(dims);
  *n_unique_host = host[0];
  return SSC_OK;
}

int ssc_unique_emit(const int32_t *coords, int64_t n, const int32_t dims[4], void *workspace,
                    size_t workspace_bytes, int64_t n_unique, int32_t *unique, int32_t *inverse,
                    int32_t *counts, ssc_stream_t stream) {
  int64_t cells;
  int rc = unique_check(dims, n, workspace, workspace_bytes, &cells);
  if (rc != SSC_OK) return rc;
  if (n == 0) return SSC_OK;
  SSC_CHECK(unique != nullptr && inverse != nullptr, SSC_EINVAL, "NULL output pointer");
  hipStream_t s = (hipStream_t)stream;
  Carver c(workspace);
  BitTable t = bit_table_carve(c, cells);
  if (counts && (rc = fill_i32(counts, n_unique, 0, s)) != SSC_OK) return rc;
  hipLaunchKernelGGL(emit_rows_kernel, dim3((unsigned)ceil_div(t.n_words, 256)), dim3(256), 0, s,
                     t.bits, t.prefix, t.n_words, dims[1], dims[2], dims[3], unique);
  SSC_LAUNCH_CHECK("emit_rows");
  hipLaunchKernelGGL(inverse_counts_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s,
                     coords, n, dims[0], dims[1], dims[2], dims[3], t.bits, t.prefix, inverse,
                     counts, (int32_t *)nullptr);
  SSC_LAUNCH_CHECK("inverse_counts");
  return SSC_OK;
}

int ssc_unique_build(const int32_t *coords, int64_t n, const int32_t dims[4], void *workspace,
                     size_t workspace_bytes, int32_t *inverse, int32_t *counts,
                     int32_t *totals_host, ssc_stream_t stream) {
  int64_t cells;
  int rc = unique_check(dims, n, workspace, workspace_bytes, &cells);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(totals_host != nullptr, SSC_EINVAL, "totals_host is NULL");
  if (n == 0) {
    totals_host[0] = totals_host[1] = 0;
    return SSC_OK;
  }
  SSC_CHECK(inverse != nullptr && counts != nullptr, SSC_EINVAL, "NULL output pointer");
  hipStream_t s = (hipStream_t)stream;
  Carver c(workspace);
  BitTable t = bit_table_carve(c, cells);
  // total[0]: the number of distinct rows (written by the scan); total[1]: flags;
  // total[2]: the largest count; all cleared with the table
  if ((rc = bit_table_clear(t, s)) != SSC_OK) return rc;
  hipLaunchKernelGGL(mark_rows_kernel<false>, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s,
                     coords, n, dims[0], dims[1], dims[2], dims[3], t.bits, t.total + 1, 0,
                     CombineJob{}, (int64_t)0);
  SSC_LAUNCH_CHECK("mark_rows");
  if ((rc = bit_table_scan(t, s)) != SSC_OK) return rc;
  if ((rc = fill_i32(counts, n, 0, s)) != SSC_OK) return rc;
  hipLaunchKernelGGL(inverse_counts_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s,
                     coords, n, dims[0], dims[1], dims[2], dims[3], t.bits, t.prefix, inverse,
                     counts, t.total + 2);
  SSC_LAUNCH_CHECK("inverse_counts");
  int32_t host[3];
  if ((rc = read_back(host, t.total, sizeof(host), s)) != SSC_OK) return rc;
  if (host[1] & kFlagBadRow) return unique_bad_row(dims);
  totals_host[0] = host[0];
  totals_host[1] = host[2];
  return SSC_OK;
}

int ssc_unique_rows(const int32_t dims[4], int64_t n, void *workspace, size_t workspace_bytes,
                    int32_t *unique, ssc_stream_t stream) {
  int64_t cells;
  int rc = unique_check(dims, n, workspace, workspace_bytes, &cells);
  if (rc != SSC_OK) return rc;
  if (n == 0) return SSC_OK;
  SSC_CHECK(unique != nullptr, SSC_EINVAL, "unique is NULL");
  Carver c(workspace);
  BitTable t = bit_table_carve(c, cells);
  hipLaunchKernelGGL(emit_rows_kernel, dim3((unsigned)ceil_div(t.n_words, 256)), dim3(256), 0,
                     (hipStream_t)stream, t.bits, t.prefix, t.n_words, dims[1], dims[2], dims[3],
                     unique);
  SSC_LAUNCH_CHECK("emit_rows");
  return SSC_OK;
}
}
