// Sparse convolution forward as an output-stationary implicit GEMM on fp32 MFMA.
//
// Outputs are cut into tiles of at most T consecutive rows.  A workgroup owns one
// tile and 64 output columns at a time; the tile's accumulators live in LDS until
// the tile is complete.  For every kernel offset k the pairs that land in the tile
// form one contiguous segment of the rulebook (pairs of an offset are ascending in
// output row), so they are packed 16 at a time into the M side of
// v_mfma_f32_16x16x4_f32: the gathered input rows are staged in LDS, the matching
// 16x16 weight fragments are held in registers, and the product is added to the
// LDS accumulators at the pairs' output rows.  Only occupied (row, offset) slots
// cost MFMA work, and because each wave owns a fixed set of columns and walks the
// offsets in ascending order the result is bit-reproducible without atomics.
//
// Host side of a call: pack the filters into MFMA fragment order; check that the
// pairs are sorted (re-order them if not); split the output rows over the
// workgroups by work and cut the ranges into tiles; build the row-block schedule;
// launch the persistent kernel.
#include "combine_element.h"
#include "conv_kernel.h"
#include "conv_pack.h"
#include "ssc_common.h"

namespace ssc {
static_assert(kPackKC == kKC, "conv_pack.h packs half filters in chunks of kKC channels");


// ---- weight packing ---------------------------------------------------------------------
// packed[((k*NCB + ncb)*NCH + cc)*1024 + q*256 + lane*4 + j] =
//     W[k][cc*64 + 16q + (lane/16)*4 + j][ncb*16 + lane%16]   (0 outside Cin/Cout)
// i.e. the weight fragments of MFMA steps 4q + j of chunk cc for column block ncb, laid
// out so that a wave reads them as four 16-byte loads per lane, each load one contiguous
// KiB (lane l at byte 16 l): 8 cache lines an instruction, where a lane-major layout
// (64 bytes per lane) touches 32.  The four steps of load q cover the 16 channels
// 16q .. 16q+15 of the chunk (lane group g has channels 16q + 4g .. +3), so a layer with
// few input channels needs only its first loads.
//
// A chunk need not hold 64 channels: with ns < 16 MFMA steps per chunk it holds 4 ns, the
// channels cc*4ns .. cc*4ns + 4ns - 1, and only the first ns of the 16 (q, j) slots carry
// weights.  The quarters below ns / 4 are laid out as above.  In the quarter that is only
// partly used (ns % 4 steps) step j must stand for four consecutive channels, one per lane
// group, so there slot (q, lane group g, j) holds channel 16q + 4j + g of the chunk (the
// rows staged in LDS follow the same rule: conv_fwd_kernel's producers), and the quarter is
// packed densely, ns % 4 floats per lane at float 256 (ns / 4) + lane (ns % 4) + j of the
// fragment: a wave fetches 256 (ns % 4) bytes for it instead of a KiB.
//
// Half-precision filters are packed for v_mfma_f32_16x16x32_f16 instead, two steps of 32
// channels per chunk (halves, 2 KiB per fragment):
// packed[((k*NCB + ncb)*NCH + cc)*1024 + q*512 + lane*8 + j] =
//     W[k][cc*64 + 32q + (lane/16)*8 + j][ncb*16 + lane%16]
// i.e. one 16-byte load per lane and step.  Which of a step's 32 channels sits in which of
// a lane's 8 slots does not matter for the sum as long as the staged rows use the same
// assignment; they do (lane group g reads channels 32q + 8g .. +7 of its row).
// Synthesis of the dense float kernel and its packing in one launch: one thread per packed
// element computes the element (combine_element), stores it at its place in the packed
// filters and in the dense [K, Cin, Cout] array (every dense element has exactly one packed
// place; padding places get zero).
__global__ void __launch_bounds__(256)
    combine_pack_kernel(PackArgs a, const float *__restrict__ weight,
                        const float *__restrict__ basis, const int32_t *__restrict__ chan_out,
                        const int32_t *__restrict__ chan_in, const int32_t *__restrict__ blocks,
                        int n_j, float *__restrict__ dense) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)a.K * a.ncb * a.nch * 1024) return;
  const CombineJob job = {a, weight, basis, chan_out, chan_in, blocks, n_j, dense};
  combine_pack_element(job, idx);
}

// (for a rulebook that was handed a CombineJob it cannot take along)
int launch_combine_pack(const CombineJob &job, hipStream_t s) {
  const int64_t n = combine_job_elements(job);
  hipLaunchKernelGGL(combine_pack_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s, job.pk,
                     job.weight, job.basis, job.chan_out, job.chan_in, job.blocks, job.n_j,
                     job.dense);
  SSC_LAUNCH_CHECK("combine_pack");
  return SSC_OK;
}

template <typename IO>
__global__ void __launch_bounds__(256) pack_filters_kernel(PackArgs a, int32_t *__restrict__ flag) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx == 0 && flag != nullptr) flag[0] = 0;  // the pair-order flag of the kernels that follow
  if (idx < (int64_t)a.K * a.ncb * a.nch * 1024) pack_filter_element<IO>(a, idx);
}

// ---- pair order -------------------------------------------------------------------------
// flag[0] |= 1 when some offset's scatter rows are not strictly ascending.
__global__ void __launch_bounds__(256)
    check_sorted_kernel(const int32_t *__restrict__ pairs, int64_t pair_stride, int plane_s,
                        const int32_t *__restrict__ pair_num, int32_t *__restrict__ flag) {
  int k = blockIdx.y;
  int n = pair_num[k];
  const int32_t *s = pairs + ((int64_t)k * 2 + plane_s) * pair_stride;
  int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j + 1 < n && s[j] >= s[j + 1]) atomicOr(flag, 1);
}

// Re-ordering of unsorted pair lists (rare: inputs not in ascending key order).
// Scatter rows are unique inside an offset, so their rank in a per-offset bit
// table over [0, n_out) is their sorted position.  Every kernel returns at once
// when flag[0] == 0.
__global__ void __launch_bounds__(256)
    resort_clear_kernel(const int32_t *__restrict__ flag, uint32_t *__restrict__ bits, int64_t n) {
  if (flag[0] == 0) return;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += step) bits[i] = 0u;
}

__global__ void __launch_bounds__(256)
    resort_mark_kernel(const int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                       int64_t pair_stride, int plane_s, const int32_t *__restrict__ pair_num,
                       uint32_t *__restrict__ bits, int64_t words_per_k) {
  if (flag[0] == 0) return;
  int k = blockIdx.y;
  int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= pair_num[k]) return;
  uint32_t o = (uint32_t)pairs[((int64_t)k * 2 + plane_s) * pair_stride + j];
  atomicOr(&bits[(int64_t)k * words_per_k + (o >> 5)], 1u << (o & 31u));
}

__global__ void __launch_bounds__(kScanThreads)
    resort_scan_kernel(const int32_t *__restrict__ flag, const uint32_t *__restrict__ bits,
                       int32_t *__restrict__ prefix, int64_t words_per_k) {
  if (flag[0] == 0) return;
  __shared__ int lds[kScanThreads / 64 + 1];
  const uint32_t *b = bits + (int64_t)blockIdx.x * words_per_k;
  int32_t *p = prefix + (int64_t)blockIdx.x * words_per_k;
  int carry = 0;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int64_t base = 0; base < words_per_k; base += kScanThreads) {
    int64_t i = base + threadIdx.x;
    int v = i < words_per_k ? __popc(b[i]) : 0;
    int incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      int o = __shfl_up(incl, d, 64);
      if (lane >= d) incl += o;
    }
    if (lane == 63) lds[wave] = incl;
    __syncthreads();
    int wave_off = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < kScanThreads / 64; ++w) {
      int x = lds[w];
      if (w < wave) wave_off += x;
      tot += x;
    }
    __syncthreads();
    if (i < words_per_k) p[i] = carry + wave_off + incl - v;
    carry += tot;
  }
}

__global__ void __launch_bounds__(256)
    resort_scatter_kernel(const int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                          int64_t pair_stride, int plane_s, const int32_t *__restrict__ pair_num,
                          const uint32_t *__restrict__ bits, const int32_t *__restrict__ prefix,
                          int64_t words_per_k, int32_t *__restrict__ sorted) {
  if (flag[0] == 0) return;
  int k = blockIdx.y;
  int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= pair_num[k]) return;
  const int32_t *ps = pairs + ((int64_t)k * 2 + plane_s) * pair_stride;
  const int32_t *pg = pairs + ((int64_t)k * 2 + (1 - plane_s)) * pair_stride;
  uint32_t o = (uint32_t)ps[j];
  int pos = bit_rank(bits + (int64_t)k * words_per_k, prefix + (int64_t)k * words_per_k, o);
  sorted[((int64_t)k * 2 + plane_s) * pair_stride + pos] = (int32_t)o;
  sorted[((int64_t)k * 2 + (1 - plane_s)) * pair_stride + pos] = pg[j];
}

// segs[t*K + k] = first pair of offset k whose scatter row is >= the first row of
// tile t (t = 0..n_tiles; tile rows from tile_row0[], tile count from n_tiles_dev[0]).
// The search starts from the cell of the tile's first row in grid_segs[], the same
// segments for a regular grid of `granule` rows (grid_segments_kernel).
// Also spill[t*K + k] = how far the last row block of tile t-1 may reach into tile t:
// the first pair at or after segs[t*K + k], at most 15 further, whose row is >=
// spill_end[t].
__global__ void __launch_bounds__(256)
    tile_segments_kernel(const int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                         const int32_t *__restrict__ sorted, int64_t pair_stride, int plane_s,
                         const int32_t *__restrict__ pair_num, int K,
                         const int32_t *__restrict__ n_tiles_dev,
                         const int32_t *__restrict__ tile_row0, int64_t n_out,
                         const int32_t *__restrict__ grid_segs, int granule,
                         const int32_t *__restrict__ spill_end, int32_t *__restrict__ segs,
                         int32_t *__restrict__ spill) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t n_tiles = n_tiles_dev[0];
  if (idx >= (n_tiles + 1) * K) return;
  int64_t t = idx / K;
  int k = (int)(idx - t * K);
  const int32_t *src = flag[0] ? sorted : pairs;
  const int32_t *s = src + ((int64_t)k * 2 + plane_s) * pair_stride;
  int64_t target = tile_row0[t];
  if (target > n_out) target = n_out;
  const int n = pair_num[k];
  const int64_t cell = target / granule;  // a cell of the grid, or its end
  int lo = grid_segs[cell * K + k];
  int hi = (cell + 1) * granule <= n_out ? grid_segs[(cell + 1) * K + k] : n;
  while (lo < hi) {
    int mid = (lo + hi) >> 1;
    if (s[mid] < target) lo = mid + 1;
    else hi = mid;
  }
  segs[idx] = lo;
  const int bound = spill_end[t];
  int cnt = 0;
#pragma unroll
  for (int j = 0; j < 15; ++j) cnt += (lo + j < n && s[lo + j] < bound) ? 1 : 0;  // rows ascend
  spill[idx] = lo + cnt;
}

// segs[c*K + k] = first pair of offset k whose scatter row is >= c*granule, for the
// cells c = 0..n_cells of a regular grid (cell n_cells being the end), computed from
// the pairs' side: one thread per pair; the pair
// that is the first of its offset at or beyond a cell boundary writes that boundary.
//
// Rows y >= K of the grid, when the launch has them, do an unrelated job that depends on
// nothing before it: they pack the filters (strided over the packed elements) and clear
// flag[0] for the kernels that follow.  Such a launch is told that the pairs are in order
// (`pairs_in_order`) and does not read the flag itself.
template <typename IO>
__global__ void __launch_bounds__(256)
    grid_segments_kernel(int32_t *__restrict__ flag, int pairs_in_order,
                         const int32_t *__restrict__ pairs, const int32_t *__restrict__ sorted,
                         int64_t pair_stride, int plane_s, const int32_t *__restrict__ pair_num,
                         int K, int64_t n_cells, int granule, int32_t *__restrict__ segs,
                         PackArgs pack) {
  if ((int)blockIdx.y >= K) {
    const int64_t total = (int64_t)pack.K * pack.ncb * pack.nch * 1024;
    const int64_t step = (int64_t)(gridDim.y - K) * gridDim.x * blockDim.x;
    int64_t idx = ((int64_t)(blockIdx.y - K) * gridDim.x + blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx == 0) flag[0] = 0;
    for (; idx < total; idx += step) pack_filter_element<IO>(pack, idx);
    return;
  }
  const int k = blockIdx.y;
  const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int n = pair_num[k];
  if (j >= n && !(j == 0 && n == 0)) return;
  const int32_t *src = (!pairs_in_order && flag[0]) ? sorted : pairs;
  const int32_t *s = src + ((int64_t)k * 2 + plane_s) * pair_stride;
  // boundary c (first row c*granule) is served by the first pair whose row is at or
  // beyond it: pair j serves the boundaries in (row[j-1], row[j]]
  int64_t c_next = 0;  // first boundary beyond this pair
  if (n > 0) {
    const int64_t c1 = s[j] / granule;
    const int64_t c0 = j > 0 ? (int64_t)s[j - 1] / granule + 1 : 0;
    for (int64_t c = c0; c <= c1 && c <= n_cells; ++c) segs[c * K + k] = (int32_t)j;
    c_next = c1 + 1;
  }
  if (n == 0 || j == n - 1)  // boundaries beyond the last pair
    for (int64_t c = c_next; c <= n_cells; ++c) segs[c * K + k] = n;
}

// ---- work split ------------------------------------------------------------------------
// Output rows are dealt to the persistent workgroups in contiguous ranges of equal
// WORK, not equal length: work(r) = pairs that land in rows < r, plus a per-row
// share of what every tile costs on top of its pairs (padding of the last row block
// of each offset, writing the tile out).  Pairs per row come from a fine grid of
// kSplitGranule rows; range boundaries lie on that grid.  Each range is then cut
// into tiles (range_tiles below: equal heights of about T at most, a higher last one).
// (16 rows where a range has fewer than 2048: with 3.5 cells of 64 rows to a range -- the
// input gradient of the 64 -> 128 benchmark layer, 57 k rows for 256 workgroups -- the
// ranges' work differed by 14 %)
constexpr int kSplitGranule = 64, kSplitGranuleSmall = 16;
constexpr int kTileSlack = 24;
// The accumulator window of a workgroup holds kSpillRows more rows than a tile is
// high: the last row block that an offset contributes to a tile may then be filled
// up with the offset's next pairs, whose rows lie in the following tile (at most
// kSpillRows into it), instead of being padded.  Rows map to accumulator slots
// modulo the window height, so what such a block adds to the next tile's rows is
// still there when that tile's turn comes.
constexpr int kSpillRows = 160;
// (the five-group form, whose window is 376 rows: 200 -> 200 channels with 125 offsets takes
// 14.3 ms with 160, 13.9 with 192 or 224, 14.7 with 128)
constexpr int kSpillRowsFive = 192;

// cost of a tile beyond its pairs, in pair slots: padding per offset, and about a stage's
// worth of time for writing it out (measured: 2 K + 128 and 3 K + 64 are as good on the
// 27-offset benchmark layers; with 125 offsets 4 K + 64 is 4 % faster than 2 K + 128, and
// more than that slower again)
__device__ __forceinline__ int64_t split_tile_cost(int K) { return (int64_t)K * 4 + 64; }

// Work in rows below cell b of the fine grid (scaled by T to stay in integers).
__device__ __forceinline__ int64_t split_work(int64_t pairs_below, int64_t b, int64_t n_out,
                                              int T, int K, int granule) {
  int64_t r = b * granule;
  if (r > n_out) r = n_out;
  return pairs_below * T + r * split_tile_cost(K);
}

// One thread per cell boundary b = 0..nb of the fine grid: the ranges whose first row
// is boundary b are those whose target (w/n_wg of the total work) lies in
// (work(b-1), work(b)].  range_row0[w], w = 0..n_wg.
__global__ void __launch_bounds__(256)
    split_bounds_kernel(const int32_t *__restrict__ fine_segs, int K, int64_t nb, int64_t n_out,
                        int T, int n_wg, int granule, int32_t *__restrict__ range_row0) {
  int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b > nb) return;
  int64_t below = 0, below_prev = 0, all = 0;
  for (int k = 0; k < K; ++k) {
    below += fine_segs[b * K + k];
    if (b > 0) below_prev += fine_segs[(b - 1) * K + k];
    all += fine_segs[nb * K + k];
  }
  const int64_t total = split_work(all, nb, n_out, T, K, granule);
  // ranges w with ceil(total * w / n_wg) <= work, i.e. w <= work * n_wg / total
  auto reached = [&](int64_t work) -> int64_t {
    if (total <= 0) return n_wg + 1;
    int64_t c = work * n_wg / total + 1;
    return c > n_wg + 1 ? n_wg + 1 : c;
  };
  const int64_t w0 = b > 0 ? reached(split_work(below_prev, b - 1, n_out, T, K, granule)) : 0;
  const int64_t w1 = reached(split_work(below, b, n_out, T, K, granule));
  int64_t r = b * granule;
  if (r > n_out) r = n_out;
  for (int64_t w = w0; w < w1; ++w)
    range_row0[w] = (w == 0) ? 0 : (w == n_wg ? (int32_t)n_out : (int32_t)r);
}

// The split again, from what the first one turned out to cost.  The schedule of the first
// split is counted by then: range_grp[w] row-block groups for range w, where the model
// above had promised every range the same work -- what a tile pads depends on how many
// offsets it meets with how many pairs each, which the model does not see, and the slowest
// workgroup sets the kernel's time.  Here a row's modelled work counts with the factor its
// range showed, groups per modelled work, and the boundaries are placed anew for equal
// corrected work: boundary b of the fine grid has
//   cum(b) = groups of the ranges before b's range + groups of that range * the part of
//            its modelled work that lies below b,
// and the ranges whose target (w / n_wg of all groups) lies in (cum(b-1), cum(b)] begin
// there.  row_old: range_row0 of the first split; row_new: that of the second.
__global__ void __launch_bounds__(256)
    split_rebalance_kernel(const int32_t *__restrict__ fine_segs, int K, int64_t nb,
                           int64_t n_out, int T, int n_wg, int granule,
                           const int32_t *__restrict__ row_old,
                           const int32_t *__restrict__ range_grp, int32_t *__restrict__ row_new) {
  __shared__ int row_s[kMaxRanges + 1];
  __shared__ double work_s[kMaxRanges + 1];  // modelled work below the first row of range w
  __shared__ double grp_s[kMaxRanges + 1];   // groups of the ranges before range w
  auto cell_of = [&](int64_t row) -> int64_t { return (row + granule - 1) / granule; };
  auto work_below = [&](int64_t cell) -> double {
    int64_t below = 0;
    for (int k = 0; k < K; ++k) below += fine_segs[cell * K + k];
    return (double)split_work(below, cell, n_out, T, K, granule);
  };
  for (int w = threadIdx.x; w <= n_wg; w += blockDim.x) {  // n_wg ranges, <= kMaxRanges
    int r = row_old[w];
    if (w == 0) r = 0;
    if (w == n_wg) r = (int)n_out;
    row_s[w] = r;
    work_s[w] = work_below(cell_of(r));  // range boundaries lie on the grid, or at the end
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double run = 0.0;
    for (int w = 0; w < n_wg; ++w) {
      grp_s[w] = run;
      run += (double)range_grp[w];
    }
    grp_s[n_wg] = run;
  }
  __syncthreads();
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b > nb) return;
  const double total = grp_s[n_wg];
  // corrected work below cell c
  auto cum = [&](int64_t c) -> double {
    if (c >= nb) return total;
    int64_t r = c * granule;
    if (r > n_out) r = n_out;
    // the last range that begins at or before row r and does not end there
    int lo = 0, hi = n_wg - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (row_s[mid] <= r) lo = mid;
      else hi = mid - 1;
    }
    const double span = work_s[lo + 1] - work_s[lo];
    const double part = span > 0.0 ? (work_below(c) - work_s[lo]) / span : 0.0;
    const double g = grp_s[lo + 1] - grp_s[lo];
    return grp_s[lo] + g * (part < 0.0 ? 0.0 : part > 1.0 ? 1.0 : part);
  };
  auto reached = [&](double c) -> int64_t {
    if (total <= 0.0) return n_wg + 1;
    const int64_t v = (int64_t)(c * (double)n_wg / total) + 1;
    return v > n_wg + 1 ? n_wg + 1 : v;
  };
  const int64_t w0 = b > 0 ? reached(cum(b - 1)) : 0;
  const int64_t w1 = reached(cum(b));
  int64_t r = b * granule;
  if (r > n_out) r = n_out;
  for (int64_t w = w0; w < w1; ++w)
    row_new[w] = (w == 0) ? 0 : (w == n_wg ? (int32_t)n_out : (int32_t)r);
}

// One block.  wg_tile[0..n_wg]: first tile of every range (n_wg of them); tile_row0[0..n_tiles]:
// first row of every tile; n_tiles_dev[0]: number of tiles; spill_end[0..n_tiles]:
// rows below spill_end[t] may be touched by the last row blocks of tile t-1 (the
// first row of tile t itself when t starts a workgroup's range: no spill across
// ranges); tile_slot0[t]: accumulator slot of the first row of tile t.  T is the
// largest tile height, window the height of the accumulator window.
// How a range of `rows` output rows is cut into tiles: nt tiles, all of height h but the last,
// which has what is left.  T is the height a tile has when the window behind it keeps the
// usual room for spilled row blocks (window - T rows).  The last tile of a range spills
// nowhere -- the next rows are another workgroup's -- so it may fill the window: it is
// given up to window - T - kTileSlack rows more than the others.  And a range a little
// longer than a whole number of tiles does not get one more: its tiles grow by up to
// kTileSlack rows in all, at the cost of as many rows of spill.  (Every tile more pads the
// last row block of every offset once more.)
__host__ __device__ __forceinline__ void range_tiles(int rows, int T, int window, int *nt, int *h) {
  if (rows <= 0) {
    *nt = 0;
    *h = 0;
    return;
  }
  const int bonus = window - T - kTileSlack;  // > 0: T <= window - 160
  const int eff = rows - bonus;
  int n = (eff - kTileSlack + T - 1) / T;
  if (eff - kTileSlack <= 0 || n < 1) n = 1;
  if (n == 1) {
    *nt = 1;
    *h = rows;
    return;
  }
  // h <= T + kTileSlack.  Tiles of that height until what is left fits the last one: with
  // hundreds of tiles to a range the rounding of h adds up to whole tiles, and n tiles of
  // height h would reach beyond the range's end.  The last tile has between bonus + 1 and
  // bonus + h rows.
  const int hh = (eff + n - 1) / n;
  *h = hh;
  *nt = (eff + hh - 1) / hh;
}

__global__ void __launch_bounds__(kMaxRanges)
    split_rows_kernel(const int32_t *__restrict__ range_row0, int64_t n_out, int T, int window,
                      int n_wg, int32_t *__restrict__ wg_tile, int32_t *__restrict__ tile_row0,
                      int32_t *__restrict__ n_tiles_dev, int32_t *__restrict__ spill_end,
                      int32_t *__restrict__ tile_slot0) {
  __shared__ int row_s[kMaxRanges + 1];
  __shared__ int tile_s[kMaxRanges + 1];
  for (int w = threadIdx.x; w <= n_wg; w += blockDim.x) {  // n_wg ranges, <= kMaxRanges
    int r = range_row0[w];
    if (w == 0) r = 0;
    if (w == n_wg) r = (int)n_out;
    row_s[w] = r;
  }
  __syncthreads();
  {
    // exclusive scan of the tile counts of the ranges, one per thread
    __shared__ int wave_sum[kMaxRanges / 64];
    const int w = threadIdx.x, lane = w & 63;
    int nt = 0, h_unused = 0;
    if (w < n_wg) range_tiles(row_s[w + 1] - row_s[w], T, window, &nt, &h_unused);
    int incl = nt;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      int o = __shfl_up(incl, d, 64);
      if (lane >= d) incl += o;
    }
    if (lane == 63) wave_sum[w >> 6] = incl;
    __syncthreads();
    int before = 0;
    for (int i = 0; i < (w >> 6); ++i) before += wave_sum[i];
    if (w < n_wg) tile_s[w] = before + incl - nt;
    if (w == kMaxRanges - 1) {
      const int run = before + incl;
      tile_s[n_wg] = run;
      n_tiles_dev[0] = run;
      n_tiles_dev[1] = 0;  // (the cursor of range_sched_kernel<true>)
      tile_row0[run] = (int32_t)n_out;
      spill_end[run] = (int32_t)n_out;
    }
  }
  __syncthreads();
  for (int w = threadIdx.x; w <= n_wg; w += blockDim.x) {
    wg_tile[w] = tile_s[w];
    if (w == n_wg) break;
    const int rows = row_s[w + 1] - row_s[w];
    int nt = 0, h = 0;
    range_tiles(rows, T, window, &nt, &h);  // nt == tile_s[w + 1] - tile_s[w]
    if (nt > 0) {
      for (int j = 0; j < nt; ++j) {
        const int r = row_s[w] + j * h;
        tile_row0[tile_s[w] + j] = r;
        // (tile and spill fill the window: a tile lower than the highest spills further)
        spill_end[tile_s[w] + j] = j == 0 ? r : min(r + window - h, row_s[w + 1]);
        tile_slot0[tile_s[w] + j] = (j * h) % window;
      }
    }
  }
}

// The tiles and their segments in one launch, from range boundaries that are there already
// (a rulebook placed them: SplitRequest) and from the pairs' side: a block takes a run of
// kSegChunk consecutive pairs of one offset, whose scatter rows ascend.  Every block first
// works out, in LDS, the rows and the first tile of every range (what split_rows_kernel
// computes); a tile is then a function of its range and its number in it.  The run holds
// the first pair at or beyond the first row of every tile whose first row lies in (row of
// the pair before the run, row of the run's last pair]: for those tiles -- a handful -- a
// thread each bisects the run's rows in LDS and writes segs[] and spill[] as
// tile_segments_kernel does.  Block (0, 0) also writes the tables of the tiles for the
// kernels that follow (wg_tile, tile_row0, spill_end, tile_slot0, n_tiles_dev) and clears
// flag[0]: the pairs are in order.
struct TileOf {
  int t;       // tile
  int row0;    // its first row
  int spill;   // spill_end of the tile
};
__device__ __forceinline__ TileOf tile_of_row(int r, const int *row_s, const int *tile_s,
                                              int n_rng, int T, int window) {
  // the last range that begins at or before r (a range without rows is never the last such)
  int lo = 0, hi = n_rng - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (row_s[mid] <= r) lo = mid;
    else hi = mid - 1;
  }
  int nt, h;
  range_tiles(row_s[lo + 1] - row_s[lo], T, window, &nt, &h);
  int j = h > 0 ? (r - row_s[lo]) / h : 0;
  if (j > nt - 1) j = nt - 1;
  if (j < 0) j = 0;
  TileOf o;
  o.t = tile_s[lo] + j;
  o.row0 = row_s[lo] + j * h;
  o.spill = j == 0 ? o.row0 : min(o.row0 + window - h, row_s[lo + 1]);
  return o;
}

// Tile t by its number: the range that holds it, then as above.
__device__ __forceinline__ TileOf tile_by_index(int t, const int *row_s, const int *tile_s,
                                                int n_rng, int T, int window) {
  int lo = 0, hi = n_rng - 1;  // the last range whose first tile is at or before t
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (tile_s[mid] <= t) lo = mid;
    else hi = mid - 1;
  }
  int nt, h;
  range_tiles(row_s[lo + 1] - row_s[lo], T, window, &nt, &h);
  const int j = t - tile_s[lo];
  TileOf o;
  o.t = t;
  o.row0 = row_s[lo] + j * h;
  o.spill = j == 0 ? o.row0 : min(o.row0 + window - h, row_s[lo + 1]);
  return o;
}

// CHUNK: pairs of one offset to a block.  LDSROWS: the run's rows are staged in LDS and a
// thread bisects them for its tile; otherwise they stay in memory and sixteen lanes find a
// tile's first pair in three rounds of sixteen probes (next to nothing in LDS: such a block
// fits beside a workgroup of the convolution, which leaves a few KB of a CU's LDS).
// Dynamic LDS: 2 (n_rng + 1) ints.
constexpr int kSegChunk = 2048;
template <int CHUNK, bool LDSROWS>
__global__ void __launch_bounds__(256)
    pair_tile_segments_kernel(int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                              int64_t pair_stride, int plane_s,
                              const int32_t *__restrict__ pair_num, int K,
                              const int32_t *__restrict__ range_row0, int n_rng, int T,
                              int window, int n_out, int32_t *__restrict__ wg_tile, int32_t *__restrict__ tile_row0,
                              int32_t *__restrict__ n_tiles_dev, int32_t *__restrict__ spill_end,
                              int32_t *__restrict__ tile_slot0, int32_t *__restrict__ segs,
                              int32_t *__restrict__ spill) {
  extern __shared__ int range_dyn[];
  int *const row_s = range_dyn, *const tile_s = range_dyn + n_rng + 1;
  __shared__ int wave_sum[4];
  // (the loads of the run's rows are issued first: they are not needed before the tables
  // of the ranges stand)
  const int k = blockIdx.y;
  const int64_t j0 = (int64_t)blockIdx.x * CHUNK;
  const int32_t *s = pairs + ((int64_t)k * 2 + plane_s) * pair_stride;
  constexpr int kPer = LDSROWS ? (CHUNK + 15 + 255) / 256 : 1;
  int held[kPer];
  if constexpr (LDSROWS) {
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
      const int64_t idx = j0 + threadIdx.x + 256 * u;
      held[u] = idx < pair_stride ? s[idx] : 0x7FFFFFFF;
    }
  }
  const int r_before = j0 > 0 && j0 <= pair_stride ? s[j0 - 1] : -1;
  const int n = pair_num[k];
  // rows and tile counts of the ranges: two ranges to a thread (n_rng <= 512)
  for (int w = threadIdx.x; w <= n_rng; w += 256) {
    int r = range_row0[w];
    if (w == 0) r = 0;
    if (w == n_rng) r = n_out;
    row_s[w] = r;
  }
  __syncthreads();
  {
    const int w0 = 2 * threadIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int nt0 = 0, nt1 = 0, h_unused = 0;
    if (w0 < n_rng) range_tiles(row_s[w0 + 1] - row_s[w0], T, window, &nt0, &h_unused);
    if (w0 + 1 < n_rng) range_tiles(row_s[w0 + 2] - row_s[w0 + 1], T, window, &nt1, &h_unused);
    const int v = nt0 + nt1;
    int incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      int o = __shfl_up(incl, d, 64);
      if (lane >= d) incl += o;
    }
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    int before = 0;
    for (int i = 0; i < wave; ++i) before += wave_sum[i];
    const int ex = before + incl - v;
    if (w0 <= n_rng) tile_s[w0] = ex;
    if (w0 + 1 <= n_rng) tile_s[w0 + 1] = ex + nt0;
    if (w0 + 2 == n_rng) tile_s[n_rng] = ex + v;  // (512 ranges: no thread has w0 = n_rng)
    __syncthreads();
  }
  const int n_tiles = tile_s[n_rng];
  if (blockIdx.x == 0 && blockIdx.y == 0) {
    if (threadIdx.x == 0) {
      flag[0] = 0;
      n_tiles_dev[0] = n_tiles;
      n_tiles_dev[1] = 0;  // (the cursor of range_sched_kernel<true>)
      tile_row0[n_tiles] = n_out;
      spill_end[n_tiles] = n_out;
    }
    for (int w = threadIdx.x; w <= n_rng; w += 256) {
      wg_tile[w] = tile_s[w];
      if (w == n_rng) break;
      int nt = 0, h = 0;
      range_tiles(row_s[w + 1] - row_s[w], T, window, &nt, &h);
      for (int j = 0; j < nt; ++j) {
        const int r = row_s[w] + j * h;
        tile_row0[tile_s[w] + j] = r;
        spill_end[tile_s[w] + j] = j == 0 ? r : min(r + window - h, row_s[w + 1]);
        tile_slot0[tile_s[w] + j] = (j * h) % window;
      }
    }
  }
  // the block's run of the offset's pairs: their rows (and those of the 15 pairs behind
  // them, for the spill) in LDS
  __shared__ int rows[LDSROWS ? CHUNK + 16 : 1];
  if (n == 0) {  // no pair: every tile's segment is empty
    if (blockIdx.x == 0)
      for (int t = threadIdx.x; t <= n_tiles; t += 256) {
        segs[(int64_t)t * K + k] = 0;
        spill[(int64_t)t * K + k] = 0;
      }
    return;
  }
  if (j0 >= n) return;
  const int cnt = n - j0 < CHUNK ? (int)(n - j0) : CHUNK;
  const int r_prev = r_before;
  int t_hi;
  if constexpr (LDSROWS) {
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
      const int i = threadIdx.x + 256 * u;
      if (i < CHUNK + 15) rows[i] = j0 + i < n ? held[u] : 0x7FFFFFFF;
    }
    __syncthreads();
    // the tiles whose first row lies in (row of the pair before the run, row of its last pair]
    const int t_lo = j0 > 0 ? tile_of_row(r_prev, row_s, tile_s, n_rng, T, window).t + 1 : 0;
    t_hi = tile_of_row(rows[cnt - 1], row_s, tile_s, n_rng, T, window).t;
    for (int t = t_lo + threadIdx.x; t <= t_hi; t += 256) {
      const TileOf tl = tile_by_index(t, row_s, tile_s, n_rng, T, window);
      int lo = 0, hi = cnt - 1;  // the first pair of the run at or beyond the tile's first row
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (rows[mid] < tl.row0) lo = mid + 1;
        else hi = mid;
      }
      int beyond = 0;
#pragma unroll
      for (int q = 0; q < 15; ++q) beyond += rows[lo + q] < tl.spill ? 1 : 0;  // rows ascend
      segs[(int64_t)t * K + k] = (int32_t)(j0 + lo);
      spill[(int64_t)t * K + k] = (int32_t)(j0 + lo + beyond);
    }
  } else {
    auto row_at = [&](int i) -> int { return j0 + i < n ? s[j0 + i] : 0x7FFFFFFF; };
    const int t_lo = j0 > 0 ? tile_of_row(r_prev, row_s, tile_s, n_rng, T, window).t + 1 : 0;
    t_hi = tile_of_row(row_at(cnt - 1), row_s, tile_s, n_rng, T, window).t;
    const int sub = threadIdx.x & 15, shift = threadIdx.x & 48;
    for (int t = t_lo + (threadIdx.x >> 4); t <= t_hi; t += 16) {
      const TileOf tl = tile_by_index(t, row_s, tile_s, n_rng, T, window);
      // the first pair of the run at or beyond the tile's first row lies in [lo, lo + len),
      // and the last pair of that stretch is at or beyond it (rows ascend; the run's last
      // pair is, t being at most the tile of its row)
      int lo = 0, len = cnt;
      while (len > 1) {
        const int step = (len + 15) >> 4;
        const int upto = (sub + 1) * step < len ? (sub + 1) * step : len;
        const bool at = row_at(lo + upto - 1) >= tl.row0;
        const unsigned m = (unsigned)(__ballot(at) >> shift) & 0xFFFFu;
        const int f = __ffs(m) - 1;  // (the stretch's last probe is set)
        lo += f * step;
        len = (f + 1) * step < len ? step : len - f * step;
      }
      const bool in_spill = sub < 15 && row_at(lo + sub) < tl.spill;
      const int beyond = __popc((unsigned)(__ballot(in_spill) >> shift) & 0xFFFFu);
      if (sub == 0) {
        segs[(int64_t)t * K + k] = (int32_t)(j0 + lo);
        spill[(int64_t)t * K + k] = (int32_t)(j0 + lo + beyond);
      }
    }
  }
  if (j0 + cnt == n)  // the offset's last run: tiles beyond its last pair
    for (int t = t_hi + 1 + threadIdx.x; t <= n_tiles; t += 256) {
      segs[(int64_t)t * K + k] = n;
      spill[(int64_t)t * K + k] = n;
    }
}

// ---- row-block schedule -----------------------------------------------------------------
// The pairs a tile works on (its share of every offset) are cut, offset by offset,
// into row blocks of 16 (the M side of one MFMA); where the share could not be
// filled up to a whole block, the last block is padded.  Four
// consecutive row blocks form a group (one pipeline stage per 64-channel chunk
// of Cin); a tile's last group is padded with empty blocks, and a tile without
// pairs still gets one empty group so that its rows are written.  The schedule
// lists, tile after tile and offset-major inside a tile:
//   sched_in [group*64 + slot]  gather row of the slot times in_scale (in_pad = padding):
//                               the row number, or the byte offset of the row
//   sched_out[group*64 + slot]  byte offset of the slot's accumulator row (accumulator
//                               slot * out_scale; slot T, a dummy, = padding)
//   grp_meta [group*8 + ...]    0..3 offset k of the 4 blocks times k_scale (the byte
//                               distance between the weight fragments of two offsets;
//                               an empty block has 0), 4 first output row of the
//                               group's tile, 5 rows of the tile, negated when the
//                               group is not the tile's last one, 6 accumulator slot
//                               of the tile's first row
// The convolution kernel streams through it without per-offset bookkeeping.
// share_first/share_cnt[t*K + k]: the pairs of offset k that tile t works on.  They
// begin where the previous tile of the same workgroup stopped and end with the last
// pair of a row of tile t, rounded up to a whole row block with pairs of the next
// tile's rows as far as spill[] allows.
//
// range_sched_kernel: one block per workgroup range.  Threads over the offsets walk the range's tiles in order
// (the shares), then a wave per tile scans its offsets -- kofs[t*K + k] = row blocks of
// tile t before offset k, tile_nmb[t] = its row blocks, its groups (at least one) -- then
// the first wave numbers the groups of the range's tiles: tile_loc[t] = groups of the range
// before tile t, tile_rng[t] = the range, range_grp[w] = groups of range w.  What is left
// of the prefix over all tiles, the sum over the ranges before a tile's own (at most 256
// numbers), every block of sched_fill_kernel takes for itself: three dependent launches
// (shares, counts, a one-block scan) became one.
// FILL (plans with one range to a workgroup and a single work split): the block goes on to
// fill its range's part of the schedule (what sched_fill_kernel does, sixteen threads to a
// (tile, offset)), at the groups it takes from a cursor that all ranges share -- in whatever
// order the blocks get there: a workgroup of the convolution finds its groups through
// wg_grp, and nothing else depends on where in the buffers they lie.
// What the schedule of one (tile, offset) is filled from and into (sched_fill_item).
struct SchedFill {
  const int32_t *pairs, *sorted, *flag;
  int64_t pair_stride;
  int plane_g;
  const int32_t *tile_row0, *tile_slot0;
  int T;
  uint32_t in_scale, in_pad;
  int out_scale, k_scale;
  int32_t *sched_in, *sched_out, *grp_meta;
};

// Lane `lane` of the 16 threads of (tile t, offset k) fills slot `lane` of each of their row
// blocks; the threads of offset 0 also write the tile's padding blocks and the tile fields of
// its groups [g0, g1).
// `first` (optional): what the loads of the first four row blocks return, issued by the
// caller together with those of other combinations (first[0..3] gather rows, [4..7] scatter
// rows, [8] tile_row0[t], [9] tile_slot0[t]).
__device__ __forceinline__ void sched_fill_item(const SchedFill &f, int64_t t, int k, int lane,
                                                int64_t g0, int64_t g1, int s0, int n, int kof,
                                                int nmb, const int *first = nullptr) {
  const int T = f.T, out_scale = f.out_scale, k_scale = f.k_scale, plane_g = f.plane_g;
  const uint32_t in_scale = f.in_scale, in_pad = f.in_pad;
  const int64_t pair_stride = f.pair_stride;
  const int32_t *__restrict__ tile_row0 = f.tile_row0, *__restrict__ tile_slot0 = f.tile_slot0;
  int32_t *__restrict__ sched_in = f.sched_in, *__restrict__ sched_out = f.sched_out,
                       *__restrict__ grp_meta = f.grp_meta;
  const int32_t *src = f.flag[0] ? f.sorted : f.pairs;
  if (k == 0) {
    for (int64_t g = g0 + lane; g < g1; g += 16) {
      const int rows = tile_row0[t + 1] - tile_row0[t];
      grp_meta[g * 8 + 4] = tile_row0[t];
      grp_meta[g * 8 + 5] = g + 1 == g1 ? rows : -rows;
      grp_meta[g * 8 + 6] = tile_slot0[t];
      grp_meta[g * 8 + 7] = 0;
    }
    for (int64_t mb = g0 * 4 + nmb; mb < g1 * 4; ++mb) {
      sched_in[mb * 16 + lane] = (int32_t)in_pad;
      sched_out[mb * 16 + lane] = T * out_scale;
      if (lane == 0) grp_meta[(mb >> 2) * 8 + (mb & 3)] = 0;
    }
  }
  if (n <= 0) return;
  const int32_t *pg = src + ((int64_t)k * 2 + plane_g) * pair_stride + s0;
  const int32_t *ps = src + ((int64_t)k * 2 + (1 - plane_g)) * pair_stride + s0;
  int64_t mb = g0 * 4 + kof;
  // accumulator slot of a row: rows map to slots modulo the window height T; the
  // rows a tile touches span less than T, so one conditional subtraction does it
  const int slot_off = first ? first[9] - first[8] : tile_slot0[t] - tile_row0[t];
  // four row blocks at a time: their loads are issued together
  const int n16 = (n + 15) & ~15;
  for (int p0 = lane; p0 < n16; p0 += 64, mb += 4) {
    int gi[4], so[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int p = p0 + 16 * u;
      if (first != nullptr && p0 == lane) {
        gi[u] = first[u];
        so[u] = first[4 + u];
      } else {
        gi[u] = p < n ? pg[p] : 0;
        so[u] = p < n ? ps[p] : 0;
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int p = p0 + 16 * u;
      if (p < n16) {
        const int64_t b = mb + u;
        sched_in[b * 16 + lane] = p < n ? (int32_t)((uint32_t)gi[u] * in_scale) : (int32_t)in_pad;
        int slot = T;
        if (p < n) {
          slot = so[u] + slot_off;
          if (slot >= T) slot -= T;
        }
        sched_out[b * 16 + lane] = slot * out_scale;
        if (lane == 0) grp_meta[(b >> 2) * 8 + (b & 3)] = k * k_scale;
      }
    }
  }
}

constexpr int kRangeSchedThreads = 1024;  // sixteen tiles at a time in the second step
constexpr int kFillItems = 2048;  // (tile, offset) combinations of a range whose shares stay in LDS
constexpr int kFillTiles = 256;   // tiles of such a range

// The steps of range_sched_kernel for one range.  LDS: shares, block offsets and the tiles'
// counts live in LDS (the FILL form, a range of at most kFillItems (tile, offset)
// combinations and kFillTiles tiles: what follows reads them without a trip to memory) --
// otherwise in the global arrays, where sched_fill_kernel finds them.
template <bool FILL, bool LDS>
__device__ __forceinline__ void range_sched_steps(
    const int32_t *__restrict__ segs, const int32_t *__restrict__ spill, int K, int w, int t0,
    int t1, int32_t *share_first, int32_t *share_cnt, int32_t *kofs, int32_t *tile_nmb,
    int32_t *tile_loc, int32_t *__restrict__ tile_rng, int32_t *__restrict__ range_grp,
    const SchedFill &fill, int32_t *__restrict__ cursor, int32_t *__restrict__ wg_grp,
    int *sf_s, int *sc_s, int *ko_s, int *tn_s, int *tl_s, int *range_base_s) {
  auto item = [&](int64_t t, int k) -> int64_t { return LDS ? (t - t0) * K + k : t * K + k; };
  int *const sf = LDS ? sf_s : share_first;
  int *const sc = LDS ? sc_s : share_cnt;
  int *const ko = LDS ? ko_s : kofs;
  // (indices, not shifted pointers: an LDS pointer must stay inside its array)
  auto tile = [&](int64_t t) -> int64_t { return LDS ? t - t0 : t; };
  int *const tn = LDS ? tn_s : tile_nmb;
  int *const tl = LDS ? tl_s : tile_loc;
  for (int k = threadIdx.x; k < K && t0 < t1; k += blockDim.x) {
    int s = segs[(int64_t)t0 * K + k];
    // eight tiles at a time: their loads are issued together, the chain through s is
    // arithmetic only
    constexpr int U = 8;
    for (int tb = t0; tb < t1; tb += U) {
      int q[U], lim[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int t = tb + u < t1 ? tb + u : t1 - 1;
        q[u] = segs[(int64_t)(t + 1) * K + k];    // first pair of a later tile's row
        lim[u] = spill[(int64_t)(t + 1) * K + k];  // >= q
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int t = tb + u;
        if (t < t1) {
          int e = s;
          if (q[u] > s) {
            e = s + ((q[u] - s + 15) & ~15);
            if (e > lim[u]) e = lim[u];
          }
          sf[item(t, k)] = s;
          sc[item(t, k)] = e - s;
          s = e;
        }
      }
    }
  }
  __threadfence_block();
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int64_t t = t0 + wave; t < t1; t += blockDim.x >> 6) {
    int run = 0;
    for (int k0 = 0; k0 < K; k0 += 64) {
      const int k = k0 + lane;
      const int nb = k < K ? (sc[item(t, k)] + 15) >> 4 : 0;
      int incl = nb;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
      }
      if (k < K) ko[item(t, k)] = run + incl - nb;
      run += __shfl(incl, 63, 64);
    }
    if (lane == 0) {
      tn[tile(t)] = run;
      const int groups = (run + 3) >> 2;
      tl[tile(t)] = groups > 0 ? groups : 1;  // a tile without pairs gets an empty group
    }
  }
  __threadfence_block();
  __syncthreads();
  if (wave == 0) {
    int carry = 0;
    for (int base = t0; base < t1; base += 64) {
      const int t = base + lane;
      const int v = t < t1 ? tl[tile(t)] : 0;
      int incl = v;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
      }
      if (t < t1) {
        tl[tile(t)] = carry + incl - v;
        if (!FILL) tile_rng[t] = w;
      }
      carry += __shfl(incl, 63, 64);
    }
    if (lane == 0) range_grp[w] = carry;
    if (FILL && lane == 0) {
      const int base = atomicAdd(cursor, carry);
      wg_grp[2 * w] = base;
      wg_grp[2 * w + 1] = base + carry;
      range_base_s[0] = base;
      range_base_s[1] = base + carry;
    }
  }
  if (!FILL) return;
  __threadfence_block();
  __syncthreads();
  const int64_t base = range_base_s[0], end = range_base_s[1];
  // A team of sixteen threads takes three (tile, offset) combinations at a time and issues
  // the loads of all three before it stores anything: a range has a few hundred combinations
  // for its 64 teams, and one after the other each would wait for its own loads.
  const int team = threadIdx.x >> 4, l16 = threadIdx.x & 15;
  constexpr int U = 3, kTeams = kRangeSchedThreads / 16;
  const int64_t tk_end = (int64_t)t1 * K;
  const int32_t *src = fill.flag[0] ? fill.sorted : fill.pairs;
  for (int64_t tk0 = (int64_t)t0 * K + team; tk0 < tk_end; tk0 += U * kTeams) {
    int first[U][10], s0[U], n[U];
    int64_t tt[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t tk = tk0 + u * kTeams;
      const bool live = tk < tk_end;
      const int64_t t = live ? tk / K : t0;
      const int k = live ? (int)(tk - t * K) : 0;
      tt[u] = t;
      s0[u] = sf[item(t, k)];
      n[u] = live ? sc[item(t, k)] : 0;
      const int32_t *pg = src + ((int64_t)k * 2 + fill.plane_g) * fill.pair_stride + s0[u];
      const int32_t *ps = src + ((int64_t)k * 2 + (1 - fill.plane_g)) * fill.pair_stride + s0[u];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int p = l16 + 16 * j;
        first[u][j] = p < n[u] ? pg[p] : 0;
        first[u][4 + j] = p < n[u] ? ps[p] : 0;
      }
      first[u][8] = fill.tile_row0[t];
      first[u][9] = fill.tile_slot0[t];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t tk = tk0 + u * kTeams;
      if (tk < tk_end) {
        const int64_t t = tt[u];
        const int k = (int)(tk - t * K);
        const int64_t g0 = base + tl[tile(t)];
        const int64_t g1 = t + 1 < t1 ? base + tl[tile(t + 1)] : end;
        sched_fill_item(fill, t, k, l16, g0, g1, s0[u], n[u], ko[item(t, k)], tn[tile(t)],
                        first[u]);
      }
    }
  }
}

template <bool FILL>
__global__ void __launch_bounds__(kRangeSchedThreads)
    range_sched_kernel(const int32_t *__restrict__ segs, const int32_t *__restrict__ spill, int K,
                       const int32_t *__restrict__ wg_tile, int32_t *share_first,
                       int32_t *share_cnt, int32_t *kofs, int32_t *tile_nmb, int32_t *tile_loc,
                       int32_t *__restrict__ tile_rng, int32_t *__restrict__ range_grp,
                       SchedFill fill, int32_t *__restrict__ cursor,
                       int32_t *__restrict__ wg_grp) {
  const int w = blockIdx.x;
  __shared__ int range_base_s[2];
  __shared__ int sf_s[FILL ? kFillItems : 1], sc_s[FILL ? kFillItems : 1],
      ko_s[FILL ? kFillItems : 1], tn_s[FILL ? kFillTiles : 1], tl_s[FILL ? kFillTiles : 1];
  const int t0 = wg_tile[w], t1 = wg_tile[w + 1];
  if (FILL && (int64_t)(t1 - t0) * K <= kFillItems && t1 - t0 <= kFillTiles)
    range_sched_steps<FILL, true>(segs, spill, K, w, t0, t1, share_first, share_cnt, kofs,
                                  tile_nmb, tile_loc, tile_rng, range_grp, fill, cursor, wg_grp,
                                  sf_s, sc_s, ko_s, tn_s, tl_s, range_base_s);
  else
    range_sched_steps<FILL, false>(segs, spill, K, w, t0, t1, share_first, share_cnt, kofs,
                                   tile_nmb, tile_loc, tile_rng, range_grp, fill, cursor, wg_grp,
                                   sf_s, sc_s, ko_s, tn_s, tl_s, range_base_s);
}

// Two ranges to a workgroup (n_rng = 2 n_wg): which two, by the row-block groups the ranges
// came to.  What a range costs is known only once its schedule is counted, and the ranges
// of equal modelled work differ by 5-10 % there.  Inside every run of 32 consecutive ranges
// (neighbours in the rows, whose gathers share an L2) the range with the most groups goes
// with the one with the fewest, the second with the last but one, ...: 16 workgroups whose
// sums differ far less than the ranges do.  One block.  range_g0[r]: first group of range r
// in the schedule, where a workgroup's two ranges follow each other, the one of the lower
// rows first; wg_grp[2 v], wg_grp[2 v + 1]: first group of workgroup v and the one behind its last.
__global__ void __launch_bounds__(kMaxRanges)
    range_assign_kernel(const int32_t *__restrict__ range_grp, int n_rng, int n_wg,
                        int32_t *__restrict__ range_g0, int32_t *__restrict__ wg_grp) {
  __shared__ int cnt_s[kMaxRanges];
  __shared__ int member_s[kMaxRanges];  // the two ranges of workgroup v: [2v], [2v + 1]
  __shared__ int sum_s[kMaxRanges / 2 + 1];
  const int r = threadIdx.x;
  const int c = r < n_rng ? range_grp[r] : 0;
  cnt_s[r] = c;
  __syncthreads();
  if (r < n_rng) {
    const int base = r & ~31;
    const int width = min(32, n_rng - base);  // even: n_rng is
    int rank = 0;
    for (int j = 0; j < width; ++j) {
      const int cj = cnt_s[base + j];
      rank += (cj > c || (cj == c && base + j < r)) ? 1 : 0;
    }
    const int q = rank < width / 2 ? rank : width - 1 - rank;
    member_s[2 * (base / 2 + q) + (rank < width / 2 ? 0 : 1)] = r;
  }
  __syncthreads();
  if (r < n_wg) {
    const int a = member_s[2 * r], b = member_s[2 * r + 1];
    if (a > b) {
      member_s[2 * r] = b;
      member_s[2 * r + 1] = a;
    }
    sum_s[r] = cnt_s[a] + cnt_s[b];
  }
  __syncthreads();
  if (r == 0) {  // at most 256 sums
    int run = 0;
    for (int v = 0; v < n_wg; ++v) {
      const int t = sum_s[v];
      sum_s[v] = run;
      run += t;
    }
    sum_s[n_wg] = run;
  }
  __syncthreads();
  if (r < n_wg) {
    wg_grp[2 * r] = sum_s[r];
    wg_grp[2 * r + 1] = sum_s[r + 1];
  }
  if (r < n_wg) {
    const int a = member_s[2 * r], b = member_s[2 * r + 1];
    range_g0[a] = sum_s[r];
    range_g0[b] = sum_s[r] + cnt_s[a];
  }
}

// 16 threads per (tile, offset): lane i fills slot i of each of its row blocks; the
// threads of offset 0 also write the tile's padding blocks and its group -> tile map.
// (Blocks that take several times 16 (tile, offset) combinations, to compute the prefix over
// the ranges they start with less often, are slower: 19 against 14 us on the benchmark layer.)
__global__ void __launch_bounds__(256)
    sched_fill_kernel(const int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                      const int32_t *__restrict__ sorted, int64_t pair_stride, int plane_g,
                      const int32_t *__restrict__ share_first,
                      const int32_t *__restrict__ share_cnt, const int32_t *__restrict__ kofs,
                      const int32_t *__restrict__ tile_nmb, const int32_t *__restrict__ tile_loc,
                      const int32_t *__restrict__ tile_rng, const int32_t *__restrict__ range_grp,
                      int n_wg, const int32_t *__restrict__ range_g0_paired,
                      int32_t *__restrict__ wg_grp, int K,
                      const int32_t *__restrict__ n_tiles_dev,
                      const int32_t *__restrict__ tile_row0,
                      const int32_t *__restrict__ tile_slot0, int T, uint32_t in_scale,
                      uint32_t in_pad, int out_scale, int k_scale,
                      int32_t *__restrict__ sched_in, int32_t *__restrict__ sched_out,
                      int32_t *__restrict__ grp_meta) {
  // groups before every range (n_wg <= 256 of them): exclusive prefix of range_grp, which
  // is also where the workgroups begin (block 0 writes that down for the convolution
  // kernel) -- or, with two ranges to a workgroup, what range_assign_kernel found
  // (range_g0_paired)
  __shared__ int range_g0[257];
  if (range_g0_paired == nullptr) {
    __shared__ int wave_sum[4];
    const int w = threadIdx.x, wl = w & 63;
    const int v = w < n_wg ? range_grp[w] : 0;
    int incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      int o = __shfl_up(incl, d, 64);
      if (wl >= d) incl += o;
    }
    if (wl == 63) wave_sum[w >> 6] = incl;
    __syncthreads();
    int before = 0;
    for (int i = 0; i < (w >> 6); ++i) before += wave_sum[i];
    range_g0[w] = before + incl - v;
    if (w == 255) range_g0[256] = before + incl;
    __syncthreads();
    if (blockIdx.x == 0) {
      for (int i = threadIdx.x; i < n_wg; i += blockDim.x) {
        wg_grp[2 * i] = range_g0[i];
        wg_grp[2 * i + 1] = range_g0[i + 1];
      }
    }
  }
  const int64_t n_tiles = n_tiles_dev[0];
  const int32_t *src = flag[0] ? sorted : pairs;
  int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t tk = gid >> 4;
  int lane = (int)(gid & 15);
  if (tk >= n_tiles * K) return;
  int64_t t = tk / K;
  int k = (int)(tk - t * K);
  const int rng = tile_rng[t];
  const int64_t rg0 = range_g0_paired ? range_g0_paired[rng] : range_g0[rng];
  const int64_t g0 = rg0 + tile_loc[t];
  const int64_t g1 = (t + 1 < n_tiles && tile_rng[t + 1] == rng) ? rg0 + tile_loc[t + 1]
                                                                : rg0 + range_grp[rng];
  SchedFill f = {pairs, sorted, flag, pair_stride, plane_g, tile_row0, tile_slot0, T, in_scale,
                 in_pad, out_scale, k_scale, sched_in, sched_out, grp_meta};
  sched_fill_item(f, t, k, lane, g0, g1, share_first[t * K + k], share_cnt[t * K + k],
                  kofs[t * K + k], tile_nmb[t]);
}


static size_t conv_lds_bytes(int T, int acc_cols) {
  return ((size_t)(T + 1) * (acc_cols + 4) + 2 * (size_t)kStage * kAStride) * 4;
}

constexpr size_t kLdsLeft = 4096 + 256;
static int pick_tile(int acc_cols, bool leave_room) {
  // One workgroup per CU: (almost) all of the 160 KB of LDS goes to the accumulators.
  // (kLdsLeft bytes stay free: the kernels of the index work -- rulebooks and plans of other
  // layers, queued on a stream of their own -- are built to fit there, beside this kernel's
  // workgroups)
  // (... unless the kernel will run for long: the index work of a neighbouring layer is
  // small change next to it, and the rows of the window are worth more)
  size_t budget = 160 * 1024 - conv_lds_bytes(0, acc_cols) - (leave_room ? kLdsLeft : 512);
  int t = (int)(budget / ((size_t)(acc_cols + 4) * 4));
  t = t / 8 * 8;
  if (t < kMinTile) t = kMinTile;
  return t;
}

static int device_cu_count() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      cus = prop.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
}

// (switched by ssc_conv_tuning, for measurements)
static bool g_conv_tail = true;       // a launch of its own for a lone last column group
static bool g_conv_five = true;       // the lone last group as a fifth one of the last block
constexpr int64_t kRebalanceStages = 1500;
// estimated groups per workgroup from which ranges are paired (the benchmark layer, 200 to
// a workgroup: 216 -> 210 in the largest but no time gained for the launch it costs; the
// third configuration, 55: one more range end each, 3499 -> 3691 groups, evens nothing out)
constexpr int64_t kPairGroups = 250;
static bool g_conv_pair = true, g_conv_pair_always = false;
static int64_t g_conv_rebalance_stages = kRebalanceStages;
static bool g_conv_fuse_fill = true;  // range_sched_kernel<true> instead of sched_fill_kernel
// Index work (rulebooks, plans) is queued on a stream of its own and runs while a convolution
// holds every CU with nearly all of its LDS: kernels are picked that need little LDS.
static thread_local bool g_index_beside_conv = false;  // (a setting of the calling host thread)
static bool g_conv_rebalance = true;  // long kernels: a second work split from the first one's counts
static bool g_conv_round8 = false;    // ranges per column block: a multiple of 8 only
static bool g_conv_small = true;      // layers of at most 8 input channels: conv_small_kernel

// The sizes that follow from the number of workgroups per column block.
// `sizing`: the plan is only being sized (the number of input rows, and with it the number
// of ranges, is not known): the finer grid, so that a buffer sized for n_out rows is large
// enough for a plan over any smaller number of rows as well.
static void plan_split(ConvPlan &p, int n_wg, int n_rng, int64_t n_out, int K,
                       int64_t pair_stride, bool sizing) {
  p.n_wg = n_wg;
  p.n_rng = n_rng;
  // upper bound of the tile count: every range ends with a partial tile
  p.n_tiles = ceil_div(n_out > 0 ? n_out : 1, p.tile_rows) + n_rng;
  p.granule = sizing || n_out / n_rng < 2048 ? kSplitGranuleSmall : kSplitGranule;
  p.n_fine = ceil_div(n_out > 0 ? n_out : 1, p.granule);
  p.words_per_k = ceil_div(n_out > 0 ? n_out : 1, 32);
  // groups: pairs/64 plus, per (tile, offset), up to one partial block, plus one
  // partial (or empty) group per tile, plus the groups the kernel's prefetches may
  // touch beyond the end of the schedule
  int64_t max_pairs_k = pair_stride < n_out ? pair_stride : n_out;
  p.grp_cap = ((int64_t)K * (max_pairs_k / 16 + 1) + p.n_tiles * K) / 4 + 2 * p.n_tiles + 4 + 16;
}

static ConvPlan make_plan(int64_t n_in, int64_t n_out, int K, int c_in, int c_out,
                          int64_t pair_stride, int elem_bytes = 4) {
  ConvPlan p;
  p.ncb = (int)ceil_div(c_out, 16);
  p.nch = (int)ceil_div(c_in, kKC);
  // chunks of equal width: the fewest steps of 4 channels that cover Cin in nch chunks,
  // rounded up to a width the kernel is built for
  p.ns = 16;
  if (elem_bytes == 4) {
    const int want = (int)ceil_div(ceil_div(c_in, p.nch), 4);
    constexpr int kBuilt[] = {1, 2, 3, 4, 6, 8, 10, 12, 13, 14, 15, 16};
    for (int b : kBuilt)
      if (b >= want) {
        p.ns = b;
        break;
      }
  }
  p.ncw = 4;
  // the five-group form: a lone last group goes along with the last full block (the
  // kernel needs four chunks for it, one for each wave's turn at the fifth group's sums)
  p.five = g_conv_five && elem_bytes == 4 && p.ncb % p.ncw == 1 && p.ncb > p.ncw && p.nch >= 4;
  p.acc_cols = p.five ? 16 * p.ncw + 16 : 16 * p.ncw;
  // the gather can be a range-checked buffer load when rows are multiples of four
  // channels and byte offsets into the features (plus the padding marker) fit 32 bits
  p.gather = 0;
  if ((c_in & 3) == 0 && (uint64_t)n_in * c_in * elem_bytes <= (uint64_t)kGatherPad)
    p.gather = (c_in % kKC) == 0 ? 1 : 2;
  // (wider layers: the launches of one column block each cost more than the lone group
  // in a block of its own does -- 128 -> 256 channels at stride 2 takes 0.255 ms as four
  // launches against 0.185 ms as one, 200 -> 200 with 125 offsets 17.6 against 16.8 ms)
  p.has_tail = !p.five && g_conv_tail && elem_bytes == 4 && p.ncb % p.ncw == 1 && p.ncb / p.ncw <= 2;
  const bool serial = p.has_tail || p.five;
  const int blocks = serial ? p.ncb / p.ncw : (int)ceil_div(p.ncb, p.ncw);
  p.n_colblk = serial ? 1 : blocks;
  p.n_launch = serial ? blocks : 1;
  int n_wg = device_cu_count() / p.n_colblk;
  if (n_wg < 1) n_wg = 1;
  if (n_wg > 256) n_wg = 256;  // the kernels of the split hold a number per workgroup in LDS
  // (every CU a workgroup, also where the column blocks do not divide the CUs by a
  // multiple of 8: the kernel then deals its workgroups to the XCDs by its general rule)
  if (n_wg >= 8 && g_conv_round8) n_wg = n_wg / 8 * 8;
  // estimates from the pairs the layer is likely to have -- N_in K where the outputs
  // outnumber the inputs (stride 1), an eighth of that where the inputs outnumber the
  // outputs (stride 2; also the input gradient of a stride-1 layer, which has N_out K), a
  // quarter of N_out K for submanifold layers and where N_in is not known: stages and
  // row-block groups per workgroup
  const int64_t est_pairs = n_in <= 0 || n_in == n_out ? n_out * K / 4
                            : n_in < n_out             ? n_in * K
                                                       : n_in * K / 8;
  const int64_t est_groups = est_pairs / kStage / n_wg;
  const int64_t est_stages = est_groups * p.nch;
  // A second work split (split_rebalance_kernel) where the kernel runs long enough for four
  // more small launches (30 us; the split evens out 3-15 % of the kernel's time, more with
  // more ranges): 1500 stages per workgroup or more.
  p.rebalance = g_conv_rebalance && est_stages >= g_conv_rebalance_stages;
  // The accumulator window: all of the LDS for kernels that run long (those that get a second
  // split: about 2 ms and up), a few KB less for the others (see pick_tile); sizing calls
  // (N_in unknown) count with the smaller window, which has more tiles.  (Kernels of middle
  // size lose and gain about the same, 10.49 against 10.48 ms for the backbone whose stages
  // they are; layers whose pairs the estimate overstates -- a strided layer with more
  // outputs than inputs -- are short kernels and gain.)
  const bool long_kernel = n_in > 0 && est_stages >= kRebalanceStages;
  p.T = pick_tile(p.acc_cols, !long_kernel);
  p.tile_rows = p.T - (p.five ? kSpillRowsFive : kSpillRows);
  // Two ranges to a workgroup, paired by what they came to (range_assign_kernel): one more
  // small launch and one more range end per workgroup, whose last row blocks cannot be
  // filled from a next tile (K / 8 groups), against the 5-10 % by which single ranges
  // differ.  Not with the second split, which leaves less than that to even out.
  // (N_in unknown: the plan is only being sized, for the larger of the two)
  const bool pair = g_conv_pair && n_wg >= 2 &&
                    (g_conv_pair_always || n_in <= 0 ||
                     (!p.rebalance && est_groups >= kPairGroups && est_groups >= (int64_t)K / 2));
  plan_split(p, n_wg, pair ? 2 * n_wg : n_wg, n_out, K, pair_stride, n_in <= 0);
  p.lds_bytes = conv_lds_bytes(p.T, p.acc_cols);
  p.small = g_conv_small && conv_small_applies(K, c_in, c_out, elem_bytes);
  if (p.small) p.rebalance = false;
  p.kvol = K;
  p.out_rows = n_out;
  return p;
}


// 4 KiB per fragment for either element type (half fragments use the first half).
static size_t conv_packed_bytes(const ConvPlan &p, int K) {
  return align_up((size_t)K * p.ncb * p.nch * 4096);
}

static size_t conv_plan_walk(void *base, const ConvPlan &p, ConvWs *w) {
  Carver c(base);
  if (p.small) {  // the plan is the table of every output row's input rows, nothing else
    int32_t *table =
        c.take<int32_t>((size_t)p.kvol * (size_t)(p.out_rows > 0 ? p.out_rows : 1));
    if (w) w->small_table = table;
    return c.used;
  }
  int32_t *wg_tile = c.take<int32_t>((size_t)p.n_rng + 1);
  int32_t *wg_grp = c.take<int32_t>(2 * (size_t)p.n_wg);
  int32_t *sched_in = c.take<int32_t>((size_t)p.grp_cap * 64);
  int32_t *sched_out = c.take<int32_t>((size_t)p.grp_cap * 64);
  int32_t *grp_meta = c.take<int32_t>((size_t)p.grp_cap * 8);
  if (w) {
    w->wg_tile = wg_tile;
    w->wg_grp = wg_grp;
    w->sched_in = sched_in;
    w->sched_out = sched_out;
    w->grp_meta = grp_meta;
  }
  return c.used;
}

// The head of the scratch buffer, whose layout does not depend on the plan: flag and
// range_row0 (a rulebook that places the range boundaries itself writes them before the
// number of output rows, and with it the plan, is known).
static size_t conv_scratch_head(void *base, ConvWs *w) {
  Carver c(base);
  w->flag = c.take<int32_t>(1);
  w->range_row0 = c.take<int32_t>((size_t)kMaxRanges + 1);
  w->range_row0_alt = c.take<int32_t>((size_t)kMaxRanges + 1);
  return c.used;
}

static size_t conv_scratch_walk(void *base, const ConvPlan &p, int K, int64_t pair_stride,
                                ConvWs *w) {
  Carver c(base);
  ConvWs t;
  t.flag = c.take<int32_t>(1);
  t.range_row0 = c.take<int32_t>((size_t)kMaxRanges + 1);
  t.range_row0_alt = c.take<int32_t>((size_t)kMaxRanges + 1);
  t.segs = c.take<int32_t>((size_t)(p.n_tiles + 1) * K);
  t.sorted = c.take<int32_t>((size_t)K * 2 * pair_stride);
  t.bits = c.take<uint32_t>((size_t)K * p.words_per_k);
  t.prefix = c.take<int32_t>((size_t)K * p.words_per_k);
  t.tile_loc = c.take<int32_t>((size_t)p.n_tiles);
  t.tile_nmb = c.take<int32_t>((size_t)p.n_tiles);
  t.kofs = c.take<int32_t>((size_t)p.n_tiles * K);
  t.fine_segs = c.take<int32_t>((size_t)(p.n_fine + 1) * K);
  t.tile_row0 = c.take<int32_t>((size_t)p.n_tiles + 1);
  t.spill_end = c.take<int32_t>((size_t)p.n_tiles + 1);
  t.tile_slot0 = c.take<int32_t>((size_t)p.n_tiles + 1);
  t.spill = c.take<int32_t>((size_t)(p.n_tiles + 1) * K);
  t.share_first = c.take<int32_t>((size_t)p.n_tiles * K);
  t.share_cnt = c.take<int32_t>((size_t)p.n_tiles * K);
  t.n_tiles_dev = c.take<int32_t>(2);  // [1]: cursor over the schedule's groups
  t.tile_rng = c.take<int32_t>((size_t)p.n_tiles + 1);
  t.range_grp = c.take<int32_t>((size_t)p.n_rng + 1);
  t.range_row1 = c.take<int32_t>((size_t)p.n_rng + 1);
  t.range_g0 = c.take<int32_t>((size_t)p.n_rng + 1);
  if (w) {
    w->flag = t.flag;
    w->segs = t.segs;
    w->sorted = t.sorted;
    w->bits = t.bits;
    w->prefix = t.prefix;
    w->tile_loc = t.tile_loc;
    w->tile_nmb = t.tile_nmb;
    w->kofs = t.kofs;
    w->fine_segs = t.fine_segs;
    w->range_row0 = t.range_row0;
    w->range_row0_alt = t.range_row0_alt;
    w->tile_row0 = t.tile_row0;
    w->spill_end = t.spill_end;
    w->tile_slot0 = t.tile_slot0;
    w->spill = t.spill;
    w->share_first = t.share_first;
    w->share_cnt = t.share_cnt;
    w->n_tiles_dev = t.n_tiles_dev;
    w->tile_rng = t.tile_rng;
    w->range_grp = t.range_grp;
    w->range_row1 = t.range_row1;
    w->range_g0 = t.range_g0;
  }
  return c.used;
}

// The one-workspace form of ssc_conv_fwd_*: packed | plan | scratch.
static size_t conv_ws_walk(void *base, const ConvPlan &p, int K, int64_t pair_stride, ConvWs *w) {
  char *b = static_cast<char *>(base);
  size_t used = 0;
  if (w) w->packed = b;
  used += conv_packed_bytes(p, K);
  used += conv_plan_walk(b ? b + used : nullptr, p, w);
  used += conv_scratch_walk(b ? b + used : nullptr, p, K, pair_stride, w);
  return used;
}

static size_t conv_ws_bytes(int64_t n_out, int K, int c_in, int c_out, int64_t pair_stride) {
  // the workspace does not depend on the number of input rows (nor on the element type,
  // which is not known here: room for the plan of either)
  ConvPlan p = make_plan(0, n_out, K, c_in, c_out, pair_stride);
  size_t bytes = conv_ws_walk(nullptr, p, K, pair_stride, nullptr);
  if (p.small) {
    p.small = false;
    const size_t other = conv_ws_walk(nullptr, p, K, pair_stride, nullptr);
    if (other > bytes) bytes = other;
  }
  return bytes;
}

// The launches of a plan (ConvPlan): the column blocks, all at once or one after the other,
// then the one-column-group form for a lone last group.
template <typename IO, int GATHER, int NS>
static int launch_all(const ConvPlan &p, const ConvWs &w, const IO *features, int64_t n_in,
                      int c_in, int K, IO *out, int c_out, const ConvEpilogue &epi,
                      hipStream_t s) {
  constexpr bool kFloat = sizeof(IO) == 4;
  const bool with_epi = epi.mode != nullptr;
  if (p.five) {
    if constexpr (kFloat) {
      for (int l = 0; l < p.n_launch; ++l) {
        const int col_base = l * 16 * p.ncw;
        int rc;
        if (l == p.n_launch - 1) {  // with the lone group as a fifth one
          const int xcol = (p.ncb - 1) * 16;
          rc = with_epi ? launch_conv_f32<GATHER, NS, true, 2>(p, w, features, n_in, c_in, K, out,
                                                               c_out, col_base, xcol, epi, s)
                        : launch_conv_f32<GATHER, NS, false, 2>(p, w, features, n_in, c_in, K, out,
                                                                c_out, col_base, xcol, epi, s);
        } else {  // the plain kernel on the plan's wider accumulator rows
          rc = with_epi ? launch_conv_f32<GATHER, NS, true, 3>(p, w, features, n_in, c_in, K, out,
                                                               c_out, col_base, -1, epi, s)
                        : launch_conv_f32<GATHER, NS, false, 3>(p, w, features, n_in, c_in, K, out,
                                                                c_out, col_base, -1, epi, s);
        }
        if (rc != SSC_OK) return rc;
      }
      return SSC_OK;
    } else {
      SSC_CHECK(false, SSC_ERUNTIME, "the five-group form is built for float rows");
    }
  }
  for (int l = 0; l < p.n_launch; ++l) {
    const int col_base = l * p.n_colblk * 16 * p.ncw;
    int rc;
    if constexpr (kFloat) {
      rc = with_epi ? launch_conv_f32<GATHER, NS, true, 0>(p, w, features, n_in, c_in, K, out,
                                                           c_out, col_base, -1, epi, s)
                    : launch_conv<float, GATHER, 4, NS, false, 0>(p, w, features, n_in, c_in, K,
                                                                  out, c_out, col_base, -1, epi, s);
    } else {
      rc = with_epi ? launch_conv<IO, GATHER, 4, NS, true, 0>(p, w, features, n_in, c_in, K, out,
                                                              c_out, col_base, -1, epi, s)
                    : launch_conv<IO, GATHER, 4, NS, false, 0>(p, w, features, n_in, c_in, K, out,
                                                               c_out, col_base, -1, epi, s);
    }
    if (rc != SSC_OK) return rc;
  }
  if (p.has_tail) {
    const int col_base = (p.ncb - 1) * 16;
    if constexpr (kFloat) {
      return with_epi ? launch_conv_f32<GATHER, NS, true, 1>(p, w, features, n_in, c_in, K, out,
                                                             c_out, col_base, -1, epi, s)
                      : launch_conv_f32<GATHER, NS, false, 1>(p, w, features, n_in, c_in, K, out,
                                                              c_out, col_base, -1, epi, s);
    } else {
      SSC_CHECK(false, SSC_ERUNTIME, "the one-column-group form is built for float rows");
    }
  }
  return SSC_OK;
}

// Optional timing of the convolution kernel alone: a ring of event pairs recorded
// on the caller's stream right around the launch of conv_fwd_kernel.
constexpr int kProfileRing = 512;
static bool g_profile_on = false;
static int g_profile_count = 0;   // launches timed so far
static int g_profile_calls = 0;   // launches seen since profiling was enabled
static int g_profile_every = 1;   // every n-th launch is timed
static hipEvent_t g_profile_ev[kProfileRing][2];
static bool g_profile_init = false;

}  // namespace ssc

using namespace ssc;

extern "C" {

int ssc_profile_conv(int32_t enable) {
  if (enable && !g_profile_init) {
    // (events that only measure time: without the system-scope fence, whose cache
    // write-back and invalidation would be charged to the kernels around them)
    for (int i = 0; i < kProfileRing; ++i) {
      SSC_HIP(hipEventCreateWithFlags(&g_profile_ev[i][0], hipEventDisableSystemFence));
      SSC_HIP(hipEventCreateWithFlags(&g_profile_ev[i][1], hipEventDisableSystemFence));
    }
    g_profile_init = true;
  }
  g_profile_on = enable != 0;
  g_profile_every = enable > 1 ? enable : 1;
  g_profile_count = 0;
  g_profile_calls = 0;
  return SSC_OK;
}

int ssc_conv_tuning(int32_t flags) {
  g_conv_by_column = (flags & 1) != 0;
  g_conv_tail = (flags & 2) == 0;
  g_conv_round8 = (flags & 4) != 0;
  g_conv_five = (flags & 8) == 0;
  g_conv_rebalance = (flags & 16) == 0;
  g_conv_rebalance_stages = (flags & 32) != 0 ? 0 : kRebalanceStages;
  g_conv_pair = (flags & 64) == 0;
  g_conv_pair_always = (flags & 128) != 0;
  g_conv_small = (flags & 256) == 0;
  g_conv_fuse_fill = (flags & 512) == 0;
  return SSC_OK;
}

int ssc_index_beside_conv(int32_t on) {
  const int old = g_index_beside_conv ? 1 : 0;
  g_index_beside_conv = on != 0;
  return old;
}

int ssc_profile_conv_read(float *ms, int32_t capacity, int32_t *count) {
  SSC_CHECK(ms != nullptr && count != nullptr, SSC_EINVAL, "NULL pointer argument");
  int n = g_profile_count < kProfileRing ? g_profile_count : kProfileRing;
  if (n > capacity) n = capacity;
  for (int i = 0; i < n; ++i) {
    SSC_HIP(hipEventSynchronize(g_profile_ev[i][1]));
    SSC_HIP(hipEventElapsedTime(&ms[i], g_profile_ev[i][0], g_profile_ev[i][1]));
  }
  *count = n;
  return SSC_OK;
}

size_t ssc_conv_workspace_bytes(int64_t n_out, int32_t kernel_volume, int32_t c_in, int32_t c_out,
                                int64_t pair_stride) {
  if (n_out < 0 || kernel_volume < 1 || c_in < 1 || c_out < 1 || pair_stride < 0) return 0;
  return conv_ws_bytes(n_out, kernel_volume, c_in, c_out, pair_stride);
}
}  // extern "C"

template <typename IO>
__global__ void __launch_bounds__(256) zero_rows_kernel(IO *__restrict__ p, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += step) p[i] = (IO)0.f;
}
template <typename IO> static int fill_zero(IO *p, int64_t n, hipStream_t s) {
  if (n <= 0) return SSC_OK;
  const int64_t blocks = ceil_div(n, 256) < 8192 ? ceil_div(n, 256) : 8192;
  hipLaunchKernelGGL(zero_rows_kernel<IO>, dim3((unsigned)blocks), dim3(256), 0, s, p, n);
  SSC_LAUNCH_CHECK("zero_rows");
  return SSC_OK;
}

// Enqueue the kernels that build the plan of a convolution over `pairs` into w (plan and
// scratch parts).  `pack`, when given, is packed on the way: beside the first kernel of the
// work split for canonical pairs, by a launch of its own otherwise.  PACK_IO: element type
// of the filters to pack (float when there is nothing to pack).
template <typename PACK_IO>
static int conv_plan_build(const ConvPlan &p, const ConvWs &w, const int32_t *pairs,
                           int64_t pair_stride, const int32_t *pair_num, int K, int inverse,
                           bool in_order, int c_in, int64_t n_out, int elem_bytes,
                           const PackArgs *pack, hipStream_t s, bool seeded = false) {
  const int plane_g = inverse ? 1 : 0;
  const int plane_s = 1 - plane_g;
  int rc;
  const int frag_bytes = elem_bytes == 2 ? Io<_Float16>::kFragBytes : Io<float>::kFragBytes;
  const SchedFill fill = {pairs, w.sorted, w.flag, pair_stride, plane_g, w.tile_row0,
                          w.tile_slot0, p.T,
                          p.gather ? (uint32_t)c_in * (uint32_t)elem_bytes : 1u,
                          p.gather ? kGatherPad : 0xFFFFFFFFu, (p.acc_cols + 4) * 4,
                          p.ncb * p.nch * frag_bytes, w.sched_in, w.sched_out, w.grp_meta};
  // One range to a workgroup and a single work split: the launch that counts a range's row
  // blocks goes on to fill its schedule (no sched_fill_kernel).
  // (not for index work queued beside a running convolution: there two small kernels that
  // fit next to its workgroups beat one that has to wait for a CU of its own)
  const bool fuse_fill =
      g_conv_fuse_fill && !g_index_beside_conv && !p.rebalance && p.n_rng == p.n_wg;
  auto range_sched = [&]() -> int {
    hipLaunchKernelGGL(fuse_fill ? range_sched_kernel<true> : range_sched_kernel<false>,
                       dim3((unsigned)p.n_rng), dim3(kRangeSchedThreads), 0, s, w.segs, w.spill,
                       K, w.wg_tile, w.share_first, w.share_cnt, w.kofs, w.tile_nmb, w.tile_loc,
                       w.tile_rng, w.range_grp, fill, w.n_tiles_dev + 1, w.wg_grp);
    SSC_LAUNCH_CHECK("range_sched");
    return SSC_OK;
  };
  if (seeded) {
    // The range boundaries are in w.range_row0 already (a rulebook placed them, see
    // SplitRequest): the tiles and their segments in one launch from the pairs' side, then
    // the schedule.  For pairs in order, plans without a second split and nothing to pack.
    SSC_CHECK(in_order && !p.rebalance && pack == nullptr, SSC_ERUNTIME,
              "a seeded plan needs pairs in order and a single work split");
    auto segments_kernel = g_index_beside_conv ? pair_tile_segments_kernel<kSegChunk, false>
                                               : pair_tile_segments_kernel<kSegChunk, true>;
    hipLaunchKernelGGL(segments_kernel, dim3((unsigned)ceil_div(pair_stride, kSegChunk), (unsigned)K), dim3(256),
                       2 * ((size_t)p.n_rng + 1) * sizeof(int), s,
                       w.flag, pairs, pair_stride, plane_s, pair_num, K, w.range_row0, p.n_rng,
                       p.tile_rows, p.T, (int)n_out, w.wg_tile, w.tile_row0, w.n_tiles_dev,
                       w.spill_end, w.tile_slot0, w.segs, w.spill);
    SSC_LAUNCH_CHECK("pair_tile_segments");
    if ((rc = range_sched()) != SSC_OK) return rc;
    if (fuse_fill) return SSC_OK;
  }
  const int64_t packed_n = pack ? (int64_t)K * p.ncb * p.nch * 1024 : 0;
  PackArgs pk = {nullptr, 0, 0, 0, 0, 0, 0, 0, 0, nullptr, 16};
  if (pack) pk = *pack;
  if (!in_order && !seeded) {  // otherwise the filters are packed beside the first kernel of the split
    if (pack) {
      hipLaunchKernelGGL(pack_filters_kernel<PACK_IO>, dim3((unsigned)ceil_div(packed_n, 256)),
                         dim3(256), 0, s, pk, w.flag);
      SSC_LAUNCH_CHECK("pack_filters");
    } else {
      int rc = fill_i32(w.flag, 1, 0, s);
      if (rc != SSC_OK) return rc;
    }
  }

  dim3 pair_grid((unsigned)ceil_div(pair_stride, 256), (unsigned)K);
  if (!in_order && !seeded) {  // otherwise flag[0] is 0: pairs in order
    hipLaunchKernelGGL(check_sorted_kernel, pair_grid, dim3(256), 0, s, pairs, pair_stride, plane_s,
                       pair_num, w.flag);
    SSC_LAUNCH_CHECK("check_sorted");
    int64_t nbits_words = (int64_t)K * p.words_per_k;
    unsigned clear_blocks =
        (unsigned)(ceil_div(nbits_words, 256) < 4096 ? ceil_div(nbits_words, 256) : 4096);
    hipLaunchKernelGGL(resort_clear_kernel, dim3(clear_blocks), dim3(256), 0, s, w.flag, w.bits,
                       nbits_words);
    hipLaunchKernelGGL(resort_mark_kernel, pair_grid, dim3(256), 0, s, w.flag, pairs, pair_stride,
                       plane_s, pair_num, w.bits, p.words_per_k);
    hipLaunchKernelGGL(resort_scan_kernel, dim3(K), dim3(kScanThreads), 0, s, w.flag, w.bits,
                       w.prefix, p.words_per_k);
    hipLaunchKernelGGL(resort_scatter_kernel, pair_grid, dim3(256), 0, s, w.flag, pairs,
                       pair_stride, plane_s, pair_num, w.bits, w.prefix, p.words_per_k, w.sorted);
    SSC_LAUNCH_CHECK("resort");
  }

  if (p.small) {
    // a layer of a handful of input channels: the plan is the table of every output row's
    // input rows (conv_small.hip); the filters, if any, by a launch of their own
    if (in_order && pack) {
      hipLaunchKernelGGL(pack_filters_kernel<PACK_IO>, dim3((unsigned)ceil_div(packed_n, 256)),
                         dim3(256), 0, s, pk, w.flag);
      SSC_LAUNCH_CHECK("pack_filters");
    }
    return conv_small_build_table(w.flag, in_order, pairs, w.sorted, pair_stride, plane_s, pair_num,
                                  K, n_out, w.small_table, s);
  }
  // work split on the fine grid, then the tiles and their segments
  dim3 seg_grid = pair_grid;
  if (in_order) {  // extra rows: pack the filters (if any) and clear flag[0]
    int64_t rows = ceil_div(ceil_div(packed_n > 0 ? packed_n : 1, 256), pair_grid.x);
    seg_grid.y += (unsigned)(rows < 4096 ? rows : 4096);
  }
  if (!seeded) {
    hipLaunchKernelGGL(grid_segments_kernel<PACK_IO>, seg_grid, dim3(256), 0, s, w.flag,
                       in_order ? 1 : 0, pairs, w.sorted, pair_stride, plane_s, pair_num, K,
                       p.n_fine, p.granule, w.fine_segs, pk);
    hipLaunchKernelGGL(split_bounds_kernel, dim3((unsigned)ceil_div(p.n_fine + 1, 256)), dim3(256),
                       0, s, w.fine_segs, K, p.n_fine, n_out, p.tile_rows, p.n_rng, p.granule,
                       w.range_row0);
  }
  // the ranges' tiles, their segments, shares and row-block counts
  const int64_t nseg = (p.n_tiles + 1) * K;
  auto tiles_of = [&](const int32_t *range_row0) -> int {
    hipLaunchKernelGGL(split_rows_kernel, dim3(1), dim3(kMaxRanges), 0, s, range_row0, n_out,
                       p.tile_rows, p.T, p.n_rng, w.wg_tile, w.tile_row0, w.n_tiles_dev, w.spill_end,
                       w.tile_slot0);
    SSC_LAUNCH_CHECK("split");
    hipLaunchKernelGGL(tile_segments_kernel, dim3((unsigned)ceil_div(nseg, 256)), dim3(256), 0, s,
                       w.flag, pairs, w.sorted, pair_stride, plane_s, pair_num, K, w.n_tiles_dev,
                       w.tile_row0, n_out, w.fine_segs, p.granule, w.spill_end, w.segs,
                       w.spill);
    SSC_LAUNCH_CHECK("tile_segments");
    return range_sched();
  };
  rc = seeded ? SSC_OK : tiles_of(w.range_row0);
  if (rc != SSC_OK) return rc;
  if (fuse_fill) return SSC_OK;
  if (p.rebalance) {  // long kernels: once more, from the groups the ranges came to
    hipLaunchKernelGGL(split_rebalance_kernel, dim3((unsigned)ceil_div(p.n_fine + 1, 256)),
                       dim3(256), 0, s, w.fine_segs, K, p.n_fine, n_out, p.tile_rows, p.n_rng,
                       p.granule, w.range_row0, w.range_grp, w.range_row1);
    SSC_LAUNCH_CHECK("split_rebalance");
    rc = tiles_of(w.range_row1);
    if (rc != SSC_OK) return rc;
  }
  const bool paired = p.n_rng != p.n_wg;
  if (paired) {
    hipLaunchKernelGGL(range_assign_kernel, dim3(1), dim3(kMaxRanges), 0, s, w.range_grp, p.n_rng,
                       p.n_wg, w.range_g0, w.wg_grp);
    SSC_LAUNCH_CHECK("range_assign");
  }
  hipLaunchKernelGGL(sched_fill_kernel, dim3((unsigned)ceil_div(p.n_tiles * K * 16, 256)),
                     dim3(256), 0, s, w.flag, pairs, w.sorted, pair_stride, plane_g,
                     w.share_first, w.share_cnt, w.kofs, w.tile_nmb, w.tile_loc, w.tile_rng,
                     w.range_grp, p.n_wg, paired ? w.range_g0 : (const int32_t *)nullptr,
                     w.wg_grp, K, w.n_tiles_dev, w.tile_row0,
                     w.tile_slot0, p.T,
                     p.gather ? (uint32_t)c_in * (uint32_t)elem_bytes : 1u,
                     p.gather ? kGatherPad : 0xFFFFFFFFu, (p.acc_cols + 4) * 4,
                     p.ncb * p.nch * frag_bytes, w.sched_in, w.sched_out, w.grp_meta);
  SSC_LAUNCH_CHECK("schedule");
  return SSC_OK;
}

// Enqueue the convolution kernel over a built plan and packed filters.
template <typename IO>
static int conv_run(const ConvPlan &p, const ConvWs &w, const IO *features, int64_t n_in, int c_in,
                    int K, IO *out, int c_out, hipStream_t s, const ConvEpilogue &epi = ConvEpilogue{}) {
  int rc;
  const bool prof = g_profile_on && (g_profile_calls++ % g_profile_every) == 0;
  const int slot = g_profile_count % kProfileRing;
  if (prof) SSC_HIP(hipEventRecord(g_profile_ev[slot][0], s));
  if (p.small) {
    if constexpr (sizeof(IO) == 4) {
      rc = conv_small_run(features, c_in, w.packed, p.ncb, p.ns, w.small_table, K, out, c_out,
                          p.out_rows, epi, s);
      if (rc != SSC_OK) return rc;
      if (prof) {
        SSC_HIP(hipEventRecord(g_profile_ev[slot][1], s));
        ++g_profile_count;
      }
      return SSC_OK;
    } else {
      SSC_CHECK(false, SSC_ERUNTIME, "the kernel for few input channels is built for float rows");
    }
  }
#define SSC_CONV_LAUNCH(G, S) \
  launch_all<IO, G, S>(p, w, features, n_in, c_in, K, out, c_out, epi, s)
#define SSC_CONV_BY_STEPS(G)                                                            \
  (p.ns == 1 ? SSC_CONV_LAUNCH(G, 1) : p.ns == 2 ? SSC_CONV_LAUNCH(G, 2)                 \
   : p.ns == 3 ? SSC_CONV_LAUNCH(G, 3) : p.ns == 4 ? SSC_CONV_LAUNCH(G, 4)               \
   : p.ns == 6 ? SSC_CONV_LAUNCH(G, 6) : p.ns == 8 ? SSC_CONV_LAUNCH(G, 8)               \
   : p.ns == 10 ? SSC_CONV_LAUNCH(G, 10) : p.ns == 12 ? SSC_CONV_LAUNCH(G, 12)           \
   : p.ns == 13 ? SSC_CONV_LAUNCH(G, 13) : p.ns == 14 ? SSC_CONV_LAUNCH(G, 14)           \
   : p.ns == 15 ? SSC_CONV_LAUNCH(G, 15) : SSC_CONV_LAUNCH(G, 16))
  if constexpr (sizeof(IO) == 2) {
    // half precision: one instance per gather mode (whole chunks)
    rc = p.gather == 1 ? SSC_CONV_LAUNCH(1, 16)
       : p.gather == 2 ? SSC_CONV_LAUNCH(2, 16) : SSC_CONV_LAUNCH(0, 16);
  } else if (p.gather == 1) {
    rc = SSC_CONV_LAUNCH(1, 16);
  } else if (p.gather == 2) {
    rc = SSC_CONV_BY_STEPS(2);
  } else {
    rc = SSC_CONV_BY_STEPS(0);
  }
#undef SSC_CONV_BY_STEPS
#undef SSC_CONV_LAUNCH
  if (rc != SSC_OK) return rc;
  if (prof) {
    SSC_HIP(hipEventRecord(g_profile_ev[slot][1], s));
    ++g_profile_count;
  }
  return SSC_OK;
}

static int conv_check_sizes(int K, int c_in, int c_out, int64_t n_in, int64_t n_out,
                            int64_t pair_stride) {
  SSC_CHECK(K >= 1 && K <= SSC_MAX_KERNEL_VOLUME, SSC_ERUNTIME, "kernel volume %d out of range", K);
  SSC_CHECK(c_in >= 1 && c_out >= 1, SSC_EINVAL, "channel counts must be positive");
  SSC_CHECK(n_in >= 0 && n_out >= 0 && pair_stride >= 0, SSC_EINVAL, "negative size");
  SSC_CHECK(n_out < ((int64_t)1 << 31) && n_in < ((int64_t)1 << 31), SSC_EINVAL,
            "row counts must fit 31 bits");
  return SSC_OK;
}

// The forward convolution for features, filters and output of element type IO.
template <typename IO>
static int conv_fwd(const IO *features, int64_t n_in, int32_t c_in, const IO *filters,
                    int64_t fs_k, int64_t fs_ci, int64_t fs_co, int32_t c_out,
                    const int32_t *pairs, int64_t pair_stride, const int32_t *pair_num,
                    int32_t kernel_volume, int32_t inverse, int32_t subm, IO *out, int64_t n_out,
                    void *workspace, size_t workspace_bytes, ssc_stream_t stream) {
  const int K = kernel_volume;
  int rc = conv_check_sizes(K, c_in, c_out, n_in, n_out, pair_stride);
  if (rc != SSC_OK) return rc;
  if (n_out == 0) return SSC_OK;
  SSC_CHECK(out != nullptr, SSC_EINVAL, "out is NULL");
  hipStream_t s = (hipStream_t)stream;
  if (pair_stride == 0 || n_in == 0) return fill_zero(out, n_out * c_out, s);
  SSC_CHECK(features && filters && pairs && pair_num && workspace, SSC_EINVAL,
            "NULL pointer argument");
  size_t need = conv_ws_bytes(n_out, K, c_in, c_out, pair_stride);
  SSC_CHECK(workspace_bytes >= need, SSC_EWORKSPACE, "conv workspace too small: %zu < %zu",
            workspace_bytes, need);

  ConvPlan p = make_plan(n_in, n_out, K, c_in, c_out, pair_stride, (int)sizeof(IO));
  ConvWs w;
  conv_ws_walk(workspace, p, K, pair_stride, &w);
  const PackArgs pack = {filters, fs_k, fs_ci, fs_co, K, c_in, c_out, p.ncb, p.nch, w.packed, p.ns};
  const bool in_order = (subm & SSC_CONV_PAIRS_CANONICAL) != 0;
  rc = conv_plan_build<IO>(p, w, pairs, pair_stride, pair_num, K, inverse, in_order, c_in, n_out,
                           (int)sizeof(IO), &pack, s);
  if (rc != SSC_OK) return rc;
  return conv_run<IO>(p, w, features, n_in, c_in, K, out, c_out, s);
}

template <typename IO>
static int conv_pack(const IO *filters, int64_t fs_k, int64_t fs_ci, int64_t fs_co, int K, int c_in,
                     int c_out, void *packed, size_t packed_bytes, hipStream_t s) {
  int rc = conv_check_sizes(K, c_in, c_out, 0, 0, 0);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(filters != nullptr && packed != nullptr, SSC_EINVAL, "NULL pointer argument");
  ConvPlan p = make_plan(0, 1, K, c_in, c_out, 0, (int)sizeof(IO));
  SSC_CHECK(packed_bytes >= conv_packed_bytes(p, K), SSC_EWORKSPACE,
            "buffer of the packed filters too small: %zu < %zu", packed_bytes,
            conv_packed_bytes(p, K));
  const PackArgs pack = {filters, fs_k, fs_ci, fs_co, K, c_in, c_out, p.ncb, p.nch, packed, p.ns};
  const int64_t packed_n = (int64_t)K * p.ncb * p.nch * 1024;
  hipLaunchKernelGGL(pack_filters_kernel<IO>, dim3((unsigned)ceil_div(packed_n, 256)), dim3(256), 0,
                     s, pack, (int32_t *)nullptr);
  SSC_LAUNCH_CHECK("pack_filters");
  return SSC_OK;
}

template <typename IO>
static int conv_planned(const IO *features, int64_t n_in, int32_t c_in, const void *packed,
                        size_t packed_bytes, const void *plan, size_t plan_bytes, int64_t pair_stride,
                        int32_t K, int32_t c_out, IO *out, int64_t n_out, hipStream_t s) {
  int rc = conv_check_sizes(K, c_in, c_out, n_in, n_out, pair_stride);
  if (rc != SSC_OK) return rc;
  if (n_out == 0) return SSC_OK;
  SSC_CHECK(out != nullptr, SSC_EINVAL, "out is NULL");
  if (pair_stride == 0 || n_in == 0) return fill_zero(out, n_out * c_out, s);
  SSC_CHECK(features && packed && plan, SSC_EINVAL, "NULL pointer argument");
  ConvPlan p = make_plan(n_in, n_out, K, c_in, c_out, pair_stride, (int)sizeof(IO));
  SSC_CHECK(packed_bytes >= conv_packed_bytes(p, K), SSC_EWORKSPACE,
            "buffer of the packed filters too small");
  SSC_CHECK(plan_bytes >= conv_plan_walk(nullptr, p, nullptr), SSC_EWORKSPACE,
            "plan buffer too small");
  ConvWs w = {};
  w.packed = const_cast<void *>(packed);
  conv_plan_walk(const_cast<void *>(plan), p, &w);
  return conv_run<IO>(p, w, features, n_in, c_in, K, out, c_out, s);
}

// conv_planned with the epilogue applied to every finished tile.
template <typename IO>
static int conv_planned_epilogue(const IO *features, int64_t n_in, int32_t c_in,
                                 const void *packed, size_t packed_bytes, const void *plan,
                                 size_t plan_bytes, int64_t pair_stride, int32_t K, int32_t c_cols,
                                 const ssc_conv_epilogue *e, IO *out, int64_t n_out,
                                 hipStream_t s) {
  int rc = conv_check_sizes(K, c_in, c_cols, n_in, n_out, pair_stride);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(e != nullptr, SSC_EINVAL, "epilogue is NULL");
  SSC_CHECK((c_cols & 3) == 0, SSC_EINVAL, "an epilogue needs a multiple of 4 filter columns");
  SSC_CHECK(e->c_dest >= 1, SSC_EINVAL, "c_dest must be positive");
  SSC_CHECK(e->act_scalar >= SSC_ACT_NONE && e->act_scalar <= SSC_ACT_TANH &&
                e->act_gate >= SSC_ACT_NONE && e->act_gate <= SSC_ACT_TANH,
            SSC_EINVAL, "unknown activation code");
  if (n_out == 0) return SSC_OK;
  SSC_CHECK(pair_stride > 0 && n_in > 0, SSC_EINVAL,
            "no pairs: apply the normalisation to rows of zeros with ssc_bnact_fwd_f32");
  SSC_CHECK(out && features && packed && plan, SSC_EINVAL, "NULL pointer argument");
  SSC_CHECK(e->shift && e->scale && e->add && e->pre_bias && e->mode && e->gate && e->dest &&
                e->gate_run,
            SSC_EINVAL, "NULL table in the epilogue");
  ConvPlan p = make_plan(n_in, n_out, K, c_in, c_cols, pair_stride, (int)sizeof(IO));
  SSC_CHECK(packed_bytes >= conv_packed_bytes(p, K), SSC_EWORKSPACE,
            "buffer of the packed filters too small");
  SSC_CHECK(plan_bytes >= conv_plan_walk(nullptr, p, nullptr), SSC_EWORKSPACE,
            "plan buffer too small");
  ConvWs w = {};
  w.packed = const_cast<void *>(packed);
  conv_plan_walk(const_cast<void *>(plan), p, &w);
  const ConvEpilogue epi = {e->shift, e->scale, e->add, e->pre_bias, e->mode, e->gate, e->dest,
                            e->gate_run, e->act_scalar, e->act_gate, e->c_dest};
  return conv_run<IO>(p, w, features, n_in, c_in, K, out, c_cols, s, epi);
}

extern "C" {

int ssc_conv_run_epilogue_f32(const float *features, int64_t n_in, int32_t c_in,
                              const void *packed, size_t packed_bytes, const void *plan,
                              size_t plan_bytes, int64_t pair_stride, int32_t kernel_volume,
                              int32_t c_cols, const ssc_conv_epilogue *epilogue, float *out,
                              int64_t n_out, ssc_stream_t stream) {
  return conv_planned_epilogue<float>(features, n_in, c_in, packed, packed_bytes, plan,
                                      plan_bytes, pair_stride, kernel_volume, c_cols, epilogue,
                                      out, n_out, (hipStream_t)stream);
}

int ssc_conv_run_epilogue_f16(const void *features, int64_t n_in, int32_t c_in,
                              const void *packed, size_t packed_bytes, const void *plan,
                              size_t plan_bytes, int64_t pair_stride, int32_t kernel_volume,
                              int32_t c_cols, const ssc_conv_epilogue *epilogue, void *out,
                              int64_t n_out, ssc_stream_t stream) {
  return conv_planned_epilogue<_Float16>(static_cast<const _Float16 *>(features), n_in, c_in,
                                         packed, packed_bytes, plan, plan_bytes, pair_stride,
                                         kernel_volume, c_cols, epilogue,
                                         static_cast<_Float16 *>(out), n_out, (hipStream_t)stream);
}

int ssc_conv_fwd_f32(const float *features, int64_t n_in, int32_t c_in, const float *filters,
                     int64_t fs_k, int64_t fs_ci, int64_t fs_co, int32_t c_out,
                     const int32_t *pairs, int64_t pair_stride, const int32_t *pair_num,
                     int32_t kernel_volume, int32_t inverse, int32_t subm, float *out,
                     int64_t n_out, void *workspace, size_t workspace_bytes,
                     ssc_stream_t stream) {
  return conv_fwd<float>(features, n_in, c_in, filters, fs_k, fs_ci, fs_co, c_out, pairs,
                         pair_stride, pair_num, kernel_volume, inverse, subm, out, n_out, workspace,
                         workspace_bytes, stream);
}

int ssc_conv_fwd_f16(const void *features, int64_t n_in, int32_t c_in, const void *filters,
                     int64_t fs_k, int64_t fs_ci, int64_t fs_co, int32_t c_out,
                     const int32_t *pairs, int64_t pair_stride, const int32_t *pair_num,
                     int32_t kernel_volume, int32_t inverse, int32_t subm, void *out,
                     int64_t n_out, void *workspace, size_t workspace_bytes,
                     ssc_stream_t stream) {
  return conv_fwd<_Float16>(static_cast<const _Float16 *>(features), n_in, c_in,
                            static_cast<const _Float16 *>(filters), fs_k, fs_ci, fs_co, c_out,
                            pairs, pair_stride, pair_num, kernel_volume, inverse, subm,
                            static_cast<_Float16 *>(out), n_out, workspace, workspace_bytes, stream);
}

int ssc_conv_tile_cut(int32_t rows, int32_t c_in, int32_t c_out, int32_t *n_tiles, int32_t *height,
                      int32_t *window) {
  SSC_CHECK(rows >= 0 && c_in >= 1 && c_out >= 1 && n_tiles && height && window, SSC_EINVAL,
            "bad argument");
  const ConvPlan p = make_plan(0, 1, 1, c_in, c_out, 0);
  int nt = 0, h = 0;
  range_tiles(rows, p.tile_rows, p.T, &nt, &h);
  *n_tiles = nt;
  *height = h;
  *window = p.T;
  return SSC_OK;
}

size_t ssc_conv_packed_bytes(int32_t kernel_volume, int32_t c_in, int32_t c_out) {
  if (kernel_volume < 1 || c_in < 1 || c_out < 1) return 0;
  return conv_packed_bytes(make_plan(0, 1, kernel_volume, c_in, c_out, 0), kernel_volume);
}

size_t ssc_conv_plan_bytes(int64_t n_out, int32_t kernel_volume, int32_t c_in, int32_t c_out,
                           int64_t pair_stride) {
  if (n_out < 0 || kernel_volume < 1 || c_in < 1 || c_out < 1 || pair_stride < 0) return 0;
  // (the element type is not known here: room for the plan of either, which differ for
  // layers of a handful of input channels)
  ConvPlan p = make_plan(0, n_out, kernel_volume, c_in, c_out, pair_stride);
  size_t bytes = conv_plan_walk(nullptr, p, nullptr);
  if (p.small) {
    p.small = false;
    const size_t other = conv_plan_walk(nullptr, p, nullptr);
    if (other > bytes) bytes = other;
  }
  return bytes;
}

size_t ssc_conv_plan_scratch_bytes(int64_t n_out, int32_t kernel_volume, int32_t c_in,
                                   int32_t c_out, int64_t pair_stride) {
  if (n_out < 0 || kernel_volume < 1 || c_in < 1 || c_out < 1 || pair_stride < 0) return 0;
  return conv_scratch_walk(nullptr, make_plan(0, n_out, kernel_volume, c_in, c_out, pair_stride),
                           kernel_volume, pair_stride, nullptr);
}

int ssc_conv_plan_build(const int32_t *pairs, int64_t pair_stride, const int32_t *pair_num,
                        int32_t kernel_volume, int32_t inverse, int32_t flags, int64_t n_in,
                        int64_t n_out, int32_t c_in, int32_t c_out, int32_t elem_bytes, void *plan,
                        size_t plan_bytes, void *scratch, size_t scratch_bytes,
                        ssc_stream_t stream) {
  const int K = kernel_volume;
  int rc = conv_check_sizes(K, c_in, c_out, n_in, n_out, pair_stride);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(elem_bytes == 4 || elem_bytes == 2, SSC_EINVAL, "elem_bytes must be 4 or 2");
  if (n_out == 0 || pair_stride == 0 || n_in == 0) return SSC_OK;  // nothing to schedule
  SSC_CHECK(pairs && pair_num && plan && scratch, SSC_EINVAL, "NULL pointer argument");
  ConvPlan p = make_plan(n_in, n_out, K, c_in, c_out, pair_stride, elem_bytes);
  SSC_CHECK(plan_bytes >= conv_plan_walk(nullptr, p, nullptr), SSC_EWORKSPACE,
            "plan buffer too small");
  SSC_CHECK(scratch_bytes >= conv_scratch_walk(nullptr, p, K, pair_stride, nullptr),
            SSC_EWORKSPACE, "plan scratch too small");
  ConvWs w = {};
  conv_plan_walk(plan, p, &w);
  conv_scratch_walk(scratch, p, K, pair_stride, &w);
  return conv_plan_build<float>(p, w, pairs, pair_stride, pair_num, K, inverse,
                                (flags & SSC_CONV_PAIRS_CANONICAL) != 0, c_in, n_out, elem_bytes,
                                nullptr, (hipStream_t)stream);
}

// The checked form of "synthesise and pack these filters".
static int combine_job_of(const float *weight, const float *basis, const int32_t *chan_out,
                          const int32_t *chan_in, const int32_t *blocks, int32_t n_irreps_in,
                          int32_t K, int32_t c_in, int32_t c_out, float *out, void *packed,
                          size_t packed_bytes, CombineJob *job) {
  int rc = conv_check_sizes(K, c_in, c_out, 0, 0, 0);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(weight && basis && chan_out && chan_in && blocks && out && packed, SSC_EINVAL,
            "NULL pointer argument");
  SSC_CHECK(n_irreps_in >= 1, SSC_EINVAL, "sizes must be positive");
  const ConvPlan p = make_plan(0, 1, K, c_in, c_out, 0, 4);
  SSC_CHECK(packed_bytes >= conv_packed_bytes(p, K), SSC_EWORKSPACE,
            "buffer of the packed filters too small");
  job->pk = PackArgs{nullptr, 0, 0, 0, K, c_in, c_out, p.ncb, p.nch, packed, p.ns};
  job->weight = weight;
  job->basis = basis;
  job->chan_out = chan_out;
  job->chan_in = chan_in;
  job->blocks = blocks;
  job->n_j = (int)n_irreps_in;
  job->dense = out;
  return SSC_OK;
}

// A rulebook between ssc_rulebook_conv_begin and ssc_rulebook_conv_finish on this host thread:
// whether the rulebook was asked to place the range boundaries, and for which cuts (number
// of ranges and tile height of the request and of its alternative; 0 ranges: none).
struct PendingLayer {
  bool seeded = false;
  int n_rng[2] = {0, 0};
  int tile_rows[2] = {0, 0};
};
static thread_local PendingLayer g_pending_layer;

int ssc_rulebook_conv_begin(const int32_t *indices, int64_t n_in, const ssc_geometry *g,
                            void *workspace, size_t workspace_bytes, int32_t *pairs,
                            int32_t *pair_num, int32_t *out_indices, int64_t out_capacity,
                            void *clean_table, size_t clean_table_bytes, int32_t c_in,
                            int32_t c_out, int32_t elem_bytes, void *scratch,
                            size_t scratch_bytes, const ssc_combine_job *filters,
                            ssc_stream_t stream) {
  g_pending_layer = PendingLayer();
  SSC_CHECK(g != nullptr, SSC_EINVAL, "geometry is NULL");
  SSC_CHECK(c_in >= 1 && c_out >= 1, SSC_EINVAL, "channel counts must be positive");
  SSC_CHECK(elem_bytes == 4 || elem_bytes == 2, SSC_EINVAL, "elem_bytes must be 4 or 2");
  CombineJob job = {};
  if (filters != nullptr) {
    int rc = combine_job_of(filters->weight, filters->basis, filters->chan_out, filters->chan_in,
                            filters->blocks, filters->n_irreps_in, filters->kernel_volume, c_in,
                            c_out, filters->out, filters->packed, filters->packed_bytes, &job);
    if (rc != SSC_OK) return rc;
  }
  SplitRequest rq = {0, 0, 0, nullptr, 0, 0, nullptr};
  const SplitRequest *ask = nullptr;
  int64_t K = 1;
  for (int a = 0; a < 3; ++a) K *= g->ksize[a] > 0 ? g->ksize[a] : 1;
  if (scratch != nullptr && n_in > 0 && K <= SSC_MAX_KERNEL_VOLUME && !g->subm && !g->transpose) {
    // What the plan will look like depends on whether the outputs outnumber the inputs
    // (make_plan's estimate of the pairs).  At stride 1 with a padded kernel they do; a
    // strided layer can go either way (a sparse cloud loses few rows to a stride of 2), so
    // its rulebook is asked for the cut of either plan where the two differ.
    bool strided = false;
    for (int a = 0; a < 3; ++a) strided = strided || g->stride[a] != 1 || g->dilation[a] != 1;
    ConvWs w = {};
    const size_t head = conv_scratch_head(scratch, &w);
    const ConvPlan more = make_plan(n_in, n_in + 1, (int)K, c_in, c_out, n_in, elem_bytes);
    const ConvPlan fewer =
        make_plan(n_in, n_in > 1 ? n_in - 1 : 1, (int)K, c_in, c_out, n_in, elem_bytes);
    const bool more_ok = !more.rebalance && !more.small;
    const bool fewer_ok = strided && n_in > 1 && !fewer.rebalance && !fewer.small &&
                          !(more_ok && fewer.n_rng == more.n_rng &&
                            fewer.tile_rows == more.tile_rows);
    if (scratch_bytes >= head && (more_ok || fewer_ok)) {
      const ConvPlan &first = more_ok ? more : fewer;
      rq.n_rng = first.n_rng;
      rq.tile_rows = first.tile_rows;
      rq.tile_cost = (long long)K * 4 + 64;  // split_tile_cost
      rq.range_row0 = w.range_row0;
      if (more_ok && fewer_ok) {
        rq.n_rng_alt = fewer.n_rng;
        rq.tile_rows_alt = fewer.tile_rows;
        rq.range_row0_alt = w.range_row0_alt;
      }
      ask = &rq;
    }
  }
  bool seeded = false;
  int rc = rulebook_begin_impl(indices, n_in, g, workspace, workspace_bytes, pairs, pair_num,
                               out_indices, out_capacity, clean_table, clean_table_bytes, ask,
                               &seeded, (hipStream_t)stream, filters ? &job : nullptr);
  if (rc != SSC_OK) return rc;
  g_pending_layer.seeded = seeded;
  g_pending_layer.n_rng[0] = rq.n_rng;
  g_pending_layer.tile_rows[0] = rq.tile_rows;
  g_pending_layer.n_rng[1] = rq.n_rng_alt;
  g_pending_layer.tile_rows[1] = rq.tile_rows_alt;
  return SSC_OK;
}

int ssc_rulebook_conv_finish(const ssc_geometry *g, int64_t n_in, int32_t *n_out_host,
                             int32_t *in_order_host, const int32_t *pairs,
                             const int32_t *pair_num, int32_t c_in, int32_t c_out,
                             int32_t elem_bytes, void *plan, size_t plan_bytes, void *scratch,
                             size_t scratch_bytes, ssc_stream_t stream) {
  const PendingLayer pending = g_pending_layer;
  g_pending_layer = PendingLayer();
  int rc = ssc_rulebook_finish(g, n_in, n_out_host, in_order_host);
  if (rc != SSC_OK) return rc;
  const int64_t n_out = *n_out_host;
  int K = 1;
  for (int a = 0; a < 3; ++a) K *= g->ksize[a];
  rc = conv_check_sizes(K, c_in, c_out, n_in, n_out, n_in);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(elem_bytes == 4 || elem_bytes == 2, SSC_EINVAL, "elem_bytes must be 4 or 2");
  if (n_out == 0 || n_in == 0) return SSC_OK;  // nothing to schedule
  SSC_CHECK(pairs && pair_num && plan && scratch, SSC_EINVAL, "NULL pointer argument");
  const ConvPlan p = make_plan(n_in, n_out, K, c_in, c_out, n_in, elem_bytes);
  SSC_CHECK(plan_bytes >= conv_plan_walk(nullptr, p, nullptr), SSC_EWORKSPACE,
            "plan buffer too small");
  SSC_CHECK(scratch_bytes >= conv_scratch_walk(nullptr, p, K, n_in, nullptr), SSC_EWORKSPACE,
            "plan scratch too small");
  ConvWs w = {};
  conv_plan_walk(plan, p, &w);
  conv_scratch_walk(scratch, p, K, n_in, &w);
  const bool in_order = *in_order_host != 0;
  // the cut the rulebook placed for this plan, if any: the one of the same tile height
  // before one that only has the plan's number of ranges (the height is a weight in the
  // work measure, not a condition)
  int cut = -1;
  if (pending.seeded && in_order && !p.rebalance && !p.small) {
    for (int c = 1; c >= 0; --c)
      if (pending.n_rng[c] == p.n_rng) cut = c;
    for (int c = 1; c >= 0; --c)
      if (pending.n_rng[c] == p.n_rng && pending.tile_rows[c] == p.tile_rows) cut = c;
  }
  const bool seeded = cut >= 0;
  if (cut == 1) w.range_row0 = w.range_row0_alt;
  return conv_plan_build<float>(p, w, pairs, n_in, pair_num, K, 0, in_order, c_in, n_out,
                                elem_bytes, nullptr, (hipStream_t)stream, seeded);
}

int ssc_kernel_combine_packed_f32(const float *weight, const float *basis,
                                  const int32_t *chan_out, const int32_t *chan_in,
                                  const int32_t *blocks, int32_t n_irreps_in,
                                  int32_t kernel_volume, int32_t c_in, int32_t c_out, float *out,
                                  void *packed, size_t packed_bytes, ssc_stream_t stream) {
  CombineJob job;
  int rc = combine_job_of(weight, basis, chan_out, chan_in, blocks, n_irreps_in, kernel_volume,
                          c_in, c_out, out, packed, packed_bytes, &job);
  if (rc != SSC_OK) return rc;
  return launch_combine_pack(job, (hipStream_t)stream);
}

int ssc_conv_pack_filters_f32(const float *filters, int64_t fs_k, int64_t fs_ci, int64_t fs_co,
                              int32_t kernel_volume, int32_t c_in, int32_t c_out, void *packed,
                              size_t packed_bytes, ssc_stream_t stream) {
  return conv_pack<float>(filters, fs_k, fs_ci, fs_co, kernel_volume, c_in, c_out, packed,
                          packed_bytes, (hipStream_t)stream);
}

int ssc_conv_pack_filters_f16(const void *filters, int64_t fs_k, int64_t fs_ci, int64_t fs_co,
                              int32_t kernel_volume, int32_t c_in, int32_t c_out, void *packed,
                              size_t packed_bytes, ssc_stream_t stream) {
  return conv_pack<_Float16>(static_cast<const _Float16 *>(filters), fs_k, fs_ci, fs_co,
                             kernel_volume, c_in, c_out, packed, packed_bytes,
                             (hipStream_t)stream);
}

int ssc_conv_run_f32(const float *features, int64_t n_in, int32_t c_in, const void *packed,
                     size_t packed_bytes, const void *plan, size_t plan_bytes, int64_t pair_stride,
                     int32_t kernel_volume, int32_t c_out, float *out, int64_t n_out,
                     ssc_stream_t stream) {
  return conv_planned<float>(features, n_in, c_in, packed, packed_bytes, plan, plan_bytes,
                             pair_stride, kernel_volume, c_out, out, n_out, (hipStream_t)stream);
}

int ssc_conv_run_f16(const void *features, int64_t n_in, int32_t c_in, const void *packed,
                     size_t packed_bytes, const void *plan, size_t plan_bytes, int64_t pair_stride,
                     int32_t kernel_volume, int32_t c_out, void *out, int64_t n_out,
                     ssc_stream_t stream) {
  return conv_planned<_Float16>(static_cast<const _Float16 *>(features), n_in, c_in, packed,
                                packed_bytes, plan, plan_bytes, pair_stride, kernel_volume, c_out,
                                static_cast<_Float16 *>(out), n_out, (hipStream_t)stream);
}
}
