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
#include "ssc_common.h"

#include <type_traits>

namespace ssc {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));

constexpr int kKC = 64;       // input channels per chunk = 16 MFMA steps of 4
constexpr int kStage = 64;    // pairs staged per barrier = 4 row blocks of 16
constexpr int kAStride = 68;  // floats per staged row (64 + 4: 16-byte aligned, bank spread)
constexpr int kMinTile = 64;

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
    ci = cc * kKC + 32 * q + (lane >> 4) * 8 + j;
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
  int k, ci, co;
  pack_decode<float>(a, idx, k, ci, co);
  float v = 0.f;
  if (ci < a.cin && co < a.cout) {
    v = combine_element(weight, basis, chan_out, chan_in, blocks, n_j, a.K, k, ci, co);
    dense[((int64_t)k * a.cin + ci) * a.cout + co] = v;
  }
  static_cast<float *>(a.packed_out)[idx] = v;
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
// into tiles of equal height <= T.
constexpr int kSplitGranule = 64;
// The accumulator window of a workgroup holds kSpillRows more rows than a tile is
// high: the last row block that an offset contributes to a tile may then be filled
// up with the offset's next pairs, whose rows lie in the following tile (at most
// kSpillRows into it), instead of being padded.  Rows map to accumulator slots
// modulo the window height, so what such a block adds to the next tile's rows is
// still there when that tile's turn comes.
constexpr int kSpillRows = 160;

// cost of a tile beyond its pairs, in pair slots: padding per offset, and about a stage's
// worth of time for writing it out (measured: 2 K + 128 and 3 K + 64 are as good on the
// 27-offset benchmark layers; with 125 offsets 4 K + 64 is 4 % faster than 2 K + 128, and
// more than that slower again)
__device__ __forceinline__ int64_t split_tile_cost(int K) { return (int64_t)K * 4 + 64; }

// Work in rows below cell b of the fine grid (scaled by T to stay in integers).
__device__ __forceinline__ int64_t split_work(int64_t pairs_below, int64_t b, int64_t n_out,
                                              int T, int K) {
  int64_t r = b * kSplitGranule;
  if (r > n_out) r = n_out;
  return pairs_below * T + r * split_tile_cost(K);
}

// One thread per cell boundary b = 0..nb of the fine grid: the ranges whose first row
// is boundary b are those whose target (w/n_wg of the total work) lies in
// (work(b-1), work(b)].  range_row0[w], w = 0..n_wg.
__global__ void __launch_bounds__(256)
    split_bounds_kernel(const int32_t *__restrict__ fine_segs, int K, int64_t nb, int64_t n_out,
                        int T, int n_wg, int32_t *__restrict__ range_row0) {
  int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b > nb) return;
  int64_t below = 0, below_prev = 0, all = 0;
  for (int k = 0; k < K; ++k) {
    below += fine_segs[b * K + k];
    if (b > 0) below_prev += fine_segs[(b - 1) * K + k];
    all += fine_segs[nb * K + k];
  }
  const int64_t total = split_work(all, nb, n_out, T, K);
  // ranges w with ceil(total * w / n_wg) <= work, i.e. w <= work * n_wg / total
  auto reached = [&](int64_t work) -> int64_t {
    if (total <= 0) return n_wg + 1;
    int64_t c = work * n_wg / total + 1;
    return c > n_wg + 1 ? n_wg + 1 : c;
  };
  const int64_t w0 = b > 0 ? reached(split_work(below_prev, b - 1, n_out, T, K)) : 0;
  const int64_t w1 = reached(split_work(below, b, n_out, T, K));
  int64_t r = b * kSplitGranule;
  if (r > n_out) r = n_out;
  for (int64_t w = w0; w < w1; ++w)
    range_row0[w] = (w == 0) ? 0 : (w == n_wg ? (int32_t)n_out : (int32_t)r);
}

// One block.  wg_tile[0..n_wg]: first tile of every workgroup; tile_row0[0..n_tiles]:
// first row of every tile; n_tiles_dev[0]: number of tiles; spill_end[0..n_tiles]:
// rows below spill_end[t] may be touched by the last row blocks of tile t-1 (the
// first row of tile t itself when t starts a workgroup's range: no spill across
// ranges); tile_slot0[t]: accumulator slot of the first row of tile t.  T is the
// largest tile height, window the height of the accumulator window.
__global__ void __launch_bounds__(256)
    split_rows_kernel(const int32_t *__restrict__ range_row0, int64_t n_out, int T, int window,
                      int n_wg, int32_t *__restrict__ wg_tile, int32_t *__restrict__ tile_row0,
                      int32_t *__restrict__ n_tiles_dev, int32_t *__restrict__ spill_end,
                      int32_t *__restrict__ tile_slot0) {
  __shared__ int row_s[257];
  __shared__ int tile_s[257];
  for (int w = threadIdx.x; w <= n_wg; w += blockDim.x) {  // n_wg <= 256
    int r = range_row0[w];
    if (w == 0) r = 0;
    if (w == n_wg) r = (int)n_out;
    row_s[w] = r;
  }
  __syncthreads();
  {
    // exclusive scan of the tile counts of the (at most 256) ranges, one per thread
    __shared__ int wave_sum[4];
    const int w = threadIdx.x, lane = w & 63;
    const int nt = w < n_wg ? (row_s[w + 1] - row_s[w] + T - 1) / T : 0;
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
    if (w == 255) {
      const int run = before + incl;
      tile_s[n_wg] = run;
      n_tiles_dev[0] = run;
      tile_row0[run] = (int32_t)n_out;
      spill_end[run] = (int32_t)n_out;
    }
  }
  __syncthreads();
  for (int w = threadIdx.x; w <= n_wg; w += blockDim.x) {
    wg_tile[w] = tile_s[w];
    if (w == n_wg) break;
    const int rows = row_s[w + 1] - row_s[w];
    const int nt = tile_s[w + 1] - tile_s[w];
    if (nt > 0) {
      const int h = (rows + nt - 1) / nt;
      for (int j = 0; j < nt; ++j) {
        const int r = row_s[w] + j * h;
        tile_row0[tile_s[w] + j] = r;
        spill_end[tile_s[w] + j] = j == 0 ? r : min(r + window - T, row_s[w + 1]);
        tile_slot0[tile_s[w] + j] = (j * h) % window;
      }
    }
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
__global__ void __launch_bounds__(256)
    range_sched_kernel(const int32_t *__restrict__ segs, const int32_t *__restrict__ spill, int K,
                       const int32_t *__restrict__ wg_tile, int32_t *__restrict__ share_first,
                       int32_t *__restrict__ share_cnt, int32_t *__restrict__ kofs,
                       int32_t *__restrict__ tile_nmb, int32_t *__restrict__ tile_loc,
                       int32_t *__restrict__ tile_rng, int32_t *__restrict__ range_grp) {
  const int w = blockIdx.x;
  const int t0 = wg_tile[w], t1 = wg_tile[w + 1];
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
          share_first[(int64_t)t * K + k] = s;
          share_cnt[(int64_t)t * K + k] = e - s;
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
      const int nb = k < K ? (share_cnt[t * K + k] + 15) >> 4 : 0;
      int incl = nb;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
      }
      if (k < K) kofs[t * K + k] = run + incl - nb;
      run += __shfl(incl, 63, 64);
    }
    if (lane == 0) {
      tile_nmb[t] = run;
      const int groups = (run + 3) >> 2;
      tile_loc[t] = groups > 0 ? groups : 1;  // a tile without pairs gets an empty group
    }
  }
  __threadfence_block();
  __syncthreads();
  if (wave == 0) {
    int carry = 0;
    for (int base = t0; base < t1; base += 64) {
      const int t = base + lane;
      const int v = t < t1 ? tile_loc[t] : 0;
      int incl = v;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
      }
      if (t < t1) {
        tile_loc[t] = carry + incl - v;
        tile_rng[t] = w;
      }
      carry += __shfl(incl, 63, 64);
    }
    if (lane == 0) range_grp[w] = carry;
  }
}

// 16 threads per (tile, offset): lane i fills slot i of each of its row blocks; the
// threads of offset 0 also write the tile's padding blocks and its group -> tile map.
__global__ void __launch_bounds__(256)
    sched_fill_kernel(const int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                      const int32_t *__restrict__ sorted, int64_t pair_stride, int plane_g,
                      const int32_t *__restrict__ share_first,
                      const int32_t *__restrict__ share_cnt, const int32_t *__restrict__ kofs,
                      const int32_t *__restrict__ tile_nmb, const int32_t *__restrict__ tile_loc,
                      const int32_t *__restrict__ tile_rng, const int32_t *__restrict__ range_grp,
                      int n_wg, int32_t *__restrict__ tile_grp, int K,
                      const int32_t *__restrict__ n_tiles_dev,
                      const int32_t *__restrict__ tile_row0,
                      const int32_t *__restrict__ tile_slot0, int T, uint32_t in_scale,
                      uint32_t in_pad, int out_scale, int k_scale,
                      int32_t *__restrict__ sched_in, int32_t *__restrict__ sched_out,
                      int32_t *__restrict__ grp_meta) {
  // groups before every range (n_wg <= 256 of them): exclusive prefix of range_grp
  __shared__ int range_g0[257];
  {
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
  }
  int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t tk = gid >> 4;
  int lane = (int)(gid & 15);
  const int64_t n_tiles = n_tiles_dev[0];
  if (tk >= n_tiles * K) return;
  int64_t t = tk / K;
  int k = (int)(tk - t * K);
  const int rng = tile_rng[t];
  const int64_t g0 = range_g0[rng] + tile_loc[t];
  const int64_t g1 = (t + 1 < n_tiles && tile_rng[t + 1] == rng) ? range_g0[rng] + tile_loc[t + 1]
                                                                : range_g0[rng + 1];
  if (k == 0 && lane == 0) {  // the tiles' first groups, for the convolution kernel
    tile_grp[t] = (int32_t)g0;
    if (t + 1 == n_tiles) tile_grp[n_tiles] = (int32_t)g1;
  }
  if (k == 0) {
    for (int64_t g = g0 + lane; g < g1; g += 16) {
      const int rows = tile_row0[t + 1] - tile_row0[t];
      grp_meta[g * 8 + 4] = tile_row0[t];
      grp_meta[g * 8 + 5] = g + 1 == g1 ? rows : -rows;
      grp_meta[g * 8 + 6] = tile_slot0[t];
      grp_meta[g * 8 + 7] = 0;
    }
    for (int64_t mb = g0 * 4 + tile_nmb[t]; mb < g1 * 4; ++mb) {
      sched_in[mb * 16 + lane] = (int32_t)in_pad;
      sched_out[mb * 16 + lane] = T * out_scale;
      if (lane == 0) grp_meta[(mb >> 2) * 8 + (mb & 3)] = 0;
    }
  }
  const int32_t *src = flag[0] ? sorted : pairs;
  int s0 = share_first[t * K + k];
  int n = share_cnt[t * K + k];
  if (n <= 0) return;
  const int32_t *pg = src + ((int64_t)k * 2 + plane_g) * pair_stride + s0;
  const int32_t *ps = src + ((int64_t)k * 2 + (1 - plane_g)) * pair_stride + s0;
  int64_t mb = g0 * 4 + kofs[t * K + k];
  // accumulator slot of a row: rows map to slots modulo the window height T; the
  // rows a tile touches span less than T, so one conditional subtraction does it
  const int slot_off = tile_slot0[t] - tile_row0[t];
  for (int p = lane; p < ((n + 15) & ~15); p += 16, ++mb) {
    sched_in[mb * 16 + lane] = p < n ? (int32_t)((uint32_t)pg[p] * in_scale) : (int32_t)in_pad;
    int slot = T;
    if (p < n) {
      slot = ps[p] + slot_off;
      if (slot >= T) slot -= T;
    }
    sched_out[mb * 16 + lane] = slot * out_scale;
    if (lane == 0) grp_meta[(mb >> 2) * 8 + (mb & 3)] = k * k_scale;
  }
}

// ---- the convolution --------------------------------------------------------------------
// Persistent kernel: one workgroup per CU walks a contiguous, work-balanced range
// of tiles.  A workgroup owns T output rows x 16*NCW output columns at a time; the
// fp32 accumulators of that tile live in LDS.
//   waves 0..NCW-1    consumers: wave w owns 16 columns of the workgroup's column
//                     range.  It multiplies the staged input rows of a stage with the
//                     weight fragments of its columns and adds the products to the
//                     accumulators.
//   waves NCW..NCW+3  producers: gather the input rows of the coming stages from
//                     global memory (several stages ahead, in registers) and stage
//                     them in LDS.
// NCW = 4 (64 columns) is what the host code launches.  NCW = 8 (128 columns, two
// consumers per SIMD, tiles half as tall) computes the same result; on the 64 -> 128
// channel benchmark layer it is 6 % slower, because the shorter tiles pack the row
// blocks less densely and the weight-fragment traffic per tile row doubles.
// A stage = one group of the schedule (4 row blocks = 64 pair slots, any mix of
// offsets) x one 64-channel chunk of Cin.  One barrier per stage hands the buffer
// filled with stage s+1 to the consumers and the buffer of stage s back to the
// producers.  After a tile's last stage all waves write the tile out and clear
// the accumulators.
//
// fp32 MFMAs and ordinary vector-ALU instructions do not overlap on a SIMD, no
// matter which wave issues them (measured: every VALU instruction next to a
// stream of v_mfma_f32_16x16x4_f32 costs about five cycles of matrix time), while
// scalar, LDS and memory instructions of another wave are free.  So the loops
// below keep vector arithmetic out of the steady state: the schedule already
// holds byte offsets, addresses are (scalar offset + constant lane offset) of
// buffer loads, per-stage bookkeeping is scalar loads and scalar arithmetic, and
// the producers do not touch the VALU except for one add per gathered row chunk.
// Buffer loads are range-checked by the hardware and return zero outside their
// buffer: padding slots carry an offset beyond the features and gather zeros,
// and the prefetches that run past the end of a workgroup's schedule are harmless.
//
// MFMA orientation: D[16 channels x 16 pairs] = W^T[16 x 4] * F^T[4 x 16], so a
// lane ends up with 4 consecutive output channels of one pair and adds them to
// the LDS accumulator row of that pair with one 16-byte read-modify-write.  A
// column group belongs to exactly one wave, which walks the schedule in order,
// so every output element sees its offsets added in ascending k: reproducible,
// no atomics.
//
// Dynamic LDS: acc[T+1][16*NCW+4] | abuf[2][64][68]
constexpr int kRowsAhead = 4;  // stages whose gathered rows are in flight in registers
constexpr int kIdxAhead = 2;   // further stages whose gather offsets are in flight
constexpr unsigned kGatherPad = 0xFFFFF000u;  // byte offset that gathers zeros (beyond any feature buffer)
constexpr int kRsrcFlags = 0x00020000;        // raw buffer of 32-bit data

__device__ __forceinline__ float4v buf_load4(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
  return __builtin_bit_cast(float4v, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
typedef int int3v __attribute__((ext_vector_type(3)));
__device__ __forceinline__ int3v buf_load3(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
  return __builtin_bit_cast(int3v, __builtin_amdgcn_raw_buffer_load_b96(r, voff, soff, 0));
}
__device__ __forceinline__ int buf_load1(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
  return (int)__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0);
}

// Element type of the features, the filters and the output.  float: fp32 rows in LDS,
// v_mfma_f32_16x16x4_f32.  _Float16: half rows in LDS, v_mfma_f32_16x16x32_f16; the
// accumulators are fp32 either way and are rounded once, when a finished tile is written.
typedef int int2v __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float float3v __attribute__((ext_vector_type(3)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
template <typename IO> struct Io;
template <> struct Io<float> {
  static constexpr int kBytes = 4;
  static constexpr int kRowBytes = kAStride * 4;  // a staged row of 64 channels in LDS
  static constexpr int kFragBytes = 4096;         // packed filters of (offset, column block, chunk)
  typedef float4v Raw;  // four channels as they are loaded
  static __device__ __forceinline__ Raw zero() { return Raw{0.f, 0.f, 0.f, 0.f}; }
  static __device__ __forceinline__ Raw gather(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    return buf_load4(r, voff, soff);
  }
  static __device__ __forceinline__ Raw load(const float *p) {
    return *reinterpret_cast<const float4v *>(p);
  }
  // the first n (possibly <= 0 or > 4) of four channels, zeros for the rest
  static __device__ __forceinline__ Raw load_first(const float *p, int n) {
    Raw v = zero();
    if (n > 0) v.x = p[0];
    if (n > 1) v.y = p[1];
    if (n > 2) v.z = p[2];
    if (n > 3) v.w = p[3];
    return v;
  }
  static __device__ __forceinline__ void store_stream(float *p, const float4v &v) {
    __builtin_nontemporal_store(v, reinterpret_cast<float4v *>(p));
  }
};
template <> struct Io<_Float16> {
  static constexpr int kBytes = 2;
  static constexpr int kRowBytes = 144;  // 128 + 16: 16-byte aligned, bank spread as for float
  static constexpr int kFragBytes = 2048;
  typedef int2v Raw;
  static __device__ __forceinline__ Raw zero() { return Raw{0, 0}; }
  static __device__ __forceinline__ Raw gather(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(int2v, __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0));
  }
  static __device__ __forceinline__ Raw load(const _Float16 *p) {
    return *reinterpret_cast<const int2v *>(p);
  }
  static __device__ __forceinline__ Raw load_first(const _Float16 *p, int n) {
    half4v v = {(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
    if (n > 0) v.x = p[0];
    if (n > 1) v.y = p[1];
    if (n > 2) v.z = p[2];
    if (n > 3) v.w = p[3];
    return __builtin_bit_cast(int2v, v);
  }
  static __device__ __forceinline__ void store_stream(_Float16 *p, const float4v &v) {
    const half4v h = __builtin_convertvector(v, half4v);  // round to nearest even
    __builtin_nontemporal_store(__builtin_bit_cast(int2v, h), reinterpret_cast<int2v *>(p));
  }
};

// Position of a stage in the schedule: group index and channel chunk.  Advanced
// with scalar arithmetic only.
struct StagePos {
  int g, cc;
  __device__ __forceinline__ void advance(int nch) {
    ++cc;
    if (cc == nch) {
      cc = 0;
      ++g;
    }
  }
};

// GATHER selects how the producers read the input rows:
//   1  Cin is a multiple of 64 and the features are smaller than 4 GiB: the schedule
//      holds byte offsets of the gather rows and the gather is a range-checked
//      buffer load;
//   2  the same with Cin a multiple of 4 only: in the last channel chunk the lanes
//      beyond Cin gather from the padding offset, i.e. zeros;
//   0  anything else: the schedule holds row numbers and the gather uses 64-bit
//      addresses with per-channel masks.
//
// The waves-per-SIMD attribute states the occupancy the workgroup size gives anyway
// (one workgroup per CU), so that the compiler uses the whole register budget.
// NS: MFMA steps (of 4 input channels) per chunk, 16 for chunks of 64 channels.  A layer
// whose input channels do not fill whole chunks of 64 is cut into ceil(Cin / 64) chunks of
// equal width 4 NS instead (200 channels: 4 chunks of 52, 13 steps each, where chunks of 64
// would run 64 steps for 50 steps' worth of channels): MFMA steps, fragment loads, gathers
// and staged-row reads beyond NS are left out.  Half precision always runs whole chunks.
// What conv_fwd_kernel applies to a finished tile instead of storing its sums: per column c
// of the accumulators z = (x - shift[c]) * scale[c] + add[c], then by mode[c]
//   0  y = z                                          2  y = z * act_gate(z_g + pre[g]),
//   1  y = act_scalar(z + pre[c])                        g = gate[c], a column of the same
//   3  nothing is stored (gates, padding)                workgroup's column range
// stored at column dest[c] of rows of c_dest columns.  The gates of a block of 64 columns
// are one run of at most 16 columns (gate_run): act_gate is evaluated once per gate and
// row, not once per gated column.  mode == nullptr: plain store.
struct ConvEpilogue {
  const float *shift, *scale, *add, *pre;  // [cout]
  const int32_t *mode, *gate, *dest;       // [cout]
  const int32_t *gate_run;                 // [2 * blocks of 64 columns]: first gate, gates
  int act_s, act_g, c_dest;
};

template <typename IO, int GATHER, int NCW, int NS, bool EPI, bool TAIL>
__global__ void __launch_bounds__((NCW + 4) * 64)
    __attribute__((amdgpu_waves_per_eu((NCW + 4) / 4, (NCW + 4) / 4)))
    conv_fwd_kernel(const IO *__restrict__ features, int cin, unsigned feat_bytes,
                    const void *__restrict__ packed, unsigned packed_bytes,
                    const int32_t *__restrict__ sched_in, const int32_t *__restrict__ sched_out,
                    const int32_t *__restrict__ grp_meta, unsigned sched_bytes, unsigned meta_bytes,
                    const int32_t *__restrict__ tile_grp, const int32_t *__restrict__ wg_tile,
                    int nch, int ncb, IO *__restrict__ out, int cout, int T, int cols_per_xcd,
                    int col_base, ConvEpilogue epi) {
  constexpr int kCN = 16 * NCW;   // output columns per workgroup
  constexpr int kEB = Io<IO>::kBytes;
  constexpr bool kHalf = kEB == 2;
  constexpr int kRowB = Io<IO>::kRowBytes;    // bytes of a staged row
  constexpr int kFragB = Io<IO>::kFragBytes;  // bytes of a packed filter fragment
  static_assert(NS >= 1 && NS <= 16 && (!kHalf || NS == 16), "steps per chunk");
  static_assert(GATHER != 1 || NS == 16, "the unchecked gather reads whole chunks of 64");
  constexpr int kChunk = kHalf ? kKC : 4 * NS;  // input channels per chunk
  constexpr int kQFull = NS / 4, kQRem = NS % 4;  // whole quarters, steps of the partial one
  typedef typename Io<IO>::Raw Raw;
  constexpr int kAS = kCN + 4;    // accumulator row stride in floats
  constexpr int NT = (NCW + 4) * 64;
  constexpr int NP = 256;  // producer threads
  constexpr int NE = kStage * 16 / NP;
  extern __shared__ __align__(16) float lds[];
  float *acc = lds;
  float *abuf = acc + (size_t)(T + 1) * kAS;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool producer = wave >= NCW;
  // Consecutive workgroup ids land on different XCDs (8 of them, one L2 each): give
  // every XCD a contiguous run of tile ranges so neighbouring tiles, which gather
  // the same input rows, share an L2.  Which column blocks an XCD works on depends on the
  // size of the packed filters.  Small ones (they stay in every L2): all column blocks of
  // a run of ranges, so that the gathered rows are shared as well.  Large ones (an L2
  // holds a fraction of them, and a workgroup walks all of its column block's fragments
  // once per tile): one column block per XCD (cols_per_xcd: XCDs per column block), so that
  // the 32 workgroups of an XCD ask for the same fragments at about the same time and
  // one fetch serves them all.
  int chunk = blockIdx.x, cblk = blockIdx.y;
  {
    const int nwg = gridDim.x;
    if (cols_per_xcd > 0) {
      const int lin = blockIdx.y * nwg + blockIdx.x;  // dispatch order: XCD = lin % 8
      const int xcd = lin & 7, slot = lin >> 3;
      const int ncol = gridDim.y;  // divides 8
      cblk = xcd % ncol;
      chunk = (xcd / ncol) * ((nwg * ncol) >> 3) + slot;
    } else if ((nwg & 7) == 0) {
      chunk = (chunk & 7) * (nwg >> 3) + (chunk >> 3);
    }
  }
  const int t_begin = wg_tile[chunk], t_end = wg_tile[chunk + 1];
  const int g_begin = tile_grp[t_begin], g_end = tile_grp[t_end];
  const int nstages = (g_end - g_begin) * nch;  // stages of this workgroup
  const int col0 = col_base + cblk * kCN;
  static_assert(!TAIL || (NCW == 4 && !kHalf), "the one-column-group form is built for float");

  {
    float4v z = {0.f, 0.f, 0.f, 0.f};
    float4v *a4 = reinterpret_cast<float4v *>(acc);
    for (int i = tid; i < (T + 1) * kAS / 4; i += NT) a4[i] = z;
  }

  // Tile `tl` is complete: write its rows, clear the accumulators.
  // (slot0 = accumulator slot of the tile's first row; slots wrap around at T)
  // Epilogue constants of this thread, loaded once: when a tile is written out a thread
  // keeps its 4 columns (c_t) and walks down the rows; lane l of a row's 16 lanes also
  // owns gate l of the workgroup's column block.
  //   z = x * e_ca + e_cb (e_cb includes the bias in front of a scalar activation);
  //   e_mg = mode | LDS column of the gate << 4;  e_dest = output column
  //   gate l: activated value = act_gate(x * e_gca + e_gcb), LDS column e_gcl (-1: none)
  float e_ca[4], e_cb[4], e_gca = 0.f, e_gcb = 0.f;
  int e_mg[4], e_dest[4], e_gcl = -1;
  bool e_any = false, e_vec = false;
  if constexpr (EPI) {
    const int c_t = (tid % (kCN / 4)) * 4, col = col0 + c_t;
    const bool col_ok = col < cout;
    static_assert(!EPI || kCN == 64, "the epilogue's gate runs are per block of 64 columns");
    const int eblk = col0 / kCN;  // block of 64 columns the workgroup's columns start
    const int gfirst = epi.gate_run[2 * eblk], gcount = min(epi.gate_run[2 * eblk + 1], 16);
    const bool run_ok = gfirst >= col0 && gfirst + gcount <= min(col0 + kCN, cout);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = col_ok ? col + i : 0;
      int mode = col_ok ? epi.mode[c] : 3;
      e_dest[i] = epi.dest[c];
      const int g = epi.gate[c];
      // tables that point outside the output row or outside the block's run of gates
      // switch the column off
      if (e_dest[i] < 0 || e_dest[i] >= epi.c_dest || mode < 0 || mode > 2 ||
          (mode == 2 && (!run_ok || g < gfirst || g >= gfirst + gcount)))
        mode = 3;
      e_mg[i] = mode | ((mode == 2 ? g - col0 : c_t + i) << 4);
      e_ca[i] = epi.scale[c];
      e_cb[i] = epi.add[c] - epi.shift[c] * e_ca[i] + (mode == 1 ? epi.pre[c] : 0.f);
    }
    e_any = (e_mg[0] & 15) != 3 || (e_mg[1] & 15) != 3 || (e_mg[2] & 15) != 3 || (e_mg[3] & 15) != 3;
    e_vec = (e_mg[0] & 15) != 3 && (e_mg[1] & 15) != 3 && (e_mg[2] & 15) != 3 &&
            (e_mg[3] & 15) != 3 && e_dest[1] == e_dest[0] + 1 && e_dest[2] == e_dest[0] + 2 &&
            e_dest[3] == e_dest[0] + 3 && ((e_dest[0] | epi.c_dest) & 3) == 0;
    const int gi = (tid % (kCN / 4));
    if (run_ok && gi < gcount) {
      const int g = gfirst + gi;
      e_gcl = g - col0;
      e_gca = epi.scale[g];
      e_gcb = epi.add[g] - epi.shift[g] * e_gca + epi.pre[g];
    }
  }
  const int e_c_dest = epi.c_dest, e_act_s = epi.act_s, e_act_g = epi.act_g;
  auto flush_tile = [&](int row0, int rows, int slot0) __attribute__((always_inline)) {
    if constexpr (TAIL) {
      // The four consumer waves each hold a partial sum of the one column group, in the
      // 16 columns a wave owns: add them up in the first 16, clear the others, and write
      // the tile out as any other.
      const float4v z = {0.f, 0.f, 0.f, 0.f};
      for (int r = tid >> 2; r < rows; r += NT / 4) {
        int sl = slot0 + r;
        if (sl >= T) sl -= T;
        float4v *ap = reinterpret_cast<float4v *>(acc + sl * kAS + (tid & 3) * 4);
        const float4v v = (ap[0] + ap[4]) + (ap[8] + ap[12]);
        ap[0] = v;
        ap[4] = z;
        ap[8] = z;
        ap[12] = z;
      }
      __syncthreads();
    }
    if constexpr (EPI) {
      // Batch norm constants and gate applied on the way out (cout % 4 == 0).  Threads,
      // columns and rows as in the plain store below.  The 16 lanes of a row sit in one wave
      // and a wave's LDS operations execute in order: first the row's gates are replaced by
      // their activated values (lane l: gate l), then every lane reads its sums and the
      // gates of its columns, then the wave clears the row.
      // FAST: scalar activation none or relu, gate activation none or sigmoid -- a few instructions
      // per element and no branch (a taken branch costs a wave more than the arithmetic of
      // a whole row); the other activations go through act_fn.
      auto rows_out = [&](auto fast_tag) __attribute__((always_inline)) {
        constexpr bool FAST = decltype(fast_tag)::value;
        constexpr int U = 2;
        constexpr int RS = NT / (kCN / 4);
        const int r_t = tid / (kCN / 4), c_t = (tid % (kCN / 4)) * 4;
        const float4v z = {0.f, 0.f, 0.f, 0.f};
        // FAST: max(t, lo) is the scalar activation where there is one, t elsewhere
        float lo[4];
        bool gated[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          lo[i] = ((e_mg[i] & 15) == 1 && e_act_s == SSC_ACT_RELU) ? 0.f : -INFINITY;
          gated[i] = (e_mg[i] & 15) == 2;
        }
        auto gate_act = [&](float x) -> float {
          const float u = x * e_gca + e_gcb;
          if constexpr (FAST)
            return e_act_g == SSC_ACT_SIGMOID ? __builtin_amdgcn_rcpf(1.f + __expf(-u)) : u;
          else
            return act_fn(e_act_g, u);
        };
        float *gp = reinterpret_cast<float *>(out) + (int64_t)(row0 + r_t) * e_c_dest;
        const int64_t gstep = (int64_t)RS * e_c_dest;
        for (int r = r_t; r < rows; r += U * RS) {
          const bool two = r + RS < rows;
          int sl0 = slot0 + r, sl1 = slot0 + r + RS;
          if (sl0 >= T) sl0 -= T;
          if (sl1 >= T) sl1 -= T;
          float *a0 = acc + sl0 * kAS, *a1 = acc + sl1 * kAS;
          if (e_gcl >= 0) {
            const float x0 = a0[e_gcl], x1 = two ? a1[e_gcl] : 0.f;
            a0[e_gcl] = gate_act(x0);
            if (two) a1[e_gcl] = gate_act(x1);
          }
          __builtin_amdgcn_sched_barrier(0);
          float4v v0 = *reinterpret_cast<float4v *>(a0 + c_t), v1 = z, g1 = z;
          float4v g0 = {a0[e_mg[0] >> 4], a0[e_mg[1] >> 4], a0[e_mg[2] >> 4], a0[e_mg[3] >> 4]};
          if (two) {
            v1 = *reinterpret_cast<float4v *>(a1 + c_t);
            g1 = float4v{a1[e_mg[0] >> 4], a1[e_mg[1] >> 4], a1[e_mg[2] >> 4], a1[e_mg[3] >> 4]};
          }
          __builtin_amdgcn_sched_barrier(0);  // the clears stay behind every read above
          *reinterpret_cast<float4v *>(a0 + c_t) = z;
          if (two) *reinterpret_cast<float4v *>(a1 + c_t) = z;
          if (e_any) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
              if (u == 1 && !two) break;
              const float4v v = u == 0 ? v0 : v1, gv = u == 0 ? g0 : g1;
              float4v y;
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const float t = v[i] * e_ca[i] + e_cb[i];
                if constexpr (FAST) {
                  y[i] = fmaxf(t, lo[i]) * (gated[i] ? gv[i] : 1.f);
                } else {  // every form, then select: no divergent branches
                  const float ts = act_fn(e_act_s, t);
                  const int m = e_mg[i] & 15;
                  y[i] = m == 1 ? ts : m == 2 ? t * gv[i] : t;
                }
              }
              float *p = gp + u * gstep;
              if (e_vec) {
                __builtin_nontemporal_store(y, reinterpret_cast<float4v *>(p + e_dest[0]));
              } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                  if ((e_mg[i] & 15) != 3) __builtin_nontemporal_store(y[i], p + e_dest[i]);
              }
            }
          }
          gp += U * gstep;
        }
      };
      if ((e_act_s == SSC_ACT_NONE || e_act_s == SSC_ACT_RELU) &&
          (e_act_g == SSC_ACT_NONE || e_act_g == SSC_ACT_SIGMOID))
        rows_out(std::true_type());
      else
        rows_out(std::false_type());
      return;
    }
    if ((cout & 3) == 0) {
      // A thread keeps its 4 columns and walks down the rows, NT / (kCN / 4) rows per
      // step: addresses advance by constants, so a step is little more than its LDS
      // read, LDS clear and store, and four reads are in flight before the first store
      // (one at a time, every step would pay the full LDS latency while the matrix
      // cores idle).
      const float4v z = {0.f, 0.f, 0.f, 0.f};
      constexpr int U = 4;
      constexpr int RS = NT / (kCN / 4);  // rows per step
      const int r_t = tid / (kCN / 4), c_t = (tid % (kCN / 4)) * 4;
      const bool col_ok = col0 + c_t < cout;
      IO *gp = out + (int64_t)(row0 + r_t) * cout + col0 + c_t;
      const int64_t gstep = (int64_t)RS * cout;
      for (int r = r_t; r < rows; r += U * RS) {
        float4v v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (r + u * RS < rows) {
            int sl = slot0 + r + u * RS;
            if (sl >= T) sl -= T;
            float4v *ap = reinterpret_cast<float4v *>(acc + sl * kAS + c_t);
            v[u] = *ap;
            *ap = z;
          }
#pragma unroll
        for (int u = 0; u < U; ++u)
          // streaming store: the output is not read again by this kernel and must not
          // push the weights and the gathered rows out of L2
          if (r + u * RS < rows && col_ok)
            Io<IO>::store_stream(gp + u * gstep, v[u]);
        gp += U * gstep;
      }
    } else {
      for (int e = tid; e < rows * kCN; e += NT) {
        int r = e / kCN, c = e % kCN;
        int sl = slot0 + r;
        if (sl >= T) sl -= T;
        if (col0 + c < cout)
          __builtin_nontemporal_store((IO)acc[sl * kAS + c], out + (int64_t)(row0 + r) * cout + col0 + c);
        acc[sl * kAS + c] = 0.f;
      }
    }
  };
  // The tile of stage `pos` (first row, rows) ends with it when the group is the
  // tile's last one and the chunk is the last chunk.  Scalar loads: the address is
  // uniform.
  auto tile_end = [&](const StagePos &pos, int &row0, int &rows, int &slot0) -> bool {
    const int32_t *m = grp_meta + (int64_t)pos.g * 8;
    row0 = m[4];
    slot0 = m[6];
    const int r = m[5];
    rows = r < 0 ? -r : r;
    return r > 0 && pos.cc == nch - 1;
  };

  if (producer) {
    // ------------------------------------------------------------------ producer
    const int pt = tid - NCW * 64;
    constexpr int RD = kRowsAhead, ID = kIdxAhead;
    static_assert(RD == 4 && ID == 2, "the rings below are sized for these distances");
    const __amdgpu_buffer_rsrc_t rs_in =
        __builtin_amdgcn_make_buffer_rsrc((void *)sched_in, 0, (int)sched_bytes, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs_feat =
        __builtin_amdgcn_make_buffer_rsrc((void *)features, 0, (int)feat_bytes, kRsrcFlags);
    const int idx_voff = (pt >> 4) * 4;    // this thread's slot (plus 16 slots per element)
    const int piece = pt & 15;                  // this thread's 4 channels of a row chunk
    const int chunk_off = piece * 4 * kEB;
    // the chunk has no such piece (fewer than 16 steps), or, in the last chunk, the piece
    // lies beyond Cin
    const bool no_piece = !kHalf && piece >= NS;
    const bool beyond_cin = (nch - 1) * kChunk + piece * 4 >= cin;
    // a piece of the partly used quarter is staged one channel per lane group
    const bool spread = !kHalf && kQRem != 0 && piece >= 4 * kQFull && piece < NS;
    typedef Raw Held;
    int idx[ID][NE];
    Held rows[RD][NE];
    // Rings indexed by stage number: rows of stage st in rows[st & 3], gather offsets
    // in idx[st & 1].  The loop is unrolled four times so that every ring index is a
    // compile-time constant: rotating a ring through register moves would read
    // registers that loads are still writing, and so wait for those loads one
    // iteration after their issue.
    auto load_idx = [&](const StagePos &pos, int s, int (&ix)[NE]) {
#pragma unroll
      for (int j = 0; j < NE; ++j) {
        int v = buf_load1(rs_in, idx_voff + j * 64, pos.g * 256);
        if (GATHER == 0) v = s < nstages ? v : -1;  // the pointer gather is not range-checked
        ix[j] = v;
      }
    };
    auto load_rows = [&](const StagePos &pos, const int (&ix)[NE], Held (&r)[NE]) {
#pragma unroll
      for (int j = 0; j < NE; ++j) {
        if constexpr (GATHER == 1) {
          r[j] = Io<IO>::gather(rs_feat, ix[j] + chunk_off, pos.cc * (kChunk * kEB));
        } else if constexpr (GATHER == 2) {
          const int off =
              (no_piece || (pos.cc == nch - 1 && beyond_cin)) ? (int)kGatherPad : ix[j];
          r[j] = Io<IO>::gather(rs_feat, off + chunk_off, pos.cc * (kChunk * kEB));
        } else {
          const int ch = pos.cc * kChunk + piece * 4;
          const int row = ix[j] < 0 ? 0 : ix[j];  // padding slots read row 0 and drop it
          const IO *fp = features + (int64_t)row * cin + ch;
          Held v = Io<IO>::zero();
          if ((cin & 3) == 0) {
            if (ch < cin) v = Io<IO>::load(fp);
          } else {  // rows are not aligned: one element at a time
            v = Io<IO>::load_first(fp, cin - ch);
          }
          if (ix[j] < 0 || no_piece) v = Io<IO>::zero();
          r[j] = v;
        }
      }
    };
    // where this thread's piece goes in a staged row: its own 16 bytes, or, for a piece of
    // the partly used quarter, element (piece - 4 kQFull) of each lane group's 16 bytes
    char *const st_base = reinterpret_cast<char *>(abuf) + (pt >> 4) * kRowB +
                          (spread ? (16 * kQFull + (piece - 4 * kQFull)) * kEB : piece * 4 * kEB);
    auto store_rows = [&](int parity, const Held (&r)[NE]) {
#pragma unroll
      for (int j = 0; j < NE; ++j) {
        char *dst = st_base + (parity * kStage + j * 16) * kRowB;
        if constexpr (!kHalf && kQRem != 0) {
          if (spread) {
            const float4v v = __builtin_bit_cast(float4v, r[j]);
            reinterpret_cast<float *>(dst)[0] = v.x;
            reinterpret_cast<float *>(dst)[4] = v.y;
            reinterpret_cast<float *>(dst)[8] = v.z;
            reinterpret_cast<float *>(dst)[12] = v.w;
            continue;
          }
        }
        if (!no_piece) *reinterpret_cast<Held *>(dst) = r[j];
      }
    };
    // Prologue.  Loads are issued in the order the loop will wait for them (offsets,
    // then rows, oldest stage first): the wait counts of the loop are static, so
    // they must also be right on its first trip.
    StagePos p_rows = {g_begin, 0};  // stage whose rows are loaded next
    StagePos p_idx = {g_begin, 0};   // stage whose gather offsets are loaded next
    StagePos p_cur = {g_begin, 0};   // stage the consumers are working on
    {
      int ix[RD + 1][NE];
#pragma unroll
      for (int j = 0; j <= RD; ++j) {
        load_idx(p_idx, j, ix[j]);
        p_idx.advance(nch);
      }
#pragma unroll
      for (int j = 1; j <= ID; ++j) {
        load_idx(p_idx, RD + j, idx[(RD + j) & 1]);
        p_idx.advance(nch);
      }
      Held r0[NE];
      load_rows(p_rows, ix[0], r0);
      p_rows.advance(nch);
#pragma unroll
      for (int j = 1; j <= RD; ++j) {
        load_rows(p_rows, ix[j], rows[j & 3]);
        p_rows.advance(nch);
      }
      store_rows(0, r0);
    }
    __syncthreads();
    // Iteration s stages the rows of stage s+1 and issues the loads of stages s+5
    // (rows) and s+7 (gather offsets).
    auto iteration = [&](int s, auto phase) {
      constexpr int ph = decltype(phase)::value;  // == s & 3
      int t_row0, t_rows, t_slot0;
      const bool last = tile_end(p_cur, t_row0, t_rows, t_slot0);
      p_cur.advance(nch);
      store_rows((ph + 1) & 1, rows[(ph + 1) & 3]);
      load_rows(p_rows, idx[(ph + 1 + RD) & 1], rows[(ph + 1 + RD) & 3]);
      p_rows.advance(nch);
      load_idx(p_idx, s + 1 + RD + ID, idx[(ph + 1 + RD + ID) & 1]);
      p_idx.advance(nch);
      __syncthreads();
      if (last) {
        flush_tile(t_row0, t_rows, t_slot0);
        __syncthreads();
      }
    };
    // Whole groups of four stages first, the remainder after the loop: an early exit
    // from the middle of the unrolled body would share the loop's back edge, and the
    // static wait counts at the top of the body would then have to allow for a trip
    // that follows a shorter one.
    int s = 0;
    for (; s + 4 <= nstages; s += 4) {
      iteration(s, std::integral_constant<int, 0>());
      iteration(s + 1, std::integral_constant<int, 1>());
      iteration(s + 2, std::integral_constant<int, 2>());
      iteration(s + 3, std::integral_constant<int, 3>());
    }
    if (s < nstages) iteration(s, std::integral_constant<int, 0>());
    if (s + 1 < nstages) iteration(s + 1, std::integral_constant<int, 1>());
    if (s + 2 < nstages) iteration(s + 2, std::integral_constant<int, 2>());
  } else {
    // ------------------------------------------------------------------ consumer
    const int g = lane >> 4;
    const int l16 = lane & 15;
    // A column group beyond Cout multiplies with the last real one's fragments; its
    // accumulator columns are never written out.
    // (The one-column-group form: every wave multiplies with the fragments of that group.)
    const int cb = TAIL ? col_base / 16 : min(col0 / 16 + wave, ncb - 1);
    const __amdgpu_buffer_rsrc_t rs_w =
        __builtin_amdgcn_make_buffer_rsrc((void *)packed, 0, (int)packed_bytes, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs_out =
        __builtin_amdgcn_make_buffer_rsrc((void *)sched_out, 0, (int)sched_bytes, kRsrcFlags);
    // 16-byte pieces of operands a lane handles per row block: weight fragment loads, and
    // as many reads of its staged row (float: 4 MFMA steps of 4 channels each, a quarter
    // of the chunk; half: one MFMA step of 32 channels, lane group g has 8 of them)
    constexpr int NF = kHalf ? 2 : (NS + 3) / 4;
    typedef std::conditional_t<kHalf, int4v, float4v> Frag;
    const int w_voff = lane * 16;  // this lane's 16 bytes of a KiB of fragments
    constexpr int kWStep = 1024;   // from one 16-byte piece to the next
    const int w_soff0 = cb * nch * kFragB;  // fragments of this wave's column block
    const char *const a_base = reinterpret_cast<const char *>(abuf) + l16 * kRowB + g * 16;
    // The accumulators are addressed with 32-bit LDS byte addresses (acc_lane includes
    // the base of acc): no pointer arithmetic left for the vector ALU.
    typedef __attribute__((address_space(3))) float4v lds_float4v;
    const int acc_base = (int)(size_t)(__attribute__((address_space(3))) char *)acc;
    auto lds_load4 = [](int addr) -> float4v { return *(lds_float4v *)(size_t)addr; };
    auto lds_store4 = [](int addr, const float4v &v) { *(lds_float4v *)(size_t)addr = v; };

    const __amdgpu_buffer_rsrc_t rs_meta =
        __builtin_amdgcn_make_buffer_rsrc((void *)grp_meta, 0, (int)meta_bytes, kRsrcFlags);
    // Per-lane state of the consumer pipeline.  Row blocks are numbered through the
    // stages (block 4s+m is block m of stage s); rings are indexed with the block or
    // stage number, and the loop is unrolled over two stages so that every ring index
    // is a compile-time constant.
    //   w[b & 3][q]   weight fragments of block b (four 16-byte loads), fetched three
    //                 blocks ahead: while block b multiplies, the slot of block b-1 is
    //                 refilled for block b+3
    //   orow[b & 3]   LDS byte offset of the accumulator row of this lane's pair in block b
    //   rec[s & 1]    the schedule record (offsets of the 4 blocks, rows of the tile)
    //                 of stage s, the same in every lane.  It travels through vector
    //                 loads and v_readfirstlane rather than scalar loads: scalar loads
    //                 return out of order, and one in flight would turn every partial
    //                 wait for LDS data below into a wait for everything.
    Frag w[4][NF];
    int orow[4];
    int4v rec[2][2];
    // Second half of a record: only its first three words are used.  A 12-byte load:
    // a wider one would still write the unused register when it lands, and whatever
    // the compiler keeps there in the meantime would have to wait for it.
    auto load_rec_tail = [&](const StagePos &pos) -> int4v {
      const int3v t = buf_load3(rs_meta, 16, pos.g * 32);
      return int4v{t.x, t.y, t.z, 0};
    };
    // First row and rows of the tile of a stage, and whether the tile ends with the
    // stage, from the second half of its record.
    struct TileEnd {
      int row0, rows, slot0;
      bool last;
    };
    auto tile_end_of = [&](const int4v &tail, const StagePos &pos) -> TileEnd {
      TileEnd e;
      e.row0 = __builtin_amdgcn_readfirstlane(tail.x);
      const int r = __builtin_amdgcn_readfirstlane(tail.y);
      e.rows = r < 0 ? -r : r;
      e.slot0 = __builtin_amdgcn_readfirstlane(tail.z);
      e.last = r > 0 && pos.cc == nch - 1;
      return e;
    };
    auto load_rec = [&](const StagePos &pos, int4v (&r)[2]) {
      r[0] = __builtin_bit_cast(int4v, buf_load4(rs_meta, 0, pos.g * 32));
      r[1] = load_rec_tail(pos);
    };
    // Byte offset of the weight fragments of a block: the offset's part comes from the
    // schedule record (0 for empty blocks and, the loads being range-checked, for
    // records beyond the schedule), `base` is the part of this wave and channel chunk.
    auto frag_soff = [&](int rec_lane, int base) -> int {
      return __builtin_amdgcn_readfirstlane(rec_lane) + base;
    };
    auto rec_k = [](const int4v &v, int b) -> int {
      return b == 0 ? v.x : b == 1 ? v.y : b == 2 ? v.z : v.w;
    };
    auto fetch_w = [&](int soff, int slot, int q) {
      if constexpr (!kHalf && kQRem != 0) {
        if (q == kQFull) {  // the partly used quarter: kQRem floats per lane, densely packed
          const int voff = kQFull * kWStep + lane * (4 * kQRem);
          // The wider loads are cast to float vectors as a whole: with per-element casts
          // of an integer vector this compiler shrinks the load to its first element.
          if constexpr (kQRem == 1) {
            w[slot][q].x = __builtin_bit_cast(float, buf_load1(rs_w, voff, soff));
          } else if constexpr (kQRem == 2) {
            const float2v t = __builtin_bit_cast(
                float2v, __builtin_amdgcn_raw_buffer_load_b64(rs_w, voff, soff, 0));
            w[slot][q].x = t.x;
            w[slot][q].y = t.y;
          } else {
            const float3v t = __builtin_bit_cast(
                float3v, __builtin_amdgcn_raw_buffer_load_b96(rs_w, voff, soff, 0));
            w[slot][q].x = t.x;
            w[slot][q].y = t.y;
            w[slot][q].z = t.z;
          }
          return;
        }
      }
      w[slot][q] = __builtin_bit_cast(Frag, buf_load4(rs_w, w_voff + q * kWStep, soff));
    };
    auto fetch_orow = [&](const StagePos &pos, int m, int slot) {
      orow[slot] = buf_load1(rs_out, l16 * 4 + m * 64, pos.g * 256);
    };
    // An accumulator update whose write is still to come: row address, the row as it
    // was read, and the product to add.
    struct Pending {
      int addr;
      float4v accr, d;
    };
    // LDS address of this lane's 4 columns in accumulator row 0
    const int acc_lane = acc_base + (wave * 16 + g * 4) * 4;
    const int dummy_addr = T * kAS * 4 + acc_lane;
    if constexpr (TAIL) {
      // One column group for four consumer waves: wave m multiplies row block m of every
      // group and keeps its products in the 16 accumulator columns it owns (a partial sum
      // of the group's columns over the pairs of its blocks; flush_tile adds the four up).
      // A stage is 1 row block of NS MFMAs per wave instead of 4; the products of a group's
      // chunks stay in registers and reach the accumulators once per group.
      // Rings indexed by stage number (the loop is unrolled over four stages):
      //   w[s & 3]     fragments of stage s, fetched three stages ahead
      //   kof[s & 3]   fragment offset of the block's kernel offset, loaded seven stages
      //                ahead (four before the fetch that needs it)
      //   orow[s & 3]  accumulator row of this lane's pair, tl[s & 3] the tile of the stage:
      //                loaded four stages ahead, into the slot the stage before just used
      int kof[4];
      int4v tl[4];
      const char *const ab_wave = a_base + wave * 16 * kRowB;
      auto load_kof = [&](const StagePos &pos) -> int {
        return buf_load1(rs_meta, wave * 4, pos.g * 32);
      };
      StagePos p_cur = {g_begin, 0};  // stage being multiplied
      StagePos p_f = {g_begin, 0};    // stage whose fragments are fetched next
      StagePos p_k = {g_begin, 0};    // stage whose fragment offset is loaded next
      StagePos p_m = {g_begin, 0};    // stage whose accumulator rows and tile are loaded next
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        kof[j] = load_kof(p_k);
        p_k.advance(nch);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        fetch_orow(p_m, wave, j);
        tl[j] = load_rec_tail(p_m);
        p_m.advance(nch);
      }
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const int soff = frag_soff(kof[j], w_soff0 + p_f.cc * kFragB);
#pragma unroll
        for (int q = 0; q < NF; ++q) fetch_w(soff, j, q);
        p_f.advance(nch);
        kof[j] = load_kof(p_k);
        p_k.advance(nch);
      }
      float4v d = float4v{0.f, 0.f, 0.f, 0.f};
      __syncthreads();
      auto stage = [&](auto phase) {
        constexpr int ph = decltype(phase)::value;  // == stage number & 3
        constexpr int nx = (ph + 3) & 3;
        {
          const int soff = frag_soff(kof[nx], w_soff0 + p_f.cc * kFragB);
#pragma unroll
          for (int q = 0; q < NF; ++q) fetch_w(soff, nx, q);
          p_f.advance(nch);
          kof[nx] = load_kof(p_k);
          p_k.advance(nch);
        }
        const char *ab = ab_wave + (ph & 1) * kStage * kRowB;
        Frag a[NF];
#pragma unroll
        for (int q = 0; q < NF; ++q) a[q] = *reinterpret_cast<const Frag *>(ab + q * 64);
        const bool commit = p_cur.cc == nch - 1;  // the group's last chunk
        const int addr = commit ? orow[ph] + acc_lane : dummy_addr;
        const float4v accr = lds_load4(addr);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < NS; ++i)
          d = __builtin_amdgcn_mfma_f32_16x16x4f32(w[ph][i >> 2][i & 3], a[i >> 2][i & 3], d, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        const TileEnd e = tile_end_of(tl[ph], p_cur);
        if (commit) {
          lds_store4(addr, accr + d);
          d = float4v{0.f, 0.f, 0.f, 0.f};
        }
        fetch_orow(p_m, wave, ph);
        tl[ph] = load_rec_tail(p_m);
        p_m.advance(nch);
        p_cur.advance(nch);
        __syncthreads();
        if (e.last) {
          flush_tile(e.row0, e.rows, e.slot0);
          __syncthreads();
        }
      };
      // whole groups of four stages first, the remainder after the loop (see the producers)
      int s = 0;
      for (; s + 4 <= nstages; s += 4) {
        stage(std::integral_constant<int, 0>());
        stage(std::integral_constant<int, 1>());
        stage(std::integral_constant<int, 2>());
        stage(std::integral_constant<int, 3>());
      }
      if (s < nstages) stage(std::integral_constant<int, 0>());
      if (s + 1 < nstages) stage(std::integral_constant<int, 1>());
      if (s + 2 < nstages) stage(std::integral_constant<int, 2>());
    } else {
    Pending pend;  // nothing pending yet: the first write adds zero to the dummy row
    pend.addr = dummy_addr;
    pend.accr = float4v{0.f, 0.f, 0.f, 0.f};
    pend.d = float4v{0.f, 0.f, 0.f, 0.f};
    // One stage = 4 row blocks of 16 MFMAs each, software-pipelined by hand.  A wave
    // issues at most one instruction every few cycles, and a dependent MFMA can only
    // issue when its predecessor is through the pipeline, so between two MFMAs of a
    // chain a handful of other instructions issue for free -- and no more than that:
    // everything else a block needs is therefore spread, one small piece per gap,
    // over the 16 gaps of the block, and scheduling barriers pin it there:
    // (gap numbers for NS = 16, i.e. 16 MFMAs a block)
    //   gap 2      fragment offset of block b+3 (from the schedule record); accumulator
    //              update of the previous block: add, write; once per stage, tile and
    //              last-of-tile of the next stage
    //   gap 3      accumulator read of this block (LDS operations of a wave execute
    //              in order, so it sees the write of gap 2 when both blocks touch
    //              the same output row)
    //   gaps 4,7,9,12  the four fragment loads of block b+3 (the slot of block b-1)
    //   gap 5      output rows of block b+3
    //   gaps 6,8,10,11  the staged rows of block m+1
    //   gaps 13,14 once per stage: the record of the stage after the next
    // The update of a stage's last block waits, across the barrier, for the first
    // block of the next stage, unless the tile ends here.
    //   cur / next / after: positions of this stage and the two that follow;
    //   returns the tile rows and last-of-tile of the NEXT stage.
    auto run_stage = [&](auto parity, bool last_cur, const StagePos &cur, const StagePos &next,
                         const StagePos &after, TileEnd &end_next) {
      constexpr int par = decltype(parity)::value;
      const char *ab = a_base + par * kStage * kRowB;
      const int base_cur = w_soff0 + cur.cc * kFragB;
      const int base_next = w_soff0 + next.cc * kFragB;
      Frag a[2][NF];
      auto load_a = [&](int m, int q, Frag (&av)[NF]) {
        av[q] = *reinterpret_cast<const Frag *>(ab + m * 16 * kRowB + q * 64);
      };
#pragma unroll
      for (int q = 0; q < NF; ++q) load_a(0, q, a[0]);
      // gaps of the pieces of a block (see above); with fewer than 16 MFMAs they move
      // closer together, in the same order
      // half: two MFMAs a block, so the pieces sit behind the first or the second
      constexpr int kSteps = kHalf ? 2 : NS;
      constexpr bool kFull = !kHalf && NS == 16;
      // no piece may be placed behind the last MFMA
      constexpr int kLast = kSteps - 1;
      auto at = [](int gap) constexpr { return gap < (kHalf ? 1 : NS - 1) ? gap : (kHalf ? 1 : NS - 1); };
      constexpr int kGapAlu = kHalf ? 0 : kFull ? 2 : at(1), kGapAcc = kHalf ? 0 : at(kGapAlu + 1);
      constexpr int kGapW[4] = {kHalf ? 0 : kFull ? 4 : at(2), kHalf ? 1 : kFull ? 7 : at(3),
                                kFull ? 9 : at(4), at(12)};
      constexpr int kGapRow = kHalf ? 0 : kFull ? 5 : at(2);  // after fragment load 0 in the same gap
      constexpr int kGapA[4] = {kHalf ? 1 : kFull ? 6 : at(kSteps / 2),
                                kHalf ? 1 : kFull ? 8 : at(kSteps / 2 + 1),
                                kFull ? 10 : at(kSteps / 2 + 2), at(11)};
      constexpr int kGapRec0 = kHalf ? 1 : kFull ? 13 : (kSteps >= 2 ? kSteps - 2 : 0);
      constexpr int kGapRec1 = kHalf ? 1 : kFull ? 14 : kLast;
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const int slot = m;                 // == (4 * s + m) & 3
        const int tslot = (m + 3) & 3;      // slot of block b+3 == slot of block b-1
        const int tm = (m + 3) & 3;         // index of block b+3 inside its stage
        const bool tnext = m > 0;           // block b+3 belongs to the next stage
        float4v d = float4v{0.f, 0.f, 0.f, 0.f};
        int soff = 0;
#pragma unroll
        for (int i = 0; i < kSteps; ++i) {
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (kHalf) {
            d = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8v, w[slot][i]),
                                                       __builtin_bit_cast(half8v, a[m & 1][i]), d,
                                                       0, 0, 0);
          } else {
            const int q = i >> 2, j = i & 3;
            d = __builtin_amdgcn_mfma_f32_16x16x4f32(w[slot][q][j], a[m & 1][q][j], d, 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
          // all vector-ALU work of the block in one gap: a vector-ALU instruction
          // next to the matrix chain costs about ten cycles for leaving and re-entering
          // the chain, whatever follows it in the same gap is cheap
          if (i == kGapAlu) {
            soff = tnext ? frag_soff(rec_k(rec[par ^ 1][0], tm), base_next)
                         : frag_soff(rec_k(rec[par][0], tm), base_cur);
            if (m == 3) end_next = tile_end_of(rec[par ^ 1][1], next);
            // pend.d = out[pair l16][channels 4g .. 4g+3] of the previous block
            lds_store4(pend.addr, pend.accr + pend.d);
            pend.addr = orow[slot] + acc_lane;
          }
          if (i == kGapAcc) pend.accr = lds_load4(pend.addr);
          if (i == kGapW[0]) fetch_w(soff, tslot, 0);
          if (i == kGapRow) fetch_orow(tnext ? next : cur, tm, tslot);
#pragma unroll
          for (int qq = 1; qq < NF; ++qq)
            if (i == kGapW[qq]) fetch_w(soff, tslot, qq);
          if (m < 3) {
#pragma unroll
            for (int qq = 0; qq < NF; ++qq)
              if (i == kGapA[qq]) load_a(m + 1, qq, a[(m + 1) & 1]);
          }
          // this stage's record was last used by block 0: refill it for the stage
          // after the next
          if (m == 1 && i == kGapRec0)
            rec[par][0] = __builtin_bit_cast(int4v, buf_load4(rs_meta, 0, after.g * 32));
          if (m == 1 && i == kGapRec1) rec[par][1] = load_rec_tail(after);
        }
        __builtin_amdgcn_sched_barrier(0);
        pend.d = d;
      }
      __builtin_amdgcn_sched_barrier(0);
      if (last_cur) {  // the tile is written out after this stage: finish its last update
        lds_store4(pend.addr, pend.accr + pend.d);
        pend.addr = dummy_addr;
      }
    };
    StagePos p_cur = {g_begin, 0};    // stage being multiplied
    StagePos p_next = {g_begin, 0};   // the stage after it
    StagePos p_after = {g_begin, 0};  // and the one after that
    p_next.advance(nch);
    p_after.advance(nch);
    p_after.advance(nch);
    TileEnd end, end_next;
    {
      // what the first stage needs before it starts: its record and the next one,
      // fragments and rows of its blocks 0..2
      load_rec(p_cur, rec[0]);
      load_rec(p_next, rec[1]);
      end = tile_end_of(rec[0][1], p_cur);
      // Loads are issued in the order of the loop (fragment 0, the output rows, the other
      // fragments, block after block) and pinned there: the wait counts of the
      // loop are static and must hold on its first trip as well, so a load that the
      // prologue issued late would make every trip wait for nearly all loads in flight.
#pragma unroll
      for (int b = 0; b < 3; ++b) {
        const int soff = frag_soff(rec_k(rec[0][0], b), w_soff0 + p_cur.cc * kFragB);
        __builtin_amdgcn_sched_barrier(0);
        fetch_w(soff, b, 0);
        __builtin_amdgcn_sched_barrier(0);
        fetch_orow(p_cur, b, b);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int q = 1; q < NF; ++q) {
          fetch_w(soff, b, q);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    __syncthreads();
    auto step = [&](auto parity) {
      run_stage(parity, end.last, p_cur, p_next, p_after, end_next);
      p_cur.advance(nch);
      p_next.advance(nch);
      p_after.advance(nch);
      __syncthreads();
      if (end.last) {
        flush_tile(end.row0, end.rows, end.slot0);
        __syncthreads();
      }
      end = end_next;
    };
    // pairs of stages first, an odd last stage after the loop (see the producer's loop)
    int s = 0;
    for (; s + 2 <= nstages; s += 2) {
      step(std::integral_constant<int, 0>());
      step(std::integral_constant<int, 1>());
    }
    if (s < nstages) step(std::integral_constant<int, 0>());
    }
  }
}

struct ConvPlan {
  int ncb, nch, T, ncw, n_wg, n_colblk;  // T: rows of the accumulator window
  int tile_rows;                         // largest tile height
  int gather;  // conv_fwd_kernel's GATHER
  int ns;      // conv_fwd_kernel's NS: MFMA steps per chunk
  int64_t n_tiles, n_fine, words_per_k, grp_cap;  // n_tiles: upper bound
  size_t lds_bytes;
  // Launches.  As a rule one, over all column blocks (n_colblk of them side by side, the
  // CUs shared out among them).  A last column group that would be alone in its block of
  // four (Cout = 72: 5 groups) behind at most two full blocks gets no column block, where
  // three of four consumer waves would multiply for nothing: the full blocks take one launch
  // each over all CUs (n_launch of them, n_colblk = 1) and the kernel's one-column-group
  // form a last one (has_tail), all over the same plan.
  int n_launch;
  bool has_tail;
};

static size_t conv_lds_bytes(int T, int ncw) {
  return ((size_t)(T + 1) * (16 * ncw + 4) + 2 * (size_t)kStage * kAStride) * 4;
}

static int pick_tile(int ncw) {
  // One workgroup per CU: (almost) all of the 160 KB of LDS goes to the accumulators.
  size_t budget = 160 * 1024 - conv_lds_bytes(0, ncw) - 512;
  int t = (int)(budget / ((size_t)(16 * ncw + 4) * 4));
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
static bool g_conv_by_column = true;  // one column block per XCD for large filters
static bool g_conv_tail = true;       // a launch of its own for a lone last column group

// The sizes that follow from the number of workgroups per column block.
static void plan_split(ConvPlan &p, int n_wg, int64_t n_out, int K, int64_t pair_stride) {
  p.n_wg = n_wg;
  // upper bound of the tile count: every workgroup's range ends with a partial tile
  p.n_tiles = ceil_div(n_out > 0 ? n_out : 1, p.tile_rows) + n_wg;
  p.n_fine = ceil_div(n_out > 0 ? n_out : 1, kSplitGranule);
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
  p.T = pick_tile(p.ncw);
  p.tile_rows = p.T - kSpillRows;
  // the gather can be a range-checked buffer load when rows are multiples of four
  // channels and byte offsets into the features (plus the padding marker) fit 32 bits
  p.gather = 0;
  if ((c_in & 3) == 0 && (uint64_t)n_in * c_in * elem_bytes <= (uint64_t)kGatherPad)
    p.gather = (c_in % kKC) == 0 ? 1 : 2;
  // (wider layers: the launches of one column block each cost more than the lone group
  // in a block of its own does -- 128 -> 256 channels at stride 2 takes 0.255 ms as four
  // launches against 0.185 ms as one, 200 -> 200 with 125 offsets 17.6 against 16.8 ms)
  p.has_tail = g_conv_tail && elem_bytes == 4 && p.ncb % p.ncw == 1 && p.ncb / p.ncw <= 2;
  const int blocks = p.has_tail ? p.ncb / p.ncw : (int)ceil_div(p.ncb, p.ncw);
  p.n_colblk = p.has_tail ? 1 : blocks;
  p.n_launch = p.has_tail ? blocks : 1;
  int n_wg = device_cu_count() / p.n_colblk;
  if (n_wg < 1) n_wg = 1;
  if (n_wg > 256) n_wg = 256;  // the split kernel is one block of 256 threads
  if (n_wg >= 8) n_wg = n_wg / 8 * 8;
  plan_split(p, n_wg, n_out, K, pair_stride);
  p.lds_bytes = conv_lds_bytes(p.T, p.ncw);
  return p;
}

// Device buffers of a convolution call, in three groups with different lifetimes:
//   packed   the filters in MFMA fragment order: as long as the filters keep their values;
//   plan     what the convolution kernel reads besides features and filters (the row-block
//            schedule and the tile ranges of the workgroups): as long as the rulebook, the
//            channel counts, the element type and the direction (`inverse`) stay the same;
//   scratch  intermediate tables of the kernels that build the plan: until it is built.
struct ConvWs {
  void *packed;
  // plan
  int32_t *tile_grp, *wg_tile;
  int32_t *sched_in, *sched_out, *grp_meta;
  // scratch
  int32_t *flag;
  int32_t *segs;
  int32_t *sorted;
  uint32_t *bits;
  int32_t *prefix;
  int32_t *tile_loc, *tile_nmb, *kofs, *tile_rng, *range_grp;
  int32_t *fine_segs, *range_row0, *tile_row0, *n_tiles_dev;
  int32_t *spill_end, *tile_slot0, *spill, *share_first, *share_cnt;
};

// 4 KiB per fragment for either element type (half fragments use the first half).
static size_t conv_packed_bytes(const ConvPlan &p, int K) {
  return align_up((size_t)K * p.ncb * p.nch * 4096);
}

static size_t conv_plan_walk(void *base, const ConvPlan &p, ConvWs *w) {
  Carver c(base);
  int32_t *tile_grp = c.take<int32_t>((size_t)p.n_tiles + 1);
  int32_t *wg_tile = c.take<int32_t>((size_t)p.n_wg + 1);
  int32_t *sched_in = c.take<int32_t>((size_t)p.grp_cap * 64);
  int32_t *sched_out = c.take<int32_t>((size_t)p.grp_cap * 64);
  int32_t *grp_meta = c.take<int32_t>((size_t)p.grp_cap * 8);
  if (w) {
    w->tile_grp = tile_grp;
    w->wg_tile = wg_tile;
    w->sched_in = sched_in;
    w->sched_out = sched_out;
    w->grp_meta = grp_meta;
  }
  return c.used;
}

static size_t conv_scratch_walk(void *base, const ConvPlan &p, int K, int64_t pair_stride,
                                ConvWs *w) {
  Carver c(base);
  ConvWs t;
  t.flag = c.take<int32_t>(1);
  t.segs = c.take<int32_t>((size_t)(p.n_tiles + 1) * K);
  t.sorted = c.take<int32_t>((size_t)K * 2 * pair_stride);
  t.bits = c.take<uint32_t>((size_t)K * p.words_per_k);
  t.prefix = c.take<int32_t>((size_t)K * p.words_per_k);
  t.tile_loc = c.take<int32_t>((size_t)p.n_tiles);
  t.tile_nmb = c.take<int32_t>((size_t)p.n_tiles);
  t.kofs = c.take<int32_t>((size_t)p.n_tiles * K);
  t.fine_segs = c.take<int32_t>((size_t)(p.n_fine + 1) * K);
  t.range_row0 = c.take<int32_t>((size_t)p.n_wg + 1);
  t.tile_row0 = c.take<int32_t>((size_t)p.n_tiles + 1);
  t.spill_end = c.take<int32_t>((size_t)p.n_tiles + 1);
  t.tile_slot0 = c.take<int32_t>((size_t)p.n_tiles + 1);
  t.spill = c.take<int32_t>((size_t)(p.n_tiles + 1) * K);
  t.share_first = c.take<int32_t>((size_t)p.n_tiles * K);
  t.share_cnt = c.take<int32_t>((size_t)p.n_tiles * K);
  t.n_tiles_dev = c.take<int32_t>(1);
  t.tile_rng = c.take<int32_t>((size_t)p.n_tiles + 1);
  t.range_grp = c.take<int32_t>((size_t)p.n_wg + 1);
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
    w->tile_row0 = t.tile_row0;
    w->spill_end = t.spill_end;
    w->tile_slot0 = t.tile_slot0;
    w->spill = t.spill;
    w->share_first = t.share_first;
    w->share_cnt = t.share_cnt;
    w->n_tiles_dev = t.n_tiles_dev;
    w->tile_rng = t.tile_rng;
    w->range_grp = t.range_grp;
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
  // the workspace does not depend on the number of input rows
  ConvPlan p = make_plan(0, n_out, K, c_in, c_out, pair_stride);
  return conv_ws_walk(nullptr, p, K, pair_stride, nullptr);
}

template <typename IO, int GATHER, int NCW, int NS, bool EPI, bool TAIL>
static int launch_conv(const ConvPlan &p, const ConvWs &w, const IO *features, int64_t n_in,
                       int c_in, int K, IO *out, int c_out, int col_base,
                       const ConvEpilogue &epi, hipStream_t s) {
  static bool attr_set = false;
  if (!attr_set) {
    SSC_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(conv_fwd_kernel<IO, GATHER, NCW, NS, EPI, TAIL>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    attr_set = true;
  }
  const uint64_t packed_bytes = (uint64_t)K * p.ncb * p.nch * Io<IO>::kFragBytes;
  const uint64_t sched_bytes = (uint64_t)p.grp_cap * 256;
  SSC_CHECK(packed_bytes < ((uint64_t)1 << 32) && sched_bytes < ((uint64_t)1 << 32), SSC_ERUNTIME,
            "convolution too large for 32-bit buffer offsets (filters %llu B, schedule %llu B)",
            (unsigned long long)packed_bytes, (unsigned long long)sched_bytes);
  const unsigned feat_bytes = GATHER != 0 ? (unsigned)((uint64_t)n_in * c_in * sizeof(IO)) : 0u;
  SSC_CHECK(p.n_wg >= 1 && p.n_colblk >= 1 && col_base % 16 == 0 &&
                col_base + (p.n_colblk - 1) * 16 * NCW < c_out,
            SSC_ERUNTIME, "convolution launch outside the output columns");
  dim3 grid((unsigned)p.n_wg, (unsigned)p.n_colblk);
  // one column block per XCD when the packed filters are larger than an L2 can keep
  // (4 MiB per XCD) and the grid divides that way (256 -> 256 channels, 7 MiB: 2.44 ->
  // 2.24 ms on the 64^3 benchmark geometry; 128 -> 256 at stride 2, 3.5 MiB, is 5 % slower
  // that way and stays with the row-major mapping)
  const bool by_column = packed_bytes > ((uint64_t)4 << 20) && p.n_colblk > 1 &&
                         8 % p.n_colblk == 0 && (p.n_wg * p.n_colblk) % 8 == 0 &&
                         g_conv_by_column;
  const int cols_per_xcd = by_column ? 8 / p.n_colblk : 0;
  hipLaunchKernelGGL((conv_fwd_kernel<IO, GATHER, NCW, NS, EPI, TAIL>), grid, dim3((NCW + 4) * 64), p.lds_bytes, s, features, c_in,
                     feat_bytes, w.packed, (unsigned)packed_bytes, w.sched_in, w.sched_out,
                     w.grp_meta, (unsigned)sched_bytes, (unsigned)(p.grp_cap * 32), w.tile_grp,
                     w.wg_tile, p.nch, p.ncb, out, c_out, p.T, cols_per_xcd, col_base, epi);
  SSC_LAUNCH_CHECK("conv_fwd");
  return SSC_OK;
}

// The launches of a plan (ConvPlan): the column blocks, all at once or one after the other,
// then the one-column-group form for a lone last group.
template <typename IO, int GATHER, int NS>
static int launch_all(const ConvPlan &p, const ConvWs &w, const IO *features, int64_t n_in,
                      int c_in, int K, IO *out, int c_out, const ConvEpilogue &epi,
                      hipStream_t s) {
  constexpr bool kFloat = sizeof(IO) == 4;
  const bool with_epi = kFloat && epi.mode != nullptr;
  for (int l = 0; l < p.n_launch; ++l) {
    const int col_base = l * p.n_colblk * 16 * p.ncw;
    const int rc = with_epi ? launch_conv<IO, GATHER, 4, NS, kFloat, false>(
                                  p, w, features, n_in, c_in, K, out, c_out, col_base, epi, s)
                            : launch_conv<IO, GATHER, 4, NS, false, false>(
                                  p, w, features, n_in, c_in, K, out, c_out, col_base, epi, s);
    if (rc != SSC_OK) return rc;
  }
  if (p.has_tail) {
    const int col_base = (p.ncb - 1) * 16;
    return with_epi ? launch_conv<IO, GATHER, 4, NS, kFloat, kFloat>(
                          p, w, features, n_in, c_in, K, out, c_out, col_base, epi, s)
                    : launch_conv<IO, GATHER, 4, NS, false, kFloat>(
                          p, w, features, n_in, c_in, K, out, c_out, col_base, epi, s);
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
    for (int i = 0; i < kProfileRing; ++i) {
      SSC_HIP(hipEventCreate(&g_profile_ev[i][0]));
      SSC_HIP(hipEventCreate(&g_profile_ev[i][1]));
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
  return SSC_OK;
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
                           const PackArgs *pack, hipStream_t s) {
  const int plane_g = inverse ? 1 : 0;
  const int plane_s = 1 - plane_g;
  const int64_t packed_n = pack ? (int64_t)K * p.ncb * p.nch * 1024 : 0;
  PackArgs pk = {nullptr, 0, 0, 0, 0, 0, 0, 0, 0, nullptr, 16};
  if (pack) pk = *pack;
  if (!in_order) {  // otherwise the filters are packed beside the first kernel of the split
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
  if (!in_order) {  // otherwise flag[0] is 0: pairs in order
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

  // work split on the fine grid, then the tiles and their segments
  dim3 seg_grid = pair_grid;
  if (in_order) {  // extra rows: pack the filters (if any) and clear flag[0]
    int64_t rows = ceil_div(ceil_div(packed_n > 0 ? packed_n : 1, 256), pair_grid.x);
    seg_grid.y += (unsigned)(rows < 4096 ? rows : 4096);
  }
  hipLaunchKernelGGL(grid_segments_kernel<PACK_IO>, seg_grid, dim3(256), 0, s, w.flag,
                     in_order ? 1 : 0, pairs, w.sorted, pair_stride, plane_s, pair_num, K, p.n_fine,
                     kSplitGranule, w.fine_segs, pk);
  hipLaunchKernelGGL(split_bounds_kernel, dim3((unsigned)ceil_div(p.n_fine + 1, 256)), dim3(256), 0,
                     s, w.fine_segs, K, p.n_fine, n_out, p.tile_rows, p.n_wg, w.range_row0);
  hipLaunchKernelGGL(split_rows_kernel, dim3(1), dim3(256), 0, s, w.range_row0, n_out, p.tile_rows,
                     p.T, p.n_wg, w.wg_tile, w.tile_row0, w.n_tiles_dev, w.spill_end,
                     w.tile_slot0);
  SSC_LAUNCH_CHECK("split");
  int64_t nseg = (p.n_tiles + 1) * K;
  hipLaunchKernelGGL(tile_segments_kernel, dim3((unsigned)ceil_div(nseg, 256)), dim3(256), 0, s,
                     w.flag, pairs, w.sorted, pair_stride, plane_s, pair_num, K, w.n_tiles_dev,
                     w.tile_row0, n_out, w.fine_segs, kSplitGranule, w.spill_end, w.segs, w.spill);
  SSC_LAUNCH_CHECK("tile_segments");
  hipLaunchKernelGGL(range_sched_kernel, dim3((unsigned)p.n_wg), dim3(256), 0, s, w.segs, w.spill,
                     K, w.wg_tile, w.share_first, w.share_cnt, w.kofs, w.tile_nmb, w.tile_loc,
                     w.tile_rng, w.range_grp);
  const int frag_bytes = elem_bytes == 2 ? Io<_Float16>::kFragBytes : Io<float>::kFragBytes;
  hipLaunchKernelGGL(sched_fill_kernel, dim3((unsigned)ceil_div(p.n_tiles * K * 16, 256)),
                     dim3(256), 0, s, w.flag, pairs, w.sorted, pair_stride, plane_g,
                     w.share_first, w.share_cnt, w.kofs, w.tile_nmb, w.tile_loc, w.tile_rng,
                     w.range_grp, p.n_wg, w.tile_grp, K, w.n_tiles_dev, w.tile_row0,
                     w.tile_slot0, p.T,
                     p.gather ? (uint32_t)c_in * (uint32_t)elem_bytes : 1u,
                     p.gather ? kGatherPad : 0xFFFFFFFFu, (16 * p.ncw + 4) * 4,
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
static int conv_planned_epilogue(const float *features, int64_t n_in, int32_t c_in,
                                 const void *packed, size_t packed_bytes, const void *plan,
                                 size_t plan_bytes, int64_t pair_stride, int32_t K, int32_t c_cols,
                                 const ssc_conv_epilogue *e, float *out, int64_t n_out,
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
  ConvPlan p = make_plan(n_in, n_out, K, c_in, c_cols, pair_stride, 4);
  SSC_CHECK(packed_bytes >= conv_packed_bytes(p, K), SSC_EWORKSPACE,
            "buffer of the packed filters too small");
  SSC_CHECK(plan_bytes >= conv_plan_walk(nullptr, p, nullptr), SSC_EWORKSPACE,
            "plan buffer too small");
  ConvWs w = {};
  w.packed = const_cast<void *>(packed);
  conv_plan_walk(const_cast<void *>(plan), p, &w);
  const ConvEpilogue epi = {e->shift, e->scale, e->add, e->pre_bias, e->mode, e->gate, e->dest,
                            e->gate_run, e->act_scalar, e->act_gate, e->c_dest};
  return conv_run<float>(p, w, features, n_in, c_in, K, out, c_cols, s, epi);
}

extern "C" {

int ssc_conv_run_epilogue_f32(const float *features, int64_t n_in, int32_t c_in,
                              const void *packed, size_t packed_bytes, const void *plan,
                              size_t plan_bytes, int64_t pair_stride, int32_t kernel_volume,
                              int32_t c_cols, const ssc_conv_epilogue *epilogue, float *out,
                              int64_t n_out, ssc_stream_t stream) {
  return conv_planned_epilogue(features, n_in, c_in, packed, packed_bytes, plan, plan_bytes,
                               pair_stride, kernel_volume, c_cols, epilogue, out, n_out,
                               (hipStream_t)stream);
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

size_t ssc_conv_packed_bytes(int32_t kernel_volume, int32_t c_in, int32_t c_out) {
  if (kernel_volume < 1 || c_in < 1 || c_out < 1) return 0;
  return conv_packed_bytes(make_plan(0, 1, kernel_volume, c_in, c_out, 0), kernel_volume);
}

size_t ssc_conv_plan_bytes(int64_t n_out, int32_t kernel_volume, int32_t c_in, int32_t c_out,
                           int64_t pair_stride) {
  if (n_out < 0 || kernel_volume < 1 || c_in < 1 || c_out < 1 || pair_stride < 0) return 0;
  return conv_plan_walk(nullptr, make_plan(0, n_out, kernel_volume, c_in, c_out, pair_stride),
                        nullptr);
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

int ssc_kernel_combine_packed_f32(const float *weight, const float *basis,
                                  const int32_t *chan_out, const int32_t *chan_in,
                                  const int32_t *blocks, int32_t n_irreps_in,
                                  int32_t kernel_volume, int32_t c_in, int32_t c_out, float *out,
                                  void *packed, size_t packed_bytes, ssc_stream_t stream) {
  const int K = kernel_volume;
  int rc = conv_check_sizes(K, c_in, c_out, 0, 0, 0);
  if (rc != SSC_OK) return rc;
  SSC_CHECK(weight && basis && chan_out && chan_in && blocks && out && packed, SSC_EINVAL,
            "NULL pointer argument");
  SSC_CHECK(n_irreps_in >= 1, SSC_EINVAL, "sizes must be positive");
  const ConvPlan p = make_plan(0, 1, K, c_in, c_out, 0, 4);
  SSC_CHECK(packed_bytes >= conv_packed_bytes(p, K), SSC_EWORKSPACE,
            "buffer of the packed filters too small");
  const PackArgs pk = {nullptr, 0, 0, 0, K, c_in, c_out, p.ncb, p.nch, packed, p.ns};
  const int64_t n = (int64_t)K * p.ncb * p.nch * 1024;
  hipLaunchKernelGGL(combine_pack_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0,
                     (hipStream_t)stream, pk, weight, basis, chan_out, chan_in, blocks,
                     (int)n_irreps_in, out);
  SSC_LAUNCH_CHECK("combine_pack");
  return SSC_OK;
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
