// Sparse convolution forward as an output-stationary implicit GEMM on fp32 MFMA.
//
// Outputs are cut into tiles of T consecutive rows.  A workgroup owns one tile
// and CN output columns; its accumulators [T, CN] live in LDS for the whole
// kernel.  For every kernel offset k the pairs that land in the tile form one
// contiguous segment of the rulebook (pairs of an offset are ascending in
// output row), so they are packed 16 at a time into the M side of
// v_mfma_f32_16x16x4_f32: the gathered input rows are staged in LDS, the
// matching 16x16 weight fragments stay in registers, and the product is added
// to the LDS accumulators at the pairs' output rows.  Only occupied
// (row, offset) slots cost MFMA work, and because each wave owns a fixed set
// of columns and walks the offsets in ascending order the result is
// bit-reproducible without atomics.
#include "ssc_common.h"

namespace ssc {

typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kKC = 64;       // input channels per chunk = 16 MFMA steps of 4
constexpr int kStage = 64;    // pairs staged per barrier = 4 row blocks of 16
constexpr int kAStride = 68;  // floats per staged row (64 + 4: 16-byte aligned, bank spread)
constexpr int kMinTile = 64;

// ---- weight packing ---------------------------------------------------------------------
// packed[((k*NCB + ncb)*NCH + cc)*1024 + lane*16 + c] =
//     W[k][cc*64 + (lane/16)*16 + c][ncb*16 + lane%16]           (0 outside Cin/Cout)
// i.e. the B fragment of MFMA step c of chunk cc for column block ncb, laid
// out so that one wave reads it as four coalesced 16-byte loads per lane.
__global__ void __launch_bounds__(256)
    pack_filters_kernel(const float *__restrict__ w, int64_t fs_k, int64_t fs_ci, int64_t fs_co,
                        int K, int cin, int cout, int ncb, int nch, float *__restrict__ packed) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)K * ncb * nch * 1024;
  if (idx >= total) return;
  int c = idx & 15;
  int lane = (idx >> 4) & 63;
  int64_t r = idx >> 10;
  int cc = r % nch;
  r /= nch;
  int cb = r % ncb;
  int k = (int)(r / ncb);
  int ci = cc * kKC + (lane >> 4) * 16 + c;
  int co = cb * 16 + (lane & 15);
  float v = 0.f;
  if (ci < cin && co < cout) v = w[k * fs_k + ci * fs_ci + co * fs_co];
  packed[idx] = v;
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

// segs[t*K + k] = first pair of offset k whose scatter row is >= t*T  (t = 0..n_tiles).
__global__ void __launch_bounds__(256)
    tile_segments_kernel(const int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                         const int32_t *__restrict__ sorted, int64_t pair_stride, int plane_s,
                         const int32_t *__restrict__ pair_num, int K, int64_t n_tiles, int T,
                         int32_t *__restrict__ segs) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (n_tiles + 1) * K) return;
  int64_t t = idx / K;
  int k = (int)(idx - t * K);
  const int32_t *src = flag[0] ? sorted : pairs;
  const int32_t *s = src + ((int64_t)k * 2 + plane_s) * pair_stride;
  int64_t target = t * (int64_t)T;
  int lo = 0, hi = pair_num[k];
  while (lo < hi) {
    int mid = (lo + hi) >> 1;
    if (s[mid] < target) lo = mid + 1;
    else hi = mid;
  }
  segs[idx] = lo;
}

// ---- row-block schedule -----------------------------------------------------------------
// The pairs that land in a tile are cut, offset by offset, into row blocks of 16
// (the M side of one MFMA); the last block of an offset is padded.  The schedule
// lists, tile after tile and offset-major inside a tile, for every row block its
// offset k, its 16 gather rows (-1 = padding) and its 16 tile-local output rows
// (T = a dummy accumulator row for padding).  The convolution kernel then
// streams through it without any per-offset bookkeeping.
__global__ void __launch_bounds__(256)
    sched_count_kernel(const int32_t *__restrict__ segs, int K, int64_t n_tiles,
                       int32_t *__restrict__ tile_cnt, int32_t *__restrict__ kofs) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n_tiles) return;
  int run = 0;
  for (int k = 0; k < K; ++k) {
    int n = segs[(t + 1) * K + k] - segs[t * K + k];
    kofs[t * K + k] = run;
    run += (n + 15) >> 4;
  }
  tile_cnt[t] = run;
}

// tile_mb[0..n_tiles]: exclusive prefix of tile_cnt (one block).
__global__ void __launch_bounds__(kScanThreads)
    sched_scan_kernel(const int32_t *__restrict__ tile_cnt, int64_t n_tiles,
                      int32_t *__restrict__ tile_mb) {
  __shared__ int lds[kScanThreads / 64 + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int carry = 0;
  for (int64_t base = 0; base < n_tiles; base += kScanThreads) {
    int64_t i = base + threadIdx.x;
    int v = i < n_tiles ? tile_cnt[i] : 0;
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
    if (i < n_tiles) tile_mb[i] = carry + wave_off + incl - v;
    carry += tot;
  }
  if (threadIdx.x == 0) tile_mb[n_tiles] = carry;
}

// 16 threads per (tile, offset): lane i fills slot i of each of its row blocks.
__global__ void __launch_bounds__(256)
    sched_fill_kernel(const int32_t *__restrict__ flag, const int32_t *__restrict__ pairs,
                      const int32_t *__restrict__ sorted, int64_t pair_stride, int plane_g,
                      const int32_t *__restrict__ segs, const int32_t *__restrict__ kofs,
                      const int32_t *__restrict__ tile_mb, int K, int64_t n_tiles, int T,
                      int32_t *__restrict__ sched_in, int32_t *__restrict__ sched_out,
                      int32_t *__restrict__ sched_k) {
  int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t tk = gid >> 4;
  int lane = (int)(gid & 15);
  if (tk >= n_tiles * K) return;
  int64_t t = tk / K;
  int k = (int)(tk - t * K);
  const int32_t *src = flag[0] ? sorted : pairs;
  int s0 = segs[t * K + k];
  int n = segs[(t + 1) * K + k] - s0;
  if (n <= 0) return;
  const int32_t *pg = src + ((int64_t)k * 2 + plane_g) * pair_stride + s0;
  const int32_t *ps = src + ((int64_t)k * 2 + (1 - plane_g)) * pair_stride + s0;
  int64_t mb = (int64_t)tile_mb[t] + kofs[t * K + k];
  int64_t row0 = t * (int64_t)T;
  for (int p = lane; p < ((n + 15) & ~15); p += 16, ++mb) {
    sched_in[mb * 16 + lane] = p < n ? pg[p] : -1;
    sched_out[mb * 16 + lane] = p < n ? (int)(ps[p] - row0) : T;
    if (lane == 0) sched_k[mb] = k;
  }
}

// ---- the convolution --------------------------------------------------------------------
// One workgroup = one tile of T output rows x 64 output columns, 8 waves:
//   waves 0-3  consumers: wave w owns output columns [16w, 16w+16) of the
//              workgroup's column range and does nothing but LDS reads, MFMAs and
//              the accumulator update;
//   waves 4-7  producers: gather the input rows of the NEXT stage from global
//              memory into LDS (rows are prefetched several stages ahead into
//              registers), so that address arithmetic and memory latency run on
//              the same SIMDs underneath the MFMA stream.
// A stage = 4 consecutive row blocks of the schedule (64 pair slots, any mix of
// offsets) x one 64-channel chunk of Cin; one barrier per stage hands a filled
// LDS buffer to the consumers and an emptied one back.
//
// MFMA orientation: D[16 channels x 16 pairs] = W^T[16 x 4] * F^T[4 x 16], so a
// lane ends up with 4 consecutive output channels of one pair and adds them to
// the LDS accumulator row of that pair with one 16-byte read-modify-write.  A
// column group belongs to exactly one wave, which walks the schedule in order,
// so every output element sees its offsets added in ascending k: reproducible,
// no atomics.
//
// Dynamic LDS: acc[T+1][68] | abuf[2][64][68] | orow[4][64] | ids[4][8]
// (output rows and fragment ids of a stage are published two stages ahead, in a
// ring of four, so the consumers know their next stage before its barrier.)
constexpr int kRowsAhead = 3;  // stages whose gathered rows are in flight in registers
constexpr int kIdxAhead = 2;   // further stages whose row indices are in flight

__device__ __forceinline__ void mfma_block(const float4v (&b)[4], const float4v (&a)[4],
                                           float4v &d) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    d = __builtin_amdgcn_mfma_f32_16x16x4f32(b[q].x, a[q].x, d, 0, 0, 0);
    d = __builtin_amdgcn_mfma_f32_16x16x4f32(b[q].y, a[q].y, d, 0, 0, 0);
    d = __builtin_amdgcn_mfma_f32_16x16x4f32(b[q].z, a[q].z, d, 0, 0, 0);
    d = __builtin_amdgcn_mfma_f32_16x16x4f32(b[q].w, a[q].w, d, 0, 0, 0);
  }
}

__global__ void __launch_bounds__(512)
    conv_fwd_kernel(const float *__restrict__ features, int cin, const float *__restrict__ packed,
                    const int32_t *__restrict__ sched_in, const int32_t *__restrict__ sched_out,
                    const int32_t *__restrict__ sched_k, const int32_t *__restrict__ tile_mb,
                    int nch, int ncb, float *__restrict__ out, int64_t n_out, int cout, int T,
                    int64_t n_tiles) {
  constexpr int CN = 64;
  constexpr int AS = CN + 4;
  constexpr int NP = 256;  // producer threads
  constexpr int NE = kStage * 16 / NP;
  extern __shared__ __align__(16) float lds[];
  float *acc = lds;
  float *abuf = acc + (size_t)(T + 1) * AS;
  int *orow = reinterpret_cast<int *>(abuf + 2 * kStage * kAStride);
  int *ids = orow + 4 * kStage;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const bool producer = wave >= 4;
  // Consecutive workgroup ids land on different XCDs (8 of them, one L2 each):
  // give every XCD a contiguous range of tiles so neighbouring tiles, which
  // gather the same input rows, share an L2.
  int64_t tile = blockIdx.x;
  {
    const int64_t per = n_tiles / 8;
    if (tile < per * 8) tile = (tile % 8) * per + tile / 8;
  }
  const int64_t row0 = tile * (int64_t)T;
  const int mb0 = tile_mb[tile];
  const int nmb = tile_mb[tile + 1] - mb0;
  const int nstages = ((nmb + 3) >> 2) * nch;

  {
    float4v z = {0.f, 0.f, 0.f, 0.f};
    float4v *a4 = reinterpret_cast<float4v *>(acc);
    for (int i = tid; i < (T + 1) * AS / 4; i += 512) a4[i] = z;
  }

  if (producer) {
    // ------------------------------------------------------------------ producer
    const int pt = tid - 256;
    const bool vec4 = (cin & 3) == 0;
    constexpr int RD = kRowsAhead, NS = kRowsAhead + kIdxAhead + 1;
    int idx[NS][NE];
    float4v rows[RD + 1][NE];
    auto load_idx = [&](int s, int (&ix)[NE]) {
      const int grp = s / nch;
#pragma unroll
      for (int j = 0; j < NE; ++j) {
        int slot = grp * 64 + ((pt + j * NP) >> 4);
        ix[j] = (s < nstages && slot < nmb * 16) ? sched_in[(int64_t)mb0 * 16 + slot] : -1;
      }
    };
    auto load_rows = [&](int s, const int (&ix)[NE], float4v (&r)[NE]) {
      const int cc = s % nch;
#pragma unroll
      for (int j = 0; j < NE; ++j) {
        int ch = cc * kKC + ((pt + j * NP) & 15) * 4;
        float4v v = {0.f, 0.f, 0.f, 0.f};
#ifdef SSC_DBG_NO_GATHER
        if (false) {
#else
        if (ix[j] >= 0) {
#endif
          const float *fp = features + (int64_t)ix[j] * cin + ch;
          if (vec4) {
            if (ch < cin) v = *reinterpret_cast<const float4v *>(fp);
          } else {
            if (ch + 0 < cin) v.x = fp[0];
            if (ch + 1 < cin) v.y = fp[1];
            if (ch + 2 < cin) v.z = fp[2];
            if (ch + 3 < cin) v.w = fp[3];
          }
        }
        r[j] = v;
      }
    };
    auto store_rows = [&](int s, const float4v (&r)[NE]) {
      float *ab = abuf + (s & 1) * kStage * kAStride;
#pragma unroll
      for (int j = 0; j < NE; ++j) {
        int e = pt + j * NP;
        *reinterpret_cast<float4v *>(ab + (e >> 4) * kAStride + (e & 15) * 4) = r[j];
      }
    };
    // Per-stage metadata handled by threads 0..68: the output row of each of the
    // 64 slots, the weight-fragment id (k * nch + cc) of the 4 row blocks and of
    // the first block of the following stage.
    auto load_meta = [&](int s) -> int {
      const int grp = s / nch;
      if (pt < kStage) {
        int slot = grp * 64 + pt;
        return (s < nstages && slot < nmb * 16) ? sched_out[(int64_t)mb0 * 16 + slot] : T;
      }
      if (pt < kStage + 5) {
        int j = pt - kStage;
        int s2 = j < 4 ? s : s + 1;
        int blk = (s2 / nch) * 4 + (j & 3);
        if (s2 < nstages && blk < nmb) return sched_k[mb0 + blk] * nch + (s2 % nch);
      }
      return -1;
    };
    auto store_meta = [&](int s, int v) {
      if (pt < kStage) orow[(s & 3) * kStage + pt] = v;
      else if (pt < kStage + 5) ids[(s & 3) * 8 + (pt - kStage)] = v;
    };
#pragma unroll
    for (int i = 0; i < NS; ++i) load_idx(i, idx[i]);
#pragma unroll
    for (int i = 0; i <= RD; ++i) load_rows(i, idx[i], rows[i]);
    store_meta(0, load_meta(0));
    store_meta(1, load_meta(1));
    // metadata is fetched two iterations before it is stored, so that waiting for
    // it never waits for the row loads issued after it (loads return in order)
    int meta0 = load_meta(2), meta1 = load_meta(3);
    store_rows(0, rows[0]);
    __syncthreads();
    for (int s = 0; s < nstages; ++s) {
      store_rows(s + 1, rows[1]);
      store_meta(s + 2, meta0);
      meta0 = meta1;
#pragma unroll
      for (int i = 0; i + 1 < NS; ++i)
#pragma unroll
        for (int j = 0; j < NE; ++j) idx[i][j] = idx[i + 1][j];
#pragma unroll
      for (int i = 1; i < RD; ++i)
#pragma unroll
        for (int j = 0; j < NE; ++j) rows[i][j] = rows[i + 1][j];
      meta1 = load_meta(s + 4);
      load_idx(s + NS, idx[NS - 1]);
      load_rows(s + 1 + RD, idx[RD], rows[RD]);
      __syncthreads();
    }
  } else {
    // ------------------------------------------------------------------ consumer
    const int cg = wave;
    const int g = lane >> 4;
    const int l16 = lane & 15;
    const int cb = blockIdx.y * 4 + cg;
    const bool live = cb < ncb;
    float *acc_lane = acc + cg * 16 + g * 4;
    auto load_b = [&](int id, float4v (&b)[4]) {
      // id = k * nch + cc
      const int k = id / nch, cc = id - k * nch;
      const float4v *bp = reinterpret_cast<const float4v *>(
          packed + (((int64_t)k * ncb + cb) * nch + cc) * 1024 + lane * 16);
#pragma unroll
      for (int q = 0; q < 4; ++q) b[q] = bp[q];
    };
    auto load_a = [&](const float *ab, int m, float4v (&a)[4]) {
      const float4v *ap =
          reinterpret_cast<const float4v *>(ab + (m * 16 + l16) * kAStride + g * 16);
#ifdef SSC_DBG_NO_A
      if (n_tiles < 0)
#endif
#pragma unroll
      for (int q = 0; q < 4; ++q) a[q] = ap[q];
    };
    auto accumulate = [&](int ol, const float4v &d) {
      // d = out[pair l16][channels 4g .. 4g+3] of this column group
      float4v *ptr = reinterpret_cast<float4v *>(acc_lane + ol * AS);
#ifdef SSC_DBG_NO_RMW
      if (d.x == 12345.f) *ptr = d;
#else
      *ptr = *ptr + d;
#endif
    };
    __syncthreads();
    // Weight fragments are fetched one whole stage ahead: stage s multiplies with
    // set (s & 1) while the fragments of stage s+1 stream into the other set.
    // idc = fragment ids of the current stage, idn = of the next one (the ring
    // publishes them two stages ahead).
    int idc[5], idn[5];
#pragma unroll
    for (int j = 0; j < 5; ++j) {
      idc[j] = __builtin_amdgcn_readfirstlane(ids[j]);
      idn[j] = __builtin_amdgcn_readfirstlane(ids[8 + j]);
    }
    float4v bx[4][4], by[4][4];
    // Only the first block of a run of equal ids is fetched; the rest of the run is
    // filled in by register copies once the data has arrived (fill_b_stage).
    auto load_b_stage = [&](const int (&id)[5], float4v (&b)[4][4]) {
#pragma unroll
      for (int m = 0; m < 4; ++m)
        if (id[m] >= 0 && (m == 0 || id[m] != id[m - 1])) load_b(id[m], b[m]);
    };
    auto fill_b_stage = [&](const int (&id)[5], float4v (&b)[4][4]) {
#pragma unroll
      for (int m = 1; m < 4; ++m)
        if (id[m] >= 0 && id[m] == id[m - 1]) {
#pragma unroll
          for (int q = 0; q < 4; ++q) b[m][q] = b[m - 1][q];
        }
    };
    // one stage out of LDS buffer (s & 1) with fragment set b; prefetches bn for s+1
    auto run_stage = [&](int s, float4v (&b)[4][4], float4v (&bn)[4][4]) {
      const float *ab = abuf + (s & 1) * kStage * kAStride;
      const int *orw = orow + (s & 3) * kStage;
      load_b_stage(idn, bn);
      if (idc[3] >= 0) {
        // full stage: straight-line code so LDS reads, MFMAs and accumulator updates
        // of neighbouring row blocks can be interleaved by the scheduler
        float4v a[4][4];
        int ol[4];
        float4v d[4];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          load_a(ab, m, a[m]);
          ol[m] = orw[m * 16 + l16];
        }
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          d[m] = float4v{0.f, 0.f, 0.f, 0.f};
          mfma_block(b[m], a[m], d[m]);
          accumulate(ol[m], d[m]);
        }
      } else {
        // last, partial stage of the tile
#pragma unroll
        for (int m = 0; m < 3; ++m) {
          if (idc[m] >= 0) {
            float4v a[4];
            load_a(ab, m, a);
            const int ol = orw[m * 16 + l16];
            float4v d = {0.f, 0.f, 0.f, 0.f};
            mfma_block(b[m], a, d);
            accumulate(ol, d);
          }
        }
      }
      fill_b_stage(idn, bn);
      const int *nx = ids + ((s + 2) & 3) * 8;
#pragma unroll
      for (int j = 0; j < 5; ++j) {
        idc[j] = idn[j];
        idn[j] = __builtin_amdgcn_readfirstlane(nx[j]);
      }
    };
    if (live) {
      load_b_stage(idc, bx);
      fill_b_stage(idc, bx);
    }
    for (int s = 0; s < nstages; s += 2) {
#ifdef SSC_DBG_NO_MFMA
      if (false) {
#else
      if (live) {
#endif
        run_stage(s, bx, by);
      }
      __syncthreads();
      if (s + 1 < nstages) {
#ifdef SSC_DBG_NO_MFMA
        if (false) {
#else
        if (live) {
#endif
          run_stage(s + 1, by, bx);
        }
        __syncthreads();
      }
    }
  }
  // write the tile
  const int col0 = blockIdx.y * CN;
  if ((cout & 3) == 0) {
    for (int e = tid; e < T * (CN / 4); e += 512) {
      int r = e / (CN / 4), c4 = e % (CN / 4);
      int64_t grow = row0 + r;
      int col = col0 + c4 * 4;
      if (grow < n_out && col < cout)
        *reinterpret_cast<float4v *>(out + grow * cout + col) =
            *reinterpret_cast<const float4v *>(acc + r * AS + c4 * 4);
    }
  } else {
    for (int e = tid; e < T * CN; e += 512) {
      int r = e / CN, c = e % CN;
      int64_t grow = row0 + r;
      if (grow < n_out && col0 + c < cout) out[grow * cout + col0 + c] = acc[r * AS + c];
    }
  }
}

struct ConvPlan {
  int ncb, nch, T;
  int64_t n_tiles, words_per_k, mb_cap;
  size_t lds_bytes;
};

static size_t conv_lds_bytes(int T) {
  return ((size_t)(T + 1) * 68 + 2 * (size_t)kStage * kAStride) * 4 + 4 * kStage * 4 + 32 * 4;
}

static int pick_tile() {
  // One workgroup per CU: (almost) all of the 160 KB of LDS goes to the accumulators.
  size_t budget = 160 * 1024 - conv_lds_bytes(0) - 1024;
  int t = (int)(budget / (68 * 4));
  t = t / 16 * 16;
  if (t < kMinTile) t = kMinTile;
  return t;
}

static ConvPlan make_plan(int64_t n_out, int K, int c_in, int c_out, int64_t pair_stride) {
  ConvPlan p;
  p.ncb = (int)ceil_div(c_out, 16);
  p.nch = (int)ceil_div(c_in, kKC);
  p.T = pick_tile();
  p.n_tiles = ceil_div(n_out > 0 ? n_out : 1, p.T);
  p.words_per_k = ceil_div(n_out > 0 ? n_out : 1, 32);
  // row blocks: at most one partial block per (tile, offset) on top of pairs / 16
  int64_t max_pairs_k = pair_stride < n_out ? pair_stride : n_out;
  p.mb_cap = (int64_t)K * (max_pairs_k / 16 + 1) + p.n_tiles * K;
  p.lds_bytes = conv_lds_bytes(p.T);
  return p;
}

struct ConvWs {
  float *packed;
  int32_t *flag;
  int32_t *segs;
  int32_t *sorted;
  uint32_t *bits;
  int32_t *prefix;
  int32_t *tile_cnt, *kofs, *tile_mb, *sched_in, *sched_out, *sched_k;
};

static size_t conv_ws_walk(void *base, const ConvPlan &p, int K, int64_t pair_stride, ConvWs *w) {
  Carver c(base);
  ConvWs t;
  t.packed = c.take<float>((size_t)K * p.ncb * p.nch * 1024);
  t.flag = c.take<int32_t>(1);
  t.segs = c.take<int32_t>((size_t)(p.n_tiles + 1) * K);
  t.sorted = c.take<int32_t>((size_t)K * 2 * pair_stride);
  t.bits = c.take<uint32_t>((size_t)K * p.words_per_k);
  t.prefix = c.take<int32_t>((size_t)K * p.words_per_k);
  t.tile_cnt = c.take<int32_t>((size_t)p.n_tiles);
  t.kofs = c.take<int32_t>((size_t)p.n_tiles * K);
  t.tile_mb = c.take<int32_t>((size_t)p.n_tiles + 1);
  t.sched_in = c.take<int32_t>((size_t)p.mb_cap * 16);
  t.sched_out = c.take<int32_t>((size_t)p.mb_cap * 16);
  t.sched_k = c.take<int32_t>((size_t)p.mb_cap);
  if (w) *w = t;
  return c.used;
}

static size_t conv_ws_bytes(int64_t n_out, int K, int c_in, int c_out, int64_t pair_stride) {
  ConvPlan p = make_plan(n_out, K, c_in, c_out, pair_stride);
  return conv_ws_walk(nullptr, p, K, pair_stride, nullptr);
}

// Optional timing of the convolution kernel alone: a ring of event pairs recorded
// on the caller's stream right around the launch of conv_fwd_kernel.
constexpr int kProfileRing = 512;
static bool g_profile_on = false;
static int g_profile_count = 0;
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
  g_profile_count = 0;
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

int ssc_conv_fwd_f32(const float *features, int64_t n_in, int32_t c_in, const float *filters,
                     int64_t fs_k, int64_t fs_ci, int64_t fs_co, int32_t c_out,
                     const int32_t *pairs, int64_t pair_stride, const int32_t *pair_num,
                     int32_t kernel_volume, int32_t inverse, int32_t subm, float *out,
                     int64_t n_out, void *workspace, size_t workspace_bytes,
                     ssc_stream_t stream) {
  (void)subm;
  const int K = kernel_volume;
  SSC_CHECK(K >= 1 && K <= SSC_MAX_KERNEL_VOLUME, SSC_ERUNTIME, "kernel volume %d out of range", K);
  SSC_CHECK(c_in >= 1 && c_out >= 1, SSC_EINVAL, "channel counts must be positive");
  SSC_CHECK(n_in >= 0 && n_out >= 0 && pair_stride >= 0, SSC_EINVAL, "negative size");
  SSC_CHECK(n_out < ((int64_t)1 << 31) && n_in < ((int64_t)1 << 31), SSC_EINVAL,
            "row counts must fit 31 bits");
  if (n_out == 0) return SSC_OK;
  SSC_CHECK(out != nullptr, SSC_EINVAL, "out is NULL");
  hipStream_t s = (hipStream_t)stream;
  if (pair_stride == 0 || n_in == 0) return fill_f32(out, n_out * c_out, 0.f, s);
  SSC_CHECK(features && filters && pairs && pair_num && workspace, SSC_EINVAL,
            "NULL pointer argument");
  size_t need = conv_ws_bytes(n_out, K, c_in, c_out, pair_stride);
  SSC_CHECK(workspace_bytes >= need, SSC_EWORKSPACE, "conv workspace too small: %zu < %zu",
            workspace_bytes, need);

  ConvPlan p = make_plan(n_out, K, c_in, c_out, pair_stride);
  ConvWs w;
  conv_ws_walk(workspace, p, K, pair_stride, &w);
  const int plane_g = inverse ? 1 : 0;
  const int plane_s = 1 - plane_g;
  int rc;

  int64_t packed_n = (int64_t)K * p.ncb * p.nch * 1024;
  hipLaunchKernelGGL(pack_filters_kernel, dim3((unsigned)ceil_div(packed_n, 256)), dim3(256), 0, s,
                     filters, fs_k, fs_ci, fs_co, K, c_in, c_out, p.ncb, p.nch, w.packed);
  SSC_LAUNCH_CHECK("pack_filters");

  if ((rc = fill_i32(w.flag, 1, 0, s)) != SSC_OK) return rc;
  dim3 pair_grid((unsigned)ceil_div(pair_stride, 256), (unsigned)K);
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

  int64_t nseg = (p.n_tiles + 1) * K;
  hipLaunchKernelGGL(tile_segments_kernel, dim3((unsigned)ceil_div(nseg, 256)), dim3(256), 0, s,
                     w.flag, pairs, w.sorted, pair_stride, plane_s, pair_num, K, p.n_tiles, p.T,
                     w.segs);
  SSC_LAUNCH_CHECK("tile_segments");
  hipLaunchKernelGGL(sched_count_kernel, dim3((unsigned)ceil_div(p.n_tiles, 256)), dim3(256), 0, s,
                     w.segs, K, p.n_tiles, w.tile_cnt, w.kofs);
  hipLaunchKernelGGL(sched_scan_kernel, dim3(1), dim3(kScanThreads), 0, s, w.tile_cnt, p.n_tiles,
                     w.tile_mb);
  hipLaunchKernelGGL(sched_fill_kernel, dim3((unsigned)ceil_div(p.n_tiles * K * 16, 256)),
                     dim3(256), 0, s, w.flag, pairs, w.sorted, pair_stride, plane_g, w.segs,
                     w.kofs, w.tile_mb, K, p.n_tiles, p.T, w.sched_in, w.sched_out, w.sched_k);
  SSC_LAUNCH_CHECK("schedule");

  static bool attr_set = false;
  if (!attr_set) {
    SSC_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(conv_fwd_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    attr_set = true;
  }
  dim3 grid((unsigned)p.n_tiles, (unsigned)ceil_div(p.ncb, 4));
  const bool prof = g_profile_on;
  const int slot = g_profile_count % kProfileRing;
  if (prof) SSC_HIP(hipEventRecord(g_profile_ev[slot][0], s));
  hipLaunchKernelGGL(conv_fwd_kernel, grid, dim3(512), p.lds_bytes, s, features, c_in, w.packed,
                     w.sched_in, w.sched_out, w.sched_k, w.tile_mb, p.nch, p.ncb, out, n_out,
                     c_out, p.T, p.n_tiles);
  SSC_LAUNCH_CHECK("conv_fwd");
  if (prof) {
    SSC_HIP(hipEventRecord(g_profile_ev[slot][1], s));
    ++g_profile_count;
  }
  return SSC_OK;
}
}
