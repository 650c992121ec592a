// The convolution kernel (conv_fwd_kernel), what a launch of it needs to know of a plan,
// and the launch itself.  Eight translation units instantiate it: conv.hip the plain form
// (float and half rows), conv_epi.hip the one with the epilogue, conv_tail.hip and
// conv_tail_epi.hip the one-column-group form without and with it, conv_five.hip and
// conv_five_epi.hip the five-group form, conv_wide.hip and conv_wide_epi.hip the plain
// kernel over plans of the five-group form -- compiled side by side, the parts of the
// instances take a third of the time.
#pragma once
#include "ssc_common.h"

#include <type_traits>

namespace ssc {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));

constexpr int kKC = 64;       // input channels per chunk = 16 MFMA steps of 4
constexpr int kStage = 64;    // pairs staged per barrier = 4 row blocks of 16
constexpr int kAStride = 68;  // floats per staged row (64 + 4: 16-byte aligned, bank spread)
constexpr int kMinTile = 64;

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

// FORM: 0 the kernel as described above; 1 the one-column-group form; 2 the five-group form
// (see the consumers); 3 the plain kernel on a plan of the five-group form, whose accumulator
// rows are 16 columns wider (the launches of such a plan that have no fifth group).
template <typename IO, int GATHER, int NCW, int NS, bool EPI, int FORM>
__global__ void __launch_bounds__((NCW + 4) * 64)
    __attribute__((amdgpu_waves_per_eu((NCW + 4) / 4, (NCW + 4) / 4)))
    conv_fwd_kernel(const IO *__restrict__ features, int cin, unsigned feat_bytes,
                    const void *__restrict__ packed, unsigned packed_bytes,
                    const int32_t *__restrict__ sched_in, const int32_t *__restrict__ sched_out,
                    const int32_t *__restrict__ grp_meta, unsigned sched_bytes, unsigned meta_bytes,
                    const int32_t *__restrict__ wg_grp,
                    int nch, int ncb, IO *__restrict__ out, int cout, int T, int cols_per_xcd,
                    int col_base, int xcol, ConvEpilogue epi) {
  constexpr bool TAIL = FORM == 1, FIVE = FORM == 2, WIDE = FORM == 3;
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
  // accumulator row stride in floats (the five-group form: 16 more columns)
  constexpr int kAS = kCN + (FIVE || WIDE ? 16 : 0) + 4;
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
    } else if (cols_per_xcd < 0) {
      // any other grid: the (range, column block) items, numbered range by range (-1) or
      // column block by column block (-2), are dealt to the XCDs in contiguous runs; XCD x
      // has the workgroups x, x + 8, ...
      const int ncol = gridDim.y, total = nwg * ncol;
      const int lin = blockIdx.y * nwg + blockIdx.x;
      const int xcd = lin & 7, slot = lin >> 3;
      const int item = xcd * (total >> 3) + min(xcd, total & 7) + slot;
      if (cols_per_xcd == -1) {
        chunk = item / ncol;
        cblk = item - chunk * ncol;
      } else {  // filters larger than an L2: column block by column block (an XCD sees few)
        cblk = item / nwg;
        chunk = item - cblk * nwg;
      }
    }
  }
  const int g_begin = wg_grp[2 * chunk], g_end = wg_grp[2 * chunk + 1];  // this workgroup's groups
  const int nstages = (g_end - g_begin) * nch;  // stages of this workgroup
  const int col0 = col_base + cblk * kCN;
  static_assert(FORM == 0 || (NCW == 4 && !kHalf), "the other forms are built for float");

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
  //   z = x * ca + cb (cb includes the bias in front of a scalar activation);
  //   mg = mode | LDS column of the gate << 4;  dest = output column
  //   gate l: activated value = act_gate(x * gca + gcb), LDS column gcl (-1: none)
  // LDS columns count from the first column of the block (a fifth group's from its own).
  // (EpiConsts: ca, cb, mg, dest per column of the thread; gca, gcb, gcl of its gate)
  struct EpiConsts {
    float ca[4], cb[4], gca, gcb;
    int mg[4], dest[4], gcl;
    bool any, vec;
  };
  // bcol0: first output column of the block of 64 the columns belong to; ncols: how many of
  // the block's columns the workgroup has (64, or the 16 of a fifth group)
  auto epi_consts = [&](int bcol0, int ncols) -> EpiConsts {
    EpiConsts e;
    e.gca = 0.f;
    e.gcb = 0.f;
    e.gcl = -1;
    const int c_t = (tid % (kCN / 4)) * 4, col = bcol0 + c_t;
    const bool col_ok = col < cout && c_t < ncols;
    static_assert(!EPI || kCN == 64, "the epilogue's gate runs are per block of 64 columns");
    const int eblk = bcol0 / kCN;  // block of 64 columns the workgroup's columns start
    const int gfirst = epi.gate_run[2 * eblk], gcount = min(epi.gate_run[2 * eblk + 1], 16);
    const bool run_ok = gfirst >= bcol0 && gfirst + gcount <= min(bcol0 + ncols, cout);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = col_ok ? col + i : 0;
      int mode = col_ok ? epi.mode[c] : 3;
      e.dest[i] = epi.dest[c];
      const int g = epi.gate[c];
      // tables that point outside the output row or outside the block's run of gates
      // switch the column off
      if (e.dest[i] < 0 || e.dest[i] >= epi.c_dest || mode < 0 || mode > 2 ||
          (mode == 2 && (!run_ok || g < gfirst || g >= gfirst + gcount)))
        mode = 3;
      e.mg[i] = mode | ((mode == 2 ? g - bcol0 : col_ok ? c_t + i : 0) << 4);
      e.ca[i] = epi.scale[c];
      e.cb[i] = epi.add[c] - epi.shift[c] * e.ca[i] + (mode == 1 ? epi.pre[c] : 0.f);
    }
    e.any = (e.mg[0] & 15) != 3 || (e.mg[1] & 15) != 3 || (e.mg[2] & 15) != 3 || (e.mg[3] & 15) != 3;
    e.vec = (e.mg[0] & 15) != 3 && (e.mg[1] & 15) != 3 && (e.mg[2] & 15) != 3 &&
            (e.mg[3] & 15) != 3 && e.dest[1] == e.dest[0] + 1 && e.dest[2] == e.dest[0] + 2 &&
            e.dest[3] == e.dest[0] + 3 && ((e.dest[0] | epi.c_dest) & 3) == 0;
    const int gi = (tid % (kCN / 4));
    if (run_ok && gi < gcount) {
      const int g = gfirst + gi;
      e.gcl = g - bcol0;
      e.gca = epi.scale[g];
      e.gcb = epi.add[g] - epi.shift[g] * e.gca + epi.pre[g];
    }
    return e;
  };
  EpiConsts ec = {}, ecx = {};  // of the workgroup's block of 64 columns; of a fifth group
  if constexpr (EPI) {
    ec = epi_consts(col0, kCN);
    if constexpr (FIVE) ecx = epi_consts(xcol, 16);
  }
  const int e_c_dest = epi.c_dest, e_act_s = epi.act_s, e_act_g = epi.act_g;
  auto flush_tile = [&](int row0, int rows, int slot0) __attribute__((always_inline)) {
    if constexpr (FIVE && !EPI) {
      // the fifth column group (accumulator columns kCN .. kCN + 15): four threads a row
      if (xcol >= 0) {
        const float4v z = {0.f, 0.f, 0.f, 0.f};
        const int c4 = (tid & 3) * 4;
        for (int r = tid >> 2; r < rows; r += NT / 4) {
          int sl = slot0 + r;
          if (sl >= T) sl -= T;
          float4v *ap = reinterpret_cast<float4v *>(acc + sl * kAS + kCN + c4);
          const float4v v = *ap;
          *ap = z;
          IO *gp = out + (int64_t)(row0 + r) * cout + xcol + c4;
          if ((cout & 3) == 0) {
            if (xcol + c4 < cout) Io<IO>::store_stream(gp, v);
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (xcol + c4 + i < cout) __builtin_nontemporal_store((IO)v[i], gp + i);
          }
        }
      }
    }
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
      // (e: the constants; XG: the pass over a fifth group, whose 16 columns begin at
      // accumulator column kCN and belong to the first four of a row's 16 threads)
      auto rows_out = [&](auto fast_tag, auto x_tag, const EpiConsts &e) __attribute__((always_inline)) {
        constexpr bool FAST = decltype(fast_tag)::value;
        constexpr bool XG = decltype(x_tag)::value;
        constexpr int U = 2;
        constexpr int RS = NT / (kCN / 4);
        const int r_t = tid / (kCN / 4), c_t = (tid % (kCN / 4)) * 4;
        const bool own = !XG || c_t < 16;  // the thread has columns
        constexpr int kCol0 = XG ? kCN : 0;
        const float4v z = {0.f, 0.f, 0.f, 0.f};
        // FAST: max(t, lo) is the scalar activation where there is one, t elsewhere
        float lo[4];
        bool gated[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          lo[i] = ((e.mg[i] & 15) == 1 && e_act_s == SSC_ACT_RELU) ? 0.f : -INFINITY;
          gated[i] = (e.mg[i] & 15) == 2;
        }
        auto gate_act = [&](float x) -> float {
          const float u = x * e.gca + e.gcb;
          if constexpr (FAST)
            return e_act_g == SSC_ACT_SIGMOID ? __builtin_amdgcn_rcpf(1.f + __expf(-u)) : u;
          else
            return act_fn(e_act_g, u);
        };
        IO *gp = out + (int64_t)(row0 + r_t) * e_c_dest;
        const int64_t gstep = (int64_t)RS * e_c_dest;
        for (int r = r_t; r < rows; r += U * RS) {
          const bool two = r + RS < rows;
          int sl0 = slot0 + r, sl1 = slot0 + r + RS;
          if (sl0 >= T) sl0 -= T;
          if (sl1 >= T) sl1 -= T;
          float *a0 = acc + sl0 * kAS + kCol0, *a1 = acc + sl1 * kAS + kCol0;
          if (e.gcl >= 0) {
            const float x0 = a0[e.gcl], x1 = two ? a1[e.gcl] : 0.f;
            a0[e.gcl] = gate_act(x0);
            if (two) a1[e.gcl] = gate_act(x1);
          }
          __builtin_amdgcn_sched_barrier(0);
          float4v v0 = own ? *reinterpret_cast<float4v *>(a0 + c_t) : z, v1 = z, g1 = z;
          float4v g0 = {a0[e.mg[0] >> 4], a0[e.mg[1] >> 4], a0[e.mg[2] >> 4], a0[e.mg[3] >> 4]};
          if (two) {
            if (own) v1 = *reinterpret_cast<float4v *>(a1 + c_t);
            g1 = float4v{a1[e.mg[0] >> 4], a1[e.mg[1] >> 4], a1[e.mg[2] >> 4], a1[e.mg[3] >> 4]};
          }
          __builtin_amdgcn_sched_barrier(0);  // the clears stay behind every read above
          if (own) *reinterpret_cast<float4v *>(a0 + c_t) = z;
          if (two && own) *reinterpret_cast<float4v *>(a1 + c_t) = z;
          if (e.any) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
              if (u == 1 && !two) break;
              const float4v v = u == 0 ? v0 : v1, gv = u == 0 ? g0 : g1;
              float4v y;
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const float t = v[i] * e.ca[i] + e.cb[i];
                if constexpr (FAST) {
                  y[i] = fmaxf(t, lo[i]) * (gated[i] ? gv[i] : 1.f);
                } else {  // every form, then select: no divergent branches
                  const float ts = act_fn(e_act_s, t);
                  const int m = e.mg[i] & 15;
                  y[i] = m == 1 ? ts : m == 2 ? t * gv[i] : t;
                }
              }
              IO *p = gp + u * gstep;
              if (e.vec) {
                Io<IO>::store_stream(p + e.dest[0], y);
              } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                  if ((e.mg[i] & 15) != 3) __builtin_nontemporal_store((IO)y[i], p + e.dest[i]);
              }
            }
          }
          gp += U * gstep;
        }
      };
      const bool fast = (e_act_s == SSC_ACT_NONE || e_act_s == SSC_ACT_RELU) &&
                        (e_act_g == SSC_ACT_NONE || e_act_g == SSC_ACT_SIGMOID);
      if constexpr (FIVE) {
        if (xcol >= 0) {
          if (fast)
            rows_out(std::true_type(), std::true_type(), ecx);
          else
            rows_out(std::false_type(), std::true_type(), ecx);
        }
      }
      if (fast)
        rows_out(std::true_type(), std::false_type(), ec);
      else
        rows_out(std::false_type(), std::false_type(), ec);
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
        if constexpr (FIVE) {  // the consumers add the last group's fifth-group products
#pragma unroll
          for (int i = 0; i < 4; ++i) __syncthreads();
        }
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
    auto fetch_frag = [&](Frag &dst, int soff, int q) {
      if constexpr (!kHalf && kQRem != 0) {
        if (q == kQFull) {  // the partly used quarter: kQRem floats per lane, densely packed
          const int voff = kQFull * kWStep + lane * (4 * kQRem);
          // The wider loads are cast to float vectors as a whole: with per-element casts
          // of an integer vector this compiler shrinks the load to its first element.
          if constexpr (kQRem == 1) {
            dst.x = __builtin_bit_cast(float, buf_load1(rs_w, voff, soff));
          } else if constexpr (kQRem == 2) {
            const float2v t = __builtin_bit_cast(
                float2v, __builtin_amdgcn_raw_buffer_load_b64(rs_w, voff, soff, 0));
            dst.x = t.x;
            dst.y = t.y;
          } else {
            const float3v t = __builtin_bit_cast(
                float3v, __builtin_amdgcn_raw_buffer_load_b96(rs_w, voff, soff, 0));
            dst.x = t.x;
            dst.y = t.y;
            dst.z = t.z;
          }
          return;
        }
      }
      dst = __builtin_bit_cast(Frag, buf_load4(rs_w, w_voff + q * kWStep, soff));
    };
    auto fetch_w = [&](int soff, int slot, int q) { fetch_frag(w[slot][q], soff, q); };
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
    // The five-group form.  Besides its own column group, of
    // which it multiplies the four row blocks of a stage, wave w multiplies row block w with
    // the fragments of a fifth group (output columns xcol .., accumulator columns kCN ..):
    // five blocks of MFMAs per stage and wave instead of four, and no SIMD that multiplies
    // for a column block of one group.  The products of a row block stay in registers over
    // the chunks of its group (dx).  Two row blocks of a group may hold the same output row,
    // so the four waves must not add to the fifth group's accumulators between the same two
    // barriers: wave w adds its products of a finished group (dprev, at aprev) during chunk
    // w of the next group (nch >= 4, the host launches the form for such layers only), in
    // the order of the row blocks, as the other column groups see their offsets; when a
    // tile ends they are added at once, a barrier between each two waves.
    //   wx[s & 1]  fragments of the fifth group for stage s, fetched one stage ahead
    //   kofx       fragment offset of row block `wave` of the next stage
    //   orowx      accumulator row of this lane's pair in row block `wave` of this stage
    Frag wx[2][NF];
    int kofx = 0, orowx = 0;
    float4v dx = float4v{0.f, 0.f, 0.f, 0.f}, dprev = float4v{0.f, 0.f, 0.f, 0.f};
    const int acc_lane_x = acc_base + (kCN + g * 4) * 4;
    const int dummy_x = T * kAS * 4 + acc_lane_x;
    int aprev = dummy_x;
    bool x_pending = false;
    constexpr bool x_on = FIVE;  // (a launch of the form has a fifth group: xcol >= 0)
    const char *const abx = a_base + wave * 16 * kRowB;
    const int w_soffx = (x_on ? xcol / 16 : 0) * nch * kFragB;
    auto load_kofx = [&](const StagePos &pos) -> int {
      return buf_load1(rs_meta, wave * 4, pos.g * 32);
    };
    auto load_orowx = [&](const StagePos &pos) -> int {
      return buf_load1(rs_out, l16 * 4 + wave * 64, pos.g * 256);
    };
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
          } else if constexpr (FIVE) {  // row block `wave`, for the fifth group
#pragma unroll
            for (int qq = 0; qq < NF; ++qq)
              if (i == kGapA[qq])
                a[0][qq] = *reinterpret_cast<const Frag *>(abx + par * kStage * kRowB + qq * 64);
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
      if constexpr (FIVE) {
        if (x_on) {
          // gaps: 0 read of the accumulator row this wave adds to in this stage (the dummy
          // row in other stages); 3 that update, fragment offset of the next stage;
          // 4, 6, 8, 10 its fragments; 11, 12 the next offset and accumulator row
          const bool mine = x_pending && cur.cc == wave;
          const int caddr = mine ? aprev : dummy_x;
          float4v accx = float4v{0.f, 0.f, 0.f, 0.f};
          int soffx = 0;
          constexpr int kGapXW[4] = {at(4), at(6), at(8), at(10)};
#pragma unroll
          for (int i = 0; i < kSteps; ++i) {
            __builtin_amdgcn_sched_barrier(0);
            dx = __builtin_amdgcn_mfma_f32_16x16x4f32(wx[par][i >> 2][i & 3], a[0][i >> 2][i & 3],
                                                      dx, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (i == at(0)) accx = lds_load4(caddr);
            if (i == at(3)) {
              soffx = frag_soff(kofx, w_soffx + next.cc * kFragB);
              lds_store4(caddr, accx + dprev);
            }
#pragma unroll
            for (int qq = 0; qq < NF; ++qq)
              if (i == kGapXW[qq]) fetch_frag(wx[par ^ 1][qq], soffx, qq);
            if (i == at(11)) kofx = load_kofx(after);
          }
          __builtin_amdgcn_sched_barrier(0);
          if (cur.cc == nch - 1) {  // the group is complete
            dprev = dx;
            aprev = orowx + acc_lane_x;
            dx = float4v{0.f, 0.f, 0.f, 0.f};
            x_pending = true;
          }
          orowx = load_orowx(next);
        }
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
      if constexpr (FIVE) {
        if (x_on) {  // in the loop's order: fragments, next offset, accumulator row
          kofx = load_kofx(p_cur);
          const int soffx = frag_soff(kofx, w_soffx + p_cur.cc * kFragB);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int q = 0; q < NF; ++q) fetch_frag(wx[0][q], soffx, q);
          __builtin_amdgcn_sched_barrier(0);
          kofx = load_kofx(p_next);
          orowx = load_orowx(p_cur);
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
        if constexpr (FIVE) {
          // the last group's products of the fifth group, wave after wave
#pragma unroll
          for (int wv = 0; wv < 4; ++wv) {
            if (x_on && wave == wv) lds_store4(aprev, lds_load4(aprev) + dprev);
            __syncthreads();
          }
          x_pending = false;
        }
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
  int n_rng;  // ranges of output rows: one for every workgroup of a column block, or two
  int tile_rows;                         // largest tile height
  int gather;  // conv_fwd_kernel's GATHER
  int ns;      // conv_fwd_kernel's NS: MFMA steps per chunk
  int64_t n_tiles, n_fine, words_per_k, grp_cap;  // n_tiles: upper bound
  int granule;  // rows per cell of the grid the work split places its boundaries on
  size_t lds_bytes;
  // Launches.  As a rule one, over all column blocks (n_colblk of them side by side, the
  // CUs shared out among them).  A last column group that would be alone in its block of
  // four (Cout = 72: 5 groups) behind at most two full blocks gets no column block, where
  // three of four consumer waves would multiply for nothing: the full blocks take one launch
  // each over all CUs (n_launch of them, n_colblk = 1) and the kernel's one-column-group
  // form a last one (has_tail), all over the same plan.
  // Or, for layers of four or more channel chunks, the last full block's launch takes the
  // lone group along as a fifth one (five): every launch is then of the five-group form,
  // whose accumulator rows are 16 columns wider (acc_cols), xcol >= 0 in the last only.
  int n_launch;
  bool has_tail, five;
  bool rebalance;  // the work split is made twice, the second time from the first one's counts
  int acc_cols;  // accumulator columns of a workgroup: 64, or 80 in the five-group form
  // a layer of a handful of input channels: no schedule, no matrix kernel -- the plan is a
  // table of every output row's input rows and the rows are computed by conv_small_kernel
  bool small;
  int kvol;           // kernel volume and number of output rows the plan was made for
  int64_t out_rows;
};

// conv_small.hip
bool conv_small_applies(int K, int c_in, int c_out, int elem_bytes);
int conv_small_build_table(const int32_t *flag, bool in_order, const int32_t *pairs,
                           const int32_t *sorted, int64_t pair_stride, int plane_s,
                           const int32_t *pair_num, int K, int64_t n_out, int32_t *table,
                           hipStream_t s);
int conv_small_run(const float *features, int c_in, const void *packed, int ncb, int ns,
                   const int32_t *table, int K, float *out, int c_out, int64_t n_out,
                   const ConvEpilogue &epi, hipStream_t s);

// Device buffers of a convolution call, in three groups with different lifetimes:
//   packed   the filters in MFMA fragment order: as long as the filters keep their values;
//   plan     what the convolution kernel reads besides features and filters (the row-block
//            schedule and the tile ranges of the workgroups): as long as the rulebook, the
//            channel counts, the element type and the direction (`inverse`) stay the same;
//   scratch  intermediate tables of the kernels that build the plan: until it is built.
struct ConvWs {
  void *packed;
  // plan
  int32_t *wg_tile, *wg_grp;  // first tile of every range; first and end group of every workgroup
  int32_t *sched_in, *sched_out, *grp_meta;
  int32_t *small_table;  // [K, n_out] (plans of ConvPlan::small, which have nothing else)
  // scratch
  int32_t *flag;
  int32_t *segs;
  int32_t *sorted;
  uint32_t *bits;
  int32_t *prefix;
  int32_t *tile_loc, *tile_nmb, *kofs, *tile_rng, *range_grp, *range_row1, *range_g0;
  int32_t *fine_segs, *range_row0, *range_row0_alt, *tile_row0, *n_tiles_dev;
  int32_t *spill_end, *tile_slot0, *spill, *share_first, *share_cnt;
};

// (switched by ssc_conv_tuning, for measurements)
inline bool g_conv_by_column = true;  // one column block per XCD for large filters

template <typename IO, int GATHER, int NCW, int NS, bool EPI, int FORM>
inline int launch_conv(const ConvPlan &p, const ConvWs &w, const IO *features, int64_t n_in,
                       int c_in, int K, IO *out, int c_out, int col_base, int xcol,
                       const ConvEpilogue &epi, hipStream_t s) {
  static bool attr_set = false;
  if (!attr_set) {
    SSC_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(conv_fwd_kernel<IO, GATHER, NCW, NS, EPI, FORM>),
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
  SSC_CHECK(FORM == 2 ? (xcol >= 0 && xcol % 16 == 0 && xcol < c_out && p.nch >= 4 &&
                         p.n_colblk == 1 && p.five)
                      : (xcol < 0 && p.five == (FORM == 3)),
            SSC_ERUNTIME, "convolution launch with a fifth column group it is not built for");
  dim3 grid((unsigned)p.n_wg, (unsigned)p.n_colblk);
  // one column block per XCD when the packed filters are larger than an L2 can keep
  // (4 MiB per XCD) and the grid divides that way (256 -> 256 channels, 7 MiB: 2.44 ->
  // 2.24 ms on the 64^3 benchmark geometry; 128 -> 256 at stride 2, 3.5 MiB, is 5 % slower
  // that way and stays with the row-major mapping)
  const bool by_column = packed_bytes > ((uint64_t)4 << 20) && p.n_colblk > 1 &&
                         8 % p.n_colblk == 0 && (p.n_wg * p.n_colblk) % 8 == 0 &&
                         g_conv_by_column;
  // (-1: a grid that is no multiple of 8 wide takes the kernel's mapping for any grid)
  const bool big = packed_bytes > ((uint64_t)4 << 20) && p.n_colblk > 1 && g_conv_by_column;
  const int cols_per_xcd = by_column ? 8 / p.n_colblk
                           : ((p.n_wg & 7) != 0 && p.n_wg * p.n_colblk >= 16) ? (big ? -2 : -1) : 0;
  hipLaunchKernelGGL((conv_fwd_kernel<IO, GATHER, NCW, NS, EPI, FORM>), grid, dim3((NCW + 4) * 64), p.lds_bytes, s, features, c_in,
                     feat_bytes, w.packed, (unsigned)packed_bytes, w.sched_in, w.sched_out,
                     w.grp_meta, (unsigned)sched_bytes, (unsigned)(p.grp_cap * 32), w.wg_grp,
                     p.nch, p.ncb, out, c_out, p.T, cols_per_xcd, col_base, xcol, epi);
  SSC_LAUNCH_CHECK("conv_fwd");
  return SSC_OK;
}

// The instances on float rows that conv.hip does not compile itself (conv_instances.h):
// with the epilogue, and the one-column-group and five-group forms with and without it.
template <int GATHER, int NS, bool EPI, int FORM>
int launch_conv_f32(const ConvPlan &p, const ConvWs &w, const float *features, int64_t n_in,
                    int c_in, int K, float *out, int c_out, int col_base, int xcol,
                    const ConvEpilogue &epi, hipStream_t s);

}  // namespace ssc
