// Sparse convolution forward for layers with a handful of input channels (the first layer of
// a network on raw point features: 3 -> 152 channels in the backbone benchmark).
//
// Such a layer is bound by writing its output: 2 P Cin Cout flops are nothing next to the
// N_out Cout floats it stores, and the matrix pipeline of conv_fwd_kernel -- one persistent
// workgroup per CU, tiles staged through LDS, a barrier per stage -- keeps too few stores in
// flight to fill the memory system.  Here every output row is computed in registers by the
// lanes that store it, four columns to a lane, from a table of the row's input rows:
//   table[k * n_out + o] = input row of the pair (k, o), or -1   (the rulebook inverted: a
//   fill and a scatter),
// with all filters, K Cin Cout floats, in LDS.  Products are added offset by offset in
// ascending k, channel by channel: a fixed order, no atomics.  The evaluation-mode batch norm
// and gate of ssc_conv_run_epilogue_f32 are applied to the row before it is stored.
#include "conv_kernel.h"
#include "ssc_common.h"

#include <type_traits>

namespace ssc {

constexpr int kSmallThreads = 512;
constexpr int kSmallFeatFloats = 1280;  // staged features of a chunk
constexpr int kSmallChunk = 128;  // most rows of a chunk: the stride of its table in LDS
constexpr size_t kSmallLdsBudget = 79104;  // two workgroups to a CU: (160 KB / 2) - 2.6 KB static - a little

// Filters as float4 over the columns: K * c_in * ceil(c_out / 4) of them.
static size_t small_filter_bytes(int K, int c_in, int c_out) {
  return (size_t)K * c_in * ((c_out + 3) / 4) * 16;
}

static size_t small_lds_bytes(int K, int c_in, int c_out, bool with_epi);

bool conv_small_applies(int K, int c_in, int c_out, int elem_bytes) {
  if (elem_bytes != 4 || c_in > 8 || c_in < 1 || c_out < 1 || K > 32) return false;
  const int cout4 = (c_out + 3) / 4;
  // (a pass of at most kSmallChunk rows, at least two)
  if (cout4 > kSmallThreads / 2 || cout4 < kSmallThreads / kSmallChunk) return false;
  return small_lds_bytes(K, c_in, c_out, true) <= kSmallLdsBudget;
}

// table[k * n_out + o] = gather row of the pair of offset k that scatters to o (the table
// is filled with -1 beforehand).  One thread per pair slot.
__global__ void __launch_bounds__(256)
    small_table_kernel(const int32_t *__restrict__ flag, int pairs_in_order,
                       const int32_t *__restrict__ pairs, const int32_t *__restrict__ sorted,
                       int64_t pair_stride, int plane_s, const int32_t *__restrict__ pair_num,
                       int64_t n_out, int32_t *__restrict__ table) {
  const int k = blockIdx.y;
  const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= pair_num[k]) return;
  // (the order of the pairs does not matter here; `sorted` is read when the plan's other
  // kernels read it, for one source of truth)
  const int32_t *src = (!pairs_in_order && flag[0]) ? sorted : pairs;
  const int64_t o = src[((int64_t)k * 2 + plane_s) * pair_stride + j];
  if (o >= 0 && o < n_out)
    table[(int64_t)k * n_out + o] = src[((int64_t)k * 2 + (1 - plane_s)) * pair_stride + j];
}

// What a lane needs of the epilogue's tables for its four columns.
struct SmallEpi {
  float ca[4], cb[4], gca[4], gcb[4];
  int mode[4], dest[4], gcol[4];
  bool any, vec;
};

// Rows are worked on in chunks of a few passes (a pass: as many rows as the workgroup's
// lanes cover at four columns a lane).  For a chunk the workgroup first reads the chunk's
// slice of the table -- K coalesced runs, all loads in flight at once, a thread holding a
// run of consecutive offsets of one row -- and finds the smallest and largest input row it
// names; output rows are in key order, so those input rows are neighbours, and their
// features (a few KB) follow into LDS as one contiguous copy.  The threads then write, row
// by row, the list of the row's pairs in ascending offset order (offset and distance of the
// input row from the smallest one, packed in a word; the four threads of a row place their
// parts by each other's counts).  The passes run out of LDS alone and touch nothing but
// real pairs: a lane reads its row's count and list, then per pair the input row's
// features and its slice of the offset's filters.  Two workgroups share a CU, so one's
// loads overlap the other's passes.  (A chunk whose input rows spread further than the
// buffer holds walks the table in memory instead.)
static inline int small_sub(int c_out) {
  const int rows_per_pass = kSmallThreads / ((c_out + 3) / 4);
  int sub = kSmallChunk / rows_per_pass;
  return sub < 1 ? 1 : sub > 8 ? 8 : sub;
}
constexpr int kSmallParts = kSmallThreads / kSmallChunk;  // threads to a row of the table: 4
constexpr int kHold = 8;                                  // offsets a thread holds: K <= 32
static inline int small_list_width(int K) { return (K + 7) / 8 * 8; }  // 16-bit entries

template <bool EPI>
__global__ void __launch_bounds__(kSmallThreads)
    __attribute__((amdgpu_waves_per_eu(4, 4)))  // two workgroups of 8 waves to a CU
    conv_small_kernel(const float *__restrict__ features, int cin,
                      const int32_t *__restrict__ table, int K, int64_t n_out,
                      const float *__restrict__ packed, int ncb, int ns,
                      float *__restrict__ out, int cout, int n_sub, ConvEpilogue epi) {
  extern __shared__ float4 lds4[];
  __shared__ int s_lo, s_hi;
  __shared__ int s_cnt[kSmallChunk * kSmallParts];
  __shared__ int s_tot[kSmallChunk];
  const int tid = threadIdx.x;
  const int cout4 = (cout + 3) >> 2;
  const int rows_per_pass = kSmallThreads / cout4;
  const int chunk_rows = rows_per_pass * n_sub;  // <= kSmallChunk
  const int lw = (K + 7) & ~7;                   // entries of a row's list (16 bits each)
  float *wf = reinterpret_cast<float *>(lds4);
  float *fbuf = wf + (size_t)K * cin * cout4 * 4;                 // [kSmallFeatFloats]
  float *rowbuf = fbuf + kSmallFeatFloats;  // [2][rows_per_pass][cout4 * 4]
  uint16_t *list =                          // [chunk_rows][lw]: offset << 11 | input row
      reinterpret_cast<uint16_t *>(rowbuf + 2 * (size_t)rows_per_pass * cout4 * 4);
  // the filters out of the packed fragments (conv.hip, "weight packing": a layer of at
  // most 8 input channels has one chunk of ns = 1 or 2 steps, packed densely in the
  // fragment's first 64 ns floats as [channel % 4][column % 16][channel / 4])
  for (int idx = tid; idx < K * cin * cout4 * 4; idx += kSmallThreads) {
    const int co = idx % (cout4 * 4);
    const int kc = idx / (cout4 * 4);
    const int ci = kc % cin, k = kc / cin;
    float v = 0.f;
    if (co < cout)
      v = packed[((int64_t)k * ncb + (co >> 4)) * 1024 + (((ci & 3) * 16 + (co & 15)) * ns) +
                 (ci >> 2)];
    wf[idx] = v;
  }
  const int r_local = tid / cout4, c4 = tid - r_local * cout4;
  const bool lane_on = r_local < rows_per_pass;
  SmallEpi e = {};
  if constexpr (EPI) {
    e.any = false;
    e.vec = true;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = c4 * 4 + i;
      const bool col_ok = lane_on && c < cout;
      const int cc = col_ok ? c : 0;
      const int blk = cc >> 6;
      const int gfirst = epi.gate_run[2 * blk], gcount = min(epi.gate_run[2 * blk + 1], 16);
      const bool run_ok = gfirst >= blk * 64 && gfirst + gcount <= min(blk * 64 + 64, cout);
      int mode = col_ok ? epi.mode[cc] : 3;
      const int g = epi.gate[cc];
      e.dest[i] = epi.dest[cc];
      if (e.dest[i] < 0 || e.dest[i] >= epi.c_dest || mode < 0 || mode > 2 ||
          (mode == 2 && (!run_ok || g < gfirst || g >= gfirst + gcount)))
        mode = 3;
      e.mode[i] = mode;
      e.ca[i] = epi.scale[cc];
      e.cb[i] = epi.add[cc] - epi.shift[cc] * e.ca[i] + (mode == 1 ? epi.pre[cc] : 0.f);
      e.gcol[i] = mode == 2 ? g : 0;
      e.gca[i] = mode == 2 ? epi.scale[g] : 0.f;
      e.gcb[i] = mode == 2 ? epi.add[g] - epi.shift[g] * e.gca[i] + epi.pre[g] : 0.f;
      e.any = e.any || mode != 3;
      e.vec = e.vec && mode != 3 && e.dest[i] == e.dest[0] + i;
    }
    e.vec = e.vec && ((e.dest[0] | epi.c_dest) & 3) == 0;
  }
  const int c_dest = EPI ? epi.c_dest : cout;
  const int act_s = epi.act_s, act_g = epi.act_g;
  const int64_t n_chunks = (n_out + chunk_rows - 1) / chunk_rows;
  // the thread's part of the table: row t_r of the chunk, offsets t_k0 .. t_k0 + kq - 1
  const int t_r = tid % kSmallChunk, t_q = tid / kSmallChunk;
  const int kq = (K + kSmallParts - 1) / kSmallParts;  // <= kHold
  const int t_k0 = t_q * kq;
  for (int64_t chunk = blockIdx.x; chunk < n_chunks; chunk += gridDim.x) {
    const int64_t row_base = chunk * chunk_rows;
    const int rows_here = n_out - row_base < chunk_rows ? (int)(n_out - row_base) : chunk_rows;
    if (tid == 0) {
      s_lo = 0x7FFFFFFF;
      s_hi = -1;
    }
    int held[kHold];
    int lo = 0x7FFFFFFF, hi = -1, cnt = 0;
#pragma unroll
    for (int u = 0; u < kHold; ++u) {
      const int k = t_k0 + u;
      held[u] = (u < kq && k < K && t_r < rows_here)
                    ? table[(int64_t)k * n_out + row_base + t_r] : -1;
    }
#pragma unroll
    for (int u = 0; u < kHold; ++u) {
      if (held[u] >= 0) {
        lo = held[u] < lo ? held[u] : lo;
        hi = held[u] > hi ? held[u] : hi;
        ++cnt;
      }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
      const int ol = __shfl_xor(lo, d, 64), oh = __shfl_xor(hi, d, 64);
      lo = ol < lo ? ol : lo;
      hi = oh > hi ? oh : hi;
    }
    __syncthreads();  // s_lo, s_hi are set; the chunk before is done with the LDS tables
    if ((tid & 63) == 0 && hi >= 0) {
      atomicMin(&s_lo, lo);
      atomicMax(&s_hi, hi);
    }
    s_cnt[t_r * kSmallParts + t_q] = cnt;
    __syncthreads();
    lo = s_lo;
    hi = s_hi;
    const bool staged = hi >= 0 && (int64_t)(hi - lo + 1) * cin <= kSmallFeatFloats &&
                        hi - lo < 2048;
    if (staged) {
      const float *src = features + (int64_t)lo * cin;
      for (int en = tid; en < (hi - lo + 1) * cin; en += kSmallThreads) fbuf[en] = src[en];
      int at = 0;
      for (int q = 0; q < t_q; ++q) at += s_cnt[t_r * kSmallParts + q];
      uint16_t *mine = list + t_r * lw;
#pragma unroll
      for (int u = 0; u < kHold; ++u)
        if (held[u] >= 0) mine[at++] = (uint16_t)(((t_k0 + u) << 11) | (held[u] - lo));
      if (t_q == kSmallParts - 1) s_tot[t_r] = at;
    }
    __syncthreads();
    for (int sub = 0; sub < n_sub; ++sub) {
      const int r = sub * rows_per_pass + r_local;
      const int64_t row = row_base + r;
      const bool on = lane_on && r < rows_here;
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
      auto add_pair = [&](int k, const float *x) {
        const float4 *w = lds4 + (size_t)k * cin * cout4 + c4;
#pragma unroll
        for (int half = 0; half < 2; ++half) {  // four channels' filters in flight
          float4 ww[4];
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (4 * half + j < cin) ww[j] = w[(size_t)(4 * half + j) * cout4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (4 * half + j < cin) {
              const float xv = x[4 * half + j];
              acc.x += xv * ww[j].x;
              acc.y += xv * ww[j].y;
              acc.z += xv * ww[j].z;
              acc.w += xv * ww[j].w;
            }
          }
        }
      };
      if (on && staged) {
        const int n = s_tot[r];
        const uint16_t *mine = list + r * lw;
        for (int base = 0; base < n; base += 4) {
          const uint2 en = *reinterpret_cast<const uint2 *>(mine + base);
          const unsigned ev[4] = {en.x & 0xFFFFu, en.x >> 16, en.y & 0xFFFFu, en.y >> 16};
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            if (base + v < n) {
              const float *f = fbuf + (ev[v] & 0x7FFu) * cin;
              float x[8];
#pragma unroll
              for (int ci = 0; ci < 8; ++ci) x[ci] = ci < cin ? f[ci] : 0.f;
              add_pair((int)(ev[v] >> 11), x);
            }
          }
        }
      } else if (on && hi >= 0) {  // input rows too far apart for the buffer: from memory
        for (int k = 0; k < K; ++k) {
          const int ix = table[(int64_t)k * n_out + row];
          if (ix >= 0) {
            float x[8];
#pragma unroll
            for (int ci = 0; ci < 8; ++ci)
              x[ci] = ci < cin ? features[(int64_t)ix * cin + ci] : 0.f;
            add_pair(k, x);
          }
        }
      }
      if constexpr (!EPI) {
        if (on) {
          float *p = out + row * cout + c4 * 4;
          if ((cout & 3) == 0) {
            __builtin_nontemporal_store(float4v{acc.x, acc.y, acc.z, acc.w},
                                        reinterpret_cast<float4v *>(p));
          } else {
            const float v[4] = {acc.x, acc.y, acc.z, acc.w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (c4 * 4 + i < cout) __builtin_nontemporal_store(v[i], p + i);
          }
        }
      } else {
        // the row's sums through LDS: a gated column needs its gate's sum, which another
        // lane of the row holds
        // (two buffers in turn: one barrier a pass)
        float *rb = rowbuf + ((size_t)(sub & 1) * rows_per_pass + r_local) * cout4 * 4;
        if (lane_on) reinterpret_cast<float4 *>(rb)[c4] = acc;
        __syncthreads();
        if (on && e.any) {
          const float v[4] = {acc.x, acc.y, acc.z, acc.w};
          float y[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float t = v[i] * e.ca[i] + e.cb[i];
            float res = t;
            if (e.mode[i] == 1) res = act_fn(act_s, t);
            if (e.mode[i] == 2) res = t * act_fn(act_g, rb[e.gcol[i]] * e.gca[i] + e.gcb[i]);
            y[i] = res;
          }
          float *p = out + row * c_dest;
          if (e.vec) {
            __builtin_nontemporal_store(float4v{y[0], y[1], y[2], y[3]},
                                        reinterpret_cast<float4v *>(p + e.dest[0]));
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (e.mode[i] != 3) __builtin_nontemporal_store(y[i], p + e.dest[i]);
          }
        }
      }
    }
  }
}

// Dynamic LDS of a launch: filters, staged features, the row buffer of the epilogue, and
// the pair lists of a chunk of rows.
static size_t small_lds_bytes(int K, int c_in, int c_out, bool with_epi) {
  (void)with_epi;  // (one layout for both forms)
  const int cout4 = (c_out + 3) / 4;
  const int rows_per_pass = kSmallThreads / cout4;
  return small_filter_bytes(K, c_in, c_out) + (size_t)kSmallFeatFloats * 4 +
         2 * (size_t)rows_per_pass * cout4 * 16 +
         (size_t)rows_per_pass * small_sub(c_out) * small_list_width(K) * 2;
}

int conv_small_build_table(const int32_t *flag, bool in_order, const int32_t *pairs,
                           const int32_t *sorted, int64_t pair_stride, int plane_s,
                           const int32_t *pair_num, int K, int64_t n_out, int32_t *table,
                           hipStream_t s) {
  int rc = fill_i32(table, (int64_t)K * n_out, -1, s);
  if (rc != SSC_OK) return rc;
  hipLaunchKernelGGL(small_table_kernel,
                     dim3((unsigned)ceil_div(pair_stride > 0 ? pair_stride : 1, 256), (unsigned)K),
                     dim3(256), 0, s, flag, in_order ? 1 : 0, pairs, sorted, pair_stride, plane_s,
                     pair_num, n_out, table);
  SSC_LAUNCH_CHECK("small_table");
  return SSC_OK;
}

int conv_small_run(const float *features, int c_in, const void *packed, int ncb, int ns,
                   const int32_t *table, int K, float *out, int c_out, int64_t n_out,
                   const ConvEpilogue &epi, hipStream_t s) {
  const bool with_epi = epi.mode != nullptr;
  const int cout4 = (c_out + 3) / 4;
  const size_t lds = small_lds_bytes(K, c_in, c_out, with_epi);
  SSC_CHECK(lds <= kSmallLdsBudget, SSC_ERUNTIME, "filters of %zu bytes do not fit LDS", lds);
  static bool attr_set = false;
  if (!attr_set) {
    SSC_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(conv_small_kernel<false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)kSmallLdsBudget));
    SSC_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(conv_small_kernel<true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)kSmallLdsBudget));
    attr_set = true;
  }
  static int cus = 0;  // (asked once: the query takes the host longer than the kernel runs)
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    cus = 256;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
        prop.multiProcessorCount > 0)
      cus = prop.multiProcessorCount;
  }
  // persistent workgroups, two to a CU (the filters are read into LDS once per workgroup)
  const int n_sub = small_sub(c_out);
  const int64_t chunks = ceil_div(n_out, (int64_t)(kSmallThreads / cout4) * n_sub);
  const int64_t blocks = chunks < 2 * cus ? chunks : 2 * cus;
  if (with_epi)
    hipLaunchKernelGGL(conv_small_kernel<true>, dim3((unsigned)blocks), dim3(kSmallThreads), lds, s,
                       features, c_in, table, K, n_out, static_cast<const float *>(packed), ncb,
                       ns, out, c_out, n_sub, epi);
  else
    hipLaunchKernelGGL(conv_small_kernel<false>, dim3((unsigned)blocks), dim3(kSmallThreads), lds,
                       s, features, c_in, table, K, n_out, static_cast<const float *>(packed), ncb,
                       ns, out, c_out, n_sub, epi);
  SSC_LAUNCH_CHECK("conv_small");
  return SSC_OK;
}

}  // namespace ssc
