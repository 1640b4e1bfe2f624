// GPU tree builder for gfx950 (MI355X): quantised bins resident in HBM, one
// stream, O(1) kernel launches per tree level and no host synchronisation
// inside a tree.
//
// Data layout.  Bins are uint8, four features packed in one uint32 ("quad"),
// stored quad-column-major: quad q of row r is bins[q * stride + r].  Every
// row pass therefore reads and writes fully coalesced 256-byte wave
// transactions.  Rows of one tree node are kept contiguous: after the split of
// level k is known, a stable partition moves (bins, grad, hess, row id) from
// the level-k order into the level-(k+1) order (ping-pong buffers).  Every
// tree starts again from the original order, so y and y_hat never move.
//
// Histograms.  One workgroup owns a contiguous row range of one node and a
// private histogram in LDS: two 64-bit words per (feature, bin),
//   word0 = count << 47 | sum of g_q   (g_q fixed point, |g_q| <= 2^30)
//   word1 = sum of h_q
// so one update costs two ds_add_u64 (one for the squared objective).  A range
// holds at most 64512 rows, which keeps both fields exact.  The LDS histogram
// is laid out in blocks of 16 features, bin-major inside a block, and every
// lane of a wave updates a different feature of its own row at a time: the 16
// lanes that one pass of the LDS atomic unit serves never share a bank pair or
// an address, whatever the bins are.  Each workgroup writes its LDS histogram
// to a private slab in HBM; a reduce kernel adds the slabs of a node, turns
// them feature-major, and derives the larger sibling as parent - smaller
// child.  All sums are integers: the result does not depend on scheduling.
//
// What replaces what (reference file:line):
//   k_bin_assign      build_histogram              src/io/io.cu:293-312
//                     (thresholds: quantiser.hip)
//   k_grad_*          update_grad                  src/core/objective.cu:15-56
//   k_root_from_hist  cub::DeviceReduce::Sum       src/core/garden.cu:432-435
//   k_hist            hist_sum_node / hist_sum_multi_node
//                                                  src/core/hist_grad_sum.cu:109-215,262-406
//   k_hist_reduce     update_multi_node + global atomics
//                                                  src/core/hist_grad_sum.cu:6-33
//   k_split_scan      DeviceScan + hist_gain_kernel
//                                                  src/core/hist_tree_grower.cu:9-35,393-416
//   k_split_select    hist_apply_candidates        src/core/hist_tree_grower.cu:37-102
//   k_part_*          apply_split, set_segment, CreatePartitioningIndexes,
//                     scatter_kernel               src/core/builder.h:51-59,107-123,287-300
//   k_leaf_*          UpdateLeafWeight, update_by_last_tree
//                                                  src/core/garden.cu:45-76,487-503
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <limits>
#include <random>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include "booster.h"
#include "gain.h"

namespace arb {
namespace {

#define HIP_OK(expr)                                                                        \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if (e_ != hipSuccess)                                                                   \
      throw std::runtime_error(std::string("HIP error: ") + hipGetErrorString(e_) + " in " #expr); \
  } while (0)

constexpr int kSlots = 256;               // histogram slots per feature (uint8 bins)
constexpr int kMaxWideSlots = 4096;       // histogram slots per feature with 16-bit bins (power of two)
constexpr int kHistThreads = 1024;        // one workgroup per CU, 16 waves
constexpr int kItemWaves = kHistThreads / 64;  // waves per work item in row passes
constexpr unsigned kPartRows = 16384;     // rows per work item of the stand-alone partition
constexpr int kMaxGroupQuads = 8;         // quads per histogram launch (compile-time variants, whole blocks)
constexpr unsigned kMaxHistRows = 64512;  // rows per histogram work item (< 2^16)
constexpr int kCountShift = 47;           // word0 = count << 47 | g
constexpr int kMaxPlanNodes = 4096;       // nodes per level the planner handles
constexpr size_t kLdsBudget = 160 * 1024;
// LDS histograms are laid out in blocks of 16 features (4 quads):
//   entry(f, bin) = (f / 16) * 4096 + bin * 16 + f % 16.
// A 64-bit LDS atomic is executed 16 lanes per pass, and two of those lanes
// collide when their addresses share a bank pair (entry % 16).  With this
// layout the bank pair is the feature, and the kernels let the 16 lanes of a
// pass work on 16 different features of their rows, so a pass never has a
// bank conflict and never two lanes on one address, whatever the bin
// distribution is (missing values, zeros, a dominant category).
constexpr int kBlockFeatures = 16;
constexpr int kBlockQuads = 4;
constexpr int kBlockEntries = kBlockFeatures * kSlots;  // 4096
constexpr int HistBlocks(int nq) { return (nq + kBlockQuads - 1) / kBlockQuads; }
// LDS bytes of a histogram of nq quads
constexpr size_t HistLdsBytes(int nq, bool pair) {
  return (size_t)HistBlocks(nq) * kBlockEntries * 8 * (pair ? 2 : 1);
}

struct NodeSum {
  long long g;
  long long h;
  unsigned long long c;
};

struct SplitRec {
  float gain;
  int fid;   // -1: not split (every row stays left)
  int bin;
  unsigned pad;
  NodeSum left;
};

struct WorkItem {
  unsigned node;
  unsigned begin;  // row range in the current order
  unsigned end;
  unsigned first;  // index of the first work item of this node
};

// --------------------------------------------------------------- quantiser
// bin(x) = first l in [0,size] with x <= v[l], v[t] = thr[t] for t < size-1,
// +INF above (src/core/cuda_helpers.h:207-222, src/io/io.cu:297-302); NaN
// compares false everywhere and lands in bin `size`.
__global__ void k_bin_assign(const float *__restrict__ x, int ncols, const float *__restrict__ thr,
                             int thr_stride, const int *__restrict__ sizes,
                             uint32_t *__restrict__ out, size_t n) {
  __shared__ float s_thr[4][kSlots];
  __shared__ int s_size[4];
  for (int i = threadIdx.x; i < 4 * kSlots; i += blockDim.x) {
    const int c = i >> 8, t = i & 255;
    float v = INFINITY;
    if (c < ncols && t < sizes[c] - 1) v = thr[(size_t)c * thr_stride + t];
    s_thr[c][t] = v;
  }
  if (threadIdx.x < 4) s_size[threadIdx.x] = threadIdx.x < ncols ? sizes[threadIdx.x] : 0;
  __syncthreads();
  for (size_t r = (size_t)blockIdx.x * blockDim.x + threadIdx.x; r < n;
       r += (size_t)gridDim.x * blockDim.x) {
    uint32_t packed = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (c < ncols) {
        const float v = x[(size_t)c * n + r];
        unsigned l = 0, h = (unsigned)s_size[c];
        while (l < h) {
          const unsigned mid = (l + h) >> 1;
          if (v <= s_thr[c][mid])
            h = mid;
          else
            l = mid + 1;
        }
        packed |= l << (8 * c);
      }
    }
    out[r] = packed;
  }
}

// The same with 16-bit bins: two features per word, thresholds of both in
// dynamic LDS (2 * thr_stride floats).
__global__ void k_bin_assign_wide(const float *__restrict__ x, int ncols, const float *__restrict__ thr,
                                  int thr_stride, const int *__restrict__ sizes,
                                  uint32_t *__restrict__ out, size_t n) {
  extern __shared__ float s_thr_wide[];
  for (int i = threadIdx.x; i < 2 * thr_stride; i += blockDim.x) {
    const int c = i / thr_stride, t = i % thr_stride;
    float v = INFINITY;
    if (c < ncols && t < sizes[c] - 1) v = thr[(size_t)c * thr_stride + t];
    s_thr_wide[i] = v;
  }
  __syncthreads();
  for (size_t r = (size_t)blockIdx.x * blockDim.x + threadIdx.x; r < n;
       r += (size_t)gridDim.x * blockDim.x) {
    uint32_t packed = 0;
    for (int c = 0; c < ncols; ++c) {
      const float v = x[(size_t)c * n + r];
      unsigned l = 0, h = (unsigned)sizes[c];
      while (l < h) {
        const unsigned mid = (l + h) >> 1;
        if (v <= s_thr_wide[c * thr_stride + mid])
          h = mid;
        else
          l = mid + 1;
      }
      packed |= l << (16 * c);
    }
    out[r] = packed;
  }
}

// row-major uint8 [n][F] -> quads
__global__ void k_pack_prebinned(const uint8_t *__restrict__ in, int F, int Q,
                                 uint32_t *__restrict__ out, size_t stride, size_t n) {
  for (size_t r = (size_t)blockIdx.x * blockDim.x + threadIdx.x; r < n;
       r += (size_t)gridDim.x * blockDim.x) {
    for (int q = 0; q < Q; ++q) {
      uint32_t packed = 0;
      for (int c = 0; c < 4; ++c) {
        const int f = q * 4 + c;
        if (f < F) packed |= (uint32_t)in[r * F + f] << (8 * c);
      }
      out[(size_t)q * stride + r] = packed;
    }
  }
}

// ------------------------------------------------------------- objectives
__device__ __forceinline__ float WaveMaxF(float v) {
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_down(v, off));
  return v;
}
__device__ __forceinline__ long long WaveSumLL(long long v) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off);
  return v;
}

// squared error: g = y - y_hat (objective.cu:28-38); also max |g| for the
// fixed-point scale
__global__ void k_grad_squared(const float *__restrict__ y, const float *__restrict__ yhat,
                               float *__restrict__ g, size_t n, unsigned *__restrict__ gmax_bits) {
  float m = 0.0f;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const float v = y[i] - yhat[i];
    g[i] = v;
    const float a = fabsf(v);
    if (a > m) m = a;  // NaN never raises the maximum
  }
  m = WaveMaxF(m);
  if ((threadIdx.x & 63) == 0) atomicMax(gmax_bits, __float_as_uint(m));
}

__global__ void k_set_shift(const unsigned *__restrict__ gmax_bits, int *__restrict__ shifts) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    shifts[0] = FixShiftFromMax(__uint_as_float(*gmax_bits));
    shifts[1] = 0;
  }
}

// logistic: s = sigmoid(y_hat), g = y - s, h = s(1-s) (objective.cu:43-56)
__global__ void k_grad_logistic(const float *__restrict__ y, const float *__restrict__ yhat,
                                float *__restrict__ g, float *__restrict__ h, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const float s = SigmoidF(yhat[i]);
    g[i] = y[i] - s;
    h[i] = s * (1.0f - s);
  }
}

// soft-max: p = softmax(y_hat[., row]), g_k = [label == k] - p_k,
// h_k = 2 p_k (1 - p_k) (formula in the comment at objective.cu:60-89).
// y_hat, g, h are class-major [K][n].
__global__ void k_grad_softmax(const uint8_t *__restrict__ labels, const float *__restrict__ yhat,
                               float *__restrict__ g, float *__restrict__ h, size_t n, int K) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    double mx = -1e300;
    for (int k = 0; k < K; ++k) mx = fmax(mx, (double)yhat[i + (size_t)k * n]);
    double sum = 0.0;
    for (int k = 0; k < K; ++k) sum += (double)ExpF((float)((double)yhat[i + (size_t)k * n] - mx));
    const int lab = labels[i];
    for (int k = 0; k < K; ++k) {
      const double e = (double)ExpF((float)((double)yhat[i + (size_t)k * n] - mx));
      const float pk = (float)(e / sum);
      g[i + (size_t)k * n] = (lab == k ? 1.0f : 0.0f) - pk;
      h[i + (size_t)k * n] = 2.0f * pk * (1.0f - pk);
    }
  }
}

__global__ void k_init_root(NodeSum *tot, unsigned *seg_start, unsigned long long n,
                            unsigned *gmax_bits) {  // gmax_bits may be NULL
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    tot[0].g = 0;
    tot[0].h = 0;
    tot[0].c = n;
    seg_start[0] = 0;
    if (gmax_bits) *gmax_bits = 0;
  }
}

__device__ __forceinline__ unsigned RankBelow(unsigned long long m) {
  // number of set bits of m below this lane
  return __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0u));
}

// ------------------------------------------------------------------ planner
// Splits the row ranges of the selected nodes of a level into work items of
// at most `rows_per_item` rows.  select: 0 = every node, 1 = the smaller
// child of each sibling pair, ties -> left (hist_grad_sum.cu:279-294).
// rows_scanned (optional) is advanced by the rows that will be accumulated
// into histograms: the selected rows, or, when `split` is given (fused
// partition + histogram over parent nodes), the smaller side of every split.
// One workgroup.
__device__ __forceinline__ void PlanBody(const NodeSum *__restrict__ tot, const unsigned *__restrict__ seg_start,
                                         int L, int select, unsigned rows_per_item,
                                         WorkItem *__restrict__ work, unsigned *__restrict__ n_work,
                                         unsigned *__restrict__ node_first, unsigned *__restrict__ node_items,
                                         unsigned long long *__restrict__ rows_scanned,
                                         const SplitRec *__restrict__ split, unsigned max_items,
                                         unsigned *__restrict__ overflow) {
  __shared__ unsigned s_base[kMaxPlanNodes + 1];
  __shared__ unsigned s_wave[16];
  __shared__ unsigned s_carry;
  __shared__ unsigned long long s_rows;
  const int tid = threadIdx.x;
  if (tid == 0) {
    s_carry = 0;
    s_rows = 0;
  }
  __syncthreads();
  for (int base = 0; base < L; base += 1024) {
    const int nd = base + tid;
    unsigned cnt = 0;
    if (nd < L) {
      const unsigned long long len = tot[nd].c;
      bool sel = true;
      if (select == 1) {
        const unsigned long long sib = tot[nd ^ 1].c;
        sel = (nd & 1) ? (len < sib) : (len <= sib);
      }
      if (sel && len > 0) {
        cnt = (unsigned)((len + rows_per_item - 1) / rows_per_item);
        unsigned long long acc = len;
        if (split) {
          const unsigned long long cl = split[nd].left.c;
          acc = min(cl, len - cl);
        }
        atomicAdd(&s_rows, acc);
      }
      node_items[nd] = sel ? cnt : 0xffffffffu;  // 0xffffffff marks "not selected"
    }
    // block exclusive scan of cnt
    unsigned incl = cnt;
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned o = __shfl_up(incl, off);
      if ((tid & 63) >= off) incl += o;
    }
    if ((tid & 63) == 63) s_wave[tid >> 6] = incl;
    __syncthreads();
    unsigned wave_off = 0;
    for (int w = 0; w < (tid >> 6); ++w) wave_off += s_wave[w];
    const unsigned excl = s_carry + wave_off + incl - cnt;
    if (nd < L) {
      s_base[nd] = excl;
      node_first[nd] = excl;
    }
    __syncthreads();
    if (tid == 1023) s_carry = excl + cnt;
    __syncthreads();
  }
  const unsigned total = s_carry;
  if (tid == 0) {
    s_base[L] = total;
    *n_work = total <= max_items ? total : 0;  // never exceed the launch bound
    if (total > max_items) *overflow = 1;      // reported as an error at the end of the tree
    if (rows_scanned) *rows_scanned += s_rows;
  }
  __syncthreads();
  if (total > max_items) return;
  for (unsigned w = tid; w < total; w += 1024) {
    int lo = 0, hi = L;  // last node whose first item is <= w
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (s_base[mid] <= w)
        lo = mid;
      else
        hi = mid;
    }
    const unsigned start = seg_start[lo];
    const unsigned len = (unsigned)tot[lo].c;
    const unsigned k = w - s_base[lo];
    WorkItem it;
    it.node = lo;
    it.begin = start + k * rows_per_item;
    it.end = min(start + len, it.begin + rows_per_item);
    it.first = s_base[lo];
    work[w] = it;
  }
}

__global__ void __launch_bounds__(1024)
k_plan(const NodeSum *__restrict__ tot, const unsigned *__restrict__ seg_start, int L, int select,
       unsigned rows_per_item, WorkItem *__restrict__ work, unsigned *__restrict__ n_work,
       unsigned *__restrict__ node_first, unsigned *__restrict__ node_items,
       unsigned long long *__restrict__ rows_scanned, const SplitRec *__restrict__ split,
       unsigned max_items, unsigned *__restrict__ overflow) {
  PlanBody(tot, seg_start, L, select, rows_per_item, work, n_work, node_first, node_items, rows_scanned, split,
           max_items, overflow);
}

// Rows of a work item are dealt to its waves in chunks of kChunkRows
// consecutive rows, round-robin: wave v takes chunks v, v + kItemWaves, ...  A
// workgroup therefore streams one contiguous block of the item per step (good
// DRAM page locality) while every wave still owns a fixed, countable row set.
constexpr unsigned kChunkRows = 128;
constexpr unsigned kChunkStep = kChunkRows * kItemWaves;

// ---------------------------------------------------------------- histogram
// LDS layout of a histogram of NQ quads: word0 of every entry, then (PAIR)
// word1 in the same order.
template <int NQ>
struct HistLds {
  static constexpr int blocks = HistBlocks(NQ);
  static constexpr int entries = blocks * kBlockEntries;
  static constexpr int word1 = entries;  // offset of word1 of the same entry
};

// Adds one row per lane (bins of its NQ quads in b) to the LDS histogram.  The
// 28 (or 4*NQ) updates of a row are issued in an order that depends on the
// lane: in step (s, t) of a block, lane l works on quad (s + (l>>2)) % 4 and
// byte (t + l) % 4 of that quad, so the 16 lanes of a pass of the LDS atomic
// touch 16 different features = 16 different bank pairs.  q_first: first quad
// of this launch (a multiple of 4).
template <bool PAIR, int NQ>
__device__ __forceinline__ void AccumulateRow(unsigned long long *__restrict__ lds,
                                              const uint32_t (&b)[NQ], float gv, float hv, int sg,
                                              int sh, int q_first, int F) {
  using L = HistLds<NQ>;
  const unsigned long long w0 = (1ull << kCountShift) + (unsigned long long)ToFixed(gv, sg);
  unsigned long long w1 = 0;
  if (PAIR) w1 = (unsigned long long)ToFixed(hv, sh);
  const unsigned j = (threadIdx.x >> 2) & 3u, i = threadIdx.x & 3u;
#pragma unroll
  for (int k = 0; k < L::blocks; ++k) {
    // quads of this block; the ones past NQ do not exist
    uint32_t r[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) r[x] = 4 * k + x < NQ ? b[4 * k + x < NQ ? 4 * k + x : 0] : 0u;
#pragma unroll
    for (int s_ = 0; s_ < 4; ++s_) {
      const unsigned qi = ((unsigned)s_ + j) & 3u;  // quad of the block this lane works on
      const uint32_t lo = (j & 1u) ? r[(s_ + 1) & 3] : r[s_];
      const uint32_t hi = (j & 1u) ? r[(s_ + 3) & 3] : r[(s_ + 2) & 3];
      const uint32_t sel = (j & 2u) ? hi : lo;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const unsigned bi = ((unsigned)t + i) & 3u;  // byte of the quad
        const unsigned bin = (sel >> (8u * bi)) & 255u;
        const unsigned f16 = 4u * qi + bi;
        // Quads past NQ do not exist.  Padding features of the last quad of
        // the matrix (bin 0 in every row) are accumulated like real ones into
        // slots nobody reads: cheaper than a per-update test.
        bool on = true;
        if (4 * k + 3 >= NQ) on = 4u * k + qi < (unsigned)NQ;
        if (on) {
          const unsigned idx = (unsigned)(k * kBlockEntries) + bin * kBlockFeatures + f16;
          atomicAdd(&lds[idx], w0);
          if (PAIR) atomicAdd(&lds[L::word1 + idx], w1);
        }
      }
    }
  }
}

// Writes the LDS histogram to the slab of work item w in LDS order.  Called by
// the whole workgroup after its last LDS update.  Slab layout per work item:
// word0[slab_entries], word1[slab_entries]; q_first is a multiple of 4.
template <bool PAIR, int NQ>
__device__ __forceinline__ void FlushSlab(const unsigned long long *__restrict__ lds,
                                          unsigned long long *__restrict__ slab, unsigned w,
                                          int slab_entries, int q_first) {
  using L = HistLds<NQ>;
  __syncthreads();
  unsigned long long *out =
      slab + (size_t)w * slab_entries * (PAIR ? 2 : 1) + (size_t)(q_first / kBlockQuads) * kBlockEntries;
  for (int e = threadIdx.x; e < L::entries; e += kHistThreads) {
    out[e] = lds[e];
    if (PAIR) out[slab_entries + e] = lds[L::word1 + e];
  }
}

// Histogram of contiguous row ranges: one workgroup per work item, quads
// [q0, q0+NQ).  LDS: NQ*1024 word0 entries, then (PAIR) as many word1 entries.
template <bool PAIR, int NQ>
__global__ void __launch_bounds__(kHistThreads)
k_hist(const uint32_t *__restrict__ bins, size_t stride, int q0, int F,
       const float *__restrict__ g, const float *__restrict__ h, const int *__restrict__ shifts,
       const WorkItem *__restrict__ work, const unsigned *__restrict__ n_work,
       unsigned long long *__restrict__ slab, int slab_entries) {
  extern __shared__ unsigned long long lds[];
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  constexpr int words = (int)(HistLdsBytes(NQ, PAIR) / 8);
  for (int i = threadIdx.x; i < words; i += kHistThreads) lds[i] = 0ull;
  __syncthreads();
  const int sg = shifts[0], sh = shifts[1];
  const uint32_t *bq = bins + (size_t)q0 * stride;
  for (unsigned base = it.begin; base < it.end; base += 2 * kHistThreads) {
    const unsigned r0 = base + threadIdx.x, r1 = r0 + kHistThreads;
    const bool v0 = r0 < it.end, v1 = r1 < it.end;
    const unsigned a0 = v0 ? r0 : it.begin, a1 = v1 ? r1 : it.begin;
    uint32_t b0[NQ], b1[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      b0[q] = __builtin_nontemporal_load(&bq[(size_t)q * stride + a0]);
      b1[q] = __builtin_nontemporal_load(&bq[(size_t)q * stride + a1]);
    }
    const float g0 = g[a0], g1 = g[a1];
    const float h0 = PAIR ? h[a0] : 0.0f, h1 = PAIR ? h[a1] : 0.0f;
    if (v0) AccumulateRow<PAIR, NQ>(lds, b0, g0, h0, sg, sh, q0, F);
    if (v1) AccumulateRow<PAIR, NQ>(lds, b1, g1, h1, sg, sh, q0, F);
  }
  FlushSlab<PAIR, NQ>(lds, slab, w, slab_entries, q0);
}

// Histogram of contiguous row ranges with 16-bit bins: features [f0, f0 + nf)
// (f0 even), `slots` histogram slots per feature, LDS layout f * slots + bin,
// word0 of every entry first, then (PAIR) word1.  The slab of a work item has
// the same feature-major order: word0[slab_entries], word1[slab_entries].
template <bool PAIR>
__global__ void __launch_bounds__(kHistThreads)
k_hist_wide(const uint32_t *__restrict__ bins, size_t stride, int f0, int nf, int slots,
            const float *__restrict__ g, const float *__restrict__ h, const int *__restrict__ shifts,
            const WorkItem *__restrict__ work, const unsigned *__restrict__ n_work,
            unsigned long long *__restrict__ slab, int slab_entries) {
  extern __shared__ unsigned long long lds[];
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const int entries = nf * slots;
  for (int i = threadIdx.x; i < entries * (PAIR ? 2 : 1); i += kHistThreads) lds[i] = 0ull;
  __syncthreads();
  const int sg = shifts[0], sh = shifts[1];
  const int words = (nf + 1) / 2;
  for (unsigned r = it.begin + threadIdx.x; r < it.end; r += kHistThreads) {
    const unsigned long long w0 = (1ull << kCountShift) + (unsigned long long)ToFixed(g[r], sg);
    unsigned long long w1 = 0;
    if (PAIR) w1 = (unsigned long long)ToFixed(h[r], sh);
    for (int k = 0; k < words; ++k) {
      const uint32_t word = bins[(size_t)(f0 / 2 + k) * stride + r];
      const unsigned lo = (unsigned)(2 * k) * slots + (word & 0xffffu);
      atomicAdd(&lds[lo], w0);
      if (PAIR) atomicAdd(&lds[entries + lo], w1);
      if (2 * k + 1 < nf) {
        const unsigned hi = (unsigned)(2 * k + 1) * slots + (word >> 16);
        atomicAdd(&lds[hi], w0);
        if (PAIR) atomicAdd(&lds[entries + hi], w1);
      }
    }
  }
  __syncthreads();
  unsigned long long *out = slab + (size_t)w * slab_entries * (PAIR ? 2 : 1) + (size_t)f0 * slots;
  for (int e = threadIdx.x; e < entries; e += kHistThreads) {
    out[e] = lds[e];
    if (PAIR) out[slab_entries + e] = lds[entries + e];
  }
}

// ---------------------------------------------------------------- partition
// How bin ids are packed in the 32-bit words of a row: 8 bits (four features
// per word) or 16 bits (two features per word).
struct BinCode {
  int wshift;  // feature -> word: fid >> wshift
  int bits;
  __host__ __device__ static BinCode Of(int bits) { return BinCode{bits == 8 ? 2 : 1, bits}; }
  __device__ __forceinline__ int Word(int fid) const { return fid >> wshift; }
  __device__ __forceinline__ unsigned Bin(uint32_t word, int fid) const {
    return (word >> (bits * (fid & ((1 << wshift) - 1)))) & ((1u << bits) - 1u);
  }
};

__device__ __forceinline__ bool GoesRight(const uint32_t *__restrict__ bins, size_t stride,
                                          const SplitRec &s, unsigned r, BinCode code = BinCode{2, 8}) {
  // builder.h:107-123: bin >= q + 1 goes right
  if (s.fid < 0) return false;
  const uint32_t word = bins[(size_t)code.Word(s.fid) * stride + r];
  return (int)code.Bin(word, s.fid) > s.bin;
}

// Rows going left, per (work item, wave range).
__global__ void __launch_bounds__(kHistThreads)
k_part_count(const uint32_t *__restrict__ bins, size_t stride, const SplitRec *__restrict__ split,
             const WorkItem *__restrict__ work, const unsigned *__restrict__ n_work,
             unsigned *__restrict__ wave_left, unsigned *__restrict__ item_left, BinCode code) {
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const SplitRec s = split[it.node];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned cnt = 0;
  if (s.fid < 0) {
    for (unsigned base = it.begin + wave * kChunkRows; base < it.end; base += kChunkStep)
      cnt += lane == 0 ? min(kChunkRows, it.end - base) : 0u;
  } else {
    const uint32_t *col = bins + (size_t)code.Word(s.fid) * stride;
    // eight chunks (16 loads) in flight per wave: the pass is latency-bound
    constexpr int kBatch = 8;
    for (unsigned base = it.begin + wave * kChunkRows; base < it.end; base += kBatch * kChunkStep) {
      uint32_t v0[kBatch], v1[kBatch];
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const unsigned r0 = base + k * kChunkStep + lane, r1 = r0 + 64;
        v0[k] = col[min(r0, it.end - 1)];
        v1[k] = col[min(r1, it.end - 1)];
      }
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const unsigned r0 = base + k * kChunkStep + lane, r1 = r0 + 64;
        if (r0 < it.end) cnt += ((int)code.Bin(v0[k], s.fid) > s.bin) ? 0u : 1u;
        if (r1 < it.end) cnt += ((int)code.Bin(v1[k], s.fid) > s.bin) ? 0u : 1u;
      }
    }
  }
  for (int off = 32; off > 0; off >>= 1) cnt += __shfl_down(cnt, off);
  if (lane == 0) wave_left[(size_t)w * kItemWaves + wave] = cnt;
  // per-item total for the offset computation of later items of the node
  __shared__ unsigned s_cnt[kItemWaves];
  if (lane == 0) s_cnt[wave] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned t = 0;
    for (int k = 0; k < kItemWaves; ++k) t += s_cnt[k];
    item_left[w] = t;
  }
}

// Rows going left in the earlier work items of the same node and in the
// earlier waves of this item.  Called by the whole workgroup; s_tmp holds
// kItemWaves + 1 words.
__device__ __forceinline__ unsigned LeftsBefore(const WorkItem &it, unsigned w, int wave,
                                                const unsigned *__restrict__ wave_left,
                                                const unsigned *__restrict__ item_left,
                                                unsigned *s_tmp) {
  unsigned part = 0;
  for (unsigned k = it.first + threadIdx.x; k < w; k += blockDim.x) part += item_left[k];
  for (int off = 32; off > 0; off >>= 1) part += __shfl_down(part, off);
  if ((threadIdx.x & 63) == 0) s_tmp[threadIdx.x >> 6] = part;
  __syncthreads();
  unsigned before = 0;
  for (int k = 0; k < kItemWaves; ++k) before += s_tmp[k];
  for (int k = 0; k < wave; ++k) before += wave_left[(size_t)w * kItemWaves + k];
  __syncthreads();
  return before;
}

// Number of rows of a work item dealt to the waves before `wave`.
__device__ __forceinline__ unsigned RowsOfEarlierWaves(const WorkItem &it, int wave) {
  const unsigned rows = it.end - it.begin;
  const unsigned full = rows / kChunkStep, rem = rows % kChunkStep;  // full rounds, rows of the last partial round
  return full * kChunkRows * (unsigned)wave + min(rem, kChunkRows * (unsigned)wave);
}

// Destination offsets of one wave: its rows going left are packed in order
// from the start of the parent's range (after those of earlier items and
// waves), its rows going right from the start of the right child's range.
__device__ __forceinline__ void WaveOffsets(const WorkItem &it, const SplitRec &s, unsigned start,
                                            unsigned lefts_before, int wave, unsigned *lo, unsigned *ro) {
  const unsigned rows_before = (it.begin - start) + RowsOfEarlierWaves(it, wave);
  *lo = start + lefts_before;
  *ro = start + (unsigned)s.left.c + rows_before - lefts_before;
}

// Position of the k-th (0-based) set bit of the wave-uniform mask m; k < popcount(m).
__device__ __forceinline__ int SelectBit(unsigned long long m, unsigned k) {
  const unsigned lo = (unsigned)m, hi = (unsigned)(m >> 32);
  unsigned c = (unsigned)__popc(lo);
  const bool up = k >= c;
  unsigned word = up ? hi : lo;
  int pos = up ? 32 : 0;
  k = up ? k - c : k;
#pragma unroll
  for (int width = 16; width >= 1; width >>= 1) {
    const unsigned low = word & ((1u << width) - 1u);
    c = (unsigned)__popc(low);
    const bool u = k >= c;
    word = u ? (word >> width) : low;
    pos += u ? width : 0;
    k = u ? k - c : k;
  }
  return pos;
}

// Two rows per lane of a wave's 128-row chunk, as loaded.
template <int NQ>
struct RowSet {
  uint32_t b0[NQ], b1[NQ];
  uint32_t s0, s1;  // word of the split feature when it is not among b0/b1
  float g0, g1, h0, h1;
};

// A wave's register-resident queue of rows on their way to one child's row
// range: lane l holds the row whose destination is base + l, lanes [0, n) are
// occupied, and on a wave's first batch lanes [0, skip) stand for the rows
// before the wave's own range (base is a multiple of 64 rows, so every batch
// is written as one aligned, fully coalesced 256-byte store per array).
template <int NQ>
struct RowQueue {
  uint32_t b[NQ];
  float g, h;
  unsigned n, skip, base;
  __device__ __forceinline__ void Init(unsigned first_row) {
#pragma unroll
    for (int q = 0; q < NQ; ++q) b[q] = 0;
    g = h = 0.0f;
    n = skip = first_row & 63u;
    base = first_row - n;
  }
};

// Writes lanes [from, to) of Q to their destination and, for the child whose
// histogram is built, adds them to the LDS histogram.
// HIST: the kernel builds a histogram; GH: the gradients move with the rows.
template <bool PAIR, int NQ, bool HIST = true, bool GH = true>
__device__ __forceinline__ void EmitRows(unsigned long long *__restrict__ lds, const RowQueue<NQ> &Q,
                                         unsigned from, unsigned to, bool built,
                                         uint32_t *__restrict__ bins_out, size_t stride,
                                         float *__restrict__ g_out, float *__restrict__ h_out, int lane,
                                         int sg, int sh, int F) {
  if ((unsigned)lane >= from && (unsigned)lane < to) {
    // streaming stores and loads: the pass touches every byte once
    const unsigned d = Q.base + (unsigned)lane;
#pragma unroll
    for (int q = 0; q < NQ; ++q) __builtin_nontemporal_store(Q.b[q], &bins_out[(size_t)q * stride + d]);
    if (GH && g_out != nullptr) {  // a group pass after the first leaves the gradients alone
      __builtin_nontemporal_store(Q.g, &g_out[d]);
      if (PAIR) __builtin_nontemporal_store(Q.h, &h_out[d]);
    }
    if (HIST && built) AccumulateRow<PAIR, NQ>(lds, Q.b, Q.g, Q.h, sg, sh, 0, F);
  }
}

// Appends the rows of X flagged in xm (wave-uniform mask, one row per lane) to
// Q in row order with one lane permute per register; a full queue is emitted
// and the rest of X starts the next batch.
template <bool PAIR, int NQ, bool HIST = true, bool GH = true>
__device__ __forceinline__ void MergeRows(unsigned long long *__restrict__ lds, RowQueue<NQ> &Q,
                                          const uint32_t (&xb)[NQ], float xg, float xh,
                                          unsigned long long xm, bool built,
                                          uint32_t *__restrict__ bins_out, size_t stride,
                                          float *__restrict__ g_out, float *__restrict__ h_out, int lane,
                                          int sg, int sh, int F) {
  const unsigned nx = (unsigned)__popcll(xm);
  if (nx == 0) return;  // wave-uniform
  // lane l receives the k-th flagged row, k = (l - n) mod 64: lanes >= n fill
  // the current batch, lanes < n hold what overflows into the next one
  const unsigned k = ((unsigned)lane - Q.n) & 63u;
  const int src = SelectBit(xm, k < nx ? k : 0u);
  uint32_t vb[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q) vb[q] = (uint32_t)__shfl((int)xb[q], src);
  const float vg = GH ? __shfl(xg, src) : 0.0f;
  const float vh = GH && PAIR ? __shfl(xh, src) : 0.0f;
  if (Q.n + nx >= 64u) {  // wave-uniform: the batch is complete
    const bool fill = (unsigned)lane >= Q.n;
#pragma unroll
    for (int q = 0; q < NQ; ++q) Q.b[q] = fill ? vb[q] : Q.b[q];
    Q.g = fill ? vg : Q.g;
    Q.h = fill ? vh : Q.h;
    EmitRows<PAIR, NQ, HIST, GH>(lds, Q, Q.skip, 64u, built, bins_out, stride, g_out, h_out, lane, sg, sh, F);
    Q.base += 64u;
    Q.skip = 0u;
#pragma unroll
    for (int q = 0; q < NQ; ++q) Q.b[q] = vb[q];
    Q.g = vg;
    Q.h = vh;
    Q.n = Q.n + nx - 64u;
  } else {
    const bool fill = (unsigned)lane >= Q.n && k < nx;
#pragma unroll
    for (int q = 0; q < NQ; ++q) Q.b[q] = fill ? vb[q] : Q.b[q];
    Q.g = fill ? vg : Q.g;
    Q.h = fill ? vh : Q.h;
    Q.n += nx;
  }
}

// Fused pass over the rows of the parent nodes of a level: stable partition
// into the children order (WRITE) and histogram of the smaller child of every
// split in LDS.  Each wave owns the 128-row chunks v, v + 16, ... of the item
// and runs without workgroup barriers.  With WRITE the rows of a chunk are
// sorted into two register queues (one per child) with lane permutes; a full
// queue is one aligned 64-row store per array, and the queue of the built
// child is added to the histogram as a full wave (LDS atomic instructions
// cost the same with one active lane as with 64).  Writing each chunk's rows
// directly, as two short unaligned runs per store, costs 40 % more time than
// the copy itself.  On the last level only the quad of the split feature is
// read for every row; the selected rows are queued by row id and read 64 at a
// time.  NQ = all quads of the matrix.
// GROUP: `bins` / `bins_out` point at quad q0 of a wider matrix (q0 a multiple
// of 4); the quad of the split feature is read from `split_bins`, the start of
// the whole matrix, and g_out may be null (the gradients moved with an
// earlier group of the same level).
template <bool PAIR, int NQ, bool WRITE, bool GROUP = false>
__global__ void __launch_bounds__(kHistThreads)
k_part_hist(const uint32_t *__restrict__ bins, uint32_t *__restrict__ bins_out, size_t stride, int F,
            const float *__restrict__ g, float *__restrict__ g_out, const float *__restrict__ h,
            float *__restrict__ h_out, const int *__restrict__ shifts,
            const SplitRec *__restrict__ split, const NodeSum *__restrict__ tot,
            const unsigned *__restrict__ seg_start, const WorkItem *__restrict__ work,
            const unsigned *__restrict__ n_work, const unsigned *__restrict__ wave_left,
            const unsigned *__restrict__ item_left, unsigned long long *__restrict__ slab,
            int slab_entries, const uint32_t *__restrict__ split_bins, int q0) {
  extern __shared__ unsigned long long lds[];
  __shared__ unsigned s_tmp[kItemWaves + 1];
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const SplitRec s = split[it.node];
  const unsigned long long cl = s.left.c, cr = tot[it.node].c - cl;
  const bool build_right = cl > cr;  // ties -> left (hist_grad_sum.cu:288-290)
  constexpr int words = (int)(HistLdsBytes(NQ, PAIR) / 8);
  for (int i = threadIdx.x; i < words; i += kHistThreads) lds[i] = 0ull;
  const int sg = shifts[0], sh = shifts[1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const unsigned wb = it.begin + wave * kChunkRows, we = it.end;
  unsigned lo = 0, ro = 0;
  if (WRITE) {
    const unsigned before = LeftsBefore(it, w, wave, wave_left, item_left, s_tmp);
    WaveOffsets(it, s, seg_start[it.node], before, wave, &lo, &ro);
  }
  __syncthreads();
  const int fq = s.fid >> 2, fs = 8 * (s.fid & 3);
  if constexpr (WRITE) {
    // QB: rows of the child whose histogram is built, QO: the other child
    RowQueue<NQ> QB, QO;
    QB.Init(build_right ? ro : lo);
    QO.Init(build_right ? lo : ro);
    // Two register sets of 128 rows each: while one is processed the other is
    // in flight.  The loads are unconditional (addresses clamped to the last
    // row of the item) and the sets are never copied, so every wait in the loop
    // is for exactly the set that is needed next.
    const uint32_t *split_col = split_bins + (size_t)(s.fid < 0 ? 0 : fq) * stride;
    auto load = [&](RowSet<NQ> &R, unsigned base) {
      const unsigned a0 = min(base + lane, we - 1), a1 = min(base + 64 + lane, we - 1);
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        R.b0[q] = __builtin_nontemporal_load(&bins[(size_t)q * stride + a0]);
        R.b1[q] = __builtin_nontemporal_load(&bins[(size_t)q * stride + a1]);
      }
      if (GROUP) {  // the quad of the split feature, wherever it lives
        R.s0 = split_col[a0];
        R.s1 = split_col[a1];
      }
      R.g0 = __builtin_nontemporal_load(&g[a0]);
      R.g1 = __builtin_nontemporal_load(&g[a1]);
      R.h0 = PAIR ? __builtin_nontemporal_load(&h[a0]) : 0.0f;
      R.h1 = PAIR ? __builtin_nontemporal_load(&h[a1]) : 0.0f;
    };
    auto process = [&](const RowSet<NQ> &R, unsigned base) {
      const unsigned r0 = base + lane, r1 = r0 + 64;
      const bool v0 = r0 < we, v1 = r1 < we;
      uint32_t s0 = 0, s1 = 0;
      if (GROUP) {
        s0 = R.s0;
        s1 = R.s1;
      } else {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          s0 = q == fq ? R.b0[q] : s0;
          s1 = q == fq ? R.b1[q] : s1;
        }
      }
      const bool right0 = v0 && s.fid >= 0 && (int)((s0 >> fs) & 255u) > s.bin;
      const bool right1 = v1 && s.fid >= 0 && (int)((s1 >> fs) & 255u) > s.bin;
      const unsigned long long b0 = __ballot(v0 && right0 == build_right), o0 = __ballot(v0 && right0 != build_right);
      const unsigned long long b1 = __ballot(v1 && right1 == build_right), o1 = __ballot(v1 && right1 != build_right);
      MergeRows<PAIR, NQ>(lds, QO, R.b0, R.g0, R.h0, o0, false, bins_out, stride, g_out, h_out, lane, sg, sh, F);
      MergeRows<PAIR, NQ>(lds, QB, R.b0, R.g0, R.h0, b0, true, bins_out, stride, g_out, h_out, lane, sg, sh, F);
      MergeRows<PAIR, NQ>(lds, QO, R.b1, R.g1, R.h1, o1, false, bins_out, stride, g_out, h_out, lane, sg, sh, F);
      MergeRows<PAIR, NQ>(lds, QB, R.b1, R.g1, R.h1, b1, true, bins_out, stride, g_out, h_out, lane, sg, sh, F);
    };
    if (wb < we) {
      RowSet<NQ> A, B;
      load(A, wb);
      for (unsigned base = wb;; base += 2 * kChunkStep) {
        load(B, base + kChunkStep);
        process(A, base);
        if (base + kChunkStep >= we) break;  // wave-uniform
        load(A, base + 2 * kChunkStep);
        process(B, base + kChunkStep);
        if (base + 2 * kChunkStep >= we) break;
      }
    }
    EmitRows<PAIR, NQ>(lds, QO, QO.skip, QO.n, false, bins_out, stride, g_out, h_out, lane, sg, sh, F);
    EmitRows<PAIR, NQ>(lds, QB, QB.skip, QB.n, true, bins_out, stride, g_out, h_out, lane, sg, sh, F);
  } else {
    // Rows selected for the histogram are queued by row id (slot 64 * j + lane
    // of the queue is lane `lane` of q[j]; slots [0, np) are occupied) and read
    // again 64 at a time: LDS atomic instructions cost the same with one active
    // lane as with 64, so only full waves are accumulated.  The second read
    // hits the cache, is requested at the start of a chunk and used at its end,
    // and the wave never waits for its LDS atomics.
    unsigned q0 = it.begin, q1 = it.begin, q2 = it.begin;
    unsigned np = 0;
    uint32_t gb[NQ];
    float gg = 0.0f, gh = 0.0f;
    auto gather = [&](bool valid) {  // requests the rows of queue slots [0, 64)
      const unsigned a = valid ? q0 : it.begin;
#pragma unroll
      for (int q = 0; q < NQ; ++q) gb[q] = bins[(size_t)q * stride + a];
      gg = g[a];
      gh = PAIR ? h[a] : 0.0f;
      q0 = q1;
      q1 = q2;
    };
    // m: wave-uniform mask of the selected rows among base + [0, 64); np < 128
    auto enqueue = [&](unsigned base, unsigned long long m) {
      const unsigned nx = (unsigned)__popcll(m);
      if (nx == 0) return;
      const unsigned r = np & 63u, j = np >> 6;
      const unsigned k = ((unsigned)lane - r) & 63u;  // slot np + k
      const unsigned id = base + (unsigned)SelectBit(m, k < nx ? k : 0u);
      const bool here = (unsigned)lane >= r && k < nx;   // lands in q[j]
      const bool next = (unsigned)lane < r && k < nx;    // lands in q[j + 1]
      q0 = (j == 0 && here) ? id : q0;
      q1 = ((j == 1 && here) || (j == 0 && next)) ? id : q1;
      q2 = (j == 1 && next) ? id : q2;
      np += nx;
    };
    // after a chunk: at most 127 rows stay queued
    auto drain = [&](unsigned limit) {
      while (np > limit) {
        const unsigned take = min(np, 64u);
        const bool valid = (unsigned)lane < take;
        gather(valid);
        if (valid) AccumulateRow<PAIR, NQ>(lds, gb, gg, gh, sg, sh, 0, F);
        np -= take;
      }
    };
    if (wb < we) {
      // last level: only the quad of the split feature decides; the selected
      // rows are read when they are accumulated
      const uint32_t *col = split_bins + (size_t)(s.fid < 0 ? 0 : fq) * stride;
      auto step = [&](uint32_t s0, uint32_t s1, uint32_t &n0, uint32_t &n1, unsigned base) {
        const bool full = np >= 64u;  // wave-uniform
        if (full) {
          gather(true);
          np -= 64u;
        }
        n0 = col[min(base + kChunkStep + lane, we - 1)];
        n1 = col[min(base + kChunkStep + 64 + lane, we - 1)];
        const unsigned r0 = base + lane, r1 = r0 + 64;
        const bool v0 = r0 < we, v1 = r1 < we;
        const bool right0 = v0 && s.fid >= 0 && (int)((s0 >> fs) & 255u) > s.bin;
        const bool right1 = v1 && s.fid >= 0 && (int)((s1 >> fs) & 255u) > s.bin;
        enqueue(base, __ballot(v0 && right0 == build_right));
        enqueue(base + 64, __ballot(v1 && right1 == build_right));
        if (full) AccumulateRow<PAIR, NQ>(lds, gb, gg, gh, sg, sh, 0, F);
        drain(127u);
      };
      uint32_t a0 = col[min(wb + lane, we - 1)], a1 = col[min(wb + 64 + lane, we - 1)], b0, b1;
      for (unsigned base = wb;; base += 2 * kChunkStep) {
        step(a0, a1, b0, b1, base);
        if (base + kChunkStep >= we) break;  // wave-uniform
        step(b0, b1, a0, a1, base + kChunkStep);
        if (base + 2 * kChunkStep >= we) break;
      }
    }
    drain(0u);
  }
  FlushSlab<PAIR, NQ>(lds, slab, w, slab_entries, q0);
}

// Stable partition alone (matrices too wide for the fused pass, 16-bit bins):
// words [q0, q0 + NQ) of every row, and with GH the gradients, go to the
// children order through the two register queues of the fused pass.  One launch
// per group of words; every launch reads the word of the split feature again.
template <bool PAIR, int NQ, bool GH>
__global__ void __launch_bounds__(kHistThreads)
k_part_rows(const uint32_t *__restrict__ bins, uint32_t *__restrict__ bins_out, size_t stride, int q0,
            const float *__restrict__ g, float *__restrict__ g_out, const float *__restrict__ h,
            float *__restrict__ h_out, const SplitRec *__restrict__ split,
            const unsigned *__restrict__ seg_start, const WorkItem *__restrict__ work,
            const unsigned *__restrict__ n_work, const unsigned *__restrict__ wave_left,
            const unsigned *__restrict__ item_left, BinCode code) {
  __shared__ unsigned s_tmp[kItemWaves + 1];
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const SplitRec s = split[it.node];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const unsigned wb = it.begin + wave * kChunkRows, we = it.end;
  unsigned lo, ro;
  const unsigned before = LeftsBefore(it, w, wave, wave_left, item_left, s_tmp);
  WaveOffsets(it, s, seg_start[it.node], before, wave, &lo, &ro);
  if (wb >= we) return;
  const uint32_t *group = bins + (size_t)q0 * stride;
  uint32_t *group_out = bins_out + (size_t)q0 * stride;
  const uint32_t *split_col = bins + (size_t)(s.fid < 0 ? 0 : code.Word(s.fid)) * stride;
  RowQueue<NQ> QL, QR;
  QL.Init(lo);
  QR.Init(ro);
  struct Rows {
    RowSet<NQ> r;
    uint32_t s0, s1;  // word of the split feature
  };
  auto load = [&](Rows &R, unsigned base) {
    const unsigned a0 = min(base + lane, we - 1), a1 = min(base + 64 + lane, we - 1);
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      R.r.b0[q] = __builtin_nontemporal_load(&group[(size_t)q * stride + a0]);
      R.r.b1[q] = __builtin_nontemporal_load(&group[(size_t)q * stride + a1]);
    }
    R.s0 = split_col[a0];
    R.s1 = split_col[a1];
    R.r.g0 = GH ? __builtin_nontemporal_load(&g[a0]) : 0.0f;
    R.r.g1 = GH ? __builtin_nontemporal_load(&g[a1]) : 0.0f;
    R.r.h0 = GH && PAIR ? __builtin_nontemporal_load(&h[a0]) : 0.0f;
    R.r.h1 = GH && PAIR ? __builtin_nontemporal_load(&h[a1]) : 0.0f;
  };
  auto process = [&](const Rows &R, unsigned base) {
    const unsigned r0 = base + lane, r1 = r0 + 64;
    const bool v0 = r0 < we, v1 = r1 < we;
    const bool right0 = v0 && s.fid >= 0 && (int)code.Bin(R.s0, s.fid) > s.bin;
    const bool right1 = v1 && s.fid >= 0 && (int)code.Bin(R.s1, s.fid) > s.bin;
    const unsigned long long lm0 = __ballot(v0 && !right0), rm0 = __ballot(right0);
    const unsigned long long lm1 = __ballot(v1 && !right1), rm1 = __ballot(right1);
    MergeRows<PAIR, NQ, false, GH>(nullptr, QL, R.r.b0, R.r.g0, R.r.h0, lm0, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
    MergeRows<PAIR, NQ, false, GH>(nullptr, QR, R.r.b0, R.r.g0, R.r.h0, rm0, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
    MergeRows<PAIR, NQ, false, GH>(nullptr, QL, R.r.b1, R.r.g1, R.r.h1, lm1, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
    MergeRows<PAIR, NQ, false, GH>(nullptr, QR, R.r.b1, R.r.g1, R.r.h1, rm1, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
  };
  Rows A, B;
  load(A, wb);
  for (unsigned base = wb;; base += 2 * kChunkStep) {
    load(B, base + kChunkStep);
    process(A, base);
    if (base + kChunkStep >= we) break;  // wave-uniform
    load(A, base + 2 * kChunkStep);
    process(B, base + kChunkStep);
    if (base + 2 * kChunkStep >= we) break;
  }
  EmitRows<PAIR, NQ, false, GH>(nullptr, QL, QL.skip, QL.n, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
  EmitRows<PAIR, NQ, false, GH>(nullptr, QR, QR.skip, QR.n, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
}

// Adds the slabs of every directly built node of a level (on top of the stored
// histogram when `accumulate`) and, with `trick`, derives its sibling as
// parent - node.  Slabs are in LDS order (16-feature blocks, bin-major); the
// histograms written here are feature-major: hist[node][f * 256 + bin].
// grid (slab_entries/64, L), 1024 threads = 64 entries x 16 slab lanes.
//   by_parent = 0: slabs belong to work items of the node itself
//               (node_items == 0xffffffff marks a derived node);
//   by_parent = 1: slabs belong to work items of the parent (fused pass); the
//               built child is the smaller one, ties -> left.
template <bool PAIR, int LANES>
__global__ void __launch_bounds__(1024)
k_hist_reduce(const unsigned long long *__restrict__ slab, int slab_entries, int nbin_total,
              const unsigned *__restrict__ node_first, const unsigned *__restrict__ node_items,
              int by_parent, const SplitRec *__restrict__ parent_split,
              const NodeSum *__restrict__ parent_tot, long long *__restrict__ hg,
              long long *__restrict__ hh, unsigned *__restrict__ hc,
              const long long *__restrict__ pg, const long long *__restrict__ ph,
              const unsigned *__restrict__ pc, int trick, int accumulate, int plain) {
  // LANES threads share the slabs of one entry; a block covers 1024 / LANES
  // consecutive entries (with 4 lanes: 16 bins x 16 features, so the
  // feature-major output is written in runs of 16 bins)
  constexpr int kEntries = 1024 / LANES;
  __shared__ long long s_g[LANES][kEntries];
  __shared__ long long s_h[LANES][kEntries];
  __shared__ unsigned s_c[LANES][kEntries];
  const int nd = blockIdx.y;
  unsigned items, first;
  if (by_parent) {
    const int p = nd >> 1;
    const unsigned long long cl = parent_split[p].left.c, cr = parent_tot[p].c - cl;
    const bool build_right = cl > cr;
    if (((nd & 1) != 0) != build_right) return;  // derived from its sibling
    items = node_items[p];
    first = node_first[p];
  } else {
    items = node_items[nd];
    first = node_first[nd];
    if (items == 0xffffffffu) return;  // derived from its sibling
  }
  const int e = threadIdx.x % kEntries, lane = threadIdx.x / kEntries;
  const int entry = blockIdx.x * kEntries + e;  // slab order
  // plain: the slabs are feature-major already (16-bit bins)
  const int f = (entry / kBlockEntries) * kBlockFeatures + (entry & (kBlockFeatures - 1));
  const int bin = (entry / kBlockFeatures) & (kSlots - 1);
  // the last 16-feature block may have fewer than 16 features
  const bool live = plain ? entry < nbin_total : f * kSlots < nbin_total;
  long long ag = 0, ah = 0;
  unsigned ac = 0;
  if (live) {
    for (unsigned s = lane; s < items; s += LANES) {
      const unsigned long long *p = slab + (size_t)(first + s) * slab_entries * (PAIR ? 2 : 1);
      const unsigned long long w0 = p[entry];
      const long long gq = ((long long)(w0 << (64 - kCountShift))) >> (64 - kCountShift);
      ag += gq;
      ac += (unsigned)((w0 - (unsigned long long)gq) >> kCountShift);
      if (PAIR) ah += (long long)p[slab_entries + entry];
    }
  }
  s_g[lane][e] = ag;
  s_h[lane][e] = ah;
  s_c[lane][e] = ac;
  __syncthreads();
  if (lane == 0 && live) {
    for (int k = 1; k < LANES; ++k) {
      ag += s_g[k][e];
      ah += s_h[k][e];
      ac += s_c[k][e];
    }
    const size_t cell = plain ? (size_t)entry : (size_t)f * kSlots + bin;
    const size_t o = (size_t)nd * nbin_total + cell;
    if (accumulate) {  // streamed matrices: one call per row block
      ag += hg[o];
      ah += hh[o];
      ac += hc[o];
    }
    hg[o] = ag;
    hh[o] = ah;
    hc[o] = ac;
    if (trick) {
      const size_t po = (size_t)(nd >> 1) * nbin_total + cell;
      const size_t so = (size_t)(nd ^ 1) * nbin_total + cell;
      hg[so] = pg[po] - ag;
      hh[so] = ph[po] - ah;
      hc[so] = pc[po] - ac;
    }
  }
}

// Root totals = sum over the slots of feature 0 of the root histogram (every
// row, NaN included, sits in exactly one slot).  Replaces the reduction over
// the gradient array of garden.cu:432-435.  One wave.
__global__ void __launch_bounds__(64)
k_root_from_hist(const long long *__restrict__ hg, const long long *__restrict__ hh,
                 NodeSum *__restrict__ tot, int slots) {
  long long a = 0, b = 0;
  for (int i = threadIdx.x; i < slots; i += 64) {
    a += hg[i];
    b += hh[i];
  }
  a = WaveSumLL(a);
  b = WaveSumLL(b);
  if (threadIdx.x == 0) {
    tot[0].g = a;
    tot[0].h = b;
  }
}

// ----------------------------------------------------- streamed row blocks
// When the bins do not live in HBM (pinned host blocks copied in at every
// level; the reference streams whole columns, hist_tree_grower.cu:335-366),
// rows are never re-ordered.  A resident node id per row is advanced with the
// parents' splits while its block is on the GPU, the rows of the nodes built
// at this level are gathered node by node into a staging buffer, and the
// ordinary histogram kernel runs on that buffer.

// Is node nd accumulated directly at this level?  With sibling subtraction
// only the smaller child of each pair, ties -> left (hist_grad_sum.cu:279-294).
__device__ __forceinline__ bool NodeIsBuilt(const NodeSum *__restrict__ tot, unsigned nd, int level, int trick) {
  if (level == 0 || !trick) return true;
  const unsigned long long c = tot[nd].c, sib = tot[nd ^ 1u].c;
  return (nd & 1u) ? (c < sib) : (c <= sib);
}

// Advances the node id of every row of the block by the parents' splits and
// counts the rows of every built node (blk_cnt, zero on entry).
__global__ void __launch_bounds__(256)
k_stream_route(const uint32_t *__restrict__ bins, size_t bstride, unsigned rows, int level, int trick,
               const SplitRec *__restrict__ split, const NodeSum *__restrict__ tot,
               unsigned *__restrict__ node_of, unsigned *__restrict__ blk_cnt) {
  __shared__ unsigned s_cnt[kMaxPlanNodes];
  const int L = 1 << level;
  for (int i = threadIdx.x; i < L; i += blockDim.x) s_cnt[i] = 0;
  __syncthreads();
  const int lane = threadIdx.x & 63;
  const unsigned step = gridDim.x * blockDim.x;
  for (unsigned r0 = blockIdx.x * blockDim.x; r0 < rows; r0 += step) {  // whole waves stay together
    const unsigned r = r0 + threadIdx.x;
    unsigned nd = 0;
    bool built = false;
    if (r < rows) {
      if (level > 0) {
        const unsigned parent = node_of[r];
        nd = parent * 2u + (GoesRight(bins, bstride, split[parent], r) ? 1u : 0u);
      }
      node_of[r] = nd;
      built = NodeIsBuilt(tot, nd, level, trick);
    }
    // one LDS atomic per distinct node of the wave (64 lanes on one address serialise)
    unsigned long long todo = __ballot(built);
    while (todo) {
      const int leader = __ffsll((long long)todo) - 1;
      const unsigned lead_nd = (unsigned)__shfl((int)nd, leader);
      const unsigned long long same = __ballot(built && nd == lead_nd);
      if (lane == leader) atomicAdd(&s_cnt[lead_nd], (unsigned)__popcll(same));
      todo &= ~same;
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < L; i += blockDim.x)
    if (s_cnt[i]) atomicAdd(&blk_cnt[i], s_cnt[i]);
}

// Row ranges of the built nodes inside the staging buffer: exclusive scan of
// blk_cnt; also the cursors of the gather and the totals the planner reads.
// Clears blk_cnt for the next block.  One workgroup.
__global__ void __launch_bounds__(1024)
k_stream_segments(unsigned *__restrict__ blk_cnt, int L, NodeSum *__restrict__ blk_tot,
                  unsigned *__restrict__ blk_seg, unsigned *__restrict__ cursor) {
  __shared__ unsigned s_wave[16];
  __shared__ unsigned s_carry;
  if (threadIdx.x == 0) s_carry = 0;
  __syncthreads();
  for (int base = 0; base < L; base += 1024) {
    const int nd = base + threadIdx.x;
    const unsigned c = nd < L ? blk_cnt[nd] : 0u;
    unsigned incl = c;
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned o = __shfl_up(incl, off);
      if ((threadIdx.x & 63) >= off) incl += o;
    }
    if ((threadIdx.x & 63) == 63) s_wave[threadIdx.x >> 6] = incl;
    __syncthreads();
    unsigned off = s_carry;
    for (int w = 0; w < (int)(threadIdx.x >> 6); ++w) off += s_wave[w];
    const unsigned excl = off + incl - c;
    if (nd < L) {
      blk_seg[nd] = excl;
      cursor[nd] = excl;
      blk_tot[nd].g = 0;
      blk_tot[nd].h = 0;
      blk_tot[nd].c = c;
      blk_cnt[nd] = 0;
    }
    __syncthreads();
    if (threadIdx.x == 1023) s_carry = excl + c;
    __syncthreads();
  }
}

// Copies the rows of the built nodes into the staging buffer, node by node.
// The order inside a node is whatever the atomics give; sums are integers.
template <bool PAIR>
__global__ void __launch_bounds__(256)
k_stream_gather(const uint32_t *__restrict__ bins, size_t bstride, int Q, unsigned rows,
                const float *__restrict__ g, const float *__restrict__ h,
                const unsigned *__restrict__ node_of, int level, int trick,
                const NodeSum *__restrict__ tot, unsigned *__restrict__ cursor,
                uint32_t *__restrict__ st_bins, size_t sstride, float *__restrict__ st_g,
                float *__restrict__ st_h) {
  const int lane = threadIdx.x & 63;
  const unsigned step = gridDim.x * blockDim.x;
  for (unsigned r0 = blockIdx.x * blockDim.x; r0 < rows; r0 += step) {  // whole waves stay together
    const unsigned r = r0 + threadIdx.x;
    unsigned nd = 0;
    bool built = false;
    if (r < rows) {
      nd = node_of[r];
      built = NodeIsBuilt(tot, nd, level, trick);
    }
    // one cursor atomic per distinct node of the wave
    unsigned d = 0;
    unsigned long long todo = __ballot(built);
    while (todo) {
      const int leader = __ffsll((long long)todo) - 1;
      const unsigned lead_nd = (unsigned)__shfl((int)nd, leader);
      const unsigned long long same = __ballot(built && nd == lead_nd);
      unsigned base = 0;
      if (lane == leader) base = atomicAdd(&cursor[lead_nd], (unsigned)__popcll(same));
      base = (unsigned)__shfl((int)base, leader);
      if (built && nd == lead_nd) d = base + RankBelow(same);
      todo &= ~same;
    }
    if (built) {
      for (int q = 0; q < Q; ++q) st_bins[(size_t)q * sstride + d] = bins[(size_t)q * bstride + r];
      st_g[d] = g[r];
      if (PAIR) st_h[d] = h[r];
    }
  }
}

// sibling = parent - built child for every node that was not built directly
__global__ void k_sibling(long long *__restrict__ hg, long long *__restrict__ hh, unsigned *__restrict__ hc,
                          const long long *__restrict__ pg, const long long *__restrict__ ph,
                          const unsigned *__restrict__ pc, const NodeSum *__restrict__ tot, int level,
                          int nbin_total) {
  const unsigned nd = blockIdx.y;
  if (NodeIsBuilt(tot, nd, level, 1)) return;
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= nbin_total) return;
  const size_t o = (size_t)nd * nbin_total + e, so = (size_t)(nd ^ 1u) * nbin_total + e,
               po = (size_t)(nd >> 1) * nbin_total + e;
  hg[o] = pg[po] - hg[so];
  hh[o] = ph[po] - hh[so];
  hc[o] = pc[po] - hc[so];
}

// --------------------------------------------------------------- split scan
struct Cand {
  float gain;
  int bin;
  NodeSum left;
};

// One wave per (feature, node): inclusive prefix over the 256 slots, gain per
// bin < hist_size, arg-max with ties to the HIGHEST bin (builder.h:39-49),
// only gains > 0 (hist_tree_grower.cu:31).
template <bool PAIR, bool F64>
__global__ void __launch_bounds__(64)
k_split_scan(const long long *__restrict__ hg, const long long *__restrict__ hh,
             const unsigned *__restrict__ hc, int nbin_total, int F, int slots,
             const NodeSum *__restrict__ tot, const int *__restrict__ shifts, GainParams gp,
             int hist_size, Cand *__restrict__ cand) {
  const int f = blockIdx.x, nd = blockIdx.y, lane = threadIdx.x;
  const NodeSum t = tot[nd];
  Cand best;
  best.gain = 0.0f;
  best.bin = -1;
  best.left.g = best.left.h = 0;
  best.left.c = 0;
  if (t.c != 0) {
    const int sg = shifts[0], sh = shifts[1];
    const double GT = FromFixed<F64>(t.g, sg);
    const double HT = PAIR ? FromFixed<F64>(t.h, sh) : 0.0;
    // sums of the slots below the current chunk of 256
    long long carry_g = 0, carry_h = 0;
    unsigned long long carry_c = 0;
    for (int chunk = 0; chunk < slots && chunk < hist_size; chunk += 256) {
      const size_t base = (size_t)nd * nbin_total + (size_t)f * slots + chunk + lane * 4;
      long long g4[4], h4[4];
      unsigned long long c4[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        g4[j] = hg[base + j];
        h4[j] = PAIR ? hh[base + j] : 0;
        c4[j] = hc[base + j];
      }
#pragma unroll
      for (int j = 1; j < 4; ++j) {
        g4[j] += g4[j - 1];
        h4[j] += h4[j - 1];
        c4[j] += c4[j - 1];
      }
      long long ig = g4[3], ih = h4[3];
      unsigned long long ic = c4[3];
      for (int off = 1; off < 64; off <<= 1) {
        const long long og = __shfl_up(ig, off);
        const long long oh = __shfl_up(ih, off);
        const unsigned long long oc = __shfl_up(ic, off);
        if (lane >= off) {
          ig += og;
          ih += oh;
          ic += oc;
        }
      }
      const long long eg = carry_g + ig - g4[3], eh = carry_h + ih - h4[3];
      const unsigned long long ec = carry_c + ic - c4[3];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int bin = chunk + lane * 4 + j;
        if (bin < hist_size) {
          const long long lg = eg + g4[j], lh = eh + h4[j];
          const unsigned long long lc = ec + c4[j];
          const double GL = FromFixed<F64>(lg, sg);
          const double HL = PAIR ? FromFixed<F64>(lh, sh) : 0.0;
          const float gn = SplitGain<PAIR, F64>(GL, HL, lc, GT, HT, t.c, gp);
          if (gn > 0.0f && gn >= best.gain) {
            best.gain = gn;
            best.bin = bin;
            best.left.g = lg;
            best.left.h = lh;
            best.left.c = lc;
          }
        }
      }
      carry_g += __shfl(ig, 63);
      carry_h += __shfl(ih, 63);
      carry_c += __shfl(ic, 63);
    }
    for (int off = 32; off > 0; off >>= 1) {
      const float og = __shfl_down(best.gain, off);
      const int ob = __shfl_down(best.bin, off);
      const long long olg = __shfl_down(best.left.g, off);
      const long long olh = __shfl_down(best.left.h, off);
      const unsigned long long olc = __shfl_down(best.left.c, off);
      if (ob >= 0 && (best.bin < 0 || og > best.gain || (og == best.gain && ob > best.bin))) {
        best.gain = og;
        best.bin = ob;
        best.left.g = olg;
        best.left.h = olh;
        best.left.c = olc;
      }
    }
  }
  if (lane == 0) cand[(size_t)nd * F + f] = best;
}

// One thread per node: best candidate over the features active at this level
// (higher gain, then lower feature id: hist_tree_grower.cu:59-60), children
// totals and row ranges, node record.  A node without a candidate keeps every
// row left.
// One wave per node: lane l looks at features l, l + 64, ...; the wave keeps
// the candidate with the highest gain, ties to the lowest feature id.
__device__ __forceinline__ void SelectNode(int nd, int lane, const Cand *__restrict__ cand, int F,
                                           const NodeSum *__restrict__ tot,
                                           const unsigned *__restrict__ seg_start,
                                           NodeSum *__restrict__ tot_next, unsigned *__restrict__ seg_next,
                                           SplitRec *__restrict__ split, int *__restrict__ t_fid,
                                           int *__restrict__ t_bin, float *__restrict__ t_gain, int heap_off,
                                           const unsigned char *__restrict__ active) {
  const NodeSum t = tot[nd];
  float gain = 0.0f;
  int fid = -1, bin = -1;
  long long lg = 0, lh = 0;
  unsigned long long lc = 0;
  if (t.c != 0) {
    for (int f = lane; f < F; f += 64) {
      if (active && !active[f]) continue;  // feature not sampled at this level
      const Cand c = cand[(size_t)nd * F + f];
      if (c.bin >= 0 && (fid < 0 || gain < c.gain)) {
        gain = c.gain;
        fid = f;
        bin = c.bin;
        lg = c.left.g;
        lh = c.left.h;
        lc = c.left.c;
      }
    }
  }
  for (int off = 32; off > 0; off >>= 1) {
    const float og = __shfl_down(gain, off);
    const int of = __shfl_down(fid, off);
    const int ob = __shfl_down(bin, off);
    const long long olg = __shfl_down(lg, off);
    const long long olh = __shfl_down(lh, off);
    const unsigned long long olc = __shfl_down(lc, off);
    if (of >= 0 && (fid < 0 || og > gain || (og == gain && of < fid))) {
      gain = og;
      fid = of;
      bin = ob;
      lg = olg;
      lh = olh;
      lc = olc;
    }
  }
  if (lane != 0) return;
  SplitRec rec;
  rec.gain = fid < 0 ? 0.0f : gain;
  rec.fid = fid;
  rec.bin = fid < 0 ? -1 : bin;
  rec.pad = 0;
  rec.left = t;
  if (fid >= 0) {
    rec.left.g = lg;
    rec.left.h = lh;
    rec.left.c = lc;
  }
  split[nd] = rec;
  NodeSum r;
  r.g = t.g - rec.left.g;
  r.h = t.h - rec.left.h;
  r.c = t.c - rec.left.c;
  tot_next[2 * nd] = rec.left;
  tot_next[2 * nd + 1] = r;
  const unsigned start = seg_start[nd];
  seg_next[2 * nd] = start;
  seg_next[2 * nd + 1] = start + (unsigned)rec.left.c;
  t_fid[heap_off + nd] = rec.fid < 0 ? 0 : rec.fid;  // garden.cu:471-481
  t_bin[heap_off + nd] = rec.fid < 0 ? -1 : rec.bin;
  t_gain[heap_off + nd] = rec.gain;
}

// grid ceil(L / 16), 1024 threads: one wave per node
__global__ void __launch_bounds__(1024)
k_split_select(const Cand *__restrict__ cand, int F, int L, const NodeSum *__restrict__ tot,
               const unsigned *__restrict__ seg_start, NodeSum *__restrict__ tot_next,
               unsigned *__restrict__ seg_next, SplitRec *__restrict__ split, int *__restrict__ t_fid,
               int *__restrict__ t_bin, float *__restrict__ t_gain, int heap_off,
               const unsigned char *__restrict__ active) {
  const int nd = blockIdx.x * 16 + (threadIdx.x >> 6);
  if (nd < L)
    SelectNode(nd, threadIdx.x & 63, cand, F, tot, seg_start, tot_next, seg_next, split, t_fid, t_bin, t_gain,
               heap_off, active);
}

// k_split_select followed, in the same workgroup, by the work plan of the
// fused pass over these nodes' rows (the plan needs the splits only for the
// row statistics).  One workgroup of 1024 threads.
__global__ void __launch_bounds__(1024)
k_select_plan(const Cand *__restrict__ cand, int F, int L, const NodeSum *__restrict__ tot,
              const unsigned *__restrict__ seg_start, NodeSum *__restrict__ tot_next,
              unsigned *__restrict__ seg_next, SplitRec *__restrict__ split, int *__restrict__ t_fid,
              int *__restrict__ t_bin, float *__restrict__ t_gain, int heap_off,
              const unsigned char *__restrict__ active, unsigned rows_per_item,
              WorkItem *__restrict__ work, unsigned *__restrict__ n_work,
              unsigned *__restrict__ node_first, unsigned *__restrict__ node_items,
              unsigned long long *__restrict__ rows_scanned, unsigned max_items,
              unsigned *__restrict__ overflow) {
  for (int nd = threadIdx.x >> 6; nd < L; nd += 16)
    SelectNode(nd, threadIdx.x & 63, cand, F, tot, seg_start, tot_next, seg_next, split, t_fid, t_bin, t_gain,
               heap_off, active);
  __syncthreads();  // the splits written above are read by the plan
  PlanBody(tot, seg_start, L, 0, rows_per_item, work, n_work, node_first, node_items, rows_scanned, split,
           max_items, overflow);
}

// --------------------------------------------------------------- leaves
// UpdateLeafWeight (garden.cu:487-503, split.cu:25-35): left = Weight(left
// sum), right = Weight(parent - left) with the subtraction in the sum type.
template <bool PAIR, bool F64>
__global__ void k_leaf_weights(const SplitRec *__restrict__ split, const NodeSum *__restrict__ tot,
                               int L, const int *__restrict__ shifts, GainParams gp, float eta,
                               float *__restrict__ weights) {
  const int nd = blockIdx.x * blockDim.x + threadIdx.x;
  if (nd >= L) return;
  const int sg = shifts[0], sh = shifts[1];
  const SplitRec s = split[nd];
  const NodeSum t = tot[nd];
  const double GL = FromFixed<F64>(s.left.g, sg), HL = PAIR ? FromFixed<F64>(s.left.h, sh) : 0.0;
  const double GP = FromFixed<F64>(t.g, sg), HP = PAIR ? FromFixed<F64>(t.h, sh) : 0.0;
  double GR, HR;
  if (F64) {
    GR = GP - GL;
    HR = HP - HL;
  } else {
    GR = (double)((float)GP - (float)GL);
    HR = (double)((float)HP - (float)HL);
  }
  weights[2 * nd] = LeafWeight<PAIR, F64>(GL, HL, (unsigned)s.left.c, gp) * eta;
  weights[2 * nd + 1] = LeafWeight<PAIR, F64>(GR, HR, (unsigned)(t.c - s.left.c), gp) * eta;
}

// End of a tree, rows in original order: walk the tree on the row's bins
// (bin >= q+1 goes right, builder.h:107-123), record the leaf, add its weight
// to y_hat (update_by_last_tree, garden.cu:45-76) and, when NEXT_GRAD is not
// 0, write the gradients of the next round (objective.cu:28-56):
// 1 = squared (also max |g|), 2 = logistic.
// NQ > 0: the matrix has NQ quads, all loaded up front (coalesced, independent
// loads) and selected in registers; NQ == 0: any width, one dependent 4-byte
// load per level.
template <int NEXT_GRAD, int NQ>
__global__ void __launch_bounds__(256)
k_final(const uint32_t *__restrict__ bins, size_t stride, const int *__restrict__ t_fid,
        const int *__restrict__ t_bin, int depth, const float *__restrict__ weights,
        float *__restrict__ yhat, const float *__restrict__ y, unsigned *__restrict__ leaf_of,
        float *__restrict__ g, float *__restrict__ h, unsigned *__restrict__ gmax_bits, size_t n,
        BinCode code) {
  extern __shared__ int s_nodes[];  // fid[internal], bin[internal]
  const int internal = (1 << (depth - 1)) - 1;
  for (int i = threadIdx.x; i < internal; i += blockDim.x) {
    s_nodes[i] = t_fid[i];
    s_nodes[internal + i] = t_bin[i];
  }
  __syncthreads();
  float m = 0.0f;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    uint32_t b[NQ > 0 ? NQ : 1];
#pragma unroll
    for (int q = 0; q < NQ; ++q) b[q] = __builtin_nontemporal_load(&bins[(size_t)q * stride + i]);
    const float yh0 = yhat[i];
    const float yv = NEXT_GRAD != 0 ? __builtin_nontemporal_load(&y[i]) : 0.0f;
    unsigned node = 0;
    for (int level = 0; level + 1 < depth; ++level) {
      const int id = (1 << level) - 1 + (int)node;
      const int fid = s_nodes[id], bin = s_nodes[internal + id];
      unsigned right = 0;
      if (bin >= 0) {
        if (NQ > 0) {  // 8-bit bins, all quads in registers
          uint32_t b4 = 0;
          const int fq = fid >> 2;
#pragma unroll
          for (int q = 0; q < NQ; ++q) b4 = q == fq ? b[q] : b4;
          right = (int)((b4 >> (8 * (fid & 3))) & 255u) > bin ? 1u : 0u;
        } else {
          right = (int)code.Bin(bins[(size_t)code.Word(fid) * stride + i], fid) > bin ? 1u : 0u;
        }
      }
      node = node * 2 + right;
    }
    __builtin_nontemporal_store(node, &leaf_of[i]);
    const float yh = yh0 + weights[node];
    yhat[i] = yh;
    if (NEXT_GRAD == 1) {
      const float v = yv - yh;
      g[i] = v;
      const float a = fabsf(v);
      if (a > m) m = a;
    } else if (NEXT_GRAD == 2) {
      const float s = SigmoidF(yh);
      g[i] = yv - s;
      h[i] = s * (1.0f - s);
    }
  }
  if (NEXT_GRAD == 1) {
    m = WaveMaxF(m);
    if ((threadIdx.x & 63) == 0) atomicMax(gmax_bits, __float_as_uint(m));
  }
}

// Last pass of a tree fused with the root histogram of the next one
// (logistic objective, resident matrix, all quads in one LDS histogram): the
// rows are read once; the leaf walk, the prediction update and the new
// gradients are bound by HBM, the histogram by LDS atomics, and they overlap.
// One workgroup per root work item; LDS: histogram, then the node arrays.
template <int NQ>
__global__ void __launch_bounds__(kHistThreads)
k_final_hist(const uint32_t *__restrict__ bins, size_t stride, int F, const int *__restrict__ t_fid,
             const int *__restrict__ t_bin, int depth, const float *__restrict__ weights,
             float *__restrict__ yhat, const float *__restrict__ y, unsigned *__restrict__ leaf_of,
             float *__restrict__ g, float *__restrict__ h, const int *__restrict__ shifts,
             const WorkItem *__restrict__ work, const unsigned *__restrict__ n_work,
             unsigned long long *__restrict__ slab, int slab_entries) {
  extern __shared__ unsigned long long lds[];
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  constexpr int words = (int)(HistLdsBytes(NQ, true) / 8);
  int *s_nodes = reinterpret_cast<int *>(lds + words);  // fid[internal], bin[internal]
  const int internal = (1 << (depth - 1)) - 1;
  for (int i = threadIdx.x; i < words; i += kHistThreads) lds[i] = 0ull;
  for (int i = threadIdx.x; i < internal; i += kHistThreads) {
    s_nodes[i] = t_fid[i];
    s_nodes[internal + i] = t_bin[i];
  }
  __syncthreads();
  const int sg = shifts[0], sh = shifts[1];
  auto row = [&](const uint32_t (&b)[NQ], float p, float yv, unsigned r) {
    unsigned node = 0;
    for (int level = 0; level + 1 < depth; ++level) {
      const int id = (1 << level) - 1 + (int)node;
      const int fid = s_nodes[id], bin = s_nodes[internal + id];
      unsigned right = 0;
      if (bin >= 0) {
        uint32_t b4 = 0;
        const int fq = fid >> 2;
#pragma unroll
        for (int q = 0; q < NQ; ++q) b4 = q == fq ? b[q] : b4;
        right = (int)((b4 >> (8 * (fid & 3))) & 255u) > bin ? 1u : 0u;
      }
      node = node * 2 + right;
    }
    __builtin_nontemporal_store(node, &leaf_of[r]);
    const float yh = p + weights[node];
    yhat[r] = yh;
    const float s = SigmoidF(yh);
    const float gv = yv - s, hv = s * (1.0f - s);
    g[r] = gv;
    h[r] = hv;
    AccumulateRow<true, NQ>(lds, b, gv, hv, sg, sh, 0, F);
  };
  for (unsigned base = it.begin; base < it.end; base += 2 * kHistThreads) {
    const unsigned r0 = base + threadIdx.x, r1 = r0 + kHistThreads;
    const bool v0 = r0 < it.end, v1 = r1 < it.end;
    const unsigned a0 = v0 ? r0 : it.begin, a1 = v1 ? r1 : it.begin;
    uint32_t b0[NQ], b1[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      b0[q] = __builtin_nontemporal_load(&bins[(size_t)q * stride + a0]);
      b1[q] = __builtin_nontemporal_load(&bins[(size_t)q * stride + a1]);
    }
    const float p0 = yhat[a0], p1 = yhat[a1];
    const float y0 = __builtin_nontemporal_load(&y[a0]), y1 = __builtin_nontemporal_load(&y[a1]);
    if (v0) row(b0, p0, y0, r0);
    if (v1) row(b1, p1, y1, r1);
  }
  FlushSlab<true, NQ>(lds, slab, w, slab_entries, 0);
}

// Tree record of the tree just grown into one slot of the record ring:
// fid[internal], bin[internal], gain[internal], weights[leaves], overflow flag.
__global__ void k_pack_record(const int *__restrict__ t_fid, const int *__restrict__ t_bin,
                              const float *__restrict__ t_gain, const float *__restrict__ weights,
                              const unsigned *__restrict__ overflow, int internal, int leaves,
                              uint32_t *__restrict__ out) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < internal) {
    out[i] = (uint32_t)t_fid[i];
    out[internal + i] = (uint32_t)t_bin[i];
    out[2 * internal + i] = __float_as_uint(t_gain[i]);
  }
  if (i < leaves) out[3 * internal + i] = __float_as_uint(weights[i]);
  if (i == 0) out[3 * internal + leaves] = *overflow;
}

__global__ void k_fill_f32(float *p, float v, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x)
    p[i] = v;
}

template <typename T>
T *DevAlloc(size_t n) {
  void *p = nullptr;
  HIP_OK(hipMalloc(&p, std::max<size_t>(n, 1) * sizeof(T)));
  return static_cast<T *>(p);
}

inline int GridFor(size_t n, int block, int cap = 4096) {
  size_t g = (n + block - 1) / block;
  return (int)std::max<size_t>(1, std::min<size_t>(g, cap));
}

}  // namespace

struct DeviceMatrix {
  size_t rows = 0, stride = 0;
  int F = 0, Q = 0;          // Q words of 32 bits per row
  int bits = 8;              // bits per bin id: 8 (four features per word) or 16 (two)
  int slots = kSlots;        // histogram slots per feature
  uint32_t *bins = nullptr;  // resident: [Q][stride] in HBM
  // streamed: pinned host blocks [Q][block_rows], block b = rows [b*block_rows, ...)
  bool streamed = false;
  size_t block_rows = 0;
  std::vector<uint32_t *> host_blocks;
};

// Plain device-to-device copy of `bytes` bytes: a kernel of exactly known HBM
// traffic, used to scale hardware traffic counters in profiles.
__global__ void k_copy_probe(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

void CopyProbe(size_t bytes) {
  const size_t n16 = bytes / 16;
  uint4 *src = nullptr, *dst = nullptr;
  HIP_OK(hipMalloc((void **)&src, n16 * 16));
  HIP_OK(hipMalloc((void **)&dst, n16 * 16));
  HIP_OK(hipMemset(src, 1, n16 * 16));
  HIP_OK(hipDeviceSynchronize());
  hipLaunchKernelGGL(k_copy_probe, dim3(4096), dim3(256), 0, 0, src, dst, n16);
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipFree(src));
  HIP_OK(hipFree(dst));
}

int DeviceCount() {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}

void FreeDeviceMatrix(DeviceMatrix *m) {
  if (!m) return;
  if (m->bins) (void)hipFree(m->bins);
  for (uint32_t *b : m->host_blocks)
    if (b) (void)hipHostFree(b);
  delete m;
}

void QuantiseOnDevice(DataMatrix *data, int hist_size, bool verbose, bool streamed, size_t block_rows) {
  if (data->quantised) {
    if (data->hist_size != hist_size) throw std::runtime_error("data matrix was quantised with another hist_size");
    return;
  }
  if (hist_size < 1) throw std::runtime_error("hist_size must be positive");
  const size_t n = data->rows;
  const int F = (int)data->columns_dense;
  if (n == 0 || F == 0) throw std::runtime_error("empty data matrix");
  if (n >= (1ull << 31)) throw std::runtime_error("too many rows");
  std::unique_ptr<DeviceMatrix, void (*)(DeviceMatrix *)> dm(new DeviceMatrix(), FreeDeviceMatrix);
  dm->rows = n;
  dm->F = F;
  dm->Q = (F + 3) / 4;
  dm->stride = (n + 63) / 64 * 64;
  dm->streamed = streamed;
  uint32_t *d_col = nullptr;  // streamed: one quad column at a time on the device
  size_t nblocks = 0;
  if (streamed) {
    // default: 16M-row blocks (2 GB of bins at 128 features), large enough that
    // the per-block fixed costs vanish against the PCIe copy
    if (block_rows == 0) block_rows = std::min<size_t>(n, (size_t)1 << 24);
    if (block_rows < 64) block_rows = 64;
    block_rows = (block_rows + 63) / 64 * 64;
    dm->block_rows = block_rows;
    nblocks = (n + block_rows - 1) / block_rows;
    dm->host_blocks.assign(nblocks, nullptr);
    for (size_t b = 0; b < nblocks; ++b)
      HIP_OK(hipHostMalloc((void **)&dm->host_blocks[b], (size_t)dm->Q * block_rows * sizeof(uint32_t), hipHostMallocDefault));
    d_col = DevAlloc<uint32_t>(dm->stride);
  } else {
    dm->bins = DevAlloc<uint32_t>((size_t)dm->Q * dm->stride);
  }
  // streamed: quad q of all rows (in d_col) -> its slice of every host block
  auto store_quad = [&](int q) {
    for (size_t b = 0; b < nblocks; ++b) {
      const size_t r0 = b * block_rows, rows = std::min(block_rows, n - r0);
      HIP_OK(hipMemcpy(dm->host_blocks[b] + (size_t)q * block_rows, d_col + r0, rows * sizeof(uint32_t),
                       hipMemcpyDeviceToHost));
    }
  };
  data->thresholds.assign(F, {});
  data->reduced_size.assign(F, 0);

  if (data->is_prebinned) {
    for (int f = 0; f < F; ++f) {
      data->thresholds[f].resize(hist_size);
      for (int k = 0; k < hist_size; ++k) data->thresholds[f][k] = (float)k + 0.5f;
      data->reduced_size[f] = std::min(hist_size, kSlots);
    }
    if (!streamed) {
      uint8_t *d_in = DevAlloc<uint8_t>(n * F);
      HIP_OK(hipMemcpy(d_in, data->prebinned.data(), n * F, hipMemcpyHostToDevice));
      hipLaunchKernelGGL(k_pack_prebinned, dim3(GridFor(n, 256)), dim3(256), 0, 0, d_in, F, dm->Q,
                         dm->bins, dm->stride, n);
      HIP_OK(hipDeviceSynchronize());
      HIP_OK(hipFree(d_in));
    } else {
      // pack block by block: row-major bytes up, quads down into the pinned block
      uint8_t *d_in = DevAlloc<uint8_t>(block_rows * F);
      uint32_t *d_out = DevAlloc<uint32_t>((size_t)dm->Q * block_rows);
      for (size_t b = 0; b < nblocks; ++b) {
        const size_t r0 = b * block_rows, rows = std::min(block_rows, n - r0);
        HIP_OK(hipMemcpy(d_in, data->prebinned.data() + r0 * F, rows * F, hipMemcpyHostToDevice));
        hipLaunchKernelGGL(k_pack_prebinned, dim3(GridFor(rows, 256)), dim3(256), 0, 0, d_in, F, dm->Q, d_out,
                           block_rows, rows);
        HIP_OK(hipMemcpy(dm->host_blocks[b], d_out, (size_t)dm->Q * block_rows * sizeof(uint32_t), hipMemcpyDeviceToHost));
      }
      HIP_OK(hipFree(d_in));
      HIP_OK(hipFree(d_out));
      std::vector<uint8_t>().swap(data->prebinned);  // the pinned blocks are the only copy from here on
    }
  } else {
    // per quad: upload four columns, thresholds by device sort, bin assignment
    std::unique_ptr<SortWorkspace, void (*)(SortWorkspace *)> ws(CreateSortWorkspace(n, hist_size), FreeSortWorkspace);
    float *d_x = DevAlloc<float>(4 * n);
    float *d_thr = DevAlloc<float>(4 * (size_t)hist_size);
    int *d_size = DevAlloc<int>(4);
    // Columns go through two pinned staging buffers: the next column is copied
    // there by host threads while the GPU sorts the current one, and the copy
    // to the device runs at the full host-to-device rate.
    float *stage[2] = {nullptr, nullptr};
    for (int k = 0; k < 2; ++k) HIP_OK(hipHostMalloc((void **)&stage[k], n * sizeof(float), hipHostMallocDefault));
    auto stage_column = [&](int f, int slot) {
      const float *src = data->data[f].data();
      float *dst = stage[slot];
      ParallelFor(n, [&](size_t b, size_t e) { std::memcpy(dst + b, src + b, (e - b) * sizeof(float)); });
    };
    // One pass over the columns with `bits` bits per bin id; false when a
    // feature needs more ids than 8 bits hold.
    auto quantise_columns = [&](int bits) -> bool {
      const int W = 32 / bits;  // features per word
      stage_column(0, 0);
      for (int q = 0; q < dm->Q; ++q) {
        const int nc = std::min(W, F - q * W);
        int sizes[4] = {0, 0, 0, 0};
        for (int c = 0; c < nc; ++c) {
          const int f = q * W + c;
          std::thread next;
          if (f + 1 < F) next = std::thread(stage_column, f + 1, (f + 1) & 1);
          struct Joiner {
            std::thread &t;
            ~Joiner() { if (t.joinable()) t.join(); }
          } joiner{next};
          HIP_OK(hipMemcpy(d_x + (size_t)c * n, stage[f & 1], n * sizeof(float), hipMemcpyHostToDevice));
          bool has_nan = false;
          DeviceThresholds(ws.get(), d_x + (size_t)c * n, &data->thresholds[f], &data->reduced_size[f], &has_nan);
          if (bits == 8 && data->reduced_size[f] + (has_nan ? 1 : 0) > kSlots) return false;
          if (verbose)
            printf("feature %d has been reduced to %d bits \n", f,
                   32 - __builtin_clz((unsigned)data->reduced_size[f]));
          HIP_OK(hipMemcpy(d_thr + (size_t)c * hist_size, data->thresholds[f].data(),
                           hist_size * sizeof(float), hipMemcpyHostToDevice));
          sizes[c] = data->reduced_size[f];
        }
        HIP_OK(hipMemcpy(d_size, sizes, sizeof(sizes), hipMemcpyHostToDevice));
        uint32_t *out = streamed ? d_col : dm->bins + (size_t)q * dm->stride;
        if (bits == 8)
          hipLaunchKernelGGL(k_bin_assign, dim3(GridFor(n, 256)), dim3(256), 0, 0, d_x, nc, d_thr, hist_size, d_size,
                             out, n);
        else
          hipLaunchKernelGGL(k_bin_assign_wide, dim3(GridFor(n, 256)), dim3(256),
                             2 * (size_t)hist_size * sizeof(float), 0, d_x, nc, d_thr, hist_size, d_size, out, n);
        HIP_OK(hipGetLastError());
        HIP_OK(hipDeviceSynchronize());
        if (streamed) store_quad(q);
      }
      return true;
    };
    if (!quantise_columns(8)) {
      // Some feature has more than 256 bin ids: 16-bit bins, two features per
      // word, hist_size + 1 slots per feature rounded up to a power of two.
      if (streamed) throw std::runtime_error("a feature needs more than 256 bin ids: 16-bit bins are not built for streamed matrices");
      int slots = kSlots;
      while (slots < hist_size + 1) slots *= 2;
      if (slots > kMaxWideSlots) throw std::runtime_error("hist_size above 4095 is not supported");
      HIP_OK(hipFree(dm->bins));
      dm->bins = nullptr;
      dm->bits = 16;
      dm->slots = slots;
      dm->Q = (F + 1) / 2;
      dm->bins = DevAlloc<uint32_t>((size_t)dm->Q * dm->stride);
      if (!quantise_columns(16)) throw std::runtime_error("internal: 16-bit quantisation failed");
    }
    HIP_OK(hipFree(d_x));
    HIP_OK(hipFree(d_thr));
    HIP_OK(hipFree(d_size));
    for (int k = 0; k < 2; ++k) HIP_OK(hipHostFree(stage[k]));
  }
  if (d_col) HIP_OK(hipFree(d_col));
  if (streamed) {
    data->stream_blocks = dm->host_blocks;
    data->stream_block_rows = block_rows;
  }
  data->device = dm.release();
  data->hist_size = hist_size;
  data->quantised = true;
}

void GetBinLayout(const DataMatrix &data, int *bits, int *slots) {
  const DeviceMatrix *dm = data.device;
  if (!dm) throw std::runtime_error("data matrix is not quantised");
  *bits = dm->bits;
  *slots = dm->slots;
}

void GetDeviceBins16(const DataMatrix &data, uint16_t *out) {
  const DeviceMatrix *dm = data.device;
  if (!dm) throw std::runtime_error("data matrix is not quantised");
  if (dm->bits != 16) throw std::runtime_error("the matrix has 8-bit bins");
  std::vector<uint32_t> q((size_t)dm->Q * dm->stride);
  HIP_OK(hipMemcpy(q.data(), dm->bins, q.size() * sizeof(uint32_t), hipMemcpyDeviceToHost));
  for (size_t r = 0; r < dm->rows; ++r)
    for (int f = 0; f < dm->F; ++f)
      out[r * dm->F + f] = (uint16_t)(q[(size_t)(f >> 1) * dm->stride + r] >> (16 * (f & 1)));
}

void GetDeviceBins(const DataMatrix &data, uint8_t *out) {
  const DeviceMatrix *dm = data.device;
  if (!dm) throw std::runtime_error("data matrix is not quantised");
  if (dm->bits != 8) throw std::runtime_error("the matrix has 16-bit bins");
  if (dm->streamed) {
    for (size_t r = 0; r < dm->rows; ++r) {
      const uint32_t *blk = dm->host_blocks[r / dm->block_rows];
      for (int f = 0; f < dm->F; ++f)
        out[r * dm->F + f] = (uint8_t)(blk[(size_t)(f >> 2) * dm->block_rows + r % dm->block_rows] >> (8 * (f & 3)));
    }
    return;
  }
  std::vector<uint32_t> q((size_t)dm->Q * dm->stride);
  HIP_OK(hipMemcpy(q.data(), dm->bins, q.size() * sizeof(uint32_t), hipMemcpyDeviceToHost));
  for (size_t r = 0; r < dm->rows; ++r)
    for (int f = 0; f < dm->F; ++f)
      out[r * dm->F + f] = (uint8_t)(q[(size_t)(f >> 2) * dm->stride + r] >> (8 * (f & 3)));
}

// ===================================================================== builder
namespace {

struct RowBuffers {
  uint32_t *bins = nullptr;
  float *g = nullptr, *h = nullptr;
};

// Raises the dynamic LDS limit of a kernel once (needed above 64 KB).
template <typename K>
void AllowLds(K kernel, size_t bytes) {
  static size_t allowed = 0;  // one instance per kernel type/pointer value below
  (void)allowed;
  HIP_OK(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
}

template <bool PAIR, int NQ>
void LaunchHistNQ(hipStream_t st, unsigned grid, const uint32_t *bins, size_t stride, int q0, int F,
                  const float *g, const float *h, const int *shifts, const WorkItem *work,
                  const unsigned *n_work, unsigned long long *slab, int slab_entries) {
  const size_t lds = HistLdsBytes(NQ, PAIR);
  static bool configured = false;
  if (!configured) {
    AllowLds(k_hist<PAIR, NQ>, lds);
    configured = true;
  }
  hipLaunchKernelGGL((k_hist<PAIR, NQ>), dim3(grid), dim3(kHistThreads), lds, st, bins, stride, q0, F, g, h,
                     shifts, work, n_work, slab, slab_entries);
}

template <bool PAIR>
void LaunchHist(int nq, hipStream_t st, unsigned grid, const uint32_t *bins, size_t stride, int q0, int F,
                const float *g, const float *h, const int *shifts, const WorkItem *work,
                const unsigned *n_work, unsigned long long *slab, int slab_entries) {
#define ARB_CASE(N) \
  case N: LaunchHistNQ<PAIR, N>(st, grid, bins, stride, q0, F, g, h, shifts, work, n_work, slab, slab_entries); break;
  switch (nq) {
    ARB_CASE(1) ARB_CASE(2) ARB_CASE(3) ARB_CASE(4) ARB_CASE(5) ARB_CASE(6) ARB_CASE(7) ARB_CASE(8)
    default: throw std::runtime_error("internal: bad quad count");
  }
#undef ARB_CASE
}

struct FusedArgs {
  const uint32_t *bins;
  uint32_t *bins_out;
  size_t stride;
  int F;
  const float *g;
  float *g_out;
  const float *h;
  float *h_out;
  const int *shifts;
  const SplitRec *split;
  const NodeSum *tot;
  const unsigned *seg_start;
  const WorkItem *work;
  const unsigned *n_work;
  const unsigned *wave_left;
  const unsigned *item_left;
  unsigned long long *slab;
  int slab_entries;
  const uint32_t *split_bins;  // start of the whole matrix
  int q0;                      // first quad of this launch
};

template <bool PAIR, int NQ, bool WRITE, bool GROUP>
void LaunchFusedNQ(hipStream_t st, unsigned grid, const FusedArgs &a) {
  const size_t lds = HistLdsBytes(NQ, PAIR);
  static bool configured = false;
  if (!configured) {
    AllowLds(k_part_hist<PAIR, NQ, WRITE, GROUP>, lds);
    configured = true;
  }
  hipLaunchKernelGGL((k_part_hist<PAIR, NQ, WRITE, GROUP>), dim3(grid), dim3(kHistThreads), lds, st,
                     a.bins + (size_t)a.q0 * a.stride, a.bins_out ? a.bins_out + (size_t)a.q0 * a.stride : nullptr,
                     a.stride, a.F, a.g, a.g_out, a.h, a.h_out, a.shifts, a.split, a.tot, a.seg_start, a.work,
                     a.n_work, a.wave_left, a.item_left, a.slab, a.slab_entries, a.split_bins, a.q0);
}

template <bool PAIR, bool WRITE, bool GROUP>
void LaunchFused(int nq, hipStream_t st, unsigned grid, const FusedArgs &a) {
#define ARB_CASE(N) \
  case N: LaunchFusedNQ<PAIR, N, WRITE, GROUP>(st, grid, a); break;
  switch (nq) {
    ARB_CASE(1) ARB_CASE(2) ARB_CASE(3) ARB_CASE(4) ARB_CASE(5) ARB_CASE(6) ARB_CASE(7) ARB_CASE(8)
    default: throw std::runtime_error("internal: bad quad count");
  }
#undef ARB_CASE
}

class HipTreeBuilder : public TreeBuilder {
 public:
  HipTreeBuilder(const Configuration &cfg, DataMatrix *data) : cfg_(cfg), data_(data) {
    dm_ = data->device;
    n_ = dm_->rows;
    F_ = dm_->F;
    Q_ = dm_->Q;
    stride_ = dm_->stride;
    K_ = (int)cfg.tree.labels_count;
    D_ = (int)cfg.tree.depth;
    pair_ = cfg.objective != kLinearRegression;
    f64_ = cfg.internal.double_precision;
    trick_ = cfg.internal.use_hist_subtraction_trick;
    wide_ = dm_->bits == 16;
    slots_ = dm_->slots;
    code_ = BinCode::Of(dm_->bits);
    if (wide_) {
      if (dm_->streamed) throw std::runtime_error("16-bit bins are not built for streamed matrices");
      nbin_total_ = F_ * slots_;
      slab_entries_ = nbin_total_;  // slabs are feature-major
    } else {
      nbin_total_ = Q_ * 4 * kSlots;
      slab_entries_ = HistBlocks(Q_) * kBlockEntries;
    }
    if (cfg.objective >= kSoftMaxOneVsAll && K_ < 2) throw std::runtime_error("soft-max needs labels_count >= 2");
    if (cfg.objective < kSoftMaxOneVsAll && K_ != 1) throw std::runtime_error("labels_count must be 1 for this objective");
    const int last_nodes = 1 << (D_ - 2);
    if (last_nodes > kMaxPlanNodes) throw std::runtime_error("unsupported depth: at most 4096 nodes per level");
    HIP_OK(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking));

    // quads per histogram launch, limited by LDS
    // whole 16-feature blocks per launch
    const size_t per_block = HistLdsBytes(kBlockQuads, pair_);
    quads_per_group_ = (int)std::min<size_t>((kLdsBudget - 1024) / per_block * kBlockQuads, kMaxGroupQuads);
    quads_per_group_ = std::min(quads_per_group_, Q_);
    // the fused partition + histogram pass holds one histogram of all
    // features and builds only the smaller child
    fused_ = trick_ && !wide_;
    single_group_ = Q_ <= quads_per_group_;
    if (wide_) {
      // features per histogram launch (an even number, two per word)
      const size_t per_feature = (size_t)slots_ * 8 * (pair_ ? 2 : 1);
      wide_group_ = (int)std::max<size_t>(2, (kLdsBudget - 1024) / per_feature / 2 * 2);
    }

    // per-row state in original order
    d_y_ = DevAlloc<float>(n_);
    d_labels_ = DevAlloc<uint8_t>(n_);
    d_yhat_ = DevAlloc<float>(n_ * K_);
    d_g_ = DevAlloc<float>(n_ * K_);
    d_h_ = DevAlloc<float>(n_ * K_);
    d_leaf_ = DevAlloc<unsigned>(n_);
    if (!data->y.empty()) HIP_OK(hipMemcpy(d_y_, data->y.data(), n_ * sizeof(float), hipMemcpyHostToDevice));
    if (!data->labels.empty()) HIP_OK(hipMemcpy(d_labels_, data->labels.data(), n_, hipMemcpyHostToDevice));
    float init = cfg.tree.initial_y;
    if (cfg.objective == kLogisticRegression) init = std::log(init / (1 - init));  // objective.h:55-57
    hipLaunchKernelGGL(k_fill_f32, dim3(GridFor(n_ * K_, 256)), dim3(256), 0, stream_, d_yhat_, init, n_ * K_);
    data->y_hat.assign(n_ * K_, init);  // garden.cu:104

    streamed_ = dm_->streamed;
    if (streamed_) {
      const size_t br = dm_->block_rows;
      HIP_OK(hipStreamCreateWithFlags(&copy_stream_, hipStreamNonBlocking));
      for (int b = 0; b < 2; ++b) {
        blk_[b] = DevAlloc<uint32_t>((size_t)Q_ * br);
        HIP_OK(hipEventCreateWithFlags(&ev_ready_[b], hipEventDisableTiming));
        HIP_OK(hipEventCreateWithFlags(&ev_free_[b], hipEventDisableTiming));
      }
      stage_.bins = DevAlloc<uint32_t>((size_t)Q_ * br);
      stage_.g = DevAlloc<float>(br);
      stage_.h = DevAlloc<float>(br);
      d_node_of_ = DevAlloc<unsigned>(n_);
      d_blk_cnt_ = DevAlloc<unsigned>(last_nodes);
      d_blk_seg_ = DevAlloc<unsigned>(last_nodes);
      d_cursor_ = DevAlloc<unsigned>(last_nodes);
      d_blk_tot_ = DevAlloc<NodeSum>(last_nodes);
      HIP_OK(hipMemsetAsync(d_blk_cnt_, 0, (size_t)last_nodes * sizeof(unsigned), stream_));
    }
    // ping-pong row buffers in node order (not needed for a single split level)
    if (D_ > 2 && !streamed_) {
      for (int b = 0; b < 2; ++b) {
        buf_[b].bins = DevAlloc<uint32_t>((size_t)Q_ * stride_);
        buf_[b].g = DevAlloc<float>(n_);
        buf_[b].h = DevAlloc<float>(n_);
      }
    }
    // level state
    const int max_nodes = 1 << (D_ - 1);
    for (int b = 0; b < 2; ++b) {
      d_tot_[b] = DevAlloc<NodeSum>(max_nodes);
      d_seg_[b] = DevAlloc<unsigned>(max_nodes);
      d_hg_[b] = DevAlloc<long long>((size_t)last_nodes * nbin_total_);
      d_hh_[b] = DevAlloc<long long>((size_t)last_nodes * nbin_total_);
      d_hc_[b] = DevAlloc<unsigned>((size_t)last_nodes * nbin_total_);
    }
    d_split_ = DevAlloc<SplitRec>(last_nodes);
    d_cand_ = DevAlloc<Cand>((size_t)last_nodes * F_);
    d_node_first_ = DevAlloc<unsigned>(last_nodes);
    d_node_items_ = DevAlloc<unsigned>(last_nodes);
    max_hist_items_ = (unsigned)(n_ / HistRowsPerItem(n_)) + last_nodes + 2;
    max_hist_items_ = std::max<unsigned>(max_hist_items_, 1024 + last_nodes + 2);
    max_part_items_ = std::max<unsigned>((unsigned)(n_ / kPartRows + 1) + last_nodes, max_hist_items_);
    d_hwork_ = DevAlloc<WorkItem>(max_hist_items_);
    d_pwork_ = DevAlloc<WorkItem>(max_part_items_);
    d_nwork_ = DevAlloc<unsigned>(2);
    d_wave_left_ = DevAlloc<unsigned>((size_t)max_part_items_ * kItemWaves);
    d_item_left_ = DevAlloc<unsigned>(max_part_items_);
    d_slab_ = DevAlloc<unsigned long long>((size_t)std::max(max_hist_items_, max_part_items_) * slab_entries_ * (pair_ ? 2 : 1));
    d_shifts_ = DevAlloc<int>(2);
    d_records_ = DevAlloc<uint32_t>(kRecordRing * RecordWords());
    d_gmax_ = DevAlloc<unsigned>(1);
    d_rows_scanned_ = DevAlloc<unsigned long long>(1);
    d_overflow_ = DevAlloc<unsigned>(1);
    HIP_OK(hipMemsetAsync(d_overflow_, 0, sizeof(unsigned), stream_));
    HIP_OK(hipMemsetAsync(d_rows_scanned_, 0, sizeof(unsigned long long), stream_));
    HIP_OK(hipMemsetAsync(d_gmax_, 0, sizeof(unsigned), stream_));
    const int internal = (1 << (D_ - 1)) - 1;
    d_tfid_ = DevAlloc<int>(internal);
    d_tbin_ = DevAlloc<int>(internal);
    d_tgain_ = DevAlloc<float>(internal);
    d_weights_ = DevAlloc<float>(max_nodes);
    d_active_ = DevAlloc<unsigned char>((size_t)(D_ - 1) * F_);
    rnd_.seed(cfg.internal.seed);  // garden.cu:87
    int shifts[2] = {30, 0};
    if (cfg.objective == kLogisticRegression) shifts[1] = 32;  // 0 <= h <= 1/4
    if (cfg.objective >= kSoftMaxOneVsAll) shifts[1] = 31;     // 0 <= h <= 1/2
    HIP_OK(hipMemcpyAsync(d_shifts_, shifts, sizeof(shifts), hipMemcpyHostToDevice, stream_));
    HIP_OK(hipStreamSynchronize(stream_));
  }

  ~HipTreeBuilder() override {
    (void)hipStreamSynchronize(stream_);
    void *ptrs[] = {d_y_, d_labels_, d_yhat_, d_g_, d_h_, d_leaf_, d_split_, d_cand_, d_node_first_,
                    d_node_items_, d_hwork_, d_pwork_, d_nwork_, d_wave_left_, d_item_left_, d_slab_,
                    d_shifts_, d_gmax_, d_rows_scanned_, d_tfid_, d_tbin_, d_tgain_, d_weights_, d_active_, d_overflow_, d_records_};
    for (void *p : ptrs)
      if (p) (void)hipFree(p);
    for (int b = 0; b < 2; ++b) {
      void *q[] = {buf_[b].bins, buf_[b].g, buf_[b].h, d_tot_[b], d_seg_[b], d_hg_[b], d_hh_[b], d_hc_[b]};
      for (void *p : q)
        if (p) (void)hipFree(p);
    }
    for (hipEvent_t e : event_pool_) (void)hipEventDestroy(e);
    if (streamed_) {
      (void)hipStreamSynchronize(copy_stream_);
      void *sp[] = {blk_[0], blk_[1], stage_.bins, stage_.g, stage_.h, d_node_of_, d_blk_cnt_, d_blk_seg_,
                    d_cursor_, d_blk_tot_};
      for (void *p : sp)
        if (p) (void)hipFree(p);
      for (int b = 0; b < 2; ++b) {
        (void)hipEventDestroy(ev_ready_[b]);
        (void)hipEventDestroy(ev_free_[b]);
      }
      (void)hipStreamDestroy(copy_stream_);
    }
    (void)hipStreamDestroy(stream_);
  }

  void GrowRound(std::vector<RegTree> *trees) override {
    // Gradients of this round, unless the last pass of the previous tree has
    // already written them (single-output objectives, inspection off).
    if (!grad_ready_) {
      Mark(kGrad);
      if (cfg_.objective == kLinearRegression) {
        hipLaunchKernelGGL(k_grad_squared, dim3(GridFor(n_, 256)), dim3(256), 0, stream_, d_y_, d_yhat_, d_g_, n_, d_gmax_);
      } else if (cfg_.objective == kLogisticRegression) {
        hipLaunchKernelGGL(k_grad_logistic, dim3(GridFor(n_, 256)), dim3(256), 0, stream_, d_y_, d_yhat_, d_g_, d_h_, n_);
      } else {
        hipLaunchKernelGGL(k_grad_softmax, dim3(GridFor(n_, 256)), dim3(256), 0, stream_, d_labels_, d_yhat_, d_g_, d_h_, n_, K_);
      }
    }
    if (cfg_.objective == kLinearRegression)
      hipLaunchKernelGGL(k_set_shift, dim3(1), dim3(64), 0, stream_, d_gmax_, d_shifts_);
    grad_ready_ = false;
    Mark(kNone);
    owner_ = trees;
    for (int k = 0; k < K_; ++k) {
      // the record stays on the device until somebody needs it: no host
      // synchronisation between trees
      trees->emplace_back((unsigned)D_, (unsigned)k);
      GrowOne(k);
      pending_.push_back(trees->size() - 1);
      if (inspect_ || pending_.size() == kRecordRing) FlushTrees();
    }
    // phase times are read back lazily as well (GetTimings), or when many events are waiting
    if (!timing_ || marks_.size() > 8192) ResolveTimings();
  }

  // Copies the records of the trees grown since the last call to the host and
  // completes their RegTree entries (garden.cu:447-503).
  void FlushTrees() override {
    if (pending_.empty()) return;
    const int internal = (1 << (D_ - 1)) - 1, leaves = 1 << (D_ - 1);
    const size_t words = RecordWords();
    std::vector<uint32_t> rec(words * pending_.size());
    HIP_OK(hipStreamSynchronize(stream_));
    HIP_OK(hipMemcpy(rec.data(), d_records_, rec.size() * sizeof(uint32_t), hipMemcpyDeviceToHost));
    bool overflow = false;
    for (size_t k = 0; k < pending_.size(); ++k) {
      RegTree &tree = (*owner_)[pending_[k]];
      const uint32_t *r = rec.data() + k * words;
      for (int i = 0; i < internal; ++i) {
        const int fid = (int)r[i], bin = (int)r[internal + i];
        tree.fid[i] = (unsigned)fid;
        tree.quantized[i] = bin;
        std::memcpy(&tree.gain[i], &r[2 * internal + i], sizeof(float));
        float thr = std::numeric_limits<float>::infinity();
        if (bin >= 0 && bin < (int)data_->thresholds[fid].size()) thr = data_->thresholds[fid][bin];
        tree.threshold[i] = thr;
      }
      std::memcpy(tree.weights.data(), r + 3 * internal, (size_t)leaves * sizeof(float));
      overflow = overflow || r[3 * internal + leaves] != 0;
    }
    pending_.clear();
    if (overflow) throw std::runtime_error("internal: work plan exceeded its launch bound");
  }

  void SetInspect(bool on) override { inspect_ = on; }
  void GetLeaves(uint32_t *out) override {
    HIP_OK(hipStreamSynchronize(stream_));
    HIP_OK(hipMemcpy(out, d_leaf_, n_ * sizeof(unsigned), hipMemcpyDeviceToHost));
  }
  void GetYHat(float *out) override {
    HIP_OK(hipStreamSynchronize(stream_));
    HIP_OK(hipMemcpy(out, d_yhat_, n_ * K_ * sizeof(float), hipMemcpyDeviceToHost));
  }
  void GetGrad(float *g, float *h) override {
    if (!inspect_) throw std::runtime_error("gradients of the last round are only kept with inspection on");
    HIP_OK(hipStreamSynchronize(stream_));
    HIP_OK(hipMemcpy(g, d_g_, n_ * K_ * sizeof(float), hipMemcpyDeviceToHost));
    if (h) {
      if (pair_)
        HIP_OK(hipMemcpy(h, d_h_, n_ * K_ * sizeof(float), hipMemcpyDeviceToHost));
      else
        for (size_t i = 0; i < n_ * K_; ++i) h[i] = 1.0f;
    }
  }
  int GetLevelHist(int level, int64_t *out) override {
    if (level < 0 || level >= (int)kept_hist_.size()) return -1;
    const std::vector<int64_t> &v = kept_hist_[level];
    std::memcpy(out, v.data(), v.size() * sizeof(int64_t));
    return (int)(v.size() / 3);
  }
  void GetShifts(int *sg, int *sh) override {
    if (!inspect_ && cfg_.objective == kLinearRegression)
      throw std::runtime_error("the scale of the last round is only kept with inspection on");
    int s[2];
    HIP_OK(hipStreamSynchronize(stream_));
    HIP_OK(hipMemcpy(s, d_shifts_, sizeof(s), hipMemcpyDeviceToHost));
    *sg = s[0];
    *sh = s[1];
  }
  void EnableTiming(bool on) override {
    ResolveTimings();
    timing_ = on;
  }
  BuilderTimings GetTimings() override {
    ResolveTimings();
    return timings_;
  }
  unsigned long long RowsScanned() override {
    unsigned long long v = 0;
    HIP_OK(hipStreamSynchronize(stream_));
    HIP_OK(hipMemcpy(&v, d_rows_scanned_, sizeof(v), hipMemcpyDeviceToHost));
    return v;
  }
  void Synchronize() override {
    HIP_OK(hipStreamSynchronize(stream_));
    FlushTrees();
  }

 private:
  enum Phase { kNone = -1, kGrad = 0, kHistRoot, kHistDeep, kReduce, kSplit, kPartition, kLeaf, kPlan, kFusedLast, kPhases };

  // Timing: an event is recorded at every phase change; the time between two
  // consecutive events is charged to the phase that was open.
  void Mark(int phase) {
    if (!timing_) return;
    hipEvent_t e;
    if (event_used_ < event_pool_.size()) {
      e = event_pool_[event_used_];
    } else {
      HIP_OK(hipEventCreate(&e));
      event_pool_.push_back(e);
    }
    ++event_used_;
    HIP_OK(hipEventRecord(e, stream_));
    marks_.push_back(phase);
  }
  void ResolveTimings() {
    if (!timing_ || marks_.empty()) {
      marks_.clear();
      event_used_ = 0;
      return;
    }
    HIP_OK(hipStreamSynchronize(stream_));
    double *slots[kPhases] = {&timings_.grad, &timings_.hist_root, &timings_.hist_deep, &timings_.reduce,
                              &timings_.split, &timings_.partition, &timings_.leaf, &timings_.plan, &timings_.fused_last};
    for (size_t i = 0; i + 1 < marks_.size(); ++i) {
      if (marks_[i] < 0) continue;
      float ms = 0;
      HIP_OK(hipEventElapsedTime(&ms, event_pool_[i], event_pool_[i + 1]));
      *slots[marks_[i]] += ms;
    }
    marks_.clear();
    event_used_ = 0;
  }

  static unsigned HistRowsPerItem(size_t rows_max, size_t items = 512) {
    // about `items` work items per level (512 = two per CU measured best for
    // the fused pass), whole 1024-row tiles, at most kMaxHistRows rows
    size_t t = (rows_max + items - 1) / items;
    t = (t + kHistThreads - 1) / kHistThreads * kHistThreads;
    return (unsigned)std::min<size_t>(std::max<size_t>(t, kHistThreads), kMaxHistRows);
  }

  void Plan(int state, int L, int select, unsigned rows_per_item, WorkItem *work, unsigned *n_work,
            bool count_rows, const SplitRec *split, unsigned max_items) {
    PlanOn(d_tot_[state], d_seg_[state], L, select, rows_per_item, work, n_work, count_rows, split, max_items);
  }
  void PlanOn(const NodeSum *tot, const unsigned *seg, int L, int select, unsigned rows_per_item, WorkItem *work,
              unsigned *n_work, bool count_rows, const SplitRec *split, unsigned max_items) {
    hipLaunchKernelGGL(k_plan, dim3(1), dim3(1024), 0, stream_, tot, seg, L, select,
                       rows_per_item, work, n_work, d_node_first_, d_node_items_,
                       count_rows ? d_rows_scanned_ : (unsigned long long *)nullptr, split, max_items, d_overflow_);
  }

  // Histograms of contiguous node ranges in `cur` (level order), feature group by group.
  void HistOfNodes(const RowBuffers &cur, int state, int L, bool select_smaller, size_t rows_max, bool root) {
    // the root level is one node: one item per CU avoids a second, partial round
    const unsigned per_item = HistRowsPerItem(rows_max, root ? 256 : 512);
    const unsigned grid = (unsigned)std::min<size_t>(rows_max / per_item + L + 1, max_hist_items_);
    Mark(kPlan);
    Plan(state, L, select_smaller ? 1 : 0, per_item, d_hwork_, d_nwork_, true, nullptr, grid);
    Mark(root ? kHistRoot : kHistDeep);
    if (wide_) {
      for (int f0 = 0; f0 < F_; f0 += wide_group_) {
        const int nf = std::min(wide_group_, F_ - f0);
        const size_t lds = (size_t)nf * slots_ * 8 * (pair_ ? 2 : 1);
        if (pair_) {
          AllowLds(k_hist_wide<true>, kLdsBudget);
          hipLaunchKernelGGL(k_hist_wide<true>, dim3(grid), dim3(kHistThreads), lds, stream_, cur.bins, stride_, f0, nf,
                             slots_, cur.g, cur.h, d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_entries_);
        } else {
          AllowLds(k_hist_wide<false>, kLdsBudget);
          hipLaunchKernelGGL(k_hist_wide<false>, dim3(grid), dim3(kHistThreads), lds, stream_, cur.bins, stride_, f0, nf,
                             slots_, cur.g, cur.h, d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_entries_);
        }
        if (timing_) ++(root ? timings_.hist_root_launches : timings_.hist_deep_launches);
      }
      if (timing_ && root) timings_.hist_root_rows += n_;
      return;
    }
    for (int q0 = 0; q0 < Q_; q0 += quads_per_group_) {
      const int nq = std::min(quads_per_group_, Q_ - q0);
      if (pair_)
        LaunchHist<true>(nq, stream_, grid, cur.bins, stride_, q0, F_, cur.g, cur.h, d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_entries_);
      else
        LaunchHist<false>(nq, stream_, grid, cur.bins, stride_, q0, F_, cur.g, cur.h, d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_entries_);
      if (timing_) ++(root ? timings_.hist_root_launches : timings_.hist_deep_launches);
    }
    if (timing_ && root) timings_.hist_root_rows += n_;
  }

  void Reduce(int L, int hb, bool by_parent, int parent_state, bool trick, bool accumulate = false) {
    Mark(kReduce);
    // many nodes: few slabs per node and the output dominates -> longer output runs per block
    const bool wide_blocks = L >= 32;
    const int entries = wide_blocks ? 256 : 64;
    dim3 grid((slab_entries_ + entries - 1) / entries, L);
#define ARB_REDUCE(P, LN)                                                                                          \
  hipLaunchKernelGGL((k_hist_reduce<P, LN>), grid, dim3(1024), 0, stream_, d_slab_, slab_entries_, nbin_total_,   \
                     d_node_first_, d_node_items_, by_parent ? 1 : 0, d_split_, d_tot_[parent_state], d_hg_[hb], \
                     d_hh_[hb], d_hc_[hb], d_hg_[hb ^ 1], d_hh_[hb ^ 1], d_hc_[hb ^ 1], trick ? 1 : 0,           \
                     accumulate ? 1 : 0, wide_ ? 1 : 0)
    if (pair_) {
      if (wide_blocks) ARB_REDUCE(true, 4);
      else ARB_REDUCE(true, 16);
    } else {
      if (wide_blocks) ARB_REDUCE(false, 4);
      else ARB_REDUCE(false, 16);
    }
#undef ARB_REDUCE
  }

  void GrowOne(int label) {
    const GainParams gp = cfg_.gain_params();
    RowBuffers orig;
    orig.bins = dm_->bins;
    orig.g = d_g_ + (size_t)label * n_;
    orig.h = d_h_ + (size_t)label * n_;
    if (inspect_) kept_hist_.assign(D_ - 1, {});
    SampleColumns();
    if (streamed_) {
      GrowOneStreamed(label, orig, gp);
      return;
    }

    // (the last pass of the previous tree has done this when it built the root histogram)
    if (!root_hist_ready_)
      hipLaunchKernelGGL(k_init_root, dim3(1), dim3(64), 0, stream_, d_tot_[0], d_seg_[0],
                         (unsigned long long)n_, (unsigned *)nullptr);
    int state = 0;  // d_tot_/d_seg_[state] describe the nodes of the current level
    for (int level = 0; level + 1 < D_; ++level) {
      const int L = 1 << level;
      const int hb = level & 1;  // histogram buffer of this level; the parent level is hb ^ 1
      const bool last = level + 2 >= D_;
      if (level == 0) {
        // the slabs of the root may have been written by the last pass of the previous tree
        if (!root_hist_ready_) HistOfNodes(orig, state, 1, false, n_, true);
        root_hist_ready_ = false;
        Reduce(1, hb, false, state, false);
        hipLaunchKernelGGL(k_root_from_hist, dim3(1), dim3(64), 0, stream_, d_hg_[hb], d_hh_[hb], d_tot_[state], slots_);
      } else {
        // rows are in the order of level-1; the parents' state is state ^ 1
        const int ps = state ^ 1, PL = L >> 1;
        const RowBuffers &src = level == 1 ? orig : buf_[level & 1];
        const RowBuffers &dst = buf_[(level & 1) ^ 1];
        if (fused_) {
          // the work plan was written together with the splits of the parents
          const unsigned grid = FusedGrid(PL);
          if (!last) {  // destination offsets; the last level moves no rows
            Mark(kPartition);
            hipLaunchKernelGGL(k_part_count, dim3(grid), dim3(kHistThreads), 0, stream_, src.bins, stride_, d_split_,
                               d_pwork_, d_nwork_ + 1, d_wave_left_, d_item_left_, code_);
          }
          Mark(last ? kFusedLast : kHistDeep);
          // matrices wider than one LDS histogram: one launch per group of
          // quads; the first one moves the gradients
          for (int q0 = 0; q0 < Q_; q0 += quads_per_group_) {
            const int nq = std::min(quads_per_group_, Q_ - q0);
            FusedArgs a{src.bins, last ? nullptr : dst.bins, stride_, F_, src.g, q0 == 0 ? dst.g : nullptr, src.h,
                        q0 == 0 ? dst.h : nullptr, d_shifts_, d_split_, d_tot_[ps], d_seg_[ps], d_pwork_,
                        d_nwork_ + 1, d_wave_left_, d_item_left_, d_slab_, slab_entries_, src.bins, q0};
#define ARB_FUSED(P, W)                                        \
  do {                                                         \
    if (single_group_) LaunchFused<P, W, false>(nq, stream_, grid, a); \
    else LaunchFused<P, W, true>(nq, stream_, grid, a);        \
  } while (0)
            if (pair_) {
              if (last) ARB_FUSED(true, false);
              else ARB_FUSED(true, true);
            } else {
              if (last) ARB_FUSED(false, false);
              else ARB_FUSED(false, true);
            }
#undef ARB_FUSED
            if (timing_) ++(last ? timings_.fused_last_launches : timings_.hist_deep_launches);
          }
          Reduce(L, hb, true, ps, true);
        } else {
          const unsigned grid = (unsigned)std::min<size_t>(n_ / kPartRows + PL + 1, max_part_items_);
          Mark(kPlan);
          Plan(ps, PL, 0, kPartRows, d_pwork_, d_nwork_ + 1, false, nullptr, grid);
          Mark(kPartition);
          hipLaunchKernelGGL(k_part_count, dim3(grid), dim3(kHistThreads), 0, stream_, src.bins, stride_, d_split_,
                             d_pwork_, d_nwork_ + 1, d_wave_left_, d_item_left_, code_);
          LaunchPartRows(grid, src, dst, ps);
          HistOfNodes(dst, state, L, trick_, trick_ ? n_ / 2 : n_, false);
          Reduce(L, hb, false, ps, trick_);
        }
      }
      if (inspect_) KeepHist(level, L, hb);
      LaunchSplit(level, L, hb, state, gp, fused_ && !last);
      if (last) LaunchLeafWeights(L, state, gp);
      state ^= 1;
    }
    // ---- leaf of every row, y_hat update, gradients of the next round
    Mark(kLeaf);
    {
      const bool next_grad = !inspect_ && K_ == 1;
      if (cfg_.objective == kLinearRegression) HIP_OK(hipMemsetAsync(d_gmax_, 0, sizeof(unsigned), stream_));
      const int internal = (1 << (D_ - 1)) - 1;
      const size_t lds = HistLdsBytes(Q_, true) + (size_t)internal * 2 * sizeof(int);
      if (next_grad && cfg_.objective == kLogisticRegression && single_group_ && !wide_ &&
          lds <= kLdsBudget) {
        // plan of the next tree's root, then one pass: leaves, predictions,
        // gradients and the root histogram of the next tree
        hipLaunchKernelGGL(k_init_root, dim3(1), dim3(64), 0, stream_, d_tot_[0], d_seg_[0],
                           (unsigned long long)n_, (unsigned *)nullptr);
        const unsigned per_item = HistRowsPerItem(n_, 256);
        const unsigned grid = (unsigned)std::min<size_t>(n_ / per_item + 2, max_hist_items_);
        Plan(0, 1, 0, per_item, d_hwork_, d_nwork_, true, nullptr, grid);
        LaunchFinalHist(grid, label, lds);
        root_hist_ready_ = true;
      } else {
        LaunchFinal(dm_->bins, stride_, 0, n_, label, next_grad);
      }
      grad_ready_ = next_grad;
    }
    EnqueueRecord();
  }

  // Tree record into the next slot of the device ring; FlushTrees reads it.
  size_t RecordWords() const { return (size_t)3 * ((1 << (D_ - 1)) - 1) + (size_t)(1 << (D_ - 1)) + 1; }
  void EnqueueRecord() {
    Mark(kNone);
    const int internal = (1 << (D_ - 1)) - 1, leaves = 1 << (D_ - 1);
    hipLaunchKernelGGL(k_pack_record, dim3((leaves + 255) / 256), dim3(256), 0, stream_, d_tfid_, d_tbin_, d_tgain_,
                       d_weights_, d_overflow_, internal, leaves, d_records_ + pending_.size() * RecordWords());
    HIP_OK(hipGetLastError());
  }

  // ---- streamed matrices -------------------------------------------------
  // Block `b` of the matrix into one of the two device buffers, on the copy
  // stream; returns the buffer index.  The compute stream waits for ev_ready_
  // before reading and records ev_free_ when it is done with the buffer.
  int CopyBlockIn(size_t b) {
    const int buf = (int)(next_copy_++ & 1);
    if (buf_used_[buf]) HIP_OK(hipStreamWaitEvent(copy_stream_, ev_free_[buf], 0));
    HIP_OK(hipMemcpyAsync(blk_[buf], dm_->host_blocks[b], (size_t)Q_ * dm_->block_rows * sizeof(uint32_t),
                          hipMemcpyHostToDevice, copy_stream_));
    HIP_OK(hipEventRecord(ev_ready_[buf], copy_stream_));
    buf_used_[buf] = true;
    return buf;
  }

  // plan_next: also plan the fused pass of the next level over these nodes
  void LaunchSplit(int level, int L, int hb, int state, const GainParams &gp, bool plan_next = false) {
    Mark(kSplit);
    dim3 grid(F_, L);
    const int hs = std::min(cfg_.internal.hist_size, slots_);
#define ARB_SCAN(P, D) \
  hipLaunchKernelGGL((k_split_scan<P, D>), grid, dim3(64), 0, stream_, d_hg_[hb], d_hh_[hb], d_hc_[hb], \
                     nbin_total_, F_, slots_, d_tot_[state], d_shifts_, gp, hs, d_cand_)
    if (pair_ && f64_) ARB_SCAN(true, true);
    else if (pair_) ARB_SCAN(true, false);
    else if (f64_) ARB_SCAN(false, true);
    else ARB_SCAN(false, false);
#undef ARB_SCAN
    const unsigned char *active = sampling_ ? d_active_ + (size_t)level * F_ : (const unsigned char *)nullptr;
    if (plan_next) {
      const unsigned per_item = HistRowsPerItem(n_);
      hipLaunchKernelGGL(k_select_plan, dim3(1), dim3(1024), 0, stream_, d_cand_, F_, L, d_tot_[state],
                         d_seg_[state], d_tot_[state ^ 1], d_seg_[state ^ 1], d_split_, d_tfid_, d_tbin_, d_tgain_,
                         L - 1, active, per_item, d_pwork_, d_nwork_ + 1, d_node_first_, d_node_items_,
                         d_rows_scanned_, FusedGrid(L), d_overflow_);
    } else {
      hipLaunchKernelGGL(k_split_select, dim3((L + 15) / 16), dim3(1024), 0, stream_, d_cand_, F_, L,
                         d_tot_[state], d_seg_[state], d_tot_[state ^ 1], d_seg_[state ^ 1], d_split_,
                         d_tfid_, d_tbin_, d_tgain_, L - 1, active);
    }
  }

  // Stand-alone partition: groups of up to eight words per launch; the first
  // launch also moves the gradients.
  void LaunchPartRows(unsigned grid, const RowBuffers &src, const RowBuffers &dst, int ps) {
    for (int q0 = 0; q0 < Q_; q0 += 8) {
      const int nq = std::min(8, Q_ - q0);
#define ARB_PART(P, N, G)                                                                                        \
  hipLaunchKernelGGL((k_part_rows<P, N, G>), dim3(grid), dim3(kHistThreads), 0, stream_, src.bins, dst.bins,    \
                     stride_, q0, src.g, dst.g, src.h, dst.h, d_split_, d_seg_[ps], d_pwork_, d_nwork_ + 1,      \
                     d_wave_left_, d_item_left_, code_)
#define ARB_PART_N(N)                                          \
  case N:                                                      \
    if (q0 == 0) {                                             \
      if (pair_) ARB_PART(true, N, true);                      \
      else ARB_PART(false, N, true);                           \
    } else {                                                   \
      ARB_PART(false, N, false);                               \
    }                                                          \
    break;
      switch (nq) {
        ARB_PART_N(1) ARB_PART_N(2) ARB_PART_N(3) ARB_PART_N(4) ARB_PART_N(5) ARB_PART_N(6) ARB_PART_N(7) ARB_PART_N(8)
      }
#undef ARB_PART_N
#undef ARB_PART
    }
  }

  // launch bound of the fused pass over PL parent nodes
  unsigned FusedGrid(int PL) const {
    return (unsigned)std::min<size_t>(n_ / HistRowsPerItem(n_) + PL + 1, max_part_items_);
  }

  void LaunchLeafWeights(int L, int state, const GainParams &gp) {
    Mark(kLeaf);
    const int blocks = (L + 127) / 128;
#define ARB_LEAF(P, D) \
  hipLaunchKernelGGL((k_leaf_weights<P, D>), dim3(blocks), dim3(128), 0, stream_, d_split_, d_tot_[state], L, \
                     d_shifts_, gp, cfg_.tree.eta, d_weights_)
    if (pair_ && f64_) ARB_LEAF(true, true);
    else if (pair_) ARB_LEAF(true, false);
    else if (f64_) ARB_LEAF(false, true);
    else ARB_LEAF(false, false);
#undef ARB_LEAF
  }

  void LaunchFinal(const uint32_t *bins, size_t stride, size_t row0, size_t rows, int label, bool next_grad) {
    const int internal = (1 << (D_ - 1)) - 1;
    const size_t lds = (size_t)internal * 2 * sizeof(int);
    float *yh = d_yhat_ + (size_t)label * n_ + row0;
    const int grid = GridFor(rows, 256, 8192);
    int mode = 0;
    if (next_grad && cfg_.objective == kLinearRegression) mode = 1;
    if (next_grad && cfg_.objective == kLogisticRegression) mode = 2;
#define ARB_FINAL(M, N) \
  hipLaunchKernelGGL((k_final<M, N>), dim3(grid), dim3(256), lds, stream_, bins, stride, d_tfid_, d_tbin_, D_, \
                     d_weights_, yh, d_y_ + row0, d_leaf_ + row0, d_g_ + row0, d_h_ + row0, d_gmax_, rows, code_)
#define ARB_FINAL_Q(N) \
  do { if (mode == 1) ARB_FINAL(1, N); else if (mode == 2) ARB_FINAL(2, N); else ARB_FINAL(0, N); } while (0)
    switch (Q_ <= 8 && !wide_ ? Q_ : 0) {
      case 1: ARB_FINAL_Q(1); break;
      case 2: ARB_FINAL_Q(2); break;
      case 3: ARB_FINAL_Q(3); break;
      case 4: ARB_FINAL_Q(4); break;
      case 5: ARB_FINAL_Q(5); break;
      case 6: ARB_FINAL_Q(6); break;
      case 7: ARB_FINAL_Q(7); break;
      case 8: ARB_FINAL_Q(8); break;
      default: ARB_FINAL_Q(0); break;
    }
#undef ARB_FINAL_Q
#undef ARB_FINAL
  }

  void LaunchFinalHist(unsigned grid, int label, size_t lds) {
    float *yh = d_yhat_ + (size_t)label * n_;
#define ARB_CASE(N)                                                                                              \
  case N: {                                                                                                      \
    static bool configured = false;                                                                              \
    if (!configured) {                                                                                           \
      AllowLds(k_final_hist<N>, kLdsBudget);                                                                     \
      configured = true;                                                                                         \
    }                                                                                                            \
    hipLaunchKernelGGL((k_final_hist<N>), dim3(grid), dim3(kHistThreads), lds, stream_, dm_->bins, stride_, F_, \
                       d_tfid_, d_tbin_, D_, d_weights_, yh, d_y_, d_leaf_, d_g_, d_h_, d_shifts_, d_hwork_,     \
                       d_nwork_, d_slab_, slab_entries_);                                                        \
  } break;
    switch (Q_) {
      ARB_CASE(1) ARB_CASE(2) ARB_CASE(3) ARB_CASE(4) ARB_CASE(5) ARB_CASE(6) ARB_CASE(7) ARB_CASE(8)
      default: throw std::runtime_error("internal: bad quad count");
    }
#undef ARB_CASE
  }

  // One tree over a streamed matrix: every level copies every block in once
  // (double buffered against the kernels of the previous block), one more pass
  // assigns the leaves.
  void GrowOneStreamed(int label, const RowBuffers &orig, const GainParams &gp) {
    const size_t br = dm_->block_rows;
    const size_t nblocks = dm_->host_blocks.size();
    hipLaunchKernelGGL(k_init_root, dim3(1), dim3(64), 0, stream_, d_tot_[0], d_seg_[0],
                       (unsigned long long)n_, (unsigned *)nullptr);
    int state = 0;
    for (int level = 0; level + 1 < D_; ++level) {
      const int L = 1 << level;
      const int hb = level & 1;
      const bool trick = trick_ && level > 0;
      for (size_t b = 0; b < nblocks; ++b) {
        const size_t row0 = b * br;
        const unsigned rows = (unsigned)std::min(br, n_ - row0);
        const int buf = CopyBlockIn(b);
        HIP_OK(hipStreamWaitEvent(stream_, ev_ready_[buf], 0));
        Mark(kPartition);
        hipLaunchKernelGGL(k_stream_route, dim3(GridFor(rows, 256, 1024)), dim3(256), 0, stream_, blk_[buf], br, rows,
                           level, trick ? 1 : 0, d_split_, d_tot_[state], d_node_of_ + row0, d_blk_cnt_);
        hipLaunchKernelGGL(k_stream_segments, dim3(1), dim3(1024), 0, stream_, d_blk_cnt_, L, d_blk_tot_, d_blk_seg_,
                           d_cursor_);
        if (pair_)
          hipLaunchKernelGGL(k_stream_gather<true>, dim3(GridFor(rows, 256, 2048)), dim3(256), 0, stream_, blk_[buf],
                             br, Q_, rows, orig.g + row0, orig.h + row0, d_node_of_ + row0, level, trick ? 1 : 0,
                             d_tot_[state], d_cursor_, stage_.bins, br, stage_.g, stage_.h);
        else
          hipLaunchKernelGGL(k_stream_gather<false>, dim3(GridFor(rows, 256, 2048)), dim3(256), 0, stream_, blk_[buf],
                             br, Q_, rows, orig.g + row0, orig.h + row0, d_node_of_ + row0, level, trick ? 1 : 0,
                             d_tot_[state], d_cursor_, stage_.bins, br, stage_.g, stage_.h);
        HIP_OK(hipEventRecord(ev_free_[buf], stream_));
        // histograms of the gathered rows, added to the level's histograms
        const unsigned per_item = HistRowsPerItem(rows);
        const unsigned grid = (unsigned)std::min<size_t>(rows / per_item + L + 1, max_hist_items_);
        Mark(kPlan);
        PlanOn(d_blk_tot_, d_blk_seg_, L, 0, per_item, d_hwork_, d_nwork_, true, nullptr, grid);
        Mark(level == 0 ? kHistRoot : kHistDeep);
        for (int q0 = 0; q0 < Q_; q0 += quads_per_group_) {
          const int nq = std::min(quads_per_group_, Q_ - q0);
          if (pair_)
            LaunchHist<true>(nq, stream_, grid, stage_.bins, br, q0, F_, stage_.g, stage_.h, d_shifts_, d_hwork_,
                             d_nwork_, d_slab_, slab_entries_);
          else
            LaunchHist<false>(nq, stream_, grid, stage_.bins, br, q0, F_, stage_.g, stage_.h, d_shifts_, d_hwork_,
                              d_nwork_, d_slab_, slab_entries_);
        }
        Reduce(L, hb, false, state, false, b > 0);
      }
      if (level == 0)
        hipLaunchKernelGGL(k_root_from_hist, dim3(1), dim3(64), 0, stream_, d_hg_[hb], d_hh_[hb], d_tot_[state], slots_);
      if (trick)
        hipLaunchKernelGGL(k_sibling, dim3((nbin_total_ + 255) / 256, L), dim3(256), 0, stream_, d_hg_[hb], d_hh_[hb],
                           d_hc_[hb], d_hg_[hb ^ 1], d_hh_[hb ^ 1], d_hc_[hb ^ 1], d_tot_[state], level, nbin_total_);
      if (inspect_) KeepHist(level, L, hb);
      LaunchSplit(level, L, hb, state, gp);
      if (level + 2 >= D_) LaunchLeafWeights(L, state, gp);
      state ^= 1;
    }
    // leaves, y_hat, next gradients: one more pass over the blocks
    Mark(kLeaf);
    const bool next_grad = !inspect_ && K_ == 1;
    if (cfg_.objective == kLinearRegression) HIP_OK(hipMemsetAsync(d_gmax_, 0, sizeof(unsigned), stream_));
    for (size_t b = 0; b < nblocks; ++b) {
      const size_t row0 = b * br;
      const size_t rows = std::min(br, n_ - row0);
      const int buf = CopyBlockIn(b);
      HIP_OK(hipStreamWaitEvent(stream_, ev_ready_[buf], 0));
      LaunchFinal(blk_[buf], br, row0, rows, label, next_grad);
      HIP_OK(hipEventRecord(ev_free_[buf], stream_));
    }
    grad_ready_ = next_grad;
    EnqueueRecord();
  }

  // Column sampling of one tree (InitGrowingTree / InitTreeLevel,
  // garden.cu:126-165, and the `take` prefix of FindBestSplits, :249-253): the
  // ids are shuffled per tree, the first floor(bytree * columns) of them again
  // per level, and the first floor(bylevel * bytree * columns) are active.
  void SampleColumns() {
    const size_t columns = data_->columns_dense + data_->columns_category;
    const int take_tree = (int)(cfg_.tree.colsample_bytree * columns);
    const unsigned take_level = (unsigned)(cfg_.tree.colsample_bylevel * cfg_.tree.colsample_bytree * columns);
    sampling_ = take_level < columns;
    if (!sampling_) return;
    std::vector<unsigned> ids(columns);
    for (size_t i = 0; i < columns; ++i) ids[i] = (unsigned)i;
    std::shuffle(ids.begin(), ids.end(), rnd_);
    active_host_.assign((size_t)(D_ - 1) * F_, 0);
    for (int level = 0; level + 1 < D_; ++level) {
      std::shuffle(ids.begin(), ids.begin() + take_tree, rnd_);
      for (unsigned j = 0; j < take_level; ++j)
        if (ids[j] < (unsigned)F_) active_host_[(size_t)level * F_ + ids[j]] = 1;
    }
    // the previous tree's kernels may still read the mask
    HIP_OK(hipStreamSynchronize(stream_));
    HIP_OK(hipMemcpy(d_active_, active_host_.data(), active_host_.size(), hipMemcpyHostToDevice));
  }

  void KeepHist(int level, int L, int hb) {
    const size_t cells = (size_t)L * nbin_total_;
    std::vector<long long> g(cells), h(cells);
    std::vector<unsigned> c(cells);
    HIP_OK(hipStreamSynchronize(stream_));
    HIP_OK(hipMemcpy(g.data(), d_hg_[hb], cells * sizeof(long long), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(h.data(), d_hh_[hb], cells * sizeof(long long), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(c.data(), d_hc_[hb], cells * sizeof(unsigned), hipMemcpyDeviceToHost));
    // keep [node][F][slots][3] (padding features of the last quad dropped)
    std::vector<int64_t> &out = kept_hist_[level];
    out.resize((size_t)L * F_ * slots_ * 3);
    for (int nd = 0; nd < L; ++nd)
      for (int f = 0; f < F_; ++f)
        for (int b = 0; b < slots_; ++b) {
          const size_t s = (size_t)nd * nbin_total_ + (size_t)f * slots_ + b;
          const size_t d = (((size_t)nd * F_ + f) * slots_ + b) * 3;
          out[d] = g[s];
          out[d + 1] = pair_ ? h[s] : 0;
          out[d + 2] = c[s];
        }
  }

  const Configuration cfg_;
  DataMatrix *data_;
  DeviceMatrix *dm_;
  size_t n_ = 0, stride_ = 0;
  int F_ = 0, Q_ = 0, K_ = 1, D_ = 2, nbin_total_ = 0;
  int slab_entries_ = 0;  // histogram entries of one work item's slab (whole 16-feature blocks)
  bool single_group_ = true;  // all quads fit one LDS histogram
  bool wide_ = false;     // 16-bit bins: two features per word, slots_ histogram slots per feature
  int slots_ = kSlots;
  int wide_group_ = 2;    // features per histogram launch with 16-bit bins
  BinCode code_ = BinCode{2, 8};
  bool root_hist_ready_ = false;  // the slabs hold the root histogram of the tree grown next
  static constexpr size_t kRecordRing = 64;  // trees whose records may wait on the device
  uint32_t *d_records_ = nullptr;
  std::vector<size_t> pending_;              // indices into *owner_ of the trees not fetched yet
  std::vector<RegTree> *owner_ = nullptr;
  bool pair_ = false, f64_ = false, trick_ = true, fused_ = false, inspect_ = false, timing_ = false;
  bool grad_ready_ = false;
  int quads_per_group_ = 1;
  hipStream_t stream_ = nullptr;
  float *d_y_ = nullptr, *d_yhat_ = nullptr, *d_g_ = nullptr, *d_h_ = nullptr, *d_weights_ = nullptr, *d_tgain_ = nullptr;
  uint8_t *d_labels_ = nullptr;
  unsigned *d_overflow_ = nullptr;     // set by the planner when a launch bound was too small
  unsigned char *d_active_ = nullptr;  // [level][feature] 1 = sampled at that level
  std::vector<unsigned char> active_host_;
  std::default_random_engine rnd_;
  bool sampling_ = false;
  unsigned *d_leaf_ = nullptr, *d_node_first_ = nullptr, *d_node_items_ = nullptr, *d_nwork_ = nullptr,
           *d_wave_left_ = nullptr, *d_item_left_ = nullptr, *d_gmax_ = nullptr;
  RowBuffers buf_[2];
  // streamed matrices: two block buffers filled by the copy stream, a staging
  // buffer with the rows of the built nodes, a resident node id per row
  bool streamed_ = false;
  hipStream_t copy_stream_ = nullptr;
  uint32_t *blk_[2] = {nullptr, nullptr};
  hipEvent_t ev_ready_[2] = {nullptr, nullptr}, ev_free_[2] = {nullptr, nullptr};
  bool buf_used_[2] = {false, false};
  size_t next_copy_ = 0;  // running block-copy counter (selects the buffer)
  RowBuffers stage_;
  unsigned *d_node_of_ = nullptr, *d_blk_cnt_ = nullptr, *d_blk_seg_ = nullptr, *d_cursor_ = nullptr;
  NodeSum *d_blk_tot_ = nullptr;
  NodeSum *d_tot_[2] = {nullptr, nullptr};
  unsigned *d_seg_[2] = {nullptr, nullptr};
  long long *d_hg_[2] = {nullptr, nullptr}, *d_hh_[2] = {nullptr, nullptr};
  unsigned *d_hc_[2] = {nullptr, nullptr};
  SplitRec *d_split_ = nullptr;
  Cand *d_cand_ = nullptr;
  WorkItem *d_hwork_ = nullptr, *d_pwork_ = nullptr;
  unsigned max_hist_items_ = 0, max_part_items_ = 0;
  unsigned long long *d_slab_ = nullptr, *d_rows_scanned_ = nullptr;
  int *d_shifts_ = nullptr, *d_tfid_ = nullptr, *d_tbin_ = nullptr;
  std::vector<std::vector<int64_t>> kept_hist_;
  std::vector<hipEvent_t> event_pool_;
  size_t event_used_ = 0;
  std::vector<int> marks_;
  BuilderTimings timings_;
};

}  // namespace

TreeBuilder *CreateTreeBuilder(const Configuration &cfg, DataMatrix *data) {
  if (!data->device) throw std::runtime_error("data matrix is not quantised");
  return new HipTreeBuilder(cfg, data);
}

}  // namespace arb
