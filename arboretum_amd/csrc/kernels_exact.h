// Exact method over sorted row lists: features with more distinct values than a histogram holds.
//
// Every feature keeps the rows of every node of the current level as one list of row ids in
// ascending order of the feature's value (the reference sorts every column once and keeps the
// node segments sorted, src/core/continuous_tree_grower.cu).  Per level and feature: the running
// sums of the gradients along the list give, at every place where the value changes, the
// candidate "values up to here go left"; the best one per (node, feature) goes to the same
// selection as the histogram method's candidates, and a stable partition by the selected splits
// turns the lists of the parents into the lists of the children.
//
// The candidates are those of a histogram with one slot per distinct value (rank): a slot that
// is empty in a node has the gain of the slot before it, and ties go to the highest slot
// (builder.h:39-49), so the candidate between two neighbouring values of a node is the slot just
// below the upper one, and its threshold is that upper value: the smallest value that goes right.
#ifndef ARBORETUM_AMD_KERNELS_EXACT_H_
#define ARBORETUM_AMD_KERNELS_EXACT_H_
#include "device_common.h"
#include "gain.h"
#include "kernels_split.h"

namespace arb {
namespace {

constexpr int kExThreads = 256;
constexpr int kExPer = 8;                          // list places per thread
constexpr unsigned kExItem = kExThreads * kExPer;  // list places per work item

struct ExSum {
  long long g, h;
};
__device__ __forceinline__ ExSum operator+(const ExSum &a, const ExSum &b) { return ExSum{a.g + b.g, a.h + b.h}; }
__device__ __forceinline__ ExSum ExShflUp(const ExSum &v, int off) {
  return ExSum{__shfl_up(v.g, off), __shfl_up(v.h, off)};
}
__device__ __forceinline__ unsigned ExShflUp(unsigned v, int off) { return __shfl_up(v, off); }
__device__ __forceinline__ ExSum ExZero(const ExSum *) { return ExSum{0, 0}; }
__device__ __forceinline__ unsigned ExZero(const unsigned *) { return 0u; }

// Inclusive scan over the workgroup's threads (kExThreads of them) of one value per thread;
// *total: the sum over all threads.  s_wave: kExThreads / 64 entries.
template <typename T>
__device__ __forceinline__ T ExBlockScan(T v, T *s_wave, T *total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int off = 1; off < 64; off <<= 1) {
    const T o = ExShflUp(v, off);
    if (lane >= off) v = v + o;
  }
  __syncthreads();  // s_wave may still be read from a scan before
  if (lane == 63) s_wave[wave] = v;
  __syncthreads();
  T before = ExZero((const T *)nullptr), all = ExZero((const T *)nullptr);
  for (int w = 0; w < kExThreads / 64; ++w) {
    if (w < wave) before = before + s_wave[w];
    all = all + s_wave[w];
  }
  *total = all;
  return before + v;
}

// The lists of a level: for every feature the rows of every node in ascending order of the
// feature's value, and next to each row id what the passes need of that row, so that they read
// it in list order instead of gathering it by row: the row's rank in this feature and its
// gradients (the root's ids and ranks are the same for every tree; its gradients are gathered
// once per tree, k_ex_gather).
struct ExLists {
  const unsigned *ids;    // [F][stride]
  const unsigned *ranks;  // [F][stride]
  const float *g, *h;     // [F][stride]; h null without hessians
};

// Eight consecutive words of a list from place p0, `fill` past `end`.
template <typename T>
__device__ __forceinline__ void ExLoad8(const T *__restrict__ base, unsigned p0, unsigned end, T fill, T *out) {
  static_assert(sizeof(T) == 4, "lists hold 32-bit words");
  if ((p0 & 3u) == 0 && p0 + kExPer <= end) {
    const uint4 a = *reinterpret_cast<const uint4 *>(base + p0);
    const uint4 b = *reinterpret_cast<const uint4 *>(base + p0 + 4);
    const unsigned w[kExPer] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int j = 0; j < kExPer; ++j) __builtin_memcpy(&out[j], &w[j], 4);
  } else {
#pragma unroll
    for (int j = 0; j < kExPer; ++j) out[j] = p0 + j < end ? base[p0 + j] : fill;
  }
}

// The fixed-point gradients of the rows at the places [p0, p0 + kExPer) of feature f's list, zero past `end`.
// PACK: one float per row holds both (logistic gradients of 0/1 labels, PackGrad); no h lists.
template <bool PAIR, bool PACK>
__device__ __forceinline__ void ExLoadSums(const ExLists &ls, size_t fbase, unsigned p0, unsigned end, int sg, int sh,
                                           ExSum *v) {
  float gv[kExPer], hv[kExPer];
  ExLoad8(ls.g + fbase, p0, end, 0.0f, gv);
  if (PAIR && !PACK) ExLoad8(ls.h + fbase, p0, end, 0.0f, hv);
#pragma unroll
  for (int j = 0; j < kExPer; ++j) {
    float g1 = gv[j], h1 = PAIR && !PACK ? hv[j] : 0.0f;
    if (PACK) UnpackGrad(gv[j], &g1, &h1);
    v[j].g = p0 + j < end ? ToFixed(g1, sg) : 0;
    v[j].h = PAIR && p0 + j < end ? ToFixed(h1, sh) : 0;
  }
}

// Sum of the fixed-point gradients of all rows from packed logistic gradients: the totals of
// the root.  tot[0].g / .h must be zero at launch; integer sums, any order.
__global__ void __launch_bounds__(256)
k_ex_sum_packed(const float *__restrict__ packed, size_t n, const int *__restrict__ shifts, NodeSum *__restrict__ tot) {
  const int sg = shifts[0], sh = shifts[1];
  long long a = 0, b = 0;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    float g1, h1;
    UnpackGrad(packed[i], &g1, &h1);
    a += ToFixed(g1, sg);
    b += ToFixed(h1, sh);
  }
  a = WaveSumLL(a);
  b = WaveSumLL(b);
  if ((threadIdx.x & 63) == 0) {
    atomicAdd(reinterpret_cast<unsigned long long *>(&tot[0].g), (unsigned long long)a);
    atomicAdd(reinterpret_cast<unsigned long long *>(&tot[0].h), (unsigned long long)b);
  }
}

// grid (items, F): the sum of the gradients over every work item's piece of every feature's list.
template <bool PAIR, bool PACK>
__global__ void __launch_bounds__(kExThreads)
k_ex_partial(const ExLists ls, size_t stride, const int *__restrict__ shifts, const WorkItem *__restrict__ work,
             const unsigned *__restrict__ n_work, ExSum *__restrict__ part, unsigned max_items) {
  __shared__ ExSum s_wave[kExThreads / 64];
  const unsigned w = blockIdx.x, f = blockIdx.y;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  ExSum v[kExPer];
  ExLoadSums<PAIR, PACK>(ls, (size_t)f * stride, it.begin + threadIdx.x * kExPer, it.end, shifts[0], shifts[1], v);
  ExSum mine = v[0];
#pragma unroll
  for (int j = 1; j < kExPer; ++j) mine = mine + v[j];
  ExSum total;
  ExBlockScan(mine, s_wave, &total);
  if (threadIdx.x == 0) part[(size_t)f * max_items + w] = total;
}

// grid (L, F), one wave: exclusive scan of `part` over the work items of every node, per feature.
template <typename T>
__global__ void __launch_bounds__(64)
k_ex_offsets(const T *__restrict__ part, T *__restrict__ off, const unsigned *__restrict__ node_first,
             const unsigned *__restrict__ node_items, unsigned max_items) {
  const unsigned nd = blockIdx.x, f = blockIdx.y, lane = threadIdx.x;
  const unsigned first = node_first[nd];
  unsigned cnt = node_items[nd];
  if (cnt == 0xffffffffu) cnt = 0;
  T carry = ExZero((const T *)nullptr);
  for (unsigned base = 0; base < cnt; base += 64) {
    const unsigned k = base + lane;
    const T own = k < cnt ? part[(size_t)f * max_items + first + k] : ExZero((const T *)nullptr);
    T v = own;
    for (int o = 1; o < 64; o <<= 1) {
      const T up = ExShflUp(v, o);
      if ((int)lane >= o) v = v + up;
    }
    // exclusive: the sum of the items before this one
    T excl = carry;
    {
      const T prev = ExShflUp(v, 1);
      if (lane > 0) excl = excl + prev;
    }
    if (k < cnt) off[(size_t)f * max_items + first + k] = excl;
    T last;
    if constexpr (sizeof(T) == sizeof(unsigned)) {
      last = __shfl(v, 63);
    } else {
      last = ExSum{__shfl(v.g, 63), __shfl(v.h, 63)};
    }
    carry = carry + last;
  }
}

// SplitGain (gain.h) with the parent's term, which is the same at every place of a node, taken
// from the caller: `parent` = SideGain of the node's totals at their leaf weight.  The same
// operations in the same order, so the same bits.
template <bool PAIR, bool F64>
__device__ __forceinline__ float ExParentGain(double gt, double ht, unsigned long long ct, const GainParams &p) {
  return SideGain<PAIR, F64>(gt, ht, ct, LeafWeight<PAIR, F64>(gt, ht, ct, p), p);
}
template <bool PAIR, bool F64>
__device__ __forceinline__ float ExSplitGain(double gl, double hl, unsigned long long cl, double gt, double ht,
                                             unsigned long long ct, const GainParams &p, float parent) {
  const unsigned long long cr = ct - cl;
  double gr, hr;
  if (F64) {
    gr = gt - gl;
    hr = ht - hl;
  } else {
    gr = (double)((float)gt - (float)gl);
    hr = (double)((float)ht - (float)hl);
  }
  if (cl < p.min_leaf_size || cr < p.min_leaf_size) return 0.0f;
  if (PAIR) {
    if (F64) {
      if (!(fabs(hl) >= (double)p.min_child_weight && fabs(hr) >= (double)p.min_child_weight)) return 0.0f;
    } else {
      if (!(fabsf((float)hl) >= p.min_child_weight && fabsf((float)hr) >= p.min_child_weight)) return 0.0f;
    }
  }
  const float l = SideGain<PAIR, F64>(gl, hl, cl, LeafWeight<PAIR, F64>(gl, hl, cl, p), p);
  const float r = SideGain<PAIR, F64>(gr, hr, cr, LeafWeight<PAIR, F64>(gr, hr, cr, p), p);
  const float diff = l + r - parent;
  return (float)(diff > p.gamma_absolute && diff > p.gamma_relative * parent) * diff;
}

__device__ __forceinline__ bool ExBetter(float og, int ob, float gain, int bin) {
  return ob >= 0 && (bin < 0 || og > gain || (og == gain && ob > bin));
}

// grid (items, F): running sums along every work item's piece of every list (on top of `off`, the
// sums of the node's items before it), the gain wherever the rank changes to the next place of the
// node, and the best candidate of the piece, ties to the highest rank.
// best: [F][max_items].
template <bool PAIR, bool F64, bool PACK>
__global__ void __launch_bounds__(kExThreads)
k_ex_scan(const ExLists ls, size_t stride, const int *__restrict__ shifts,
          const WorkItem *__restrict__ work, const unsigned *__restrict__ n_work, const ExSum *__restrict__ off,
          const NodeSum *__restrict__ tot, const unsigned *__restrict__ seg_start, GainParams gp,
          Cand *__restrict__ best, unsigned max_items) {
  __shared__ ExSum s_wave[kExThreads / 64];
  __shared__ Cand s_best[kExThreads / 64];
  const unsigned w = blockIdx.x, f = blockIdx.y;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const NodeSum t = tot[it.node];
  const unsigned node_start = seg_start[it.node], node_end = node_start + (unsigned)t.c;
  const size_t fbase = (size_t)f * stride;
  const int sg = shifts[0], sh = shifts[1];
  const unsigned p0 = it.begin + threadIdx.x * kExPer;
  ExSum v[kExPer];
  ExLoadSums<PAIR, PACK>(ls, fbase, p0, it.end, sg, sh, v);
  // ranks at this thread's places and at the one after them (which may lie in the next item)
  unsigned rk[kExPer + 1];
  ExLoad8(ls.ranks + fbase, p0, node_end, 0u, rk);
  rk[kExPer] = p0 + kExPer < node_end ? ls.ranks[fbase + p0 + kExPer] : 0u;
#pragma unroll
  for (int j = 1; j < kExPer; ++j) v[j] = v[j] + v[j - 1];
  ExSum total;
  const ExSum incl = ExBlockScan(v[kExPer - 1], s_wave, &total);
  const ExSum base = off[(size_t)f * max_items + w];
  const long long eg = base.g + incl.g - v[kExPer - 1].g, eh = base.h + incl.h - v[kExPer - 1].h;

  Cand mine;
  mine.gain = 0.0f;
  mine.bin = -1;
  mine.left.g = mine.left.h = 0;
  mine.left.c = 0;
  const double GT = FromFixed<F64>(t.g, sg);
  const double HT = PAIR ? FromFixed<F64>(t.h, sh) : 0.0;
  const float parent = ExParentGain<PAIR, F64>(GT, HT, t.c, gp);
#pragma unroll
  for (int j = 0; j < kExPer; ++j) {
    const unsigned p = p0 + j;
    if (p < it.end && p + 1 < node_end && rk[j] != rk[j + 1]) {
      const long long lg = eg + v[j].g, lh = eh + v[j].h;
      const unsigned long long lc = p - node_start + 1;
      const double GL = FromFixed<F64>(lg, sg);
      const double HL = PAIR ? FromFixed<F64>(lh, sh) : 0.0;
      const float gn = ExSplitGain<PAIR, F64>(GL, HL, lc, GT, HT, t.c, gp, parent);
      if (gn > 0.0f && gn >= mine.gain) {
        mine.gain = gn;
        mine.bin = (int)(rk[j + 1] - 1u);
        mine.left.g = lg;
        mine.left.h = lh;
        mine.left.c = lc;
      }
    }
  }
  for (int o = 32; o > 0; o >>= 1) {
    const float og = __shfl_down(mine.gain, o);
    const int ob = __shfl_down(mine.bin, o);
    const long long olg = __shfl_down(mine.left.g, o);
    const long long olh = __shfl_down(mine.left.h, o);
    const unsigned long long olc = __shfl_down(mine.left.c, o);
    if (ExBetter(og, ob, mine.gain, mine.bin)) {
      mine.gain = og;
      mine.bin = ob;
      mine.left.g = olg;
      mine.left.h = olh;
      mine.left.c = olc;
    }
  }
  if ((threadIdx.x & 63) == 0) s_best[threadIdx.x >> 6] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < kExThreads / 64; ++k)
      if (ExBetter(s_best[k].gain, s_best[k].bin, mine.gain, mine.bin)) mine = s_best[k];
    best[(size_t)f * max_items + w] = mine;
  }
}

// grid (L, F), one wave: the best candidate of a node's work items -> cand[node * F + feature].
__global__ void __launch_bounds__(64)
k_ex_merge(const Cand *__restrict__ best, const unsigned *__restrict__ node_first,
           const unsigned *__restrict__ node_items, unsigned max_items, int F, Cand *__restrict__ cand) {
  const unsigned nd = blockIdx.x, f = blockIdx.y, lane = threadIdx.x;
  const unsigned first = node_first[nd];
  unsigned cnt = node_items[nd];
  if (cnt == 0xffffffffu) cnt = 0;
  Cand mine;
  mine.gain = 0.0f;
  mine.bin = -1;
  mine.left.g = mine.left.h = 0;
  mine.left.c = 0;
  for (unsigned k = lane; k < cnt; k += 64) {
    const Cand c = best[(size_t)f * max_items + first + k];
    if (ExBetter(c.gain, c.bin, mine.gain, mine.bin)) mine = c;
  }
  for (int o = 32; o > 0; o >>= 1) {
    const float og = __shfl_down(mine.gain, o);
    const int ob = __shfl_down(mine.bin, o);
    const long long olg = __shfl_down(mine.left.g, o);
    const long long olh = __shfl_down(mine.left.h, o);
    const unsigned long long olc = __shfl_down(mine.left.c, o);
    if (ExBetter(og, ob, mine.gain, mine.bin)) {
      mine.gain = og;
      mine.bin = ob;
      mine.left.g = olg;
      mine.left.h = olh;
      mine.left.c = olc;
    }
  }
  if (lane == 0) cand[(size_t)nd * F + f] = mine;
}

// Every row to its child: node_of[row] = 2 * node + (rank of the split feature > split rank).
// went_right: one bit per row (64 rows per word), small enough to stay in L2 while the lists are
// partitioned.  ranks: [F][stride] by row.  Launched with whole waves over 64-aligned rows.
__global__ void __launch_bounds__(256)
k_ex_decide(const unsigned *__restrict__ ranks, size_t stride, const SplitRec *__restrict__ split,
            unsigned *__restrict__ node_of, unsigned long long *__restrict__ went_right, size_t n) {
  const size_t padded = (n + 63) / 64 * 64;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < padded; i += (size_t)gridDim.x * blockDim.x) {
    bool right = false;
    if (i < n) {
      const unsigned nd = node_of[i];
      const SplitRec s = split[nd];
      right = s.fid >= 0 && ranks[(size_t)s.fid * stride + i] > (unsigned)s.bin;
      node_of[i] = 2 * nd + (right ? 1u : 0u);
    }
    const unsigned long long m = __ballot(right);
    if ((threadIdx.x & 63) == 0) went_right[i >> 6] = m;
  }
}

__device__ __forceinline__ unsigned ExGoesLeft(const unsigned long long *__restrict__ went_right, unsigned id) {
  return (unsigned)(~(went_right[id >> 6] >> (id & 63u)) & 1ull);
}

// grid (items, F): rows of every piece that go left; left_bits: for every thread of every piece
// the decisions of its kExPer places (bit j: place j goes left), which the partition reads back
// instead of looking the rows up again.
__global__ void __launch_bounds__(kExThreads)
k_ex_count(const unsigned *__restrict__ ids, size_t stride, const unsigned long long *__restrict__ went_right,
           const WorkItem *__restrict__ work, const unsigned *__restrict__ n_work, unsigned *__restrict__ lefts,
           uint8_t *__restrict__ left_bits, unsigned max_items) {
  static_assert(kExPer == 8, "one byte of decisions per thread");
  __shared__ unsigned s_wave[kExThreads / 64];
  const unsigned w = blockIdx.x, f = blockIdx.y;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const unsigned p0 = it.begin + threadIdx.x * kExPer;
  unsigned id[kExPer];
  ExLoad8(ids + (size_t)f * stride, p0, it.end, 0u, id);
  unsigned bits = 0;
#pragma unroll
  for (int j = 0; j < kExPer; ++j)
    if (p0 + j < it.end) bits |= ExGoesLeft(went_right, id[j]) << j;
  left_bits[((size_t)f * max_items + w) * kExThreads + threadIdx.x] = (uint8_t)bits;
  unsigned total;
  ExBlockScan((unsigned)__builtin_popcount(bits), s_wave, &total);
  if (threadIdx.x == 0) lefts[(size_t)f * max_items + w] = total;
}

// grid (items, F): the stable partition of every piece into the lists of the two children, with
// the rank and the gradients of every row next to its id (PAIR here: the lists hold h beside g;
// packed gradients are one word, like g alone).  The piece is put in order in LDS
// (the rows that go left, then the others) and written out from there, so that the stores of a
// wave are consecutive.
// left_off: rows of the node's earlier pieces that go left; seg_start / seg_next: first place of
// the parents / of the children.
template <bool PAIR>
__global__ void __launch_bounds__(kExThreads)
k_ex_scatter(const ExLists ls, unsigned *__restrict__ ids_out, unsigned *__restrict__ ranks_out,
             float *__restrict__ g_out, float *__restrict__ h_out, size_t stride,
             const uint8_t *__restrict__ left_bits, const WorkItem *__restrict__ work,
             const unsigned *__restrict__ n_work, const unsigned *__restrict__ left_off,
             const unsigned *__restrict__ seg_start, const unsigned *__restrict__ seg_next, unsigned max_items) {
  __shared__ unsigned s_wave[kExThreads / 64];
  __shared__ unsigned s_id[kExItem], s_rk[kExItem];
  __shared__ float s_g[kExItem], s_h[PAIR ? kExItem : 1];
  const unsigned w = blockIdx.x, f = blockIdx.y;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const size_t fbase = (size_t)f * stride;
  const unsigned p0 = it.begin + threadIdx.x * kExPer;
  unsigned id[kExPer], rk[kExPer];
  float gv[kExPer], hv[kExPer];
  ExLoad8(ls.ids + fbase, p0, it.end, 0u, id);
  ExLoad8(ls.ranks + fbase, p0, it.end, 0u, rk);
  ExLoad8(ls.g + fbase, p0, it.end, 0.0f, gv);
  if (PAIR) ExLoad8(ls.h + fbase, p0, it.end, 0.0f, hv);
  const unsigned bits = left_bits[((size_t)f * max_items + w) * kExThreads + threadIdx.x];
  const unsigned mine = (unsigned)__builtin_popcount(bits);
  unsigned total;
  const unsigned incl = ExBlockScan(mine, s_wave, &total);
  // places of this thread's rows in the ordered piece
  unsigned l_at = incl - mine;
  unsigned r_at = total + threadIdx.x * kExPer - l_at;
#pragma unroll
  for (int j = 0; j < kExPer; ++j) {
    if (p0 + j < it.end) {
      const unsigned at = ((bits >> j) & 1u) ? l_at++ : r_at++;
      s_id[at] = id[j];
      s_rk[at] = rk[j];
      s_g[at] = gv[j];
      if (PAIR) s_h[at] = hv[j];
    }
  }
  __syncthreads();
  const unsigned before = left_off[(size_t)f * max_items + w];
  const unsigned count = it.end - it.begin;
  const size_t l_to = fbase + seg_next[2 * it.node] + before;
  const size_t r_to = fbase + seg_next[2 * it.node + 1] + ((it.begin - seg_start[it.node]) - before);
  for (unsigned k = threadIdx.x; k < count; k += kExThreads) {
    const size_t at = k < total ? l_to + k : r_to + (k - total);
    ids_out[at] = s_id[k];
    ranks_out[at] = s_rk[k];
    g_out[at] = s_g[k];
    if (PAIR) h_out[at] = s_h[k];
  }
}

// (g, h) of every row side by side, so that one access fetches both.
__global__ void k_ex_pair(const float *__restrict__ g, const float *__restrict__ h, float2 *__restrict__ gh, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    gh[i] = make_float2(g[i], h[i]);
}

// grid (ceil(n / kExItem), F): the gradients of this tree in the order of the root's lists.
template <bool PAIR>
__global__ void __launch_bounds__(kExThreads)
k_ex_gather(const unsigned *__restrict__ ids, size_t stride, const float *__restrict__ g,
            const float2 *__restrict__ gh, float *__restrict__ g_out, float *__restrict__ h_out, size_t n) {
  const size_t fbase = (size_t)blockIdx.y * stride;
#pragma unroll
  for (int j = 0; j < kExPer; ++j) {
    const size_t p = (size_t)blockIdx.x * kExItem + (size_t)j * kExThreads + threadIdx.x;
    if (p < n) {
      const unsigned id = ids[fbase + p];
      if (PAIR) {
        const float2 v = gh[id];
        g_out[fbase + p] = v.x;
        h_out[fbase + p] = v.y;
      } else {
        g_out[fbase + p] = g[id];
      }
    }
  }
}

// The leaf of every row and its prediction (update_by_last_tree, src/core/garden.cu:45-76).
__global__ void k_ex_final(const unsigned *__restrict__ node_of, const float *__restrict__ weights,
                           float *__restrict__ yhat, unsigned *__restrict__ leaf_of, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const unsigned leaf = node_of[i];
    leaf_of[i] = leaf;
    yhat[i] += weights[leaf];
  }
}

}  // namespace
}  // namespace arb
#endif  // ARBORETUM_AMD_KERNELS_EXACT_H_
