// Leaf weights, last pass of a tree (leaf ids, predictions, next gradients), probes.
#ifndef ARBORETUM_AMD_KERNELS_FINAL_H_
#define ARBORETUM_AMD_KERNELS_FINAL_H_
#include "device_common.h"
#include "kernels_hist.h"

namespace arb {
namespace {

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
  weights[2 * nd] = LeafWeight<PAIR, F64>(GL, HL, s.left.c, gp) * eta;
  weights[2 * nd + 1] = LeafWeight<PAIR, F64>(GR, HR, t.c - s.left.c, gp) * eta;
}

// Leaf weights of a finished tree and, in the same launch, what would
// otherwise be three more one-wave kernels in front of the last pass: the
// tree's record into its slot of the record ring (layout of k_pack_record) and
// the state and work plan of the next tree's root histogram over all n rows
// (k_init_root + k_plan for one node starting at row 0).
// grid ceil(L / 128) + 1, 128 threads: the last block writes the plan.
template <bool PAIR, bool F64>
__global__ void __launch_bounds__(128)
k_tree_end(const SplitRec *__restrict__ split, const NodeSum *__restrict__ tot, int L,
           const int *__restrict__ shifts, GainParams gp, float eta, float *__restrict__ weights,
           const int *__restrict__ t_fid, const int *__restrict__ t_bin, const float *__restrict__ t_gain,
           const unsigned *__restrict__ overflow, uint32_t *__restrict__ record,
           NodeSum *__restrict__ root_tot, unsigned *__restrict__ root_seg, unsigned n, unsigned rows_per_item,
           WorkItem *__restrict__ work, unsigned *__restrict__ n_work, unsigned *__restrict__ node_first,
           unsigned *__restrict__ node_items, unsigned long long *__restrict__ rows_scanned) {
  const int internal = 2 * L - 1, leaves = 2 * L;
  const int node_blocks = (int)gridDim.x - 1;
  if ((int)blockIdx.x == node_blocks) {
    const unsigned items = (n + rows_per_item - 1) / rows_per_item;
    for (unsigned w = threadIdx.x; w < items; w += blockDim.x) {
      WorkItem it;
      it.node = 0;
      it.begin = w * rows_per_item;
      it.end = min(n, it.begin + rows_per_item);
      it.first = 0;
      work[w] = it;
    }
    if (threadIdx.x == 0) {
      node_first[0] = 0;
      node_items[0] = items;
      *n_work = items;
      *rows_scanned += n;
      record[3 * internal + leaves] = *overflow;
    }
    return;
  }
  const int nd = blockIdx.x * blockDim.x + threadIdx.x;
  for (int i = nd; i < internal; i += node_blocks * (int)blockDim.x) {
    record[i] = (uint32_t)t_fid[i];
    record[internal + i] = (uint32_t)t_bin[i];
    record[2 * internal + i] = __float_as_uint(t_gain[i]);
  }
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
  if (nd == 0) {
    // root_tot may be the array `tot` of this level: entry 0 has been read above, by this thread
    root_tot[0].g = 0;
    root_tot[0].h = 0;
    root_tot[0].c = n;
    root_seg[0] = 0;
  }
  const float wl = LeafWeight<PAIR, F64>(GL, HL, s.left.c, gp) * eta;
  const float wr = LeafWeight<PAIR, F64>(GR, HR, t.c - s.left.c, gp) * eta;
  weights[2 * nd] = wl;
  weights[2 * nd + 1] = wr;
  record[3 * internal + 2 * nd] = __float_as_uint(wl);
  record[3 * internal + 2 * nd + 1] = __float_as_uint(wr);
}

// End of a tree, rows in original order: walk the tree on the row's bins
// (bin >= q+1 goes right, builder.h:107-123), record the leaf, add its weight
// to y_hat (update_by_last_tree, garden.cu:45-76) and, when NEXT_GRAD is not
// 0, write the gradients of the next round (objective.cu:28-56):
// 1 = squared (also max |g|), 2 = logistic (h == nullptr: packed into g, PackGrad).
// NQ > 0: the matrix has NQ quads, all loaded up front (coalesced, independent
// loads) and selected in registers; NQ == 0: any width, one dependent load per
// level, from the byte columns when the matrix has them (bytes != null).
// hi_word >= 0: column of the rows' first ninth-bit word; a split at bin 255
// sends right only the rows whose id is 256 (SplitTest).
template <int NEXT_GRAD, int NQ>
__global__ void __launch_bounds__(256)
k_final(const uint32_t *__restrict__ bins, size_t stride, const int *__restrict__ t_fid,
        const int *__restrict__ t_bin, int depth, const float *__restrict__ weights,
        float *__restrict__ yhat, const float *__restrict__ y, unsigned *__restrict__ leaf_of,
        float *__restrict__ g, float *__restrict__ h, unsigned *__restrict__ gmax_bits, size_t n,
        BinCode code, const uint8_t *__restrict__ bytes, size_t stride8, int hi_word) {
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
      if (bin >= 255 && hi_word >= 0) {
        right = (bins[(size_t)(hi_word + (fid >> 5)) * stride + i] >> (fid & 31)) & 1u;
      } else if (bin >= 0) {
        if (NQ > 0) {  // 8-bit bins, all quads in registers
          uint32_t b4 = 0;
          const int fq = fid >> 2;
#pragma unroll
          for (int q = 0; q < NQ; ++q) b4 = q == fq ? b[q] : b4;
          right = (int)((b4 >> (8 * (fid & 3))) & 255u) > bin ? 1u : 0u;
        } else if (bytes != nullptr) {  // byte columns [F][stride8] of a wide matrix: a quarter of the bytes fetched
          right = (int)bytes[(size_t)fid * stride8 + i] > bin ? 1u : 0u;
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
      if (h != nullptr) {
        g[i] = yv - s;
        h[i] = s * (1.0f - s);
      } else {
        g[i] = PackGrad(s, yv);
      }
    }
  }
  if (NEXT_GRAD == 1) {
    m = WaveMaxF(m);
    if ((threadIdx.x & 63) == 0) atomicMax(gmax_bits, __float_as_uint(m));
  }
}

// LDS bytes of k_final_hist: histogram, node table, exp table, leaf weights
constexpr size_t FinalHistLdsBytes(int nq, int depth, bool hi = false) {
  return HistLdsBytes(nq, true, hi) + (size_t)((1 << (depth - 1)) - 1) * 8 + 32 * 8 + ((size_t)1 << (depth - 1)) * 4;
}

// Last pass of a tree fused with the root histogram of the next one
// (logistic objective, resident matrix, all quads in one LDS histogram): the
// rows are read once.  The histogram updates set the duration (the LDS is
// busy three quarters of it); the leaf walk, the prediction update and the
// new gradients run in their shadow as far as the waves of a CU interleave.
// One workgroup per root work item; LDS: FinalHistLdsBytes.
// leaf_of may be null: the leaf ids are then not recorded (k_leaf_ids
// computes them on demand).  root_tot (may be null): the gradient totals of
// the next root are added to root_tot[0].g / .h, which the caller has zeroed.
// HI: column NQ of the rows is their ninth-bit word (SplitTest).
template <int NQ, int HI = 0>
__global__ void __launch_bounds__(kHistThreads)
k_final_hist(const uint32_t *__restrict__ bins, size_t stride, int F, const int *__restrict__ t_fid,
             const int *__restrict__ t_bin, int depth, const float *__restrict__ weights,
             float *__restrict__ yhat, const float *__restrict__ y, unsigned *__restrict__ leaf_of,
             float *__restrict__ g, float *__restrict__ h, const int *__restrict__ shifts,
             const WorkItem *__restrict__ work, const unsigned *__restrict__ n_work,
             unsigned long long *__restrict__ slab, int slab_entries, NodeSum *__restrict__ root_tot) {
  extern __shared__ unsigned long long lds[];
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  constexpr int NW = NQ + HI;
  constexpr int words = (int)(HistLdsBytes(NQ, true, HI != 0) / 8);
  // Node table for the walk, two words per internal node: a byte selector for
  // v_perm_b32 that picks byte fid % 8 out of a pair of quads (the other three
  // result bytes are zero), and the split bin in bits 0-7 with the pair fid / 8
  // in bits 8-9.  A node that was not split compares against 255: no byte is
  // larger, so every row stays left.  HI: a node split at bin 255 has bit 31
  // set and the feature in bits 16-20: the row goes right when that bit of its
  // ninth-bit word is set (its id is 256).
  uint2 *s_tree = reinterpret_cast<uint2 *>(lds + words);
  const int internal = (1 << (depth - 1)) - 1, leaves = internal + 1;
  // the exp table and the leaf weights are read from LDS as well
  double *s_exp = reinterpret_cast<double *>(s_tree + internal);
  float *s_weight = reinterpret_cast<float *>(s_exp + 32);
  for (int i = threadIdx.x; i < words; i += kHistThreads) lds[i] = 0ull;
  if (threadIdx.x < 32) s_exp[threadIdx.x] = Exp2Table()[threadIdx.x];
  for (int i = threadIdx.x; i < leaves; i += kHistThreads) s_weight[i] = weights[i];
  for (int i = threadIdx.x; i < internal; i += kHistThreads) {
    const int fid = t_fid[i], bin = t_bin[i];
    uint2 nd;
    nd.x = 0x0c0c0c00u | (unsigned)(fid & 7);
    nd.y = (bin < 0 ? 255u : (unsigned)bin) | ((unsigned)(fid >> 3) << 8);
    if (HI && bin >= 255) nd.y |= 0x80000000u | ((unsigned)fid << 16);
    s_tree[i] = nd;
  }
  __syncthreads();
  const int sg = shifts[0], sh = shifts[1];
  // quad q of a row, zero past the last one
  auto quad = [](const uint32_t (&b)[NW], int q) { return q < NQ ? b[q < NQ ? q : 0] : 0u; };
  // one step of the walk of a row from `node`, whose table entry is nd
  auto step_at = [&](const uint32_t (&b)[NW], unsigned node, uint2 nd) {
    // the row's bin of the split feature: byte fid % 8 of each pair of quads, then the pair
    const uint32_t t0 = __builtin_amdgcn_perm(quad(b, 1), quad(b, 0), nd.x);
    const uint32_t t1 = __builtin_amdgcn_perm(quad(b, 3), quad(b, 2), nd.x);
    const uint32_t t2 = __builtin_amdgcn_perm(quad(b, 5), quad(b, 4), nd.x);
    const uint32_t t3 = __builtin_amdgcn_perm(quad(b, 7), quad(b, 6), nd.x);
    const unsigned pair = nd.y >> 8;
    const uint32_t lo = pair == 1u ? t1 : t0, hi = pair == 3u ? t3 : t2;
    const uint32_t v = pair >= 2u ? hi : lo;
    unsigned right = v > (nd.y & 255u) ? 1u : 0u;  // bin >= q + 1 goes right (builder.h:107-123)
    if (HI) right = (int)nd.y < 0 ? (b[NW - 1] >> ((nd.y >> 16) & 31u)) & 1u : right;
    return node * 2 + right;
  };
  auto step = [&](const uint32_t (&b)[NW], unsigned node, int level) {
    return step_at(b, node, s_tree[(1 << level) - 1 + (int)node]);
  };
  // The entries of the two top levels stay in registers: every row passes
  // them, and a table read waits behind the histogram updates of the other
  // waves in the LDS queue.
  const uint2 top0 = s_tree[0];
  const uint2 top1 = internal > 2 ? s_tree[1] : top0, top2 = internal > 2 ? s_tree[2] : top0;
  // records leaf, prediction and gradients of row r
  auto record = [&](unsigned node, float yh, float s, float yv, float gv, float hv, unsigned r) {
    if (leaf_of != nullptr) __builtin_nontemporal_store(node, &leaf_of[r]);  // uniform
    yhat[r] = yh;
    if (h != nullptr) {  // uniform
      g[r] = gv;
      h[r] = hv;
    } else {
      g[r] = PackGrad(s, yv);
    }
  };
  for (unsigned base = it.begin; base < it.end; base += 2 * kHistThreads) {
    const unsigned r0 = base + threadIdx.x, r1 = r0 + kHistThreads;
    const bool v0 = r0 < it.end, v1 = r1 < it.end;
    const unsigned a0 = v0 ? r0 : it.begin, a1 = v1 ? r1 : it.begin;
    uint32_t b0[NW], b1[NW];
#pragma unroll
    for (int q = 0; q < NW; ++q) {
      b0[q] = __builtin_nontemporal_load(&bins[(size_t)q * stride + a0]);
      b1[q] = __builtin_nontemporal_load(&bins[(size_t)q * stride + a1]);
    }
    const float p0 = yhat[a0], p1 = yhat[a1];
    const float y0 = __builtin_nontemporal_load(&y[a0]), y1 = __builtin_nontemporal_load(&y[a1]);
    // the two rows of a thread walk side by side: their table lookups overlap
    unsigned n0 = 0, n1 = 0;
    if (depth > 1) {
      n0 = step_at(b0, 0u, top0);
      n1 = step_at(b1, 0u, top0);
    }
    if (depth > 2) {
      uint2 e0, e1;
      e0.x = n0 ? top2.x : top1.x;
      e0.y = n0 ? top2.y : top1.y;
      e1.x = n1 ? top2.x : top1.x;
      e1.y = n1 ? top2.y : top1.y;
      n0 = step_at(b0, n0, e0);
      n1 = step_at(b1, n1, e1);
    }
    for (int level = 2; level + 1 < depth; ++level) {
      n0 = step(b0, n0, level);
      n1 = step(b1, n1, level);
    }
    // leaf weights, predictions and gradients of the two rows, side by side
    // as well
    const float yh0 = p0 + s_weight[n0], yh1 = p1 + s_weight[n1];
    const float s0 = SigmoidFrom(yh0, s_exp), s1 = SigmoidFrom(yh1, s_exp);
    const float g0 = y0 - s0, g1 = y1 - s1;
    const float h0 = s0 * (1.0f - s0), h1 = s1 * (1.0f - s1);
    if (v0) record(n0, yh0, s0, y0, g0, h0, r0);
    if (v1) record(n1, yh1, s1, y1, g1, h1, r1);
    if (v0) AccumulateRow<true, NQ, HI>(lds, b0, g0, h0, sg, sh, 0, F);
    if (v1) AccumulateRow<true, NQ, HI>(lds, b1, g1, h1, sg, sh, 0, F);
  }
  FlushSlab<true, NQ, HI>(lds, slab, w, slab_entries, 0);
  // Totals of the next root (garden.cu:432-435 reduces the gradient array):
  // every row sits in exactly one slot of feature 0, so this item's share is
  // the sum of that feature's slots; integers, so the order of the adds over
  // the work items does not matter.  root_tot starts at zero.
  if (root_tot != nullptr && threadIdx.x < 64) {
    long long a = 0, b = 0;
    for (int bin = threadIdx.x; bin < kSlots + HI; bin += 64) {  // (bin 256: the row behind the 256 bins)
      const unsigned word = (unsigned)bin * (2u * kBlockFeatures * HistLds<NQ>::blocks);  // feature 0
      const unsigned long long w0 = lds[word];
      a += ((long long)(w0 << (64 - kCountShift))) >> (64 - kCountShift);
      b += (long long)lds[word + kWord1];
    }
    a = WaveSumLL(a);
    b = WaveSumLL(b);
    if (threadIdx.x == 0) {
      atomicAdd(reinterpret_cast<unsigned long long *>(&root_tot[0].g), (unsigned long long)a);
      atomicAdd(reinterpret_cast<unsigned long long *>(&root_tot[0].h), (unsigned long long)b);
    }
  }
}

// Leaf of every row under the tree in t_fid / t_bin (heap order), for a
// caller that asks after a last pass that did not record the leaves.
__global__ void __launch_bounds__(256)
k_leaf_ids(const uint32_t *__restrict__ bins, size_t stride, const int *__restrict__ t_fid,
           const int *__restrict__ t_bin, int depth, unsigned *__restrict__ leaf_of, size_t n, BinCode code,
           int hi_word) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    unsigned node = 0;
    for (int level = 0; level + 1 < depth; ++level) {
      const int id = (1 << level) - 1 + (int)node;
      const int fid = t_fid[id], bin = t_bin[id];
      unsigned right = 0;
      if (bin >= 255 && hi_word >= 0) right = (bins[(size_t)(hi_word + (fid >> 5)) * stride + i] >> (fid & 31)) & 1u;
      else if (bin >= 0) right = (int)code.Bin(bins[(size_t)code.Word(fid) * stride + i], fid) > bin ? 1u : 0u;
      node = node * 2 + right;
    }
    leaf_of[i] = node;
  }
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
}  // namespace arb
#endif  // ARBORETUM_AMD_KERNELS_FINAL_H_
