// Split search: prefix scan and gain per feature, best feature per node.
#ifndef ARBORETUM_AMD_KERNELS_SPLIT_H_
#define ARBORETUM_AMD_KERNELS_SPLIT_H_
#include "device_common.h"
#include "kernels_plan.h"

namespace arb {
namespace {

// --------------------------------------------------------------- split scan
struct Cand {
  float gain;
  int bin;
  NodeSum left;
};

// One wave scans one (feature, node): inclusive prefix over the slots, gain
// per bin < hist_size, arg-max with ties to the HIGHEST bin (builder.h:39-49),
// only gains > 0 (hist_tree_grower.cu:31).  `first` is the index of the
// feature's slot 0 in the histogram arrays.  The result is valid in lane 0.
template <bool PAIR, bool F64>
__device__ __forceinline__ Cand ScanFeature(const long long *__restrict__ hg, const long long *__restrict__ hh,
                                            const unsigned long long *__restrict__ hc, size_t first, int slots,
                                            const NodeSum &t, const int *__restrict__ shifts,
                                            const GainParams &gp, int hist_size, int lane) {
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
      const size_t base = first + chunk + lane * 4;
      long long g4[4], h4[4];
      unsigned long long c4[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) g4[j] = h4[j] = 0, c4[j] = 0;
      // lanes whose four slots all lie at or past hist_size (missing values, unused slots) hold no
      // candidate and are in no candidate's prefix: they read nothing
      if (chunk + lane * 4 < hist_size) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          g4[j] = hg[base + j];
          h4[j] = PAIR ? hh[base + j] : 0;
          c4[j] = hc[base + j];
        }
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
  return best;
}

// grid (F, L), 64 threads: one wave per (feature, node), candidates to `cand`.
template <bool PAIR, bool F64>
__global__ void __launch_bounds__(64)
k_split_scan(const long long *__restrict__ hg, const long long *__restrict__ hh,
             const unsigned long long *__restrict__ hc, int nbin_total, int F, int slots,
             const NodeSum *__restrict__ tot, const int *__restrict__ shifts, GainParams gp,
             int hist_size, Cand *__restrict__ cand) {
  const int f = blockIdx.x, nd = blockIdx.y, lane = threadIdx.x;
  const NodeSum t = tot[nd];
  const Cand best = ScanFeature<PAIR, F64>(hg, hh, hc, (size_t)nd * nbin_total + (size_t)f * slots, slots, t, shifts,
                                           gp, hist_size, lane);
  if (lane == 0) cand[(size_t)nd * F + f] = best;
}

// Record of one node from its best candidate (fid < 0: none, every row stays
// left): split, totals and row ranges of the two children, tree arrays.
__device__ __forceinline__ SplitRec WriteNode(int nd, const NodeSum &t, float gain, int fid, int bin, long long lg,
                                          long long lh, unsigned long long lc,
                                          const unsigned *__restrict__ seg_start, NodeSum *__restrict__ tot_next,
                                          unsigned *__restrict__ seg_next, SplitRec *__restrict__ split,
                                          int *__restrict__ t_fid, int *__restrict__ t_bin,
                                          float *__restrict__ t_gain, int heap_off) {
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
  return rec;
}

// What a fused pass over the rows of a level's nodes needs to select the splits of those nodes
// itself, in its prologue, from the per-feature candidates of the split scan (k_split_scan)
// instead of reading them from a selection kernel launched before it: one launch less per level
// on the critical path.  Every workgroup of the pass selects for ITS node; the node's first work
// item also writes the node's record.  cand == null: the splits are read from `split` as before.
struct LevelScan {
  const Cand *cand;
  int F, L;
  NodeSum *tot_next;
  unsigned *seg_next;
  SplitRec *split;
  int *t_fid, *t_bin;
  float *t_gain;
  int heap_off;
  const unsigned char *active;
  const unsigned *node_first;         // first work item of every node: that item writes the node's record
  unsigned long long *rows_scanned;   // advanced by the rows of the smaller side of every split
};

// Split of node nd (totals t) from its candidates: wave 0 of the workgroup keeps the candidate
// with the highest gain, ties to the lowest feature id (hist_tree_grower.cu:59-60), over the
// features active at this level; every thread returns the node's record.  `write`: this
// workgroup also stores the record, the children's totals and row ranges and the tree arrays
// (WriteNode).  Called by all threads of the workgroup; s_rec holds one record.
__device__ __forceinline__ SplitRec SelectInPass(const LevelScan &a, int nd, const NodeSum &t,
                                                 const unsigned *__restrict__ seg_start, bool write,
                                                 SplitRec *s_rec) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (wave == 0) {
    float gain = 0.0f;
    int fid = -1, bin = -1;
    long long lg = 0, lh = 0;
    unsigned long long lc = 0;
    if (t.c != 0) {
      for (int f = lane; f < a.F; f += 64) {
        if (a.active && !a.active[f]) continue;  // feature not sampled at this level
        const Cand c = a.cand[(size_t)nd * a.F + f];
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
    if (lane == 0) {
      SplitRec rec;
      if (write) {
        rec = WriteNode(nd, t, gain, fid, bin, lg, lh, lc, seg_start, a.tot_next, a.seg_next, a.split, a.t_fid,
                        a.t_bin, a.t_gain, a.heap_off);
        if (a.rows_scanned && t.c != 0) {
          const unsigned long long cl = fid < 0 ? t.c : lc;
          atomicAdd(a.rows_scanned, min(cl, t.c - cl));
        }
      } else {
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
      }
      *s_rec = rec;
    }
  }
  __syncthreads();
  // the record as wave-uniform values (it steers the whole pass)
  SplitRec r;
  r.gain = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(s_rec->gain)));
  r.fid = __builtin_amdgcn_readfirstlane(s_rec->fid);
  r.bin = __builtin_amdgcn_readfirstlane(s_rec->bin);
  r.pad = 0;
  const unsigned long long *p = reinterpret_cast<const unsigned long long *>(&s_rec->left);
  unsigned long long v[3];
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)p[k]);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(p[k] >> 32));
    v[k] = ((unsigned long long)hi << 32) | lo;
  }
  r.left.g = (long long)v[0];
  r.left.h = (long long)v[1];
  r.left.c = v[2];
  return r;
}

// Records of the nodes of a level that hold no row (no work item of the pass stands for them):
// not split, both children empty.  Called by one workgroup.
__device__ __forceinline__ void WriteEmptyNodes(const LevelScan &a, const NodeSum *__restrict__ tot,
                                                const unsigned *__restrict__ seg_start) {
  for (int nd = threadIdx.x; nd < a.L; nd += blockDim.x) {
    const NodeSum t = tot[nd];
    if (t.c == 0)
      WriteNode(nd, t, 0.0f, -1, -1, 0, 0, 0, seg_start, a.tot_next, a.seg_next, a.split, a.t_fid, a.t_bin, a.t_gain,
                a.heap_off);
  }
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
  WriteNode(nd, t, gain, fid, bin, lg, lh, lc, seg_start, tot_next, seg_next, split, t_fid, t_bin, t_gain, heap_off);
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
              unsigned *__restrict__ overflow, unsigned *__restrict__ cursor) {
  for (int nd = threadIdx.x >> 6; nd < L; nd += 16)
    SelectNode(nd, threadIdx.x & 63, cand, F, tot, seg_start, tot_next, seg_next, split, t_fid, t_bin, t_gain,
               heap_off, active);
  __syncthreads();  // the splits written above are read by the plan
  PlanBody(tot, seg_start, L, 0, rows_per_item, work, n_work, node_first, node_items, rows_scanned, split,
           max_items, overflow, cursor);
}

// Split scan and selection in one launch: workgroup `nd` < L scans the
// features of node nd (wave w takes features w, w + 16, ...), keeps the
// candidate with the highest gain, ties to the lowest feature id, and writes
// the node's record; with `plan` set, workgroup L cuts the row ranges of these
// nodes into the work items of the fused pass that follows, and every node adds
// the rows of its smaller side to rows_scanned.  grid L (+ 1), 1024 threads.
template <bool PAIR, bool F64>
__global__ void __launch_bounds__(1024)
k_scan_select(const long long *__restrict__ hg, const long long *__restrict__ hh,
              const unsigned long long *__restrict__ hc, int nbin_total, int F, int slots, int L,
              const NodeSum *__restrict__ tot, const int *__restrict__ shifts, GainParams gp, int hist_size,
              const unsigned *__restrict__ seg_start, NodeSum *__restrict__ tot_next,
              unsigned *__restrict__ seg_next, SplitRec *__restrict__ split, int *__restrict__ t_fid,
              int *__restrict__ t_bin, float *__restrict__ t_gain, int heap_off,
              const unsigned char *__restrict__ active, int plan, unsigned rows_per_item,
              WorkItem *__restrict__ work, unsigned *__restrict__ n_work, unsigned *__restrict__ node_first,
              unsigned *__restrict__ node_items, unsigned long long *__restrict__ rows_scanned,
              unsigned max_items, unsigned *__restrict__ overflow, unsigned *__restrict__ cursor) {
  if ((int)blockIdx.x >= L) {  // uniform per workgroup
    PlanBody(tot, seg_start, L, 0, rows_per_item, work, n_work, node_first, node_items, nullptr, nullptr, max_items,
             overflow, cursor);
    return;
  }
  __shared__ Cand s_cand[16];
  __shared__ int s_fid[16];
  const int nd = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const NodeSum t = tot[nd];
  Cand mine;
  mine.gain = 0.0f;
  mine.bin = -1;
  mine.left.g = mine.left.h = 0;
  mine.left.c = 0;
  int mine_fid = -1;
  for (int f = wave; f < F; f += 16) {
    if (active && !active[f]) continue;  // feature not sampled at this level
    const Cand c = ScanFeature<PAIR, F64>(hg, hh, hc, (size_t)nd * nbin_total + (size_t)f * slots, slots, t, shifts,
                                          gp, hist_size, lane);
    if (c.bin >= 0 && (mine_fid < 0 || mine.gain < c.gain)) {  // features ascend: ties keep the lower id
      mine = c;
      mine_fid = f;
    }
  }
  if (lane == 0) {
    s_cand[wave] = mine;
    s_fid[wave] = mine_fid;
  }
  __syncthreads();
  if (wave != 0) return;
  float gain = 0.0f;
  int fid = -1, bin = -1;
  long long lg = 0, lh = 0;
  unsigned long long lc = 0;
  if (lane < 16 && s_fid[lane] >= 0) {
    const Cand c = s_cand[lane];
    gain = c.gain;
    fid = s_fid[lane];
    bin = c.bin;
    lg = c.left.g;
    lh = c.left.h;
    lc = c.left.c;
  }
  for (int off = 8; off > 0; off >>= 1) {
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
  WriteNode(nd, t, gain, fid, bin, lg, lh, lc, seg_start, tot_next, seg_next, split, t_fid, t_bin, t_gain, heap_off);
  if (plan && rows_scanned && t.c != 0) {
    const unsigned long long cl = fid < 0 ? t.c : lc;
    atomicAdd(rows_scanned, min(cl, t.c - cl));
  }
}

}  // namespace
}  // namespace arb
#endif  // ARBORETUM_AMD_KERNELS_SPLIT_H_
