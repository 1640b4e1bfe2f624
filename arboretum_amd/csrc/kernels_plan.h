// Work planning on the device: row ranges of nodes cut into work items.
#ifndef ARBORETUM_AMD_KERNELS_PLAN_H_
#define ARBORETUM_AMD_KERNELS_PLAN_H_
#include "device_common.h"

namespace arb {
namespace {

// Rows per work item for `rows` rows in `nodes` node ranges on `cus` compute units that hold
// one work item at a time (one LDS histogram): a launch then runs in rounds of `cus` items, and
// a round with a single item costs as much as a full one.
// Few nodes (at most cus / 8): the fewest rounds r such that r * cus items of at most `cap`
// rows cover the rows when every node adds up to two short items; the items of those rounds
// are equally long, so the rounds are full.
// Many nodes: their short items would unbalance such rounds, so the items are a quarter of a
// compute unit's share of the rows and the units even out over several items each.
// Item sizes are multiples of 1024 rows.  *items: a bound on the items of the plan.
__host__ __device__ inline unsigned BalancedRowsPerItem(unsigned long long rows, unsigned nodes, unsigned cap,
                                                        unsigned cus, unsigned *items) {
  if (nodes <= cus / 8) {
    for (unsigned r = 1; r <= 64; ++r) {
      const long long slots = (long long)r * cus - 2ll * nodes - 2;
      if (slots <= 0) continue;
      unsigned long long per = (rows + (unsigned long long)slots - 1) / (unsigned long long)slots;
      per = (per + 1023) / 1024 * 1024;
      if (per < 1024) per = 1024;
      if (per <= cap) {
        *items = r * cus;
        return (unsigned)per;
      }
    }
  }
  unsigned long long per = (rows + 4ull * cus - 1) / (4ull * cus);
  per = (per + 1023) / 1024 * 1024;
  if (per < 1024) per = 1024;
  if (per > cap) per = cap;
  *items = (unsigned)(rows / per) + 2 * nodes + 2;
  return (unsigned)per;
}
// The most items a plan by that rule can have for at most `rows` rows in at most `nodes` nodes.
inline unsigned BalancedPlanItems(unsigned long long rows, unsigned nodes, unsigned cap, unsigned cus) {
  unsigned few = 0, many = 0;
  BalancedRowsPerItem(rows, nodes <= cus / 8 ? nodes : cus / 8, cap, cus, &few);  // fewer nodes selected than present
  const unsigned at_cap = (unsigned)(rows / cap) + 2 * nodes + 2;
  many = 4 * cus + 2 * nodes + 2;
  unsigned most = few > many ? few : many;
  return most > at_cap ? most : at_cap;
}

// ------------------------------------------------------------------ planner
// Splits the row ranges of the selected nodes of a level into work items of
// at most `rows_per_item` rows (a multiple of 64; at most len / rows_per_item
// + 2 items per node).  select: 0 = every node, 1 = the smaller
// child of each sibling pair, ties -> left (hist_grad_sum.cu:279-294).
// rows_scanned (optional) is advanced by the rows that will be accumulated
// into histograms: the selected rows, or, when `split` is given (fused
// partition + histogram over parent nodes), the smaller side of every split.
// cursor (optional): two words per node, cleared here; the fused pass claims
// the destination ranges of its work items on them.
// balance_cus (optional): rows_per_item is then the most an item may hold, and
// the item size is chosen here from the rows and nodes actually selected
// (BalancedRowsPerItem); the launch must hold the rounds that the same rule
// gives for the largest row and node counts the caller can have.
// One workgroup.
__device__ __forceinline__ void PlanBody(const NodeSum *__restrict__ tot, const unsigned *__restrict__ seg_start,
                                         int L, int select, unsigned rows_per_item,
                                         WorkItem *__restrict__ work, unsigned *__restrict__ n_work,
                                         unsigned *__restrict__ node_first, unsigned *__restrict__ node_items,
                                         unsigned long long *__restrict__ rows_scanned,
                                         const SplitRec *__restrict__ split, unsigned max_items,
                                         unsigned *__restrict__ overflow,
                                         unsigned *__restrict__ cursor = nullptr, unsigned balance_cus = 0) {
  __shared__ unsigned s_base[kMaxPlanNodes + 1];
  __shared__ unsigned s_wave[16];
  __shared__ unsigned s_carry;
  __shared__ unsigned long long s_rows;
  __shared__ unsigned long long s_sel_rows;
  __shared__ unsigned s_sel_nodes, s_per;
  const int tid = threadIdx.x;
  if (tid == 0) {
    s_carry = 0;
    s_rows = 0;
    s_sel_rows = 0;
    s_sel_nodes = 0;
  }
  __syncthreads();
  if (balance_cus != 0) {  // uniform over the workgroup
    for (int nd = tid; nd < L; nd += 1024) {
      const unsigned long long len = tot[nd].c;
      bool sel = true;
      if (select == 1) {
        const unsigned long long sib = tot[nd ^ 1].c;
        sel = (nd & 1) ? (len < sib) : (len <= sib);
      }
      if (sel && len > 0) {
        atomicAdd(&s_sel_rows, len);
        atomicAdd(&s_sel_nodes, 1u);
      }
    }
    __syncthreads();
    if (tid == 0) {
      unsigned bound;
      s_per = BalancedRowsPerItem(s_sel_rows, s_sel_nodes, rows_per_item, balance_cus, &bound);
    }
    __syncthreads();
    rows_per_item = s_per;
  }
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
        // item boundaries sit at multiples of 64 rows from the node's start
        // rounded down to one, so that every item but a node's first begins on
        // a 256-byte boundary of the row arrays
        cnt = (unsigned)(((seg_start[nd] & 63u) + len + rows_per_item - 1) / rows_per_item);
        unsigned long long acc = len;
        if (split) {
          const unsigned long long cl = split[nd].left.c;
          acc = min(cl, len - cl);
        }
        atomicAdd(&s_rows, acc);
      }
      node_items[nd] = sel ? cnt : 0xffffffffu;  // 0xffffffff marks "not selected"
      if (cursor) {  // destination cursors of the node's two children in the fused pass
        cursor[2 * nd] = 0;
        cursor[2 * nd + 1] = 0;
      }
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
    const unsigned origin = start - (start & 63u);
    WorkItem it;
    it.node = lo;
    it.begin = max(start, origin + k * rows_per_item);
    it.end = min(start + len, origin + (k + 1) * rows_per_item);
    it.first = s_base[lo];
    work[w] = it;
  }
}

__global__ void __launch_bounds__(1024)
k_plan(const NodeSum *__restrict__ tot, const unsigned *__restrict__ seg_start, int L, int select,
       unsigned rows_per_item, WorkItem *__restrict__ work, unsigned *__restrict__ n_work,
       unsigned *__restrict__ node_first, unsigned *__restrict__ node_items,
       unsigned long long *__restrict__ rows_scanned, const SplitRec *__restrict__ split,
       unsigned max_items, unsigned *__restrict__ overflow, unsigned balance_cus,
       unsigned *__restrict__ cursor = nullptr) {
  PlanBody(tot, seg_start, L, select, rows_per_item, work, n_work, node_first, node_items, rows_scanned, split,
           max_items, overflow, cursor, balance_cus);
}


}  // namespace
}  // namespace arb
#endif  // ARBORETUM_AMD_KERNELS_PLAN_H_
