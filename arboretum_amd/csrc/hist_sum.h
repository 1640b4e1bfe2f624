// Stand-alone histogram sums of node segments on the device (hist_sum.hip).
#ifndef ARBORETUM_AMD_HIST_SUM_H_
#define ARBORETUM_AMD_HIST_SUM_H_
#include <cstddef>
#include <cstdint>

namespace arb {

// Arguments of HistTreeGrower::HistSum (src/core/hist_tree_grower.h:17-23),
// widened from one feature column to a quad-packed matrix.  Every pointer is a
// device pointer.
struct HistSumArgs {
  const uint32_t *bins;        // [Q][stride] words, four 8-bit bin ids each, rows in node order
  unsigned long long stride;   // words between the quad columns (>= nrow)
  int ncol;                    // features; Q = ceil(ncol / 4)
  long long nrow;
  const float *grad;           // [nrow]
  const float *hess;           // [nrow], or null: the row count is the hessian (squared error)
  const unsigned *node_size;   // nodes + 1 non-decreasing row offsets: node k = rows [node_size[k], node_size[k+1])
  int nodes;
  int use_trick;               // build the smaller node of each sibling pair (ties -> left), derive the other
  const long long *parent_g;   // with use_trick: [nodes / 2][4 Q * 256], as sum_g
  const long long *parent_h;
  const unsigned *parent_c;
  int shift_g, shift_h;        // sums are integers: value * 2^shift rounded to nearest
  long long *sum_g;            // out [nodes][4 Q][256]
  long long *sum_h;            // out, may be null without hessians
  unsigned *bin_count;         // out [nodes][4 Q][256]
  void *stream;                // hipStream_t, null = the default stream
};

// Allocates its work memory (plan, per-work-item slabs), runs and waits.
void HistSum(const HistSumArgs &args);
// Rows per work item HistSum plans for nrow rows in `nodes` segments (host arithmetic only).
unsigned HistSumRowsPerItem(size_t nrow, int nodes);

// The same without any allocation: plan and slabs live in a static device
// array of 32 MB + 192 KB per GPU; enqueues on args.stream and returns without
// waiting.  status (device, may be null): 0, 1 = bad node offsets, 2 = internal.
// Throws for sizes the array cannot hold.
void HistSumNoAlloc(const HistSumArgs &args, unsigned *status);

}  // namespace arb
#endif  // ARBORETUM_AMD_HIST_SUM_H_
