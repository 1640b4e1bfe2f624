// Histogram sums of node segments as a stand-alone device operation: the
// counterpart of HistTreeGrower::HistSum (src/core/hist_tree_grower.h:17-23,
// src/core/hist_tree_grower.cu:200-301, kernels src/core/hist_grad_sum.cu:109-406),
// which the reference's own tests call directly (tests/cpp/test_hist_sum.cu).
// The reference runs it once per feature column; here one call covers every
// feature of a quad-packed matrix with the tree builder's own kernels: k_plan
// cuts the node segments into work items, k_hist builds one LDS histogram per
// work item and writes it to a slab, k_hist_reduce adds the slabs of a node
// and, with the subtraction trick, derives the larger sibling from the parent.
// All pointers of the entry points are device pointers.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <mutex>
#include <stdexcept>
#include <string>

#include "device_common.h"
#include "hist_sum.h"
#include "kernels_hist.h"
#include "kernels_launch.h"
#include "kernels_partition.h"
#include "kernels_plan.h"

namespace arb {
namespace {

// Everything the kernels of one call need besides the caller's arrays.
struct HistSumScratch {
  NodeSum *tot;
  unsigned *seg;
  unsigned *node_first;
  unsigned *node_items;
  unsigned *n_work;
  unsigned *overflow;
  int *shifts;
  WorkItem *work;
  unsigned long long *slab;
};

constexpr size_t Align256(size_t v) { return (v + 255) / 256 * 256; }

// Bytes of the small arrays in front of the slabs (for up to max_nodes nodes
// and max_items work items).
size_t HistSumHeadBytes(int max_nodes, unsigned max_items) {
  return Align256((size_t)max_nodes * sizeof(NodeSum)) + 3 * Align256((size_t)max_nodes * sizeof(unsigned)) +
         Align256(64) + Align256((size_t)max_items * sizeof(WorkItem));
}

HistSumScratch Carve(unsigned char *base, int max_nodes, unsigned max_items) {
  HistSumScratch s;
  unsigned char *p = base;
  s.tot = reinterpret_cast<NodeSum *>(p);
  p += Align256((size_t)max_nodes * sizeof(NodeSum));
  s.seg = reinterpret_cast<unsigned *>(p);
  p += Align256((size_t)max_nodes * sizeof(unsigned));
  s.node_first = reinterpret_cast<unsigned *>(p);
  p += Align256((size_t)max_nodes * sizeof(unsigned));
  s.node_items = reinterpret_cast<unsigned *>(p);
  p += Align256((size_t)max_nodes * sizeof(unsigned));
  s.n_work = reinterpret_cast<unsigned *>(p);
  s.overflow = s.n_work + 1;
  s.shifts = reinterpret_cast<int *>(s.n_work + 2);
  p += Align256(64);
  s.work = reinterpret_cast<WorkItem *>(p);
  p += Align256((size_t)max_items * sizeof(WorkItem));
  s.slab = reinterpret_cast<unsigned long long *>(p);
  return s;
}

// Node sizes and segment starts from the offsets the caller passes (the
// reference's node_size array: nodes + 1 non-decreasing row offsets), the
// fixed-point shifts, cleared counters.  status (optional): 0, or 1 when the
// offsets are not non-decreasing within [0, nrow].  One workgroup.
__global__ void __launch_bounds__(1024)
k_hist_sum_setup(const unsigned *__restrict__ node_size, int nodes, unsigned nrow, int shift_g, int shift_h,
                 NodeSum *__restrict__ tot, unsigned *__restrict__ seg, unsigned *__restrict__ n_work,
                 unsigned *__restrict__ overflow, int *__restrict__ shifts, unsigned *__restrict__ status) {
  __shared__ unsigned s_bad;
  if (threadIdx.x == 0) s_bad = 0;
  __syncthreads();
  for (int nd = threadIdx.x; nd < nodes; nd += blockDim.x) {
    const unsigned b = node_size[nd], e = node_size[nd + 1];
    const bool ok = b <= e && e <= nrow;
    if (!ok) s_bad = 1;
    NodeSum t;
    t.g = 0;
    t.h = 0;
    t.c = ok ? e - b : 0;  // a bad segment is skipped, never read
    tot[nd] = t;
    seg[nd] = ok ? b : 0;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    *n_work = 0;
    *overflow = 0;
    shifts[0] = shift_g;
    shifts[1] = shift_h;
    if (status) *status = s_bad;
  }
}

// A work plan that did not fit its launch bound is reported as status 2.
__global__ void k_hist_sum_status(const unsigned *__restrict__ overflow, unsigned *__restrict__ status) {
  if (threadIdx.x == 0 && blockIdx.x == 0 && *overflow != 0 && *status == 0) *status = 2;
}

struct Shape {
  int Q, quads_per_group, slab_entries, nbin_total;
  size_t slab_words;  // 64-bit words of one work item's slab
};

Shape ShapeOf(int ncol, bool pair) {
  Shape s;
  s.Q = (ncol + 3) / 4;
  const size_t per_block = HistLdsBytes(kBlockQuads, pair);
  s.quads_per_group = (int)std::min<size_t>((kLdsBudget - 1024) / per_block * kBlockQuads, kMaxGroupQuads);
  s.quads_per_group = std::min(s.quads_per_group, s.Q);
  s.slab_entries = HistBlocks(s.Q) * kBlockEntries;
  s.nbin_total = s.Q * 4 * kSlots;
  s.slab_words = (size_t)s.slab_entries * (pair ? 2 : 1);
  return s;
}

// Rows per work item so that a plan over `nodes` node segments of nrow rows
// in all has at most max_items items; 0 when that is impossible.
unsigned RowsPerItem(size_t nrow, int nodes, unsigned max_items) {
  if (max_items < 2u * (unsigned)nodes + 2u) return 0;
  const size_t row_items = max_items - 2u * (unsigned)nodes - 1u;
  size_t t = std::max<size_t>((nrow + row_items - 1) / row_items, 1);
  t = (t + kHistThreads - 1) / kHistThreads * kHistThreads;
  if (t > kMaxHistRows) return 0;
  return (unsigned)t;
}

void Validate(const HistSumArgs &a) {
  if (!a.bins || !a.grad || !a.node_size || !a.sum_g || !a.bin_count) throw std::runtime_error("null pointer argument");
  if (a.hess && !a.sum_h) throw std::runtime_error("sum_h is needed with hessians");
  if (a.ncol < 1 || a.nodes < 1 || a.nodes > kMaxPlanNodes) throw std::runtime_error("bad feature or node count");
  if (a.nrow < 1 || a.nrow >= (1ll << 31) || a.stride < (unsigned long long)a.nrow) throw std::runtime_error("bad row count or stride");
  if (a.use_trick) {
    if (a.nodes % 2 != 0) throw std::runtime_error("the subtraction trick needs sibling pairs");
    if (!a.parent_g || !a.parent_c || (a.hess && !a.parent_h)) throw std::runtime_error("the subtraction trick needs the parents' histograms");
  }
  if (a.shift_g < -64 || a.shift_g > 96 || a.shift_h < -64 || a.shift_h > 96) throw std::runtime_error("bad fixed-point shift");
}

// Enqueues the kernels of one call on `st`.  `mem` holds HistSumHeadBytes(...)
// + max_items * slab bytes, or the slabs start at slab_base.
void Enqueue(const HistSumArgs &a, const Shape &sh, unsigned char *mem, unsigned max_items, unsigned per_item,
             unsigned *status, hipStream_t st, unsigned char *slab_base = nullptr) {
  const bool pair = a.hess != nullptr;
  HistSumScratch s = Carve(mem, a.nodes, max_items);
  if (slab_base) s.slab = reinterpret_cast<unsigned long long *>(slab_base);
  hipLaunchKernelGGL(k_hist_sum_setup, dim3(1), dim3(1024), 0, st, a.node_size, a.nodes, (unsigned)a.nrow, a.shift_g,
                     a.shift_h, s.tot, s.seg, s.n_work, s.overflow, s.shifts, status);
  hipLaunchKernelGGL(k_plan, dim3(1), dim3(1024), 0, st, s.tot, s.seg, a.nodes, a.use_trick ? 1 : 0, per_item, s.work,
                     s.n_work, s.node_first, s.node_items, (unsigned long long *)nullptr, (const SplitRec *)nullptr,
                     max_items, s.overflow, 0u);
  const unsigned grid = (unsigned)std::min<size_t>((size_t)a.nrow / per_item + 2 * (size_t)a.nodes + 1, max_items);
  for (int q0 = 0; q0 < sh.Q; q0 += sh.quads_per_group) {
    const int nq = std::min(sh.quads_per_group, sh.Q - q0);
    if (pair)
      LaunchHist<true>(nq, st, grid, a.bins, (size_t)a.stride, q0, a.ncol, a.grad, a.hess, s.shifts, s.work, s.n_work,
                       s.slab, sh.slab_entries);
    else
      LaunchHist<false>(nq, st, grid, a.bins, (size_t)a.stride, q0, a.ncol, a.grad, a.hess, s.shifts, s.work, s.n_work,
                        s.slab, sh.slab_entries);
  }
  dim3 rgrid((sh.slab_entries + 63) / 64, a.nodes);
  if (pair)
    hipLaunchKernelGGL((k_hist_reduce<true, 16>), rgrid, dim3(1024), 0, st, s.slab, sh.slab_entries, sh.nbin_total,
                       s.node_first, s.node_items, 0, (const SplitRec *)nullptr, (const NodeSum *)nullptr, a.sum_g,
                       a.sum_h, a.bin_count, a.parent_g, a.parent_h, a.parent_c, a.use_trick ? 1 : 0, 0, 0,
                       HistBlocks(sh.quads_per_group));
  else
    hipLaunchKernelGGL((k_hist_reduce<false, 16>), rgrid, dim3(1024), 0, st, s.slab, sh.slab_entries, sh.nbin_total,
                       s.node_first, s.node_items, 0, (const SplitRec *)nullptr, (const NodeSum *)nullptr, a.sum_g,
                       a.sum_h, a.bin_count, a.parent_g, a.parent_h, a.parent_c, a.use_trick ? 1 : 0, 0, 0,
                       HistBlocks(sh.quads_per_group));
  if (status) hipLaunchKernelGGL(k_hist_sum_status, dim3(1), dim3(64), 0, st, s.overflow, status);
  HIP_OK(hipGetLastError());
}

// ---- work memory of the entry point that allocates nothing -----------------
// One array per GPU (each device that loads this library holds its own copy
// until the process ends): the plan and counters of a call, then the slabs.
// Its name is only a handle on the host; the address on the current device
// comes from hipGetSymbolAddress, once per device.
constexpr size_t kStaticSlabBytes = (size_t)32 << 20;
constexpr unsigned kStaticMaxItems = 1024;
constexpr size_t kStaticHeadBytes = (size_t)192 << 10;  // >= HistSumHeadBytes(kMaxPlanNodes, kStaticMaxItems)
constexpr size_t kStaticBytes = kStaticHeadBytes + kStaticSlabBytes;
static __device__ __align__(256) unsigned char scratch[kStaticBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
unsigned char *g_scratch_ptr[kMaxDevices] = {};

unsigned char *ScratchOfCurrentDevice() {
  int dev = 0;
  HIP_OK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) throw std::runtime_error("device index out of range");
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    HIP_OK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) throw std::runtime_error("no device address for the static work memory");
    g_scratch_ptr[dev] = static_cast<unsigned char *>(p);
  }
  return g_scratch_ptr[dev];
}

}  // namespace

void HistSumNoAlloc(const HistSumArgs &a, unsigned *status) {
  Validate(a);
  const bool pair = a.hess != nullptr;
  const Shape sh = ShapeOf(a.ncol, pair);
  const size_t slab_bytes = sh.slab_words * 8;
  static_assert(kStaticHeadBytes >= (size_t)kMaxPlanNodes * (sizeof(NodeSum) + 3 * sizeof(unsigned)) + 5 * 256 +
                                        (size_t)kStaticMaxItems * sizeof(WorkItem) + 256,
                "head of the static work memory too small");
  const unsigned max_items = (unsigned)std::min<size_t>(kStaticMaxItems, kStaticSlabBytes / slab_bytes);
  const unsigned per_item = RowsPerItem((size_t)a.nrow, a.nodes, max_items);
  if (per_item == 0)
    throw std::runtime_error(
        "too large for the static work memory: it holds " + std::to_string(max_items) + " work items of " +
        std::to_string(slab_bytes >> 10) + " KB for this width, each of at most " + std::to_string(kMaxHistRows) +
        " rows, and every node takes two of them (use AHistSum)");
  unsigned char *mem = ScratchOfCurrentDevice();
  // the caller's status word, or one in the work memory that nobody reads
  unsigned *st_word = status ? status : reinterpret_cast<unsigned *>(mem + kStaticHeadBytes - 256);
  Enqueue(a, sh, mem, max_items, per_item, st_word, static_cast<hipStream_t>(a.stream),
          mem + kStaticHeadBytes);
}

// Rows per work item of AHistSum: about 512 items where items of at most kMaxHistRows rows
// allow it, else items of that many rows (more than 512 x 64512 rows: more items, never
// smaller ones).
unsigned HistSumRowsPerItem(size_t nrow, int nodes) {
  const unsigned want = 512u + 2u * (unsigned)nodes + 2u;
  const unsigned fit = RowsPerItem(nrow, nodes, want);
  return fit != 0 ? std::max(fit, (unsigned)kHistThreads) : kMaxHistRows;
}

void HistSum(const HistSumArgs &a) {
  Validate(a);
  const bool pair = a.hess != nullptr;
  const Shape sh = ShapeOf(a.ncol, pair);
  // one work item per CU and round where the rows allow it, as the tree builder plans a level
  const unsigned per_item = HistSumRowsPerItem((size_t)a.nrow, a.nodes);
  const unsigned max_items = (unsigned)((size_t)a.nrow / per_item + 2 * (size_t)a.nodes + 2);
  const size_t bytes = HistSumHeadBytes(a.nodes, max_items) + (size_t)max_items * sh.slab_words * 8 + 256;
  unsigned char *mem = nullptr;
  HIP_OK(hipMalloc((void **)&mem, bytes));
  unsigned *status = reinterpret_cast<unsigned *>(mem + bytes - 256);
  unsigned host_status = 0;
  hipStream_t st = static_cast<hipStream_t>(a.stream);
  try {
    Enqueue(a, sh, mem, max_items, per_item, status, st);
    HIP_OK(hipStreamSynchronize(st));
    HIP_OK(hipMemcpy(&host_status, status, sizeof(unsigned), hipMemcpyDeviceToHost));
  } catch (...) {
    (void)hipFree(mem);
    throw;
  }
  HIP_OK(hipFree(mem));
  if (host_status == 1) throw std::runtime_error("node_size must hold non-decreasing row offsets within the matrix");
  if (host_status != 0) throw std::runtime_error("internal: work plan exceeded its launch bound");
}

}  // namespace arb
