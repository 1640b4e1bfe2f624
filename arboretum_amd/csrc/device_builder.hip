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
// is laid out bin-major, the features of a bin in blocks of 16, and every
// lane of a wave updates a different feature of its own row at a time: the 16
// lanes that one pass of the LDS atomic unit serves never share a bank pair or
// an address, whatever the bins are.  Each workgroup writes its LDS histogram
// to a private slab in HBM; a reduce kernel adds the slabs of a node, turns
// them feature-major, and derives the larger sibling as parent - smaller
// child.  All sums are integers: the result does not depend on scheduling.
//
// The kernels live in kernels_*.h (one header per stage), shared constants
// and records in device_common.h.  What replaces what (reference file:line):
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
#include "device_common.h"
#include "gain.h"
#include "kernels_final.h"
#include "kernels_hist.h"
#include "kernels_indexed.h"
#include "kernels_launch.h"
#include "kernels_objective.h"
#include "kernels_partition.h"
#include "kernels_plan.h"
#include "kernels_quantise.h"
#include "kernels_split.h"
#include "kernels_stream.h"

namespace arb {

struct DeviceMatrix {
  size_t rows = 0, stride = 0;
  int F = 0, Q = 0;          // Q words of 32 bits per row
  int bits = 8;              // bits per bin id: 8 (four features per word) or 16 (two)
  int slots = kSlots;        // histogram slots per feature
  // 8-bit ids with ninth-bit words per row in columns Q .. Q + H - 1 (ids up to 256; a word per 32
  // features): a feature that fills 256 value bins and has missing values besides (SplitTest)
  bool hi = false;
  int H = 0;                 // ninth-bit words per row in use (0 without ninth bits)
  int W() const { return Q + H; }  // words of a row that kernels read and move
  int cols = 0;              // columns allocated per row (Q, or more when ninth bits might be needed)
  // matrices of several ninth-bit words whose rows stay in place: the bits as bit columns [F][strideb]
  uint8_t *hibits = nullptr;
  size_t strideb = 0;
  uint32_t *bins = nullptr;  // resident: [cols][stride] in HBM
  // wide resident matrices, built on first use: the same bins row-major, RS words per row
  uint32_t *rec = nullptr;
  unsigned rec_largest_id = 0;  // the largest bin id (byte) seen while the records were built
  int RS = 0;
  // and column-major with one byte per bin id: [4 Q][stride8]
  uint8_t *bytes = nullptr;
  size_t stride8 = 0;
  // streamed: pinned host blocks [cols][block_rows], block b = rows [b*block_rows, ...)
  bool streamed = false;
  size_t block_rows = 0;
  std::vector<uint32_t *> host_blocks;
  bool owns_blocks = true;  // false: the caller's blocks (ACreateFromQuantizedBlocks)
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
  if (m->rec) (void)hipFree(m->rec);
  if (m->bytes) (void)hipFree(m->bytes);
  if (m->hibits) (void)hipFree(m->hibits);
  if (m->owns_blocks)
    for (uint32_t *b : m->host_blocks)
      if (b) (void)hipHostFree(b);
  delete m;
}

// Exact method (DataMatrix::InitExact, src/io/io.cu:437-482): every value becomes its rank
// among the sorted distinct values of its column.  Returns the ranks row-major [rows][F] and
// fills data->thresholds / reduced_size: the split "ranks <= q left" separates at the value
// of rank q + 1 (the smallest value that goes right, src/core/garden.cu:463-467).
// A feature with more distinct values than the histograms hold: an error, or with allow_more an
// empty result (the caller then keeps sorted row lists instead of bin ids).
static std::vector<uint16_t> ExactRanks(DataMatrix *data, size_t *most_distinct, bool allow_more) {
  const size_t n = data->rows;
  const int F = (int)data->columns_dense;
  std::vector<uint16_t> ranks(n * F);
  std::vector<std::vector<float>> mapping(F);
  std::atomic<bool> has_nan{false};
  std::atomic<int> too_many{-1};
  ParallelTasks((size_t)F, [&](size_t f) {
    if (has_nan || too_many >= 0) return;
    std::vector<float> m(data->data[f]);
    for (float v : m)
      if (v != v) has_nan = true;
    if (has_nan) return;
    std::sort(m.begin(), m.end());
    m.erase(std::unique(m.begin(), m.end()), m.end());
    if (m.size() > (size_t)kMaxWideSlots) {
      too_many = (int)f;
      return;
    }
    const float *col = data->data[f].data();
    for (size_t i = 0; i < n; ++i)
      ranks[i * F + f] = (uint16_t)(std::lower_bound(m.begin(), m.end(), col[i]) - m.begin());
    mapping[f].swap(m);
  });
  if (has_nan) throw std::runtime_error("the exact method does not take missing values (NaN); use method 1 (hist)");
  if (too_many >= 0) {
    if (allow_more) {
      *most_distinct = (size_t)kMaxWideSlots + 1;
      return {};
    }
    throw std::runtime_error("the exact method handles up to " + std::to_string(kMaxWideSlots) +
                             " distinct values per feature without internals.exact_sort; feature " +
                             std::to_string((int)too_many) + " has more: use method 1 (hist)");
  }
  size_t most = 1;
  for (int f = 0; f < F; ++f) most = std::max(most, mapping[f].size());
  *most_distinct = most;
  for (int f = 0; f < F; ++f) {
    data->reduced_size[f] = (int)mapping[f].size();
    data->thresholds[f].assign(most, std::numeric_limits<float>::infinity());
    for (size_t k = 0; k + 1 < mapping[f].size(); ++k) data->thresholds[f][k] = mapping[f][k + 1];
  }
  return ranks;
}

void QuantiseOnDevice(DataMatrix *data, int hist_size, bool verbose, bool streamed, size_t block_rows, bool exact,
                      int exact_sort) {
  if (data->quantised) {
    if (data->quantised_exact != exact) throw std::runtime_error("data matrix was prepared for the other method");
    if (!exact && data->hist_size != hist_size) throw std::runtime_error("data matrix was quantised with another hist_size");
    return;
  }
  if (exact && data->is_prebinned) throw std::runtime_error("the exact method needs float features, not bin ids");
  if (exact) hist_size = 1;  // set below from the data
  if (hist_size < 1) throw std::runtime_error("hist_size must be positive");
  const size_t n = data->rows;
  const int F = (int)data->columns_dense;
  if (n == 0 || F == 0) throw std::runtime_error("empty data matrix");
  // Rows are indexed with 32 bits inside a block of a streamed matrix and with 64 bits across
  // blocks; a resident matrix and the quantiser's sort index whole columns with 32 bits.
  if (n >= (1ull << 31) && !(streamed && data->is_prebinned))
    throw std::runtime_error("too many rows: 2^31 and more need bin ids (ACreateFromQuantized...) and "
                             "internals.upload_features = false");
  if (data->external_blocks) {
    if (!streamed) throw std::runtime_error("a matrix over caller-owned blocks is streamed: set internals.upload_features to false");
    std::unique_ptr<DeviceMatrix, void (*)(DeviceMatrix *)> ext(new DeviceMatrix(), FreeDeviceMatrix);
    ext->rows = n;
    ext->F = F;
    ext->Q = (F + 3) / 4;
    ext->cols = ext->Q;
    ext->stride = (n + 63) / 64 * 64;
    ext->streamed = true;
    ext->owns_blocks = false;
    ext->block_rows = data->stream_block_rows;
    ext->host_blocks = data->stream_blocks;
    data->thresholds.assign(F, {});
    data->reduced_size.assign(F, 0);
    for (int f = 0; f < F; ++f) {
      data->thresholds[f].resize(hist_size);
      for (int k = 0; k < hist_size; ++k) data->thresholds[f][k] = (float)k + 0.5f;
      data->reduced_size[f] = std::min(hist_size, kSlots);
    }
    data->device = ext.release();
    data->hist_size = hist_size;
    data->quantised = true;
    return;
  }
  std::unique_ptr<DeviceMatrix, void (*)(DeviceMatrix *)> dm(new DeviceMatrix(), FreeDeviceMatrix);
  dm->rows = n;
  dm->F = F;
  dm->Q = (F + 3) / 4;
  dm->stride = (n + 63) / 64 * 64;
  dm->streamed = streamed;
  // Only a quantiser run at hist_size 256 and more can hand out the id 256; the matrix then gets
  // room for ninth-bit words, one per 32 features (used if some feature turns out to need them).
  const bool may_need_hi = !exact && !data->is_prebinned && hist_size >= kSlots;
  const int hi_words = (F + 31) / 32;
  dm->cols = dm->Q + (may_need_hi ? hi_words : 0);
  uint32_t *d_col = nullptr;  // streamed: one quad column at a time on the device
  uint32_t *d_hi = nullptr;   // the column of ninth-bit words while the features are quantised
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
      HIP_OK(hipHostMalloc((void **)&dm->host_blocks[b], (size_t)dm->cols * block_rows * sizeof(uint32_t), hipHostMallocDefault));
    d_col = DevAlloc<uint32_t>(dm->stride);
    if (may_need_hi) d_hi = DevAlloc<uint32_t>((size_t)hi_words * dm->stride);
  } else {
    dm->bins = DevAlloc<uint32_t>((size_t)dm->cols * dm->stride);
    if (may_need_hi) d_hi = dm->bins + (size_t)dm->Q * dm->stride;
  }
  if (d_hi) HIP_OK(hipMemset(d_hi, 0, (size_t)hi_words * dm->stride * sizeof(uint32_t)));
  // streamed: quad q of all rows (in d_col) -> its slice of every host block
  auto store_quad = [&](int q, const uint32_t *col) {
    for (size_t b = 0; b < nblocks; ++b) {
      const size_t r0 = b * block_rows, rows = std::min(block_rows, n - r0);
      HIP_OK(hipMemcpy(dm->host_blocks[b] + (size_t)q * block_rows, col + r0, rows * sizeof(uint32_t),
                       hipMemcpyDeviceToHost));
    }
  };
  data->thresholds.assign(F, {});
  data->reduced_size.assign(F, 0);

  if (exact) {
    size_t most = 1;
    std::vector<uint16_t> ranks;
    if (exact_sort <= 0) ranks = ExactRanks(data, &most, exact_sort < 0);
    if (ranks.empty()) {
      // sorted row lists per feature instead of bin ids (exact_builder.hip)
      if (streamed) throw std::runtime_error("the exact method over sorted row lists is not built for streamed matrices");
      dm.reset();
      PrepareExactSort(data);
      return;
    }
    hist_size = (int)most;
    if (most <= (size_t)kSlots) {
      // 8-bit ids: through the pre-quantised path below
      data->prebinned.resize(n * F);
      for (size_t i = 0; i < n * F; ++i) data->prebinned[i] = (uint8_t)ranks[i];
    } else {
      if (streamed) throw std::runtime_error("a feature has more than 256 distinct values: 16-bit ids are not built for streamed matrices");
      int slots = kSlots;
      while ((size_t)slots < most) slots *= 2;
      dm->bits = 16;
      dm->slots = slots;
      dm->Q = dm->cols = (F + 1) / 2;
      HIP_OK(hipFree(dm->bins));
      dm->bins = DevAlloc<uint32_t>((size_t)dm->Q * dm->stride);
      uint16_t *d_in = DevAlloc<uint16_t>(n * F);
      HIP_OK(hipMemcpy(d_in, ranks.data(), n * F * sizeof(uint16_t), hipMemcpyHostToDevice));
      hipLaunchKernelGGL(k_pack_prebinned16, dim3(GridFor(n, 256)), dim3(256), 0, 0, d_in, F, dm->Q, dm->bins,
                         dm->stride, n);
      HIP_OK(hipDeviceSynchronize());
      HIP_OK(hipFree(d_in));
    }
  }
  if (exact && dm->bits == 16) {
    // done above
  } else if (data->is_prebinned || exact) {
    for (int f = 0; f < F && !exact; ++f) {
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
          if (bits == 8 && data->reduced_size[f] + (has_nan ? 1 : 0) > kSlots) {
            // id 256: the ninth-bit words take it, where the matrix has them
            if (d_hi == nullptr || data->reduced_size[f] + 1 > kSlots + 1) return false;
            dm->hi = true;
            dm->H = hi_words;
          }
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
                             out, n, d_hi ? d_hi + (size_t)((q * W) >> 5) * dm->stride : nullptr, (q * W) & 31);
        else
          hipLaunchKernelGGL(k_bin_assign_wide, dim3(GridFor(n, 256)), dim3(256),
                             2 * (size_t)hist_size * sizeof(float), 0, d_x, nc, d_thr, hist_size, d_size, out, n);
        HIP_OK(hipGetLastError());
        HIP_OK(hipDeviceSynchronize());
        if (streamed) store_quad(q, d_col);
      }
      for (int w = 0; streamed && w < dm->H; ++w) store_quad(dm->Q + w, d_hi + (size_t)w * dm->stride);
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
      dm->hi = false;
      dm->H = 0;
      d_hi = nullptr;  // (was a part of dm->bins: a resident matrix)
      dm->Q = dm->cols = (F + 1) / 2;
      dm->bins = DevAlloc<uint32_t>((size_t)dm->Q * dm->stride);
      if (!quantise_columns(16)) throw std::runtime_error("internal: 16-bit quantisation failed");
    }
    HIP_OK(hipFree(d_x));
    HIP_OK(hipFree(d_thr));
    HIP_OK(hipFree(d_size));
    for (int k = 0; k < 2; ++k) HIP_OK(hipHostFree(stage[k]));
  }
  if (d_col) HIP_OK(hipFree(d_col));
  if (streamed && d_hi) HIP_OK(hipFree(d_hi));
  if (dm->hi) dm->slots = kSlots + 1;
  if (streamed) {
    data->stream_blocks = dm->host_blocks;
    data->stream_block_rows = block_rows;
  }
  // the largest bin id of the matrix: bin ids from the quantiser stop at a feature's number of
  // real bins (the missing-value bin), ranks at the largest number of distinct values less one,
  // bin ids handed in are looked at
  data->max_bin = 255;
  if (dm->bits == 8) {
    if (exact) {
      data->max_bin = hist_size - 1;
    } else if (!data->is_prebinned) {
      data->max_bin = 0;
      for (int f = 0; f < F; ++f) data->max_bin = std::max(data->max_bin, std::min(data->reduced_size[f], 255));
    } else if (!data->prebinned.empty()) {
      std::atomic<int> most{0};
      ParallelFor(data->prebinned.size(), [&](size_t b, size_t e) {
        int m = 0;
        for (size_t i = b; i < e; ++i) m = std::max(m, (int)data->prebinned[i]);
        int seen = most.load();
        while (m > seen && !most.compare_exchange_weak(seen, m)) {
        }
      });
      data->max_bin = most;
    }
  }
  if (exact) std::vector<uint8_t>().swap(data->prebinned);  // prediction walks the float columns
  data->device = dm.release();
  data->hist_size = hist_size;
  data->quantised = true;
  data->quantised_exact = exact;
}

void GetBinLayout(const DataMatrix &data, int *bits, int *slots) {
  if (data.exact_sort) throw std::runtime_error("the matrix is kept as sorted row lists (exact method): it has no bin ids");
  const DeviceMatrix *dm = data.device;
  if (!dm) throw std::runtime_error("data matrix is not quantised");
  *bits = dm->bits;
  *slots = dm->slots;
}

void GetDeviceBins16(const DataMatrix &data, uint16_t *out) {
  const DeviceMatrix *dm = data.device;
  if (!dm) throw std::runtime_error("data matrix is not quantised");
  if (dm->bits == 8 && dm->hi) {
    // byte + ninth bit; resident or in pinned blocks
    std::vector<uint32_t> q;
    if (!dm->streamed) {
      q.resize((size_t)dm->W() * dm->stride);
      HIP_OK(hipMemcpy(q.data(), dm->bins, q.size() * sizeof(uint32_t), hipMemcpyDeviceToHost));
    }
    for (size_t r = 0; r < dm->rows; ++r) {
      const uint32_t *base = dm->streamed ? dm->host_blocks[r / dm->block_rows] : q.data();
      const size_t st = dm->streamed ? dm->block_rows : dm->stride, at = dm->streamed ? r % dm->block_rows : r;
      for (int f = 0; f < dm->F; ++f) {
        const uint32_t hi = base[(size_t)(dm->Q + (f >> 5)) * st + at];
        out[r * dm->F + f] = (uint16_t)(((base[(size_t)(f >> 2) * st + at] >> (8 * (f & 3))) & 255u) + ((hi >> (f & 31)) & 1u));
      }
    }
    return;
  }
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
  if (dm->hi) throw std::runtime_error("the matrix has bin ids up to 256: ask for 16-bit ids");
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
  unsigned *ids = nullptr;  // indexed mode: the row at each position (null: position = row)
};

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
  unsigned *cursor;     // claims destinations (null: read item_base)
  unsigned *item_base;  // claimed destination bases, two per work item
  unsigned long long *slab;
  int slab_entries;
  const uint32_t *split_bins;  // start of the whole matrix
  int q0;                      // first quad of this launch
  LevelScan scan;              // hg set: the pass finds the splits of its parents itself
};

template <bool PAIR, int NQ, bool WRITE, bool GROUP, bool PACK, int HI>
void LaunchFusedNQ(hipStream_t st, unsigned grid, const FusedArgs &a) {
  const size_t lds = HistLdsBytes(NQ, PAIR, HI != 0);
  static std::once_flag configured;
  AllowLdsOnce(configured, k_part_hist<PAIR, NQ, WRITE, GROUP, PACK, HI>, lds);
  hipLaunchKernelGGL((k_part_hist<PAIR, NQ, WRITE, GROUP, PACK, HI>), dim3(grid), dim3(kHistThreads), lds, st,
                     a.bins + (size_t)a.q0 * a.stride, a.bins_out ? a.bins_out + (size_t)a.q0 * a.stride : nullptr,
                     a.stride, a.F, a.g, a.g_out, a.h, a.h_out, a.shifts, a.split, a.tot, a.seg_start, a.work,
                     a.n_work, a.cursor, a.item_base, a.slab, a.slab_entries, a.split_bins, a.q0, a.scan);
}

template <bool PAIR, bool WRITE, bool GROUP, bool PACK, int HI = 0>
void LaunchFused(int nq, hipStream_t st, unsigned grid, const FusedArgs &a) {
#define ARB_CASE(N) \
  case N: LaunchFusedNQ<PAIR, N, WRITE, GROUP, PACK, HI>(st, grid, a); break;
  switch (nq) {
    ARB_CASE(1) ARB_CASE(2) ARB_CASE(3) ARB_CASE(4) ARB_CASE(5) ARB_CASE(6) ARB_CASE(7) ARB_CASE(8)
    default: throw std::runtime_error("internal: bad quad count");
  }
#undef ARB_CASE
}

class HipTreeBuilder : public TreeBuilder {
 public:
  HipTreeBuilder(const Configuration &cfg, DataMatrix *data) : cfg_(cfg), data_(data) {
    try {
      Construct(cfg, data);
    } catch (...) {  // e.g. out of device memory: give back what was allocated so far
      Release();
      throw;
    }
  }

  ~HipTreeBuilder() override { Release(); }

 private:
  void Construct(const Configuration &cfg, DataMatrix *data) {
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
    hi_ = dm_->hi;
    // one ninth-bit word (at most 32 features, one LDS histogram): ids of 256 are accumulated in a
    // 257th row of entries; several words: they are left out of the histograms (AccumulateRow)
    hi_rows_ = hi_ && dm_->H == 1;
    hi_skip_ = hi_ && !hi_rows_;
    W_ = dm_->W();
    hi_word_ = hi_ ? Q_ : -1;
    report_slots_ = dm_->slots;
    slots_ = hi_ ? kSlots : dm_->slots;  // bin 256 lives in a cell of its own behind the 256-bin histograms
    code_ = BinCode::Of(dm_->bits);
    if (wide_) {
      if (dm_->streamed) throw std::runtime_error("16-bit bins are not built for streamed matrices");
      nbin_total_ = F_ * slots_;
      slab_entries_ = nbin_total_;  // slabs are feature-major
    } else {
      hi_base_ = hi_rows_ ? Q_ * 4 * kSlots : 0;
      nbin_total_ = Q_ * 4 * kSlots + (hi_rows_ ? Q_ * 4 : 0);
      slab_entries_ = HistBlocks(Q_) * kBlockEntries;
    }
    // entries between the slabs of two work items: with ninth bits one more row, bin 256
    slab_stride_ = wide_ ? slab_entries_ : HistBlocks(Q_) * (kBlockEntries + (hi_rows_ ? kBlockFeatures : 0));
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
    single_group_ = Q_ <= quads_per_group_;
    if (hi_rows_ && (!single_group_ || HistLdsBytes(Q_, pair_, true) > kLdsBudget - 1024))
      throw std::runtime_error("internal: ninth-bit ids in a 257th row need a matrix of one group of quads");
    if (hi_skip_ && !dm_->streamed && D_ > 2 && Q_ > 256)
      throw std::runtime_error("more than 1024 features with 257 bin ids per feature: use hist_size 255");
    // Matrices wider than one group of quads: rows stay in place as records, only (row id,
    // gradients) are re-ordered (kernels_indexed.h).
    // Taken when every feature fits ONE LDS histogram of the bins in use (a record is then read
    // once per level, whole): e.g. 200 features of 65 bins with one word per cell.
    rec_slots_ = std::min(kSlots, data->max_bin + 1);
    const size_t rec_lds = (size_t)HistBlocks(Q_) * kBlockFeatures * rec_slots_ * 8 * (pair_ ? 2 : 1);
    rec_one_launch_ = rec_lds <= kLdsBudget - 1024;  // else groups of quads_per_group_ quads at 256 bins
    // Measured per tree at 10.5 M rows, 256 bins, max_depth 8 (rows in place / rows moved once per
    // group of eight quads): 33 features 2.47 / 2.39 ms, 40: 2.52 / 2.44, 44: 2.69 / 2.54, 48: 2.56 /
    // 2.68, 64: 2.59 / 3.27, 128: 3.88 / 6.21; with the bins in use in one LDS histogram (64 bins)
    // 33: 2.10 / 2.40, 44: 2.24 / 2.53.  So rows stay in place from 48 features (twelve quads) on,
    // and at any width when one launch builds the whole histogram.
    const bool in_place_pays = rec_one_launch_ || Q_ >= 12;
    // (with ninth bits in several words the rows always stay in place: the row-moving group passes do not carry them)
    indexed_ = !wide_ && !dm_->streamed && !single_group_ && D_ > 2 && Q_ <= 256 &&  // at most 64 pieces of 16 bytes per record
               (hi_skip_ || cfg.internal.wide_rows_in_place >= 2 ||
                (cfg.internal.wide_rows_in_place == 1 && in_place_pays));
    // one launch: a power of two of blocks between the bins of the LDS image when that still fits
    rec_lay_blocks_ = 0;
    if (rec_one_launch_) {
      int p2 = 1;
      while (p2 < HistBlocks(Q_)) p2 *= 2;
      // ... in the LDS and in the slab of a work item, which holds 256 bins of the blocks the matrix has
      if ((size_t)p2 * kBlockFeatures * rec_slots_ * 8 * (pair_ ? 2 : 1) <= kLdsBudget - 1024 &&
          (size_t)p2 * rec_slots_ <= (size_t)HistBlocks(Q_) * kSlots)
        rec_lay_blocks_ = p2;
    }
    fused_ = trick_ && !wide_ && !indexed_;
    if (wide_) {
      // features per histogram launch (an even number, two per word)
      const size_t per_feature = (size_t)slots_ * 8 * (pair_ ? 2 : 1);
      wide_group_ = (int)std::max<size_t>(2, (kLdsBudget - 1024) / per_feature / 2 * 2);
    }

    // per-row state in original order
    d_y_ = DevAlloc<float>(n_);
    d_labels_ = DevAlloc<uint8_t>(n_);
    d_yhat_ = DevAlloc<float>(n_ * K_);
    streamed_ = dm_->streamed;
    // Logistic gradients of 0/1 labels travel as one float per row (PackGrad):
    // there is no h array then, and kernels given h == nullptr unpack g.
    // (never together with rows kept in place: those kernels take g and h as two arrays)
    pack_ = cfg.objective == kLogisticRegression && !streamed_ && !wide_ && !indexed_ && Q_ <= kMaxGroupQuads &&
            data->y.size() == n_ &&
            std::all_of(data->y.begin(), data->y.end(), [](float v) { return v == 0.0f || v == 1.0f; });
    d_g_ = DevAlloc<float>(n_ * K_);
    d_h_ = pack_ ? nullptr : DevAlloc<float>(n_ * K_);
    d_leaf_ = DevAlloc<unsigned>(n_);
    if (!data->y.empty()) HIP_OK(hipMemcpy(d_y_, data->y.data(), n_ * sizeof(float), hipMemcpyHostToDevice));
    if (!data->labels.empty()) HIP_OK(hipMemcpy(d_labels_, data->labels.data(), n_, hipMemcpyHostToDevice));
    float init = cfg.tree.initial_y;
    if (cfg.objective == kLogisticRegression) init = std::log(init / (1 - init));  // objective.h:55-57
    hipLaunchKernelGGL(k_fill_f32, dim3(GridFor(n_ * K_, 256)), dim3(256), 0, stream_, d_yhat_, init, n_ * K_);
    data->y_hat.assign(n_ * K_, init);  // garden.cu:104

    if (streamed_) {
      const size_t br = dm_->block_rows;
      HIP_OK(hipStreamCreateWithFlags(&copy_stream_, hipStreamNonBlocking));
      for (int b = 0; b < 2; ++b) {
        blk_[b] = DevAlloc<uint32_t>((size_t)W_ * br);
        HIP_OK(hipEventCreateWithFlags(&ev_ready_[b], hipEventDisableTiming));
        HIP_OK(hipEventCreateWithFlags(&ev_free_[b], hipEventDisableTiming));
      }
      stage_.bins = DevAlloc<uint32_t>((size_t)W_ * br);
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
        if (indexed_) buf_[b].ids = DevAlloc<unsigned>(n_);
        else buf_[b].bins = DevAlloc<uint32_t>((size_t)W_ * stride_);
        buf_[b].g = DevAlloc<float>(n_);
        buf_[b].h = pack_ ? nullptr : DevAlloc<float>(n_);
      }
    }
    if (indexed_) {
      if (!dm_->rec) {  // records: whole 64-byte units (what memory answers a gather with), built once per matrix
        dm_->RS = (W_ + 15) / 16 * 16;  // (the ninth-bit words of a row follow its quads, in the columns and in the record)
        dm_->rec = DevAlloc<uint32_t>(n_ * (size_t)dm_->RS);
        AllowLds(k_to_records, (size_t)64 * (dm_->RS + 1) * sizeof(uint32_t));
        unsigned *d_largest = DevAlloc<unsigned>(1);
        HIP_OK(hipMemsetAsync(d_largest, 0, sizeof(unsigned), stream_));
        hipLaunchKernelGGL(k_to_records, dim3((unsigned)((n_ + 63) / 64)), dim3(256),
                           (size_t)64 * (dm_->RS + 1) * sizeof(uint32_t), stream_, dm_->bins, stride_, W_, dm_->rec,
                           dm_->RS, n_, Q_, d_largest);
        HIP_OK(hipGetLastError());
        HIP_OK(hipMemcpyAsync(&dm_->rec_largest_id, d_largest, sizeof(unsigned), hipMemcpyDeviceToHost, stream_));
        HIP_OK(hipStreamSynchronize(stream_));
        HIP_OK(hipFree(d_largest));
      }
      // the histogram over the records is sized by max_bin and does not look at the ids again
      if ((int)dm_->rec_largest_id > data->max_bin)
        throw std::runtime_error("internal: the matrix holds bin id " + std::to_string(dm_->rec_largest_id) +
                                 ", more than the " + std::to_string(data->max_bin) + " it was prepared for");
      if (hi_skip_ && !dm_->hibits) {
        dm_->strideb = (n_ + 7) / 8;
        dm_->strideb = (dm_->strideb + 63) / 64 * 64;
        dm_->hibits = DevAlloc<uint8_t>((size_t)F_ * dm_->strideb);
        hipLaunchKernelGGL(k_to_hi_bits, dim3((unsigned)((n_ / 8 + 256) / 256)), dim3(256), 0, stream_,
                           dm_->bins + (size_t)Q_ * stride_, stride_, F_, dm_->hibits, dm_->strideb, n_);
        HIP_OK(hipGetLastError());
      }
      if (!dm_->bytes) {
        dm_->stride8 = (n_ + 255) / 256 * 256;
        dm_->bytes = DevAlloc<uint8_t>((size_t)Q_ * 4 * dm_->stride8);
        hipLaunchKernelGGL(k_to_byte_columns, dim3((unsigned)((n_ + 255) / 256)), dim3(256), 0, stream_, dm_->bins,
                           stride_, Q_, dm_->bytes, dm_->stride8, n_);
        HIP_OK(hipGetLastError());
      }
    }
    // level state
    const int max_nodes = 1 << (D_ - 1);
    for (int b = 0; b < 2; ++b) {
      d_tot_[b] = DevAlloc<NodeSum>(max_nodes);
      d_seg_[b] = DevAlloc<unsigned>(max_nodes);
      d_hg_[b] = DevAlloc<long long>((size_t)last_nodes * nbin_total_);
      d_hh_[b] = DevAlloc<long long>((size_t)last_nodes * nbin_total_);
      d_hc_[b] = DevAlloc<unsigned long long>((size_t)last_nodes * nbin_total_);
      // cells of bins that no row can have are never written (rows in place with fewer than 256
      // bins in use) and must read as zero
      HIP_OK(hipMemsetAsync(d_hg_[b], 0, (size_t)last_nodes * nbin_total_ * sizeof(long long), stream_));
      HIP_OK(hipMemsetAsync(d_hh_[b], 0, (size_t)last_nodes * nbin_total_ * sizeof(long long), stream_));
      HIP_OK(hipMemsetAsync(d_hc_[b], 0, (size_t)last_nodes * nbin_total_ * sizeof(unsigned long long), stream_));
    }
    d_split_ = DevAlloc<SplitRec>(last_nodes);
    d_cand_ = DevAlloc<Cand>((size_t)last_nodes * F_);
    // two sets of (first item, items) per node: a slab reduction reads the plan of the pass before it
    // while it writes the plan of the pass after it
    d_node_first2_ = DevAlloc<unsigned>((size_t)2 * last_nodes);
    d_node_items2_ = DevAlloc<unsigned>((size_t)2 * last_nodes);
    d_node_first_ = d_node_first2_;
    d_node_items_ = d_node_items2_;
    own_scan_ = fused_ && single_group_;
    // row passes of a streamed matrix cover one block at a time
    const size_t plan_rows = dm_->streamed ? std::min(n_, dm_->block_rows) : n_;
    max_hist_items_ = (unsigned)(plan_rows / HistRowsPerItem(plan_rows)) + 2 * last_nodes + 2;
    max_hist_items_ = std::max<unsigned>(max_hist_items_, 1024 + 2 * last_nodes + 2);
    {
      hipDeviceProp_t prop;
      int dev = 0;
      HIP_OK(hipGetDevice(&dev));
      HIP_OK(hipGetDeviceProperties(&prop, dev));
      cus_ = (unsigned)std::max(prop.multiProcessorCount, 1);
      // the balanced plans of un-fused histogram launches: whole rounds of cus_ items
      // records read once per group of quads: the groups of a work item run side by side, on
      // that many compute units
      rec_groups_ = rec_one_launch_ ? 1 : (HistBlocks(Q_) + HistBlocks(quads_per_group_) - 1) / HistBlocks(quads_per_group_);
      hist_cus_ = indexed_ ? std::max(1u, cus_ / (unsigned)rec_groups_) : cus_;
      for (int level = 0; level + 1 < D_; ++level)
        max_hist_items_ = std::max(max_hist_items_, BalancedPlanItems(plan_rows, 1u << level, kMaxHistRows, hist_cus_));
      max_hist_items_ = std::max(max_hist_items_, BalancedPlanItems(plan_rows, 1u, kMaxHistRows, cus_));
    }
    max_part_items_ = std::max<unsigned>((unsigned)(plan_rows / kPartRows + 1) + 2 * last_nodes, max_hist_items_);
    d_hwork_ = DevAlloc<WorkItem>(max_hist_items_);
    d_pwork_ = DevAlloc<WorkItem>(max_part_items_);
    d_nwork_ = DevAlloc<unsigned>(2);
    d_wave_left_ = DevAlloc<unsigned>((size_t)max_part_items_ * kItemWaves);
    d_item_left_ = DevAlloc<unsigned>((size_t)2 * max_part_items_);  // also the claimed bases of the fused pass
    d_cursor2_ = DevAlloc<unsigned>((size_t)2 * last_nodes);
    d_slab_ = DevAlloc<unsigned long long>((size_t)std::max(max_hist_items_, max_part_items_) * slab_stride_ * (pair_ ? 2 : 1));
    d_shifts_ = DevAlloc<int>(2);
    d_records_ = DevAlloc<uint32_t>(kRecordRing * RecordWords());
    d_gmax_ = DevAlloc<unsigned>(1);
    d_rows_scanned_ = DevAlloc<unsigned long long>(kScanLevels);  // one counter per tree level
    d_overflow_ = DevAlloc<unsigned>(1);
    HIP_OK(hipMemsetAsync(d_overflow_, 0, sizeof(unsigned), stream_));
    HIP_OK(hipMemsetAsync(d_rows_scanned_, 0, kScanLevels * sizeof(unsigned long long), stream_));
    HIP_OK(hipMemsetAsync(d_gmax_, 0, sizeof(unsigned), stream_));
    const int internal = (1 << (D_ - 1)) - 1;
    d_tfid_ = DevAlloc<int>(internal);
    d_tbin_ = DevAlloc<int>(internal);
    d_tgain_ = DevAlloc<float>(internal);
    d_weights_ = DevAlloc<float>(max_nodes);
    d_active_ = DevAlloc<unsigned char>((size_t)(D_ - 1) * F_);
    rnd_.seed(cfg.internal.seed);  // garden.cu:87
    int shifts[2] = {30, 0};
    if (cfg.objective == kLogisticRegression) {
      shifts[1] = 32;  // 0 <= h <= 1/4
      // labels outside [0, 1] widen the gradient range
      float ymin = 0.0f, ymax = 1.0f;
      for (float v : data->y) {
        ymin = std::min(ymin, v);
        ymax = std::max(ymax, v);
      }
      shifts[0] = LogisticGradShift(ymin, ymax);
    }
    if (cfg.objective >= kSoftMaxOneVsAll) shifts[1] = 31;     // 0 <= h <= 1/2
    HIP_OK(hipMemcpyAsync(d_shifts_, shifts, sizeof(shifts), hipMemcpyHostToDevice, stream_));
    HIP_OK(hipStreamSynchronize(stream_));
    if (streamed_) KeepBlocksResident(cfg.internal.stream_resident_bytes);
  }

  void Release() noexcept {
    if (stream_) (void)hipStreamSynchronize(stream_);
    void *ptrs[] = {d_y_, d_labels_, d_yhat_, d_g_, d_h_, d_leaf_, d_split_, d_cand_, d_node_first2_,
                    d_node_items2_, d_hwork_, d_pwork_, d_nwork_, d_wave_left_, d_item_left_, d_slab_,
                    d_shifts_, d_gmax_, d_rows_scanned_, d_tfid_, d_tbin_, d_tgain_, d_weights_, d_active_, d_overflow_, d_records_, d_cursor2_};
    for (void *p : ptrs)
      if (p) (void)hipFree(p);
    for (int b = 0; b < 2; ++b) {
      void *q[] = {buf_[b].bins, buf_[b].g, buf_[b].h, buf_[b].ids, d_tot_[b], d_seg_[b], d_hg_[b], d_hh_[b], d_hc_[b]};
      for (void *p : q)
        if (p) (void)hipFree(p);
    }
    for (hipEvent_t e : event_pool_) (void)hipEventDestroy(e);
    for (uint32_t *p : resident_)
      if (p) (void)hipFree(p);
    if (streamed_) {
      if (copy_stream_) (void)hipStreamSynchronize(copy_stream_);
      void *sp[] = {blk_[0], blk_[1], stage_.bins, stage_.g, stage_.h, d_node_of_, d_blk_cnt_, d_blk_seg_,
                    d_cursor_, d_blk_tot_};
      for (void *p : sp)
        if (p) (void)hipFree(p);
      for (int b = 0; b < 2; ++b) {
        if (ev_ready_[b]) (void)hipEventDestroy(ev_ready_[b]);
        if (ev_free_[b]) (void)hipEventDestroy(ev_free_[b]);
      }
      if (copy_stream_) (void)hipStreamDestroy(copy_stream_);
    }
    if (stream_) (void)hipStreamDestroy(stream_);
  }

 public:
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
      ++trees_grown_;
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
    if (!leaf_valid_) {  // the last pass did not record them: walk the last tree now
      hipLaunchKernelGGL(k_leaf_ids, dim3(GridFor(n_, 256, 8192)), dim3(256), 0, stream_, dm_->bins, stride_, d_tfid_,
                         d_tbin_, D_, d_leaf_, n_, code_, hi_word_);
      HIP_OK(hipGetLastError());
      leaf_valid_ = true;
    }
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
    if (pack_) {
      for (size_t i = 0; i < n_; ++i) {
        float gv, hv;
        UnpackGrad(g[i], &gv, &hv);
        g[i] = gv;
        if (h) h[i] = hv;
      }
    } else if (h) {
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
  void EnableTiming(int level) override {
    ResolveTimings();
    timing_ = level != 0;
    dominant_only_ = level >= 2;
    sample_every_ = level == 3 ? 4 : 1;
    deep_open_ = false;
  }
  BuilderTimings GetTimings() override {
    ResolveTimings();
    return timings_;
  }
  unsigned long long RowsScanned() override {
    unsigned long long v[kScanLevels], sum = 0;
    RowsScannedByLevel(v);
    for (int k = 0; k < kScanLevels; ++k) sum += v[k];
    return sum;
  }
  void RowsScannedByLevel(unsigned long long *out) override {  // kScanLevels entries
    HIP_OK(hipStreamSynchronize(stream_));
    HIP_OK(hipMemcpy(out, d_rows_scanned_, kScanLevels * sizeof(unsigned long long), hipMemcpyDeviceToHost));
  }
  void StreamResidency(unsigned long long *resident, unsigned long long *blocks) override {
    *resident = resident_blocks_;
    *blocks = resident_.size();
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
    if (dominant_only_) {
      // only the fused pass is bracketed: an event where it starts, one where it
      // ends (level 3: on every fourth tree)
      if (phase == kHistDeep && trees_grown_ % sample_every_ != 0) return;
      if (phase != kHistDeep && !deep_open_) return;
      deep_open_ = phase == kHistDeep;
      if (!deep_open_) phase = kNone;
    }
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

  // the counter of rows accumulated into histograms at `level` (levels past the last counter share it)
  unsigned long long *ScanCounter(int level) { return d_rows_scanned_ + std::min(level, kScanLevels - 1); }
  // count_level >= 0: the planned rows are histogram work of that tree level
  // cursor: two claim cursors per node, cleared by the plan (passes that claim their output ranges)
  void Plan(int state, int L, int select, unsigned rows_per_item, WorkItem *work, unsigned *n_work,
            int count_level, const SplitRec *split, unsigned max_items, unsigned balance_cus = 0,
            unsigned *cursor = nullptr) {
    PlanOn(d_tot_[state], d_seg_[state], L, select, rows_per_item, work, n_work, count_level, split, max_items,
           balance_cus, cursor);
  }
  void PlanOn(const NodeSum *tot, const unsigned *seg, int L, int select, unsigned rows_per_item, WorkItem *work,
              unsigned *n_work, int count_level, const SplitRec *split, unsigned max_items,
              unsigned balance_cus = 0, unsigned *cursor = nullptr) {
    hipLaunchKernelGGL(k_plan, dim3(1), dim3(1024), 0, stream_, tot, seg, L, select,
                       rows_per_item, work, n_work, d_node_first_, d_node_items_,
                       count_level >= 0 ? ScanCounter(count_level) : (unsigned long long *)nullptr, split, max_items,
                       d_overflow_, balance_cus, cursor);
  }

  // Histograms of contiguous node ranges in `cur` (level order), feature group by group.
  void HistOfNodes(const RowBuffers &cur, int state, int L, bool select_smaller, size_t rows_max, bool root, int level) {
    // A CU holds one work item at a time, so the launch runs in rounds of cus_ items: the planner
    // sizes the items from the rows and nodes it finds selected so that the rounds are full
    // (one item per CU at the root); the grid holds the rounds of the largest case.
    // Rows in place in groups of quads: the root, whose rows are the matrix in its own order,
    // is read from the quad columns like a narrow matrix (one launch per group streams its
    // columns once; the groups of the record kernel share only half of their reads there).
    const bool records = indexed_ && (rec_one_launch_ || !root);
    const unsigned cus = records ? hist_cus_ : cus_;
    const unsigned grid = std::min(BalancedPlanItems(rows_max, (unsigned)L, kMaxHistRows, cus), max_hist_items_);
    Mark(kPlan);
    Plan(state, L, select_smaller ? 1 : 0, kMaxHistRows, d_hwork_, d_nwork_, level, nullptr, grid, cus);
    Mark(root ? kHistRoot : kHistDeep);
    if (wide_) {
      for (int f0 = 0; f0 < F_; f0 += wide_group_) {
        const int nf = std::min(wide_group_, F_ - f0);
        const size_t lds = (size_t)nf * slots_ * 8 * (pair_ ? 2 : 1);
        if (pair_) {
          static std::once_flag configured;
          AllowLdsOnce(configured, k_hist_wide<true>, kLdsBudget);
          hipLaunchKernelGGL(k_hist_wide<true>, dim3(grid), dim3(kHistThreads), lds, stream_, cur.bins, stride_, f0, nf,
                             slots_, cur.g, cur.h, d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_entries_);
        } else {
          static std::once_flag configured;
          AllowLdsOnce(configured, k_hist_wide<false>, kLdsBudget);
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
      if (records) {
        // one launch: every feature in one LDS histogram at rec_slots_ bins, or the groups of
        // quads at 256 bins side by side (a workgroup per work item and group)
        const int total = HistBlocks(Q_);
        const int pieces = rec_one_launch_ ? total : HistBlocks(quads_per_group_);
        const int ngroups = (total + pieces - 1) / pieces;
        const int slots = rec_one_launch_ ? rec_slots_ : kSlots;
        const int lay = rec_one_launch_ ? rec_lay_blocks_ : 0;   // blocks the LDS image is laid out for
        const size_t lds = (size_t)(lay > 0 ? lay : pieces) * kBlockFeatures * slots * 8 * (pair_ ? 2 : 1);
        const size_t item_words = rec_one_launch_ ? lds / 8 : (size_t)slab_entries_ * (pair_ ? 2 : 1);
        if (lds > kLdsBudget || (size_t)total * 4 > (size_t)dm_->RS || ngroups != rec_groups_ ||
            item_words > (size_t)slab_entries_ * (pair_ ? 2 : 1))
          throw std::runtime_error("internal: record histogram launch does not fit");
        const unsigned blocks = (grid + 7u) / 8u * 8u * (unsigned)ngroups;
        // a power of two of blocks in every group (the last may hold fewer), or in the padded layout
        const int last_pieces = total - (ngroups - 1) * pieces;
        const bool pow2 = lay > 0 ? (lay & (lay - 1)) == 0
                                  : (pieces & (pieces - 1)) == 0 && (last_pieces & (last_pieces - 1)) == 0;
#define ARB_REC(P, POW2, H)                                                                                      \
  do {                                                                                                            \
    static std::once_flag configured;                                                                             \
    AllowLdsOnce(configured, (k_hist_rec<P, POW2, H>), kLdsBudget);                                               \
    hipLaunchKernelGGL((k_hist_rec<P, POW2, H>), dim3(blocks), dim3(kHistThreads), lds, stream_, dm_->rec,        \
                       dm_->RS, cur.ids, Q_, slots, cur.g, cur.h, d_shifts_, d_hwork_, d_nwork_, d_slab_, pieces, \
                       total, ngroups, item_words, lay);                                                          \
  } while (0)
#define ARB_REC_P(P)                                   \
  do {                                                 \
    if (hi_skip_ && pow2) ARB_REC(P, true, true);      \
    else if (hi_skip_) ARB_REC(P, false, true);        \
    else if (pow2) ARB_REC(P, true, false);            \
    else ARB_REC(P, false, false);                     \
  } while (0)
        if (pair_) ARB_REC_P(true);
        else ARB_REC_P(false);
#undef ARB_REC_P
#undef ARB_REC
        if (timing_) ++(root ? timings_.hist_root_launches : timings_.hist_deep_launches);
        break;
      } else {
        HistLaunch(nq, grid, cur.bins, stride_, q0, cur.g, cur.h);
      }
      if (timing_) ++(root ? timings_.hist_root_launches : timings_.hist_deep_launches);
    }
    if (timing_ && root) timings_.hist_root_rows += n_;
  }

  // Gradient totals of the root: the sum over the slots of feature 0 of the root histogram, or, when
  // ids of 256 are left out of the histograms, over the gradients themselves (tot[0].g / .h are
  // zero: k_init_root).
  void RootTotals(int hb, int state, const RowBuffers &orig) {
    if (hi_skip_)
      hipLaunchKernelGGL(k_sum_grad, dim3(GridFor(n_, 256, 2048)), dim3(256), 0, stream_, orig.g, pair_ ? orig.h : nullptr,
                         n_, d_shifts_, d_tot_[state]);
    else
      hipLaunchKernelGGL(k_root_from_hist, dim3(1), dim3(64), 0, stream_, d_hg_[hb], d_hh_[hb], d_tot_[state], slots_,
                         hi_base_);
  }

  // k_hist over quads [q0, q0 + nq) of rows laid out with `stride` words between columns
  void HistLaunch(int nq, unsigned grid, const uint32_t *bins, size_t stride, int q0, const float *g, const float *h) {
    // the ninth-bit words of the 32 features of a group of eight quads: column Q_ + q0 / 8
    const uint32_t *hi_col = hi_ ? bins + (size_t)(Q_ + q0 / 8) * stride : nullptr;
    if (hi_skip_ && pair_)
      LaunchHist<true, 2>(nq, stream_, grid, bins, stride, q0, F_, g, h, d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_stride_, hi_col);
    else if (hi_skip_)
      LaunchHist<false, 2>(nq, stream_, grid, bins, stride, q0, F_, g, h, d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_stride_, hi_col);
    else if (hi_rows_ && pair_)
      LaunchHist<true, 1>(nq, stream_, grid, bins, stride, q0, F_, g, h, d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_stride_, hi_col);
    else if (hi_rows_)
      LaunchHist<false, 1>(nq, stream_, grid, bins, stride, q0, F_, g, h, d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_stride_, hi_col);
    else if (pair_)
      LaunchHist<true>(nq, stream_, grid, bins, stride, q0, F_, g, h, d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_stride_);
    else
      LaunchHist<false>(nq, stream_, grid, bins, stride, q0, F_, g, h, d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_stride_);
  }

  // plan_state >= 0: one more block plans the fused pass over this level's nodes (d_tot_ / d_seg_
  // [plan_state]) into the other set of (first item, items) per node, which is in use afterwards
  void Reduce(int L, int hb, bool by_parent, int parent_state, bool trick, bool accumulate = false,
              int plan_state = -1) {
    Mark(kReduce);
    const size_t last_nodes = (size_t)1 << (D_ - 2);
    unsigned *next_first = d_node_first_ == d_node_first2_ ? d_node_first2_ + last_nodes : d_node_first2_;
    unsigned *next_items = d_node_items_ == d_node_items2_ ? d_node_items2_ + last_nodes : d_node_items2_;
    NextPlan plan;
    if (plan_state >= 0) {
      plan.tot = d_tot_[plan_state];
      plan.seg_start = d_seg_[plan_state];
      plan.L = L;
      plan.rows_per_item = FusedRowsPerItem(L);
      plan.work = d_pwork_;
      plan.n_work = d_nwork_ + 1;
      plan.node_first = next_first;
      plan.node_items = next_items;
      plan.max_items = FusedGrid(L);
      plan.overflow = d_overflow_;
      plan.cursor = d_cursor2_;
    }
    // many nodes: few slabs per node and the output dominates -> longer output runs per block
    const bool wide_blocks = L >= 32;
    const int entries = wide_blocks ? 256 : 64;
    const int lds_slots = indexed_ && rec_one_launch_ ? rec_slots_ : kSlots;
    const int lay_blocks = indexed_ && rec_one_launch_ ? rec_lay_blocks_ : 0;
    // 16-bit bins: feature-major slabs; else the entries of the bins in use of every 16-feature block
    dim3 grid(wide_ ? (slab_entries_ + entries - 1) / entries
                    : slab_entries_ / kBlockEntries * ((lds_slots * kBlockFeatures + entries - 1) / entries) + (hi_rows_ ? 1 : 0),
              L);
    if (plan_state >= 0) grid.x += 1;
#define ARB_REDUCE(P, LN)                                                                                          \
  hipLaunchKernelGGL((k_hist_reduce<P, LN, unsigned long long>), grid, dim3(1024), 0, stream_, d_slab_, slab_entries_, nbin_total_,   \
                     d_node_first_, d_node_items_, by_parent ? 1 : 0, d_split_, d_tot_[parent_state], d_hg_[hb], \
                     d_hh_[hb], d_hc_[hb], d_hg_[hb ^ 1], d_hh_[hb ^ 1], d_hc_[hb ^ 1], trick ? 1 : 0,           \
                     accumulate ? 1 : 0, wide_ ? 1 : 0,                                                           \
                     indexed_ && rec_one_launch_ ? HistBlocks(Q_) : HistBlocks(quads_per_group_),                \
                     lds_slots, lay_blocks, hi_base_, plan)
    if (pair_) {
      if (wide_blocks) ARB_REDUCE(true, 4);
      else ARB_REDUCE(true, 16);
    } else {
      if (wide_blocks) ARB_REDUCE(false, 4);
      else ARB_REDUCE(false, 16);
    }
#undef ARB_REDUCE
    if (plan_state >= 0) {
      d_node_first_ = next_first;
      d_node_items_ = next_items;
    }
  }

  void GrowOne(int label) {
    const GainParams gp = cfg_.gain_params();
    RowBuffers orig;
    orig.bins = dm_->bins;
    orig.g = d_g_ + (size_t)label * n_;
    orig.h = d_h_ ? d_h_ + (size_t)label * n_ : nullptr;
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
    // The last pass of the tree can also build the root histogram of the next
    // one: logistic objective, gradients of the next round wanted, all quads in
    // one LDS histogram next to the node arrays.
    const bool next_grad = !inspect_ && K_ == 1;
    const size_t final_lds = FinalHistLdsBytes(Q_, D_, hi_rows_);
    const bool final_hist = next_grad && cfg_.objective == kLogisticRegression && single_group_ && !wide_ &&
                            final_lds <= kLdsBudget;
    int state = 0;  // d_tot_/d_seg_[state] describe the nodes of the current level
    for (int level = 0; level + 1 < D_; ++level) {
      const int L = 1 << level;
      const int hb = level & 1;  // histogram buffer of this level; the parent level is hb ^ 1
      const bool last = level + 2 >= D_;
      if (level == 0) {
        // the slabs of the root may have been written by the last pass of the previous tree
        if (!root_hist_ready_) HistOfNodes(orig, state, 1, false, n_, true, 0);
        root_hist_ready_ = false;
        Reduce(1, hb, false, state, false, false, own_scan_ && !last ? state : -1);
        // (the last pass of the previous tree has also summed the root's totals)
        if (!root_totals_ready_) RootTotals(hb, state, orig);
        root_totals_ready_ = false;
      } else {
        // rows are in the order of level-1; the parents' state is state ^ 1
        const int ps = state ^ 1, PL = L >> 1;
        const RowBuffers &src = level == 1 ? orig : buf_[level & 1];
        const RowBuffers &dst = buf_[(level & 1) ^ 1];
        if (fused_) {
          // the work plan was written together with the splits of the parents
          const unsigned grid = FusedGrid(PL);
          Mark(last ? kFusedLast : kHistDeep);
          // matrices wider than one LDS histogram: one launch per group of
          // quads; the first one moves the gradients
          for (int q0 = 0; q0 < Q_; q0 += quads_per_group_) {
            const int nq = std::min(quads_per_group_, Q_ - q0);
            LevelScan scan{};
            if (own_scan_) {  // the parents' splits are selected by the pass itself, from the scan's candidates
              scan.cand = d_cand_;
              scan.F = F_;
              scan.L = PL;
              scan.tot_next = d_tot_[state];
              scan.seg_next = d_seg_[state];
              scan.split = d_split_;
              scan.t_fid = d_tfid_;
              scan.t_bin = d_tbin_;
              scan.t_gain = d_tgain_;
              scan.heap_off = PL - 1;
              scan.active = sampling_ ? d_active_ + (size_t)(level - 1) * F_ : (const unsigned char *)nullptr;
              scan.node_first = d_node_first_;
              scan.rows_scanned = ScanCounter(level);
            }
            FusedArgs a{src.bins, last ? nullptr : dst.bins, stride_, F_, src.g, q0 == 0 ? dst.g : nullptr, src.h,
                        q0 == 0 ? dst.h : nullptr, d_shifts_, d_split_, d_tot_[ps], d_seg_[ps], d_pwork_,
                        d_nwork_ + 1, q0 == 0 ? d_cursor2_ : nullptr, d_item_left_, d_slab_, slab_stride_, src.bins,
                        q0, scan};
#define ARB_FUSED(P, W)                                                       \
  do {                                                                        \
    if (hi_rows_ && P && pack_) LaunchFused<P, W, false, P, 1>(nq, stream_, grid, a); \
    else if (hi_rows_) LaunchFused<P, W, false, false, 1>(nq, stream_, grid, a);   \
    else if (P && pack_ && single_group_) LaunchFused<P, W, false, P>(nq, stream_, grid, a); \
    else if (P && pack_) LaunchFused<P, W, true, P>(nq, stream_, grid, a);    \
    else if (single_group_) LaunchFused<P, W, false, false>(nq, stream_, grid, a); \
    else LaunchFused<P, W, true, false>(nq, stream_, grid, a);                \
  } while (0)
            if (pair_) {
              if (last) ARB_FUSED(true, false);
              else ARB_FUSED(true, true);
            } else {
              if (last) ARB_FUSED(false, false);
              else ARB_FUSED(false, true);
            }
#undef ARB_FUSED
            if (timing_ && (last || !dominant_only_ || trees_grown_ % sample_every_ == 0))
            ++(last ? timings_.fused_last_launches : timings_.hist_deep_launches);
          }
          Reduce(L, hb, true, ps, true, false, own_scan_ && !last ? state : -1);
        } else {
          const unsigned grid = (unsigned)std::min<size_t>(n_ / kPartRows + 2 * PL + 1, max_part_items_);
          Mark(kPlan);
          Plan(ps, PL, 0, kPartRows, d_pwork_, d_nwork_ + 1, -1, nullptr, grid, 0, indexed_ ? d_cursor2_ : nullptr);
          Mark(kPartition);
          if (indexed_) {
            // decisions, claims of the children's ranges and the move of (row id, g, h) in one launch
            if (pair_)
              hipLaunchKernelGGL(k_ix_part<true>, dim3(grid), dim3(kHistThreads), 0, stream_, dm_->bytes, dm_->stride8,
                                 src.ids, dst.ids, src.g, dst.g, src.h, dst.h, d_split_, d_seg_[ps], d_pwork_,
                                 d_nwork_ + 1, d_cursor2_, d_item_left_, dm_->hibits, dm_->strideb);
            else
              hipLaunchKernelGGL(k_ix_part<false>, dim3(grid), dim3(kHistThreads), 0, stream_, dm_->bytes, dm_->stride8,
                                 src.ids, dst.ids, src.g, dst.g, src.h, dst.h, d_split_, d_seg_[ps], d_pwork_,
                                 d_nwork_ + 1, d_cursor2_, d_item_left_, dm_->hibits, dm_->strideb);
          } else {
            hipLaunchKernelGGL(k_part_count, dim3(grid), dim3(kHistThreads), 0, stream_, src.bins, stride_, d_split_,
                               d_pwork_, d_nwork_ + 1, d_wave_left_, d_item_left_, code_, hi_word_);
            LaunchPartRows(grid, src, dst, ps);
          }
          HistOfNodes(dst, state, L, trick_, trick_ ? n_ / 2 : n_, false, level);
          Reduce(L, hb, false, ps, trick_);
        }
      }
      if (inspect_) KeepHist(level, L, hb, state);
      // (own_scan_: only the scan; the pass of the next level selects the splits of this level's nodes)
      LaunchSplit(level, L, hb, state, gp, fused_ && !last, own_scan_ && !last);
      if (last && !final_hist) LaunchLeafWeights(L, state, gp);
      state ^= 1;
    }
    // ---- leaf of every row, y_hat update, gradients of the next round
    Mark(kLeaf);
    bool record_written = false;
    {
      if (cfg_.objective == kLinearRegression) HIP_OK(hipMemsetAsync(d_gmax_, 0, sizeof(unsigned), stream_));
      if (final_hist) {
        // leaf weights, tree record, state and plan of the next tree's root in
        // one launch, then one pass: leaves, predictions, gradients and the
        // root histogram of the next tree
        const int last_L = 1 << (D_ - 2), last_state = state ^ 1;
        const unsigned per_item = HistRowsPerItem(n_, 256);
        const unsigned grid = (unsigned)std::min<size_t>(n_ / per_item + 2, max_hist_items_);
        if ((n_ + per_item - 1) / per_item > grid) throw std::runtime_error("internal: root plan exceeds its grid");
#define ARB_END(D)                                                                                                \
  hipLaunchKernelGGL((k_tree_end<true, D>), dim3((last_L + 127) / 128 + 1), dim3(128), 0, stream_, d_split_,      \
                     d_tot_[last_state], last_L, d_shifts_, gp, cfg_.tree.eta, d_weights_, d_tfid_, d_tbin_,      \
                     d_tgain_, d_overflow_, d_records_ + pending_.size() * RecordWords(), d_tot_[0], d_seg_[0],   \
                     (unsigned)n_, per_item, d_hwork_, d_nwork_, d_node_first_, d_node_items_, d_rows_scanned_)
        if (f64_) ARB_END(true);
        else ARB_END(false);
#undef ARB_END
        record_written = true;
        LaunchFinalHist(grid, label, final_lds);
        root_hist_ready_ = true;
        root_totals_ready_ = true;
        leaf_valid_ = false;  // not recorded by this pass; GetLeaves walks the tree when asked
      } else {
        LaunchFinal(dm_->bins, stride_, 0, n_, label, next_grad);
        leaf_valid_ = true;
      }
      grad_ready_ = next_grad;
    }
    if (record_written) Mark(kNone);
    else
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
  // Blocks that stay in device memory (the reference keeps as many columns as fit into 0.9 of the
  // free memory and streams the others, src/io/io.cu:496-507, src/core/garden.cu:296-347; here the
  // unit is the row block).  budget < 0: that rule; else at most `budget` bytes.  The resident
  // blocks are spread evenly over the matrix, so that the copies of the others run while the
  // kernels work on resident ones.
  void KeepBlocksResident(long long budget) {
    const size_t nblocks = dm_->host_blocks.size();
    const size_t block_bytes = (size_t)W_ * dm_->block_rows * sizeof(uint32_t);
    size_t free_b = 0, total_b = 0;
    HIP_OK(hipMemGetInfo(&free_b, &total_b));
    size_t allowed = (size_t)(0.9 * (double)free_b);
    if (budget >= 0) allowed = std::min(allowed, (size_t)budget);
    const size_t keep = std::min(nblocks, allowed / block_bytes);
    resident_.assign(nblocks, nullptr);
    for (size_t b = 0; b < nblocks; ++b) {
      if ((b + 1) * keep / nblocks == b * keep / nblocks) continue;  // keep of nblocks, evenly spread
      resident_[b] = DevAlloc<uint32_t>((size_t)W_ * dm_->block_rows);
      HIP_OK(hipMemcpy(resident_[b], dm_->host_blocks[b], block_bytes, hipMemcpyHostToDevice));
      ++resident_blocks_;
    }
  }

  // Block b in device memory for the kernels enqueued next: its resident copy, or one of the two
  // copy buffers, filled on the copy stream (the compute stream then waits for the copy).
  // Returns the buffer index, -1 for a resident block; DoneWithBlock after the last kernel that
  // reads it.
  const uint32_t *BlockOnDevice(size_t b, int *buf) {
    if (resident_[b]) {
      *buf = -1;
      return resident_[b];
    }
    *buf = CopyBlockIn(b);
    HIP_OK(hipStreamWaitEvent(stream_, ev_ready_[*buf], 0));
    return blk_[*buf];
  }
  void DoneWithBlock(int buf) {
    if (buf >= 0) HIP_OK(hipEventRecord(ev_free_[buf], stream_));
  }

  int CopyBlockIn(size_t b) {
    const int buf = (int)(next_copy_++ & 1);
    if (buf_used_[buf]) HIP_OK(hipStreamWaitEvent(copy_stream_, ev_free_[buf], 0));
    HIP_OK(hipMemcpyAsync(blk_[buf], dm_->host_blocks[b], (size_t)W_ * dm_->block_rows * sizeof(uint32_t),
                          hipMemcpyHostToDevice, copy_stream_));
    HIP_OK(hipEventRecord(ev_ready_[buf], copy_stream_));
    buf_used_[buf] = true;
    return buf;
  }

  // plan_next: also plan the fused pass of the next level over these nodes
  // scan_only: candidates per (node, feature) only (k_split_scan); the next fused pass selects
  void LaunchSplit(int level, int L, int hb, int state, const GainParams &gp, bool plan_next = false,
                   bool scan_only = false) {
    Mark(kSplit);
    const int hs = std::min(data_->hist_size, slots_);  // data_->hist_size: the configuration's, or the distinct values (exact method)
    const unsigned char *active = sampling_ ? d_active_ + (size_t)level * F_ : (const unsigned char *)nullptr;
    const unsigned per_item = FusedRowsPerItem(L);
    // From 32 nodes on, one launch: a workgroup per node scans its features and
    // selects.  With fewer nodes that would leave the gain arithmetic (28
    // features x 256 bins in double precision per node) on a few CUs, and the
    // scan over (feature, node) waves followed by the selection is faster.
    if (L >= 32 && !scan_only) {
#define ARB_SCAN_SELECT(P, D)                                                                                     \
  hipLaunchKernelGGL((k_scan_select<P, D>), dim3(L + (plan_next ? 1 : 0)), dim3(1024), 0, stream_, d_hg_[hb],     \
                     d_hh_[hb], d_hc_[hb], nbin_total_, F_, slots_, L, d_tot_[state], d_shifts_, gp, hs,          \
                     d_seg_[state], d_tot_[state ^ 1], d_seg_[state ^ 1], d_split_, d_tfid_, d_tbin_, d_tgain_,   \
                     L - 1, active, plan_next ? 1 : 0, per_item, d_pwork_, d_nwork_ + 1, d_node_first_,           \
                     d_node_items_, ScanCounter(level + 1), FusedGrid(L), d_overflow_, d_cursor2_)
      if (pair_ && f64_) ARB_SCAN_SELECT(true, true);
      else if (pair_) ARB_SCAN_SELECT(true, false);
      else if (f64_) ARB_SCAN_SELECT(false, true);
      else ARB_SCAN_SELECT(false, false);
#undef ARB_SCAN_SELECT
      return;
    }
    dim3 grid(F_, L);
#define ARB_SCAN(P, D) \
  hipLaunchKernelGGL((k_split_scan<P, D>), grid, dim3(64), 0, stream_, d_hg_[hb], d_hh_[hb], d_hc_[hb], \
                     nbin_total_, F_, slots_, d_tot_[state], d_shifts_, gp, hs, d_cand_)
    if (pair_ && f64_) ARB_SCAN(true, true);
    else if (pair_) ARB_SCAN(true, false);
    else if (f64_) ARB_SCAN(false, true);
    else ARB_SCAN(false, false);
#undef ARB_SCAN
    if (scan_only) return;
    if (plan_next) {
      hipLaunchKernelGGL(k_select_plan, dim3(1), dim3(1024), 0, stream_, d_cand_, F_, L, d_tot_[state],
                         d_seg_[state], d_tot_[state ^ 1], d_seg_[state ^ 1], d_split_, d_tfid_, d_tbin_, d_tgain_,
                         L - 1, active, per_item, d_pwork_, d_nwork_ + 1, d_node_first_, d_node_items_,
                         ScanCounter(level + 1), FusedGrid(L), d_overflow_, d_cursor2_);
    } else {
      hipLaunchKernelGGL(k_split_select, dim3((L + 15) / 16), dim3(1024), 0, stream_, d_cand_, F_, L,
                         d_tot_[state], d_seg_[state], d_tot_[state ^ 1], d_seg_[state ^ 1], d_split_,
                         d_tfid_, d_tbin_, d_tgain_, L - 1, active);
    }
  }

  // Stand-alone partition: groups of up to eight words per launch; the first
  // launch also moves the gradients.
  void LaunchPartRows(unsigned grid, const RowBuffers &src, const RowBuffers &dst, int ps) {
    for (int q0 = 0; q0 < W_; q0 += 8) {  // (the ninth-bit word moves like a quad)
      const int nq = std::min(8, W_ - q0);
#define ARB_PART(P, N, G)                                                                                        \
  hipLaunchKernelGGL((k_part_rows<P, N, G>), dim3(grid), dim3(kHistThreads), 0, stream_, src.bins, dst.bins,    \
                     stride_, q0, src.g, dst.g, src.h, dst.h, d_split_, d_seg_[ps], d_pwork_, d_nwork_ + 1,      \
                     d_wave_left_, d_item_left_, code_, hi_word_)
#define ARB_PART_N(N)                                          \
  case N:                                                      \
    if (q0 == 0) {                                             \
      if (pair_ && !pack_) ARB_PART(true, N, true);            \
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
    return (unsigned)std::min<size_t>(n_ / FusedRowsPerItem(PL) + 2 * PL + 1, max_part_items_);
  }
  // Rows per work item of the fused pass over PL parents.  A CU runs one
  // workgroup at a time, so the pass takes as many rounds as items / CUs rounded
  // up, and a round with a single item costs as much as a full one (measured:
  // 513 items take 18 % longer than 489).  Items are cut at multiples of the
  // item size from a node's start, so every parent adds at most one item to
  // rows / size (its last, short one); the size is chosen so that all items
  // fit one round (fewer, larger slabs as well) up to 32 parents and two rounds
  // beyond.
  unsigned FusedRowsPerItem(int PL) const {
    const size_t target = PL <= 32 ? (size_t)(254 - PL) : (size_t)std::max(256, 508 - PL);
    return HistRowsPerItem(n_, target);
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
    // the byte columns of a matrix whose rows stay in place (whole matrix only)
    const uint8_t *walk_bytes = indexed_ && bins == dm_->bins && row0 == 0 ? dm_->bytes : nullptr;
    int mode = 0;
    if (next_grad && cfg_.objective == kLinearRegression) mode = 1;
    if (next_grad && cfg_.objective == kLogisticRegression) mode = 2;
#define ARB_FINAL(M, N) \
  hipLaunchKernelGGL((k_final<M, N>), dim3(grid), dim3(256), lds, stream_, bins, stride, d_tfid_, d_tbin_, D_, \
                     d_weights_, yh, d_y_ + row0, d_leaf_ + row0, d_g_ + row0, d_h_ ? d_h_ + row0 : nullptr, d_gmax_, rows, code_, \
                     walk_bytes, dm_->stride8, hi_word_)
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
#define ARB_FH(N, H)                                                                                             \
  do {                                                                                                           \
    static std::once_flag configured;                                                                            \
    AllowLdsOnce(configured, k_final_hist<N, H>, kLdsBudget);                                                    \
    hipLaunchKernelGGL((k_final_hist<N, H>), dim3(grid), dim3(kHistThreads), lds, stream_, dm_->bins, stride_,  \
                       F_, d_tfid_, d_tbin_, D_, d_weights_, yh, d_y_, (unsigned *)nullptr, d_g_, d_h_,          \
                       d_shifts_, d_hwork_, d_nwork_, d_slab_, slab_stride_, d_tot_[0]);                         \
  } while (0)
#define ARB_CASE(N)           \
  case N:                     \
    if (hi_rows_) ARB_FH(N, 1);    \
    else ARB_FH(N, 0);        \
    break;
    switch (Q_) {
      ARB_CASE(1) ARB_CASE(2) ARB_CASE(3) ARB_CASE(4) ARB_CASE(5) ARB_CASE(6) ARB_CASE(7) ARB_CASE(8)
      default: throw std::runtime_error("internal: bad quad count");
    }
#undef ARB_CASE
#undef ARB_FH
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
        int buf = -1;
        const uint32_t *blk = BlockOnDevice(b, &buf);
        Mark(kPartition);
        hipLaunchKernelGGL(k_stream_route, dim3(GridFor(rows, 256, 1024)), dim3(256), 0, stream_, blk, br, rows,
                           level, trick ? 1 : 0, d_split_, d_tot_[state], d_node_of_ + row0, d_blk_cnt_, hi_word_);
        hipLaunchKernelGGL(k_stream_segments, dim3(1), dim3(1024), 0, stream_, d_blk_cnt_, L, d_blk_tot_, d_blk_seg_,
                           d_cursor_);
        // the root's rows are the block as it is; deeper, the rows of the built nodes are gathered
        // node by node into the staging buffer
        const bool in_place = level == 0;
        const uint32_t *hist_bins = in_place ? blk : stage_.bins;
        const float *hist_g = in_place ? orig.g + row0 : stage_.g, *hist_h = in_place ? orig.h + row0 : stage_.h;
        if (!in_place) {
          const unsigned tiles = (rows + kGatherTile - 1) / kGatherTile;
          const size_t lds = GatherLdsBytes(L);
          static std::once_flag configured;
          std::call_once(configured, [] {
            AllowLds(k_stream_gather<true>, kLdsBudget);
            AllowLds(k_stream_gather<false>, kLdsBudget);
          });
          if (pair_)
            hipLaunchKernelGGL(k_stream_gather<true>, dim3(tiles), dim3(1024), lds, stream_, blk, br, W_, rows,
                               orig.g + row0, orig.h + row0, d_node_of_ + row0, level, trick ? 1 : 0, d_tot_[state],
                               d_cursor_, stage_.bins, br, stage_.g, stage_.h);
          else
            hipLaunchKernelGGL(k_stream_gather<false>, dim3(tiles), dim3(1024), lds, stream_, blk, br, W_, rows,
                               orig.g + row0, orig.h + row0, d_node_of_ + row0, level, trick ? 1 : 0, d_tot_[state],
                               d_cursor_, stage_.bins, br, stage_.g, stage_.h);
          DoneWithBlock(buf);
        }
        // histograms of the gathered rows, added to the level's histograms
        const unsigned per_item = HistRowsPerItem(rows);
        const unsigned grid = (unsigned)std::min<size_t>(rows / per_item + 2 * L + 1, max_hist_items_);
        Mark(kPlan);
        PlanOn(d_blk_tot_, d_blk_seg_, L, 0, per_item, d_hwork_, d_nwork_, level, nullptr, grid);
        Mark(level == 0 ? kHistRoot : kHistDeep);
        for (int q0 = 0; q0 < Q_; q0 += quads_per_group_) {
          const int nq = std::min(quads_per_group_, Q_ - q0);
          HistLaunch(nq, grid, hist_bins, br, q0, hist_g, hist_h);
        }
        if (in_place) DoneWithBlock(buf);
        Reduce(L, hb, false, state, false, b > 0);
      }
      if (level == 0) RootTotals(hb, state, orig);
      if (trick)
        hipLaunchKernelGGL(k_sibling, dim3((nbin_total_ + 255) / 256, L), dim3(256), 0, stream_, d_hg_[hb], d_hh_[hb],
                           d_hc_[hb], d_hg_[hb ^ 1], d_hh_[hb ^ 1], d_hc_[hb ^ 1], d_tot_[state], level, nbin_total_);
      if (inspect_) KeepHist(level, L, hb, state);
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
      int buf = -1;
      const uint32_t *blk = BlockOnDevice(b, &buf);
      LaunchFinal(blk, br, row0, rows, label, next_grad);
      DoneWithBlock(buf);
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

  void KeepHist(int level, int L, int hb, int state) {
    const size_t cells = (size_t)L * nbin_total_;
    std::vector<long long> g(cells), h(cells);
    std::vector<unsigned long long> c(cells);
    HIP_OK(hipStreamSynchronize(stream_));
    HIP_OK(hipMemcpy(g.data(), d_hg_[hb], cells * sizeof(long long), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(h.data(), d_hh_[hb], cells * sizeof(long long), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(c.data(), d_hc_[hb], cells * sizeof(unsigned long long), hipMemcpyDeviceToHost));
    // keep [node][F][slots][3] (padding features of the last quad dropped)
    std::vector<NodeSum> tot;
    if (hi_skip_) {  // ids of 256 were left out: a feature's bin 256 holds what its other bins lack of the node
      tot.resize(L);
      HIP_OK(hipMemcpy(tot.data(), d_tot_[state], (size_t)L * sizeof(NodeSum), hipMemcpyDeviceToHost));
    }
    std::vector<int64_t> &out = kept_hist_[level];
    out.resize((size_t)L * F_ * report_slots_ * 3);
    for (int nd = 0; nd < L; ++nd)
      for (int f = 0; f < F_; ++f)
        for (int b = 0; b < report_slots_; ++b) {
          // (ninth bits: bin 256 of feature f is cell hi_base_ + f of the node)
          const size_t s = (size_t)nd * nbin_total_ + (b < slots_ ? (size_t)f * slots_ + b : (size_t)hi_base_ + f);
          const size_t d = (((size_t)nd * F_ + f) * report_slots_ + b) * 3;
          if (hi_skip_ && b >= slots_) {
            long long sg = 0, sh = 0;
            unsigned long long sc = 0;
            for (int k = 0; k < slots_; ++k) {
              const size_t e = (size_t)nd * nbin_total_ + (size_t)f * slots_ + k;
              sg += g[e];
              sh += pair_ ? h[e] : 0;
              sc += c[e];
            }
            out[d] = tot[nd].g - sg;
            out[d + 1] = pair_ ? tot[nd].h - sh : 0;
            out[d + 2] = (int64_t)(tot[nd].c - sc);
            continue;
          }
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
  unsigned cus_ = 256;        // compute units of the device
  unsigned hist_cus_ = 256;   // work items of an un-fused histogram launch that run at a time
  int rec_groups_ = 1;        // groups of quads a record is read in (rows in place)
  bool single_group_ = true;  // all quads fit one LDS histogram
  bool indexed_ = false;      // wide matrix: rows stay in place, (row id, gradients) are re-ordered
  int rec_slots_ = kSlots;    // bins per feature of the one LDS histogram of that mode
  bool rec_one_launch_ = true;  // every feature fits one LDS histogram at rec_slots_ bins
  int rec_lay_blocks_ = 0;      // blocks that histogram is laid out for (a power of two), 0: as many as the matrix has
  bool wide_ = false;     // 16-bit bins: two features per word, slots_ histogram slots per feature
  bool hi_ = false;       // 8-bit bins plus ninth-bit words per row (ids up to 256)
  bool hi_rows_ = false;  // ... one word: ids of 256 have a 257th row of entries in LDS histograms and slabs
  bool hi_skip_ = false;  // ... several words: ids of 256 are left out of the histograms
  int W_ = 0;             // words of a row: Q_, one more with ninth bits
  int hi_word_ = -1;      // column of the ninth-bit word, -1: none
  int hi_base_ = 0;       // first cell of the bin-256 cells of a node's histogram, 0: none
  int slab_stride_ = 0;   // histogram entries from one work item's slab to the next
  int report_slots_ = kSlots;  // slots per feature as GetLevelHist reports them
  int slots_ = kSlots;
  int wide_group_ = 2;    // features per histogram launch with 16-bit bins
  BinCode code_ = BinCode{2, 8};
  bool root_hist_ready_ = false;  // the slabs hold the root histogram of the tree grown next
  static constexpr int kScanLevels = 32;      // per-level counters of rows accumulated into histograms
  static constexpr size_t kRecordRing = 64;  // trees whose records may wait on the device
  uint32_t *d_records_ = nullptr;
  std::vector<size_t> pending_;              // indices into *owner_ of the trees not fetched yet
  std::vector<RegTree> *owner_ = nullptr;
  bool pair_ = false, f64_ = false, trick_ = true, fused_ = false, inspect_ = false, timing_ = false;
  bool dominant_only_ = false, deep_open_ = false;  // timing of the fused pass only
  unsigned sample_every_ = 1;
  unsigned long long trees_grown_ = 0;
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
  unsigned *d_node_first2_ = nullptr, *d_node_items2_ = nullptr;  // both sets; d_node_first_ / d_node_items_: the one in use
  bool own_scan_ = false;  // the fused passes find the splits of their parents themselves (LevelScan)
  unsigned *d_leaf_ = nullptr, *d_node_first_ = nullptr, *d_node_items_ = nullptr, *d_nwork_ = nullptr,
           *d_wave_left_ = nullptr, *d_item_left_ = nullptr, *d_gmax_ = nullptr, *d_cursor2_ = nullptr;
  RowBuffers buf_[2];
  // streamed matrices: two block buffers filled by the copy stream, a staging
  // buffer with the rows of the built nodes, a resident node id per row
  bool streamed_ = false;
  bool root_totals_ready_ = false;  // d_tot_[0][0] holds the gradient totals of the tree grown next
  bool leaf_valid_ = true;  // d_leaf_ holds the leaves of the last tree
  bool pack_ = false;  // logistic gradients packed into one float per row, no h arrays
  hipStream_t copy_stream_ = nullptr;
  uint32_t *blk_[2] = {nullptr, nullptr};
  std::vector<uint32_t *> resident_;  // per block: its copy in device memory, or null (copied in when needed)
  size_t resident_blocks_ = 0;
  hipEvent_t ev_ready_[2] = {nullptr, nullptr}, ev_free_[2] = {nullptr, nullptr};
  bool buf_used_[2] = {false, false};
  size_t next_copy_ = 0;  // running block-copy counter (selects the buffer)
  RowBuffers stage_;
  unsigned *d_node_of_ = nullptr, *d_blk_cnt_ = nullptr, *d_blk_seg_ = nullptr, *d_cursor_ = nullptr;
  NodeSum *d_blk_tot_ = nullptr;
  NodeSum *d_tot_[2] = {nullptr, nullptr};
  unsigned *d_seg_[2] = {nullptr, nullptr};
  long long *d_hg_[2] = {nullptr, nullptr}, *d_hh_[2] = {nullptr, nullptr};
  unsigned long long *d_hc_[2] = {nullptr, nullptr};  // 64-bit: a cell of a streamed matrix may hold 2^32 rows and more
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
  if (data->exact_sort) return CreateExactSortBuilder(cfg, data);
  if (!data->device) throw std::runtime_error("data matrix is not quantised");
  return new HipTreeBuilder(cfg, data);
}

}  // namespace arb
