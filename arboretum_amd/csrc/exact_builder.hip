// The exact method for features with more distinct values than the rank histograms hold:
// every feature keeps its rows sorted by value, per node (kernels_exact.h).
//
// Replaces, for that case, ContinuousTreeGrower (src/core/continuous_tree_grower.cu: one
// segmented sort per feature and level, a scan of the sorted gradients, gain_kernel at the
// places where the value changes) and DataMatrix::InitExact (src/io/io.cu:437-482: values to
// ranks among the sorted distinct values).  Here each column is sorted once; a level partitions
// the sorted lists stably instead of sorting them again.  Sums are fixed-point integers as in
// the histogram method, so the trees do not depend on the order of the additions, and the
// candidates, gains and tie rules are those of a rank histogram with one slot per distinct
// value: where both paths can run they grow the same trees bit for bit.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <limits>
#include <memory>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

#include "booster.h"
#include "device_common.h"
#include "gain.h"
#include "kernels_exact.h"
#include "kernels_final.h"
#include "kernels_indexed.h"
#include "kernels_objective.h"
#include "kernels_plan.h"
#include "kernels_split.h"

namespace arb {

struct ExactSortData {
  size_t rows = 0, stride = 0;
  int F = 0;
  uint32_t *ranks = nullptr;       // [F][stride] by row: rank of the row's value among the feature's distinct values
  uint32_t *lists = nullptr;       // [F][stride]: the rows in ascending order of the feature's value
  uint32_t *list_ranks = nullptr;  // [F][stride]: the ranks in that order
};

void FreeExactSortData(ExactSortData *d) {
  if (!d) return;
  if (d->ranks) (void)hipFree(d->ranks);
  if (d->lists) (void)hipFree(d->lists);
  if (d->list_ranks) (void)hipFree(d->list_ranks);
  delete d;
}

// Sorts every column once on the host: ranks, sorted row lists, and the thresholds of the ranks
// (the split "ranks <= q left" separates at the value of rank q + 1, the smallest value that goes
// right, src/core/garden.cu:463-467).
void PrepareExactSort(DataMatrix *data) {
  const size_t n = data->rows;
  const int F = (int)data->columns_dense;
  const size_t stride = (n + 63) / 64 * 64;
  std::vector<uint32_t> ranks((size_t)F * stride, 0u), lists((size_t)F * stride, 0u), list_ranks((size_t)F * stride, 0u);
  std::vector<std::vector<float>> mapping(F);
  std::atomic<bool> has_nan{false};
  // one column per thread at a time (the columns are few and long)
  ParallelTasks((size_t)F, [&](size_t f) {
    if (has_nan) return;
    // (value, row) packed into one integer that sorts like the pair: the float's bits with the
    // sign folded so that unsigned order is numeric order, above the row id
    std::vector<uint64_t> keyed(n);
    const float *col = data->data[f].data();
    for (size_t i = 0; i < n; ++i) {
      if (col[i] != col[i]) has_nan = true;
      uint32_t u;
      std::memcpy(&u, &col[i], sizeof(u));
      if (u == 0x80000000u) u = 0;  // -0 and +0 are one value
      u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
      keyed[i] = ((uint64_t)u << 32) | (uint64_t)i;
    }
    if (has_nan) return;
    std::sort(keyed.begin(), keyed.end());
    uint32_t *rk = ranks.data() + f * stride, *ls = lists.data() + f * stride, *lr = list_ranks.data() + f * stride;
    std::vector<float> &m = mapping[f];
    for (size_t k = 0; k < n; ++k) {
      const uint32_t row = (uint32_t)keyed[k];
      const float v = col[row];
      if (k == 0 || v != m.back()) m.push_back(v);
      ls[k] = row;
      lr[k] = rk[row] = (uint32_t)(m.size() - 1);
    }
  });
  if (has_nan) throw std::runtime_error("the exact method does not take missing values (NaN); use method 1 (hist)");
  size_t most = 1;
  data->thresholds.assign(F, {});
  data->reduced_size.assign(F, 0);
  for (int f = 0; f < F; ++f) {
    most = std::max(most, mapping[f].size());
    data->reduced_size[f] = (int)mapping[f].size();
    // one entry per rank: the value of the next rank; nothing lies above the last one
    data->thresholds[f].assign(mapping[f].size(), std::numeric_limits<float>::infinity());
    for (size_t k = 0; k + 1 < mapping[f].size(); ++k) data->thresholds[f][k] = mapping[f][k + 1];
  }
  std::unique_ptr<ExactSortData, void (*)(ExactSortData *)> d(new ExactSortData(), FreeExactSortData);
  d->rows = n;
  d->stride = stride;
  d->F = F;
  d->ranks = DevAlloc<uint32_t>(ranks.size());
  d->lists = DevAlloc<uint32_t>(lists.size());
  d->list_ranks = DevAlloc<uint32_t>(list_ranks.size());
  HIP_OK(hipMemcpy(d->ranks, ranks.data(), ranks.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d->lists, lists.data(), lists.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d->list_ranks, list_ranks.data(), list_ranks.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
  data->exact_sort = d.release();
  data->hist_size = (int)most;
  data->max_bin = (int)std::min<size_t>(most - 1, (size_t)std::numeric_limits<int>::max());
  data->quantised = true;
  data->quantised_exact = true;
}

namespace {

class ExactSortBuilder : public TreeBuilder {
 public:
  ExactSortBuilder(const Configuration &cfg, DataMatrix *data) : cfg_(cfg), data_(data) {
    try {
      Construct(cfg, data);
    } catch (...) {  // e.g. out of device memory: give back what was allocated so far
      Release();
      throw;
    }
  }
  ~ExactSortBuilder() override { Release(); }

 private:
  void Construct(const Configuration &cfg, DataMatrix *data) {
    sd_ = data->exact_sort;
    n_ = sd_->rows;
    F_ = sd_->F;
    stride_ = sd_->stride;
    K_ = (int)cfg.tree.labels_count;
    D_ = (int)cfg.tree.depth;
    pair_ = cfg.objective != kLinearRegression;
    f64_ = cfg.internal.double_precision;
    if (cfg.objective >= kSoftMaxOneVsAll && K_ < 2) throw std::runtime_error("soft-max needs labels_count >= 2");
    if (cfg.objective < kSoftMaxOneVsAll && K_ != 1) throw std::runtime_error("labels_count must be 1 for this objective");
    if (D_ < 2) throw std::runtime_error("max_depth must be at least 1");
    if (F_ > 65535) throw std::runtime_error("the exact method over sorted lists takes at most 65535 features");
    const int last_nodes = 1 << (D_ - 2);
    if (last_nodes > kMaxPlanNodes) throw std::runtime_error("unsupported depth: at most 4096 nodes per level");
    HIP_OK(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking));
    max_items_ = (unsigned)(n_ / kExItem) + 2u * (unsigned)last_nodes + 2u;

    d_y_ = DevAlloc<float>(n_);
    d_labels_ = DevAlloc<uint8_t>(n_);
    d_yhat_ = DevAlloc<float>(n_ * K_);
    // Logistic gradients of 0/1 labels travel as one float per row (PackGrad): no h array, and
    // 12 instead of 16 bytes per place of the lists.
    pack_ = cfg.objective == kLogisticRegression && data->y.size() == n_ &&
            std::all_of(data->y.begin(), data->y.end(), [](float v) { return v == 0.0f || v == 1.0f; });
    harr_ = pair_ && !pack_;
    d_g_ = DevAlloc<float>(n_ * K_);
    d_h_ = harr_ ? DevAlloc<float>(n_ * K_) : nullptr;
    d_leaf_ = DevAlloc<unsigned>(n_);
    HIP_OK(hipMemsetAsync(d_leaf_, 0, n_ * sizeof(unsigned), stream_));  // (asked for before the first tree: the root)
    d_node_of_ = DevAlloc<unsigned>(n_);
    if (!data->y.empty()) HIP_OK(hipMemcpy(d_y_, data->y.data(), n_ * sizeof(float), hipMemcpyHostToDevice));
    if (!data->labels.empty()) HIP_OK(hipMemcpy(d_labels_, data->labels.data(), n_, hipMemcpyHostToDevice));
    float init = cfg.tree.initial_y;
    if (cfg.objective == kLogisticRegression) init = std::log(init / (1 - init));  // objective.h:55-57
    hipLaunchKernelGGL(k_fill_f32, dim3(GridFor(n_ * K_, 256)), dim3(256), 0, stream_, d_yhat_, init, n_ * K_);
    data->y_hat.assign(n_ * K_, init);  // garden.cu:104

    d_went_right_ = DevAlloc<unsigned long long>(stride_ / 64);
    d_gh_ = harr_ ? DevAlloc<float2>(n_) : nullptr;
    // two sets of lists (ids, ranks, gradients in list order), written and read in turn by the
    // levels; the gradients of the second set also serve the root's lists
    const size_t words = (size_t)F_ * stride_;
    for (int b = 0; b < 2; ++b) {
      if (D_ > 2) {
        d_ids_[b] = DevAlloc<uint32_t>(words);
        d_ranks_[b] = DevAlloc<uint32_t>(words);
      }
      if (D_ > 2 || b == 1) {
        d_lg_[b] = DevAlloc<float>(words);
        d_lh_[b] = harr_ ? DevAlloc<float>(words) : nullptr;
      }
    }
    const int max_nodes = 1 << (D_ - 1);
    for (int s = 0; s < 2; ++s) {
      d_tot_[s] = DevAlloc<NodeSum>(max_nodes);
      d_seg_[s] = DevAlloc<unsigned>(max_nodes);
    }
    d_split_ = DevAlloc<SplitRec>(last_nodes);
    d_cand_ = DevAlloc<Cand>((size_t)last_nodes * F_);
    d_work_ = DevAlloc<WorkItem>(max_items_);
    d_n_work_ = DevAlloc<unsigned>(1);
    d_node_first_ = DevAlloc<unsigned>(last_nodes);
    d_node_items_ = DevAlloc<unsigned>(last_nodes);
    d_part_ = DevAlloc<ExSum>((size_t)F_ * max_items_);
    d_off_ = DevAlloc<ExSum>((size_t)F_ * max_items_);
    d_best_ = DevAlloc<Cand>((size_t)F_ * max_items_);
    d_lefts_ = DevAlloc<unsigned>((size_t)F_ * max_items_);
    d_left_off_ = DevAlloc<unsigned>((size_t)F_ * max_items_);
    d_left_bits_ = DevAlloc<uint8_t>((size_t)F_ * max_items_ * kExThreads);
    d_shifts_ = DevAlloc<int>(2);
    d_records_ = DevAlloc<uint32_t>(kRecordRing * RecordWords());
    d_gmax_ = DevAlloc<unsigned>(1);
    d_overflow_ = DevAlloc<unsigned>(1);
    HIP_OK(hipMemsetAsync(d_overflow_, 0, sizeof(unsigned), stream_));
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
      float ymin = 0.0f, ymax = 1.0f;  // labels outside [0, 1] widen the gradient range
      for (float v : data->y) {
        ymin = std::min(ymin, v);
        ymax = std::max(ymax, v);
      }
      shifts[0] = LogisticGradShift(ymin, ymax);
    }
    if (cfg.objective >= kSoftMaxOneVsAll) shifts[1] = 31;  // 0 <= h <= 1/2
    HIP_OK(hipMemcpyAsync(d_shifts_, shifts, sizeof(shifts), hipMemcpyHostToDevice, stream_));
    HIP_OK(hipStreamSynchronize(stream_));
  }

  void Release() noexcept {
    if (stream_) (void)hipStreamSynchronize(stream_);
    void *all[] = {d_y_, d_labels_, d_yhat_, d_g_, d_h_, d_leaf_, d_node_of_, d_went_right_, d_gh_, d_ids_[0], d_ids_[1], d_ranks_[0],
                   d_ranks_[1], d_lg_[0], d_lg_[1], d_lh_[0], d_lh_[1], d_tot_[0],
                   d_tot_[1], d_seg_[0], d_seg_[1], d_split_, d_cand_, d_work_, d_n_work_, d_node_first_,
                   d_node_items_, d_part_, d_off_, d_best_, d_lefts_, d_left_off_, d_left_bits_, d_shifts_, d_records_, d_gmax_,
                   d_overflow_, d_tfid_, d_tbin_, d_tgain_, d_weights_, d_active_};
    for (void *p : all)
      if (p) (void)hipFree(p);
    if (stream_) (void)hipStreamDestroy(stream_);
  }

 public:
  void GrowRound(std::vector<RegTree> *trees) override {
    if (cfg_.objective == kLinearRegression) {
      HIP_OK(hipMemsetAsync(d_gmax_, 0, sizeof(unsigned), stream_));
      hipLaunchKernelGGL(k_grad_squared, dim3(GridFor(n_, 256)), dim3(256), 0, stream_, d_y_, d_yhat_, d_g_, n_, d_gmax_);
      hipLaunchKernelGGL(k_set_shift, dim3(1), dim3(64), 0, stream_, d_gmax_, d_shifts_);
    } else if (cfg_.objective == kLogisticRegression) {
      hipLaunchKernelGGL(k_grad_logistic, dim3(GridFor(n_, 256)), dim3(256), 0, stream_, d_y_, d_yhat_, d_g_, d_h_, n_);  // (no d_h_: packed)
    } else {
      hipLaunchKernelGGL(k_grad_softmax, dim3(GridFor(n_, 256)), dim3(256), 0, stream_, d_labels_, d_yhat_, d_g_, d_h_, n_, K_);
    }
    owner_ = trees;
    for (int k = 0; k < K_; ++k) {
      trees->emplace_back((unsigned)D_, (unsigned)k);
      GrowOne(k);
      pending_.push_back(trees->size() - 1);
      if (inspect_ || pending_.size() == kRecordRing) FlushTrees();
    }
  }

  // Records of the trees grown since the last call -> their RegTree entries (garden.cu:447-503).
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
        if (bin >= 0 && (size_t)bin < data_->thresholds[fid].size()) thr = data_->thresholds[fid][bin];
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
  int GetLevelHist(int, int64_t *) override { return -1; }  // no histograms on this path
  void GetShifts(int *sg, int *sh) override {
    int s[2];
    HIP_OK(hipStreamSynchronize(stream_));
    HIP_OK(hipMemcpy(s, d_shifts_, sizeof(s), hipMemcpyDeviceToHost));
    *sg = s[0];
    *sh = s[1];
  }
  void EnableTiming(int) override {}
  BuilderTimings GetTimings() override { return BuilderTimings(); }
  unsigned long long RowsScanned() override { return 0; }
  void RowsScannedByLevel(unsigned long long *out) override {
    for (int k = 0; k < 32; ++k) out[k] = 0;  // one entry per tree level
  }
  void StreamResidency(unsigned long long *resident, unsigned long long *blocks) override {
    *resident = 0;
    *blocks = 0;
  }
  void Synchronize() override {
    HIP_OK(hipStreamSynchronize(stream_));
    FlushTrees();
  }

 private:
  static constexpr size_t kRecordRing = 64;  // trees whose records may wait on the device
  size_t RecordWords() const { return (size_t)3 * ((1 << (D_ - 1)) - 1) + (size_t)(1 << (D_ - 1)) + 1; }

  // The features a tree may split on at every level (garden.cu:142-146, 162-165, 252-253).
  void SampleColumns() {
    const size_t columns = data_->columns_dense + data_->columns_category;
    const int take_tree = (int)(cfg_.tree.colsample_bytree * columns);
    const unsigned take_level = (unsigned)(cfg_.tree.colsample_bylevel * cfg_.tree.colsample_bytree * columns);
    sampling_ = take_level < columns;
    if (!sampling_) return;
    std::vector<unsigned> ids(columns);
    for (size_t i = 0; i < columns; ++i) ids[i] = (unsigned)i;
    std::shuffle(ids.begin(), ids.end(), rnd_);
    std::vector<unsigned char> active((size_t)(D_ - 1) * F_, 0);
    for (int level = 0; level + 1 < D_; ++level) {
      std::shuffle(ids.begin(), ids.begin() + take_tree, rnd_);
      for (unsigned j = 0; j < take_level; ++j)
        if (ids[j] < (unsigned)F_) active[(size_t)level * F_ + ids[j]] = 1;
    }
    HIP_OK(hipStreamSynchronize(stream_));  // the previous tree's kernels may still read the mask
    HIP_OK(hipMemcpy(d_active_, active.data(), active.size(), hipMemcpyHostToDevice));
  }

  void GrowOne(int label) {
    const GainParams gp = cfg_.gain_params();
    const float *g = d_g_ + (size_t)label * n_;
    const float *h = d_h_ ? d_h_ + (size_t)label * n_ : nullptr;
    SampleColumns();
    hipLaunchKernelGGL(k_init_root, dim3(1), dim3(64), 0, stream_, d_tot_[0], d_seg_[0], (unsigned long long)n_,
                       (unsigned *)nullptr);
    if (pack_)
      hipLaunchKernelGGL(k_ex_sum_packed, dim3(GridFor(n_, 256, 1024)), dim3(256), 0, stream_, g, n_, d_shifts_, d_tot_[0]);
    else
      hipLaunchKernelGGL(k_sum_grad, dim3(GridFor(n_, 256, 1024)), dim3(256), 0, stream_, g, h, n_, d_shifts_, d_tot_[0]);
    HIP_OK(hipMemsetAsync(d_node_of_, 0, n_ * sizeof(unsigned), stream_));
    int state = 0;
    // the root's lists: every row, sorted once; this tree's gradients in that order
    const dim3 whole((unsigned)((n_ + kExItem - 1) / kExItem), (unsigned)F_);
    if (harr_) {
      hipLaunchKernelGGL(k_ex_pair, dim3(GridFor(n_, 256)), dim3(256), 0, stream_, g, h, d_gh_, n_);
      hipLaunchKernelGGL((k_ex_gather<true>), whole, dim3(kExThreads), 0, stream_, sd_->lists, stride_, g, d_gh_,
                         d_lg_[1], d_lh_[1], n_);
    } else {
      hipLaunchKernelGGL((k_ex_gather<false>), whole, dim3(kExThreads), 0, stream_, sd_->lists, stride_, g,
                         (const float2 *)nullptr, d_lg_[1], d_lh_[1], n_);
    }
    ExLists lists{sd_->lists, sd_->list_ranks, d_lg_[1], d_lh_[1]};
    for (int level = 0; level + 1 < D_; ++level) {
      const int L = 1 << level;
      const bool last = level + 2 >= D_;
      const unsigned grid_items = (unsigned)(n_ / kExItem) + 2u * (unsigned)L + 2u;
      const dim3 per_item(grid_items, (unsigned)F_), per_node((unsigned)L, (unsigned)F_);
      hipLaunchKernelGGL(k_plan, dim3(1), dim3(1024), 0, stream_, d_tot_[state], d_seg_[state], L, 0, kExItem, d_work_,
                         d_n_work_, d_node_first_, d_node_items_, (unsigned long long *)nullptr,
                         (const SplitRec *)nullptr, grid_items, d_overflow_, 0u, (unsigned *)nullptr);
#define ARB_EX(P, D, K)                                                                                               \
  do {                                                                                                                \
    hipLaunchKernelGGL((k_ex_partial<P, K>), per_item, dim3(kExThreads), 0, stream_, lists, stride_, d_shifts_,      \
                       d_work_, d_n_work_, d_part_, max_items_);                                                      \
    hipLaunchKernelGGL((k_ex_offsets<ExSum>), per_node, dim3(64), 0, stream_, d_part_, d_off_, d_node_first_,        \
                       d_node_items_, max_items_);                                                                    \
    hipLaunchKernelGGL((k_ex_scan<P, D, K>), per_item, dim3(kExThreads), 0, stream_, lists, stride_, d_shifts_,      \
                       d_work_, d_n_work_, d_off_, d_tot_[state], d_seg_[state], gp, d_best_, max_items_);            \
  } while (0)
      if (pack_ && f64_) ARB_EX(true, true, true);
      else if (pack_) ARB_EX(true, false, true);
      else if (pair_ && f64_) ARB_EX(true, true, false);
      else if (pair_) ARB_EX(true, false, false);
      else if (f64_) ARB_EX(false, true, false);
      else ARB_EX(false, false, false);
#undef ARB_EX
      hipLaunchKernelGGL(k_ex_merge, per_node, dim3(64), 0, stream_, d_best_, d_node_first_, d_node_items_, max_items_,
                         F_, d_cand_);
      hipLaunchKernelGGL(k_split_select, dim3((L + 15) / 16), dim3(1024), 0, stream_, d_cand_, F_, L, d_tot_[state],
                         d_seg_[state], d_tot_[state ^ 1], d_seg_[state ^ 1], d_split_, d_tfid_, d_tbin_, d_tgain_,
                         L - 1, sampling_ ? d_active_ + (size_t)level * F_ : (const unsigned char *)nullptr);
      hipLaunchKernelGGL(k_ex_decide, dim3(GridFor(n_, 256)), dim3(256), 0, stream_, sd_->ranks, stride_, d_split_,
                         d_node_of_, d_went_right_, n_);
      if (last) {
        const int blocks = (L + 127) / 128;
#define ARB_LEAF(P, D)                                                                                          \
  hipLaunchKernelGGL((k_leaf_weights<P, D>), dim3(blocks), dim3(128), 0, stream_, d_split_, d_tot_[state], L, \
                     d_shifts_, gp, cfg_.tree.eta, d_weights_)
        if (pair_ && f64_) ARB_LEAF(true, true);
        else if (pair_) ARB_LEAF(true, false);
        else if (f64_) ARB_LEAF(false, true);
        else ARB_LEAF(false, false);
#undef ARB_LEAF
        hipLaunchKernelGGL(k_ex_final, dim3(GridFor(n_, 256)), dim3(256), 0, stream_, d_node_of_, d_weights_,
                           d_yhat_ + (size_t)label * n_, d_leaf_, n_);
      } else {
        const int b = level & 1;
        hipLaunchKernelGGL(k_ex_count, per_item, dim3(kExThreads), 0, stream_, lists.ids, stride_, d_went_right_,
                           d_work_, d_n_work_, d_lefts_, d_left_bits_, max_items_);
        hipLaunchKernelGGL((k_ex_offsets<unsigned>), per_node, dim3(64), 0, stream_, d_lefts_, d_left_off_,
                           d_node_first_, d_node_items_, max_items_);
        if (harr_)
          hipLaunchKernelGGL((k_ex_scatter<true>), per_item, dim3(kExThreads), 0, stream_, lists, d_ids_[b], d_ranks_[b],
                             d_lg_[b], d_lh_[b], stride_, d_left_bits_, d_work_, d_n_work_, d_left_off_,
                             d_seg_[state], d_seg_[state ^ 1], max_items_);
        else
          hipLaunchKernelGGL((k_ex_scatter<false>), per_item, dim3(kExThreads), 0, stream_, lists, d_ids_[b], d_ranks_[b],
                             d_lg_[b], d_lh_[b], stride_, d_left_bits_, d_work_, d_n_work_, d_left_off_,
                             d_seg_[state], d_seg_[state ^ 1], max_items_);
        lists = ExLists{d_ids_[b], d_ranks_[b], d_lg_[b], d_lh_[b]};
        state ^= 1;
      }
      HIP_OK(hipGetLastError());
    }
    const int internal = (1 << (D_ - 1)) - 1, leaves = 1 << (D_ - 1);
    hipLaunchKernelGGL(k_pack_record, dim3((leaves + 255) / 256), dim3(256), 0, stream_, d_tfid_, d_tbin_, d_tgain_,
                       d_weights_, d_overflow_, internal, leaves, d_records_ + pending_.size() * RecordWords());
    HIP_OK(hipGetLastError());
  }

  const Configuration cfg_;
  DataMatrix *data_;
  const ExactSortData *sd_ = nullptr;
  size_t n_ = 0, stride_ = 0;
  int F_ = 0, K_ = 1, D_ = 2;
  bool pair_ = false, f64_ = false, inspect_ = false, sampling_ = false;
  bool pack_ = false;  // logistic gradients packed into one float per row
  bool harr_ = false;  // the gradients are two arrays (g, h)
  unsigned max_items_ = 0;
  hipStream_t stream_ = nullptr;
  std::default_random_engine rnd_;
  std::vector<RegTree> *owner_ = nullptr;
  std::vector<size_t> pending_;

  float *d_y_ = nullptr, *d_yhat_ = nullptr, *d_g_ = nullptr, *d_h_ = nullptr, *d_tgain_ = nullptr, *d_weights_ = nullptr;
  uint8_t *d_labels_ = nullptr;
  unsigned *d_leaf_ = nullptr, *d_node_of_ = nullptr, *d_seg_[2] = {nullptr, nullptr}, *d_n_work_ = nullptr,
           *d_node_first_ = nullptr, *d_node_items_ = nullptr, *d_lefts_ = nullptr, *d_left_off_ = nullptr,
           *d_gmax_ = nullptr, *d_overflow_ = nullptr;
  uint32_t *d_ids_[2] = {nullptr, nullptr}, *d_ranks_[2] = {nullptr, nullptr}, *d_records_ = nullptr;
  float *d_lg_[2] = {nullptr, nullptr}, *d_lh_[2] = {nullptr, nullptr};
  unsigned long long *d_went_right_ = nullptr;
  uint8_t *d_left_bits_ = nullptr;
  float2 *d_gh_ = nullptr;  // (g, h) of the tree's label side by side: one gather per row
  NodeSum *d_tot_[2] = {nullptr, nullptr};
  SplitRec *d_split_ = nullptr;
  Cand *d_cand_ = nullptr, *d_best_ = nullptr;
  WorkItem *d_work_ = nullptr;
  ExSum *d_part_ = nullptr, *d_off_ = nullptr;
  int *d_shifts_ = nullptr, *d_tfid_ = nullptr, *d_tbin_ = nullptr;
  unsigned char *d_active_ = nullptr;
};

}  // namespace

TreeBuilder *CreateExactSortBuilder(const Configuration &cfg, DataMatrix *data) {
  if (!data->exact_sort) throw std::runtime_error("data matrix holds no sorted lists");
  return new ExactSortBuilder(cfg, data);
}

}  // namespace arb
