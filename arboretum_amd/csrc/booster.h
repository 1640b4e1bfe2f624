// Host-side objects behind the C-ABI: the data matrix, the regression tree,
// the booster ("Garden") and the interface of the GPU tree builder.
// Counterparts in the reference: io::DataMatrix (src/io/io.h:15-83), RegTree
// (src/core/garden.h:32-127), Garden (src/core/garden.h:141-160).
#ifndef ARBORETUM_AMD_BOOSTER_H_
#define ARBORETUM_AMD_BOOSTER_H_

#include <cstdint>
#include <functional>
#include <memory>
#include <string>
#include <vector>

#include "config.h"

namespace arb {

// Runs fn(begin, end) over [0, n) on a few host threads.
void ParallelFor(size_t n, const std::function<void(size_t, size_t)> &fn);
// fn(i) for every i in [0, n), a few long tasks (columns) handed out one at a time to up to 16 threads.
void ParallelTasks(size_t n, const std::function<void(size_t)> &fn);

struct DeviceMatrix;  // quantised bins resident in HBM (device_builder.hip)
struct ExactSortData;  // ranks and sorted row lists of every feature (exact_builder.hip)

class DataMatrix {
 public:
  DataMatrix(size_t rows, size_t columns, size_t columns_category);
  ~DataMatrix();

  const size_t rows;
  const size_t columns_dense;
  const size_t columns_category;
  // Distinguishes this matrix from any other, also from one created later at
  // the same address (device-side caches are keyed by it).
  const uint64_t uid;

  // Column-major host store, one contiguous vector per feature (io.h:22).
  std::vector<std::vector<float>> data;
  // Pre-quantised input: row-major [rows][columns_dense] bin ids instead of
  // floats (extension; `data` is then empty).
  std::vector<uint8_t> prebinned;
  bool is_prebinned = false;
  std::vector<std::vector<unsigned>> data_categories;

  std::vector<float> y;
  std::vector<float> y_hat;
  std::vector<unsigned char> labels;
  std::vector<float> weights;

  // Quantiser output (io.h:24, 32): thresholds[f] has hist_size entries,
  // reduced_size[f] real bins.
  bool quantised = false;
  bool quantised_exact = false;  // bin ids are ranks among the distinct values (exact method)
  int hist_size = 0;             // exact method: the largest number of distinct values of a feature
  std::vector<std::vector<float>> thresholds;
  std::vector<int> reduced_size;
  int max_bin = 255;  // largest bin id in the quantised matrix (the missing-value bin included)
  DeviceMatrix *device = nullptr;
  // Exact method over sorted row lists (features with more distinct values than a histogram
  // holds): set instead of `device`.
  ExactSortData *exact_sort = nullptr;
  // Streamed matrices (bins in pinned host blocks instead of HBM): block b
  // holds rows [b * stream_block_rows, ...) as quads [Q][stream_block_rows].
  std::vector<uint32_t *> stream_blocks;
  size_t stream_block_rows = 0;
  // The blocks belong to the caller (ACreateFromQuantizedBlocks): never copied, never freed.
  bool external_blocks = false;

  // Feature value as seen by host prediction.
  inline float value(size_t f, size_t i) const {
    if (!is_prebinned) return data[f][i];
    if (!prebinned.empty()) return (float)prebinned[i * columns_dense + f];
    const uint32_t q = stream_blocks[i / stream_block_rows][(f >> 2) * stream_block_rows + i % stream_block_rows];
    return (float)((q >> (8 * (f & 3))) & 255u);
  }
};

// Heap-ordered tree (src/core/reg_tree.h:16-45, garden.h:32-67).
struct RegTree {
  unsigned depth = 0;  // internal depth: depth-1 split levels, 2^(depth-1) leaves
  unsigned label = 0;
  std::vector<unsigned> fid;      // 2^(depth-1)-1 internal nodes
  std::vector<float> threshold;
  std::vector<int> quantized;     // split bin, -1 when the node was not split
  std::vector<float> gain;
  std::vector<float> weights;     // 2^(depth-1)

  RegTree() {}
  RegTree(unsigned depth, unsigned label);
  // RegTree::Predict, garden.h:70-90: x < threshold -> left; adds the leaf
  // weight to out[i + label * rows].
  void Predict(const DataMatrix &data, float *out) const;
  // The same for rows [begin, end) only, on the calling thread.
  void PredictRows(const DataMatrix &data, size_t begin, size_t end, float *out) const;
};

// Accumulated GPU milliseconds per kernel class.  hist_root: histogram kernel
// of the root level; hist_deep: histogram work of the deeper levels (the fused
// partition + histogram kernel, or the histogram kernel after a stand-alone
// partition); fused_last: the fused kernel of the last level, which moves no
// rows; partition: left counts, offset scan and the stand-alone partition.
struct BuilderTimings {
  double grad = 0, hist_root = 0, hist_deep = 0, reduce = 0, split = 0, partition = 0, leaf = 0, plan = 0,
         fused_last = 0;
  unsigned long long hist_root_launches = 0, hist_deep_launches = 0, fused_last_launches = 0;
  unsigned long long hist_root_rows = 0;
};

// GPU tree builder bound to one (configuration, data matrix) pair.
class TreeBuilder {
 public:
  virtual ~TreeBuilder() {}
  // One boosting round: gradients, labels_count trees, prediction update.
  // The trees are appended to `trees` at once, but their contents may stay on
  // the device until FlushTrees() is called.
  virtual void GrowRound(std::vector<RegTree> *trees) = 0;
  virtual void FlushTrees() = 0;
  // Inspection (tests, benchmark).
  virtual void SetInspect(bool on) = 0;
  virtual void GetLeaves(uint32_t *out) = 0;               // leaf of every row, last tree
  virtual void GetYHat(float *out) = 0;                    // labels_count * rows
  virtual void GetGrad(float *g, float *h) = 0;            // labels_count * rows each
  virtual int GetLevelHist(int level, int64_t *out) = 0;   // [node][F][256][3], needs inspect
  virtual void GetShifts(int *shift_g, int *shift_h) = 0;
  // 0: off; 1: every phase; 2: only the dominant kernel (the fused pass), which
  // costs a third of the event records; 3: that on every fourth tree
  virtual void EnableTiming(int level) = 0;
  virtual BuilderTimings GetTimings() = 0;
  virtual unsigned long long RowsScanned() = 0;            // rows accumulated into histograms
  virtual void RowsScannedByLevel(unsigned long long *out) = 0;  // the same per tree level, 32 entries
  // streamed matrix: row blocks kept in device memory and row blocks in all (0, 0: not streamed)
  virtual void StreamResidency(unsigned long long *resident, unsigned long long *blocks) = 0;
  virtual void Synchronize() = 0;
};

// quantiser.hip: thresholds of one column by a device radix sort
struct SortWorkspace;
SortWorkspace *CreateSortWorkspace(size_t n, int hist_size);
void FreeSortWorkspace(SortWorkspace *ws);
void DeviceThresholds(SortWorkspace *ws, const float *d_col, std::vector<float> *thr, int *size, bool *has_nan);

// device_builder.hip
// streamed = false: bins resident in HBM; true: bins in pinned host blocks of
// block_rows rows, copied to the GPU block by block at every tree level.
// exact: no quantisation, every distinct value of a feature is a bin (the exact method).  Up to
// 4096 distinct values per feature the ranks are bin ids of the histogram kernels; beyond that,
// or always with exact_sort > 0, the matrix is kept as sorted row lists per feature
// (exact_builder.hip); exact_sort == 0 makes more than 4096 distinct values an error.
void QuantiseOnDevice(DataMatrix *data, int hist_size, bool verbose, bool streamed = false,
                      size_t block_rows = 0, bool exact = false, int exact_sort = -1);
void PrepareExactSort(DataMatrix *data);
void FreeExactSortData(ExactSortData *d);
TreeBuilder *CreateExactSortBuilder(const Configuration &cfg, DataMatrix *data);
void FreeDeviceMatrix(DeviceMatrix *m);
void GetDeviceBins(const DataMatrix &data, uint8_t *out);  // row-major [rows][F], 8-bit bins
void GetDeviceBins16(const DataMatrix &data, uint16_t *out);  // row-major [rows][F], 16-bit bins
void GetBinLayout(const DataMatrix &data, int *bits, int *slots);  // bits per bin id, histogram slots per feature
TreeBuilder *CreateTreeBuilder(const Configuration &cfg, DataMatrix *data);
int DeviceCount();
void CopyProbe(size_t bytes);

// predictor.hip: tree walks of a matrix (floats or bin ids) on the GPU.  Returns [labels][rows]
// sums of leaf weights of trees[0, use) on top of `init`, bit-identical to the
// host walk (RegTree::Predict in tree order), in pinned host memory that the
// predictor owns and overwrites on its next call.
struct DevicePredictor;
DevicePredictor *CreateDevicePredictor();
void FreeDevicePredictor(DevicePredictor *p);
const float *PredictOnDevice(DevicePredictor *p, const DataMatrix &data, const std::vector<RegTree> &trees,
                             size_t use, size_t labels, float init);

class Garden {
 public:
  explicit Garden(const Configuration &cfg);
  ~Garden();
  const Configuration cfg;

  void GrowTree(DataMatrix *data, const float *grad);        // garden.cu:585-625
  // out: rows * labels_count floats
  void Predict(const DataMatrix *data, float *out, int n_rounds) const;  // :643-657
  void UpdateByLastTree(DataMatrix *data);                   // :627-635
  void GetY(const DataMatrix *data, std::vector<float> *out) const;  // :637-641
  const char *GetModel();                                    // :659-665
  void Restore(const char *json_model);                      // :667-677

  float IntoInternal(float v) const;                         // objective.h:20,55-57
  void FromInternal(const std::vector<float> &in, std::vector<float> *out) const;
  void FromInternal(const float *in, size_t count, float *out) const;  // count = rows * labels_count

  // Inspection / timing switches; they also apply to a builder created later.
  void SetInspect(bool on) { inspect_ = on; if (builder_) builder_->SetInspect(on); }
  void SetTiming(int level) { timing_ = level; if (builder_) builder_->EnableTiming(level); }
  // Predict walks the trees on the GPU when one is present (default), or on
  // the host as the reference does.
  void SetPredictOnDevice(bool on) { predict_on_device_ = on; }

  TreeBuilder *builder() { return builder_.get(); }
  size_t num_trees() const { return trees_.size(); }
  const RegTree &tree(size_t i) const {
    SyncTrees();
    return trees_[i];
  }

 private:
  std::unique_ptr<TreeBuilder> builder_;
  DataMatrix *bound_ = nullptr;
  // Records of freshly grown trees are fetched from the GPU on first use.
  void SyncTrees() const { if (builder_) builder_->FlushTrees(); }
  mutable std::vector<RegTree> trees_;
  std::string model_;
  bool inspect_ = false;
  int timing_ = 0;
  bool predict_on_device_ = true;
  mutable std::unique_ptr<DevicePredictor, void (*)(DevicePredictor *)> predictor_{nullptr, FreeDevicePredictor};
};

}  // namespace arb
#endif  // ARBORETUM_AMD_BOOSTER_H_
