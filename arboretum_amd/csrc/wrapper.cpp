// extern "C" boundary: marshalling only.  Mirrors
// python-wrapper/arboretum_wrapper.cu:16-205 (same names, argument meaning and
// error convention) plus the extensions declared in arboretum_ext.h.
#include <cstring>
#include <limits>
#include <new>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include "../../include/arboretum_ext.h"
#include "booster.h"
#include "hist_sum.h"

using namespace arb;

namespace {

thread_local std::string g_error;

const char *Fail(const char *what) {
  g_error = what ? what : "unknown error";
  return g_error.c_str();
}

template <typename Fn>
const char *Guard(Fn &&fn) {
  try {
    fn();
    return nullptr;
  } catch (const std::exception &e) {
    return Fail(e.what());
  } catch (const char *msg) {
    return Fail(msg);
  } catch (...) {
    return Fail("unknown error");
  }
}

struct GardenHandle {
  explicit GardenHandle(const Configuration &cfg) : garden(cfg) {}
  Garden garden;
};

DataMatrix *AsData(VoidPointer p) {
  if (!p) throw std::runtime_error("null data matrix handle");
  return static_cast<DataMatrix *>(p);
}
GardenHandle *AsGarden(VoidPointer p) {
  if (!p) throw std::runtime_error("null booster handle");
  return static_cast<GardenHandle *>(p);
}
TreeBuilder *BuilderOf(VoidPointer p) {
  TreeBuilder *b = AsGarden(p)->garden.builder();
  if (!b) throw std::runtime_error("no tree has been grown yet");
  return b;
}

const char *CopyOut(const std::vector<float> &v, const float **out) {
  float *p = new (std::nothrow) float[v.size() ? v.size() : 1];
  if (!p) return Fail("unable to allocate array");
  if (!v.empty()) std::memcpy(p, v.data(), v.size() * sizeof(float));
  *out = p;
  return nullptr;
}

}  // namespace

extern "C" {

const char *ACreateFromDenseMatrix(const float *data, const unsigned int *categories, int nrow,
                                   int ncol, int ccol, float /*missing*/, VoidPointer *out) {
  return Guard([&] {
    if (!data || !out || nrow < 0 || ncol < 0 || ccol < 0) throw std::runtime_error("bad arguments");
    DataMatrix *mat = new DataMatrix((size_t)nrow, (size_t)ncol, (size_t)ccol);
    const size_t rows = (size_t)nrow, cols = (size_t)ncol;
    // the columns are allocated (and their pages first touched) by several threads
    mat->data.resize(cols);
    {
      const size_t nt = std::min<size_t>(cols, 16);
      std::vector<std::thread> th;
      for (size_t t = 0; t < nt; ++t)
        th.emplace_back([&, t] {
          for (size_t f = t; f < cols; f += nt) mat->data[f].resize(rows);
        });
      for (auto &x : th) x.join();
    }
    // row-major -> column-major in tiles of 256 rows, so that a tile's lines of every
    // column stay in cache while its rows are read once
    ParallelFor(rows, [&](size_t b, size_t e) {
      for (size_t r0 = b; r0 < e; r0 += 256) {
        const size_t r1 = std::min(e, r0 + 256);
        for (size_t f = 0; f < cols; ++f) {
          float *dst = mat->data[f].data();
          for (size_t i = r0; i < r1; ++i) dst[i] = data[i * cols + f];
        }
      }
    });
    if (ccol > 0 && categories) {
      mat->data_categories.assign(ccol, std::vector<unsigned>(rows));
      for (size_t i = 0; i < rows; ++i)
        for (int c = 0; c < ccol; ++c) mat->data_categories[c][i] = categories[i * ccol + c];
    }
    *out = mat;
  });
}

const char *ASetY(VoidPointer data, const float *y) {
  return Guard([&] {
    DataMatrix *d = AsData(data);
    if (!y) throw std::runtime_error("null y");
    d->y.assign(y, y + d->rows);
  });
}

const char *ASetLabel(VoidPointer data, const unsigned char *labels) {
  return Guard([&] {
    DataMatrix *d = AsData(data);
    if (!labels) throw std::runtime_error("null labels");
    d->labels.assign(labels, labels + d->rows);
  });
}

const char *ASetWeights(VoidPointer data, const float *weights) {
  return Guard([&] {
    DataMatrix *d = AsData(data);
    if (!weights) throw std::runtime_error("null weights");
    d->weights.assign(weights, weights + d->rows);
  });
}

const char *AInitGarden(const char *configuration, VoidPointer *out) {
  return Guard([&] {
    if (!configuration || !out) throw std::runtime_error("bad arguments");
    *out = new GardenHandle(Configuration::Parse(configuration));
  });
}

const char *AGrowTree(VoidPointer garden, VoidPointer data, const float *grad) {
  return Guard([&] {
    AsGarden(garden)->garden.GrowTree(AsData(data), grad);
  });
}

const char *APredict(VoidPointer garden, VoidPointer data, const float **out, const int n_rounds) {
  float *result = nullptr;
  const char *err = Guard([&] {
    if (!out) throw std::runtime_error("bad arguments");
    Garden &g = AsGarden(garden)->garden;
    const DataMatrix *d = AsData(data);
    const size_t count = d->rows * g.cfg.tree.labels_count;
    result = new (std::nothrow) float[count ? count : 1];
    if (!result) throw std::runtime_error("unable to allocate array");
    g.Predict(d, result, n_rounds == -1 ? std::numeric_limits<int>::max() : n_rounds);
  });
  if (err) {
    delete[] result;
    return err;
  }
  *out = result;
  return nullptr;
}

const char *ADumpModel(const char **model, VoidPointer garden) {
  return Guard([&] {
    if (!model) throw std::runtime_error("bad arguments");
    *model = AsGarden(garden)->garden.GetModel();
  });
}

const char *ALoadModel(const char *model, VoidPointer garden) {
  return Guard([&] {
    if (!model) throw std::runtime_error("bad arguments");
    AsGarden(garden)->garden.Restore(model);
  });
}

const char *AGetY(VoidPointer garden, VoidPointer data, const float **out) {
  std::vector<float> result;
  const char *err = Guard([&] {
    if (!out) throw std::runtime_error("bad arguments");
    AsGarden(garden)->garden.GetY(AsData(data), &result);
  });
  return err ? err : CopyOut(result, out);
}

const char *AAppendLastTree(VoidPointer garden, VoidPointer data) {
  return Guard([&] { AsGarden(garden)->garden.UpdateByLastTree(AsData(data)); });
}

const char *AFreeDMatrix(VoidPointer ptr) {
  return Guard([&] { delete static_cast<DataMatrix *>(ptr); });
}
const char *AFreeGarden(VoidPointer ptr) {
  return Guard([&] { delete static_cast<GardenHandle *>(ptr); });
}
const char *ADeleteArray(float *in) {
  delete[] in;
  return nullptr;
}

// ------------------------------------------------------------- extensions
const char *ADeviceCount(int *out) {
  return Guard([&] { *out = DeviceCount(); });
}

const char *ADeviceCopyProbe(unsigned long long bytes) {
  return Guard([&] {
    if (DeviceCount() <= 0) throw std::runtime_error("no HIP device available");
    CopyProbe((size_t)bytes);
  });
}

const char *ACreateFromQuantized(const unsigned char *bins, long long nrow, int ncol, VoidPointer *out) {
  return Guard([&] {
    if (!bins || !out || nrow <= 0 || ncol <= 0) throw std::runtime_error("bad arguments");
    DataMatrix *mat = new DataMatrix((size_t)nrow, (size_t)ncol, 0);
    mat->is_prebinned = true;
    mat->prebinned.assign(bins, bins + (size_t)nrow * ncol);
    *out = mat;
  });
}

const char *ACreateFromQuantizedBlocks(const unsigned *const *blocks, int nblocks, long long block_rows,
                                       long long nrow, int ncol, VoidPointer *out) {
  return Guard([&] {
    if (!blocks || !out || nblocks <= 0 || block_rows <= 0 || nrow <= 0 || ncol <= 0)
      throw std::runtime_error("bad arguments");
    if (block_rows % 64 != 0) throw std::runtime_error("block_rows must be a multiple of 64");
    if (block_rows >= (1ll << 31)) throw std::runtime_error("a block holds fewer than 2^31 rows");
    // gradients are added as integers of up to 2^30 in magnitude: 2^33 of them can leave 64 bits
    if (nrow >= (1ll << 33)) throw std::runtime_error("too many rows: a matrix holds fewer than 2^33 rows");
    if ((long long)(nblocks - 1) * block_rows >= nrow || (long long)nblocks * block_rows < nrow)
      throw std::runtime_error("nrow does not match nblocks blocks of block_rows rows (the last one may be shorter)");
    for (int b = 0; b < nblocks; ++b)
      if (!blocks[b]) throw std::runtime_error("null block pointer");
    DataMatrix *mat = new DataMatrix((size_t)nrow, (size_t)ncol, 0);
    mat->is_prebinned = true;
    mat->external_blocks = true;
    mat->stream_block_rows = (size_t)block_rows;
    mat->stream_blocks.resize(nblocks);
    for (int b = 0; b < nblocks; ++b) mat->stream_blocks[b] = const_cast<uint32_t *>(blocks[b]);
    *out = mat;
  });
}

const char *AQuantize(VoidPointer data, int hist_size) {
  return Guard([&] {
    if (DeviceCount() <= 0) throw std::runtime_error("no HIP device available: the quantiser needs an MI355X");
    QuantiseOnDevice(AsData(data), hist_size, false);
  });
}

const char *AGetBins(VoidPointer data, unsigned char *out) {
  return Guard([&] { GetDeviceBins(*AsData(data), out); });
}

const char *AGetBins16(VoidPointer data, unsigned short *out) {
  return Guard([&] { GetDeviceBins16(*AsData(data), out); });
}

const char *AGetBinLayout(VoidPointer data, int *bits, int *slots) {
  return Guard([&] { GetBinLayout(*AsData(data), bits, slots); });
}

const char *AGetThresholds(VoidPointer data, int fid, float *thr, int *size) {
  return Guard([&] {
    DataMatrix *d = AsData(data);
    if (!d->quantised) throw std::runtime_error("data matrix is not quantised");
    if (fid < 0 || (size_t)fid >= d->columns_dense) throw std::runtime_error("feature id out of range");
    if (thr) std::memcpy(thr, d->thresholds[fid].data(), d->thresholds[fid].size() * sizeof(float));
    if (size) *size = d->reduced_size[fid];
  });
}

const char *AGardenSetInspect(VoidPointer garden, int on) {
  return Guard([&] {
    AsGarden(garden)->garden.SetInspect(on != 0);
  });
}

const char *AGardenPredictOnDevice(VoidPointer garden, int on) {
  return Guard([&] {
    AsGarden(garden)->garden.SetPredictOnDevice(on != 0);
  });
}

const char *AGardenNumTrees(VoidPointer garden, int *out) {
  return Guard([&] { *out = (int)AsGarden(garden)->garden.num_trees(); });
}

const char *AGardenGetTree(VoidPointer garden, int t, int *fid, int *bin, float *threshold, float *gain,
                           float *weights) {
  return Guard([&] {
    Garden &g = AsGarden(garden)->garden;
    if (t < 0 || (size_t)t >= g.num_trees()) throw std::runtime_error("tree index out of range");
    const RegTree &tr = g.tree(t);
    for (size_t i = 0; i < tr.fid.size(); ++i) {
      if (fid) fid[i] = (int)tr.fid[i];
      if (bin) bin[i] = tr.quantized[i];
      if (threshold) threshold[i] = tr.threshold[i];
      if (gain) gain[i] = tr.gain[i];
    }
    if (weights) std::memcpy(weights, tr.weights.data(), tr.weights.size() * sizeof(float));
  });
}

const char *AGardenGetTreeDepth(VoidPointer garden, int t, int *depth) {
  return Guard([&] {
    Garden &g = AsGarden(garden)->garden;
    if (t < 0 || (size_t)t >= g.num_trees()) throw std::runtime_error("tree index out of range");
    if (!depth) throw std::runtime_error("bad arguments");
    *depth = (int)g.tree(t).depth;
  });
}

const char *AGardenGetLeaves(VoidPointer garden, unsigned *out) {
  return Guard([&] { BuilderOf(garden)->GetLeaves(out); });
}
const char *AGardenGetTrainYHat(VoidPointer garden, float *out) {
  return Guard([&] { BuilderOf(garden)->GetYHat(out); });
}
const char *AGardenGetGrad(VoidPointer garden, float *g, float *h) {
  return Guard([&] { BuilderOf(garden)->GetGrad(g, h); });
}
const char *AGardenGetLevelHist(VoidPointer garden, int level, long long *out, int *cells) {
  return Guard([&] {
    const int n = BuilderOf(garden)->GetLevelHist(level, (int64_t *)out);
    if (n < 0) throw std::runtime_error("level histogram not kept (inspect off or bad level)");
    if (cells) *cells = n;
  });
}
const char *AGardenGetShifts(VoidPointer garden, int *shift_g, int *shift_h) {
  return Guard([&] { BuilderOf(garden)->GetShifts(shift_g, shift_h); });
}
const char *AGardenEnableTiming(VoidPointer garden, int on) {
  return Guard([&] {
    AsGarden(garden)->garden.SetTiming(on);
  });
}
const char *AGardenGetTimings(VoidPointer garden, double *out) {
  return Guard([&] {
    const BuilderTimings t = BuilderOf(garden)->GetTimings();
    out[0] = t.grad;
    out[1] = t.hist_root;
    out[2] = t.hist_deep;
    out[3] = t.reduce;
    out[4] = t.split;
    out[5] = t.partition;
    out[6] = t.leaf;
    out[7] = t.plan;
    out[8] = (double)t.hist_root_launches;
    out[9] = (double)t.hist_root_rows;
    out[10] = (double)t.hist_deep_launches;
    out[11] = t.fused_last;
    out[12] = (double)t.fused_last_launches;
  });
}
const char *AGardenRowsScanned(VoidPointer garden, unsigned long long *out) {
  return Guard([&] { *out = BuilderOf(garden)->RowsScanned(); });
}
const char *AGardenRowsScannedByLevel(VoidPointer garden, unsigned long long *out) {
  return Guard([&] { BuilderOf(garden)->RowsScannedByLevel(out); });
}
const char *AGardenStreamResidency(VoidPointer garden, unsigned long long *resident, unsigned long long *blocks) {
  return Guard([&] { BuilderOf(garden)->StreamResidency(resident, blocks); });
}
const char *AGardenSynchronize(VoidPointer garden) {
  return Guard([&] { BuilderOf(garden)->Synchronize(); });
}

const char *AHistSum(long long *sum_g, long long *sum_h, unsigned *bin_count, const long long *parent_g,
                     const long long *parent_h, const unsigned *parent_c, const float *grad, const float *hess,
                     const unsigned *node_size, const unsigned *bins, unsigned long long stride, long long nrow,
                     int ncol, int nodes, int use_trick, int shift_g, int shift_h, void *stream) {
  return Guard([&] {
    if (DeviceCount() <= 0) throw std::runtime_error("no HIP device available");
    HistSumArgs a{bins, stride, ncol, nrow, grad, hess, node_size, nodes, use_trick, parent_g, parent_h, parent_c,
                  shift_g, shift_h, sum_g, sum_h, bin_count, stream};
    HistSum(a);
  });
}

const char *AHistSumPlan(long long nrow, int nodes, unsigned *rows_per_item, unsigned *work_items) {
  return Guard([&] {
    if (nrow < 1 || nodes < 1 || !rows_per_item || !work_items) throw std::runtime_error("bad arguments");
    *rows_per_item = HistSumRowsPerItem((size_t)nrow, nodes);
    *work_items = (unsigned)((size_t)nrow / *rows_per_item + 2 * (size_t)nodes + 2);
  });
}

const char *AHistSumNoAlloc(long long *sum_g, long long *sum_h, unsigned *bin_count, const long long *parent_g,
                            const long long *parent_h, const unsigned *parent_c, const float *grad,
                            const float *hess, const unsigned *node_size, const unsigned *bins,
                            unsigned long long stride, long long nrow, int ncol, int nodes, int use_trick,
                            int shift_g, int shift_h, void *stream, unsigned *status) {
  return Guard([&] {
    HistSumArgs a{bins, stride, ncol, nrow, grad, hess, node_size, nodes, use_trick, parent_g, parent_h, parent_c,
                  shift_g, shift_h, sum_g, sum_h, bin_count, stream};
    HistSumNoAlloc(a, status);
  });
}

}  // extern "C"
