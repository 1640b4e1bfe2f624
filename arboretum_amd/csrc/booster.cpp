#include "booster.h"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <exception>
#include <limits>
#include <mutex>
#include <stdexcept>
#include <thread>

namespace arb {

namespace {
// Runs the workers on threads of their own (the caller's included) and hands the first
// exception of any of them back to the caller instead of ending the process.
void RunWorkers(size_t workers, const std::function<void(size_t)> &work) {
  std::exception_ptr failed;
  std::mutex guard;
  auto run = [&](size_t t) {
    try {
      work(t);
    } catch (...) {
      std::lock_guard<std::mutex> lock(guard);
      if (!failed) failed = std::current_exception();
    }
  };
  std::vector<std::thread> th;
  for (size_t t = 1; t < workers; ++t) th.emplace_back(run, t);
  run(0);
  for (auto &t : th) t.join();
  if (failed) std::rethrow_exception(failed);
}
}  // namespace

void ParallelFor(size_t n, const std::function<void(size_t, size_t)> &fn) {
  unsigned hw = std::thread::hardware_concurrency();
  size_t nt = std::max<size_t>(1, std::min<size_t>(hw ? hw : 1, 16));
  if (n < 65536 || nt == 1) {
    fn(0, n);
    return;
  }
  const size_t chunk = (n + nt - 1) / nt;
  RunWorkers(nt, [&](size_t t) {
    const size_t b = t * chunk, e = std::min(n, b + chunk);
    if (b < e) fn(b, e);
  });
}

void ParallelTasks(size_t n, const std::function<void(size_t)> &fn) {
  const unsigned hw = std::thread::hardware_concurrency();
  const size_t nt = std::max<size_t>(1, std::min<size_t>({(size_t)(hw ? hw : 1), (size_t)16, n}));
  std::atomic<size_t> next{0};
  RunWorkers(nt, [&](size_t) {
    for (size_t i = next++; i < n; i = next++) fn(i);
  });
}

namespace {
std::atomic<uint64_t> g_next_matrix_uid{1};
}

DataMatrix::DataMatrix(size_t rows, size_t columns, size_t columns_category)
    : rows(rows), columns_dense(columns), columns_category(columns_category), uid(g_next_matrix_uid++) {}

DataMatrix::~DataMatrix() {
  if (device) FreeDeviceMatrix(device);
  if (exact_sort) FreeExactSortData(exact_sort);
}

RegTree::RegTree(unsigned depth, unsigned label) : depth(depth), label(label) {
  const size_t internal = ((size_t)1 << (depth - 1)) - 1;
  fid.assign(internal, 0);
  threshold.assign(internal, std::numeric_limits<float>::infinity());
  quantized.assign(internal, -1);
  gain.assign(internal, 0.0f);
  weights.assign((size_t)1 << (depth - 1), 0.0f);
}

void RegTree::PredictRows(const DataMatrix &data, size_t begin, size_t end, float *out) const {
  const size_t offset = ((size_t)1 << (depth - 1)) - 1;
  const size_t F = data.columns_dense;
  if (!data.is_prebinned) {
    // float columns: no per-value dispatch, no branch on the comparison
    bool foreign = false;  // a feature id outside the matrix (foreign model) behaves like NaN: right
    for (unsigned f : fid) foreign = foreign || f >= F;
    if (!foreign) {
      std::vector<const float *> cols(F);
      for (size_t f = 0; f < F; ++f) cols[f] = data.data[f].data();
      const unsigned *fids = fid.data();
      const float *thr = threshold.data();
      float *dst = out + (size_t)label * data.rows;
      for (size_t i = begin; i < end; ++i) {
        size_t id = 0;
        for (unsigned j = 1; j < depth; ++j) id = 2 * id + 2 - (size_t)(cols[fids[id]][i] < thr[id]);
        dst[i] += weights[id - offset];
      }
      return;
    }
  }
  for (size_t i = begin; i < end; ++i) {
    size_t id = 0;
    for (unsigned j = 1; j < depth; ++j) {
      const unsigned f = fid[id];
      // a feature id outside the matrix (foreign model) behaves like NaN: right
      const bool left = f < F && data.value(f, i) < threshold[id];
      id = left ? 2 * id + 1 : 2 * id + 2;
    }
    out[i + (size_t)label * data.rows] += weights[id - offset];
  }
}

void RegTree::Predict(const DataMatrix &data, float *out) const {
  ParallelFor(data.rows, [&](size_t b, size_t e) { PredictRows(data, b, e, out); });
}

Garden::Garden(const Configuration &c) : cfg(c) {
  // src/core/garden.cu:571-583 accepts objectives 0 and 1 only; the soft-max
  // ids (param.h:12-13) are implemented here from the formula the reference
  // leaves in a comment (objective.cu:60-89).
  switch (cfg.objective) {
    case kLinearRegression:
    case kLogisticRegression:
    case kSoftMaxOneVsAll:
    case kSoftMaxOptimal:
      break;
    default:
      throw std::runtime_error("Unknown objective function");
  }
  if (cfg.tree.depth < 2) throw std::runtime_error("max_depth must be at least 1");
  if (cfg.tree.depth >= 32) throw std::runtime_error("unsupported depth");  // garden.cu:536
  if (cfg.tree.labels_count < 1) throw std::runtime_error("labels_count must be at least 1");
}

Garden::~Garden() {}

float Garden::IntoInternal(float v) const {
  if (cfg.objective == kLogisticRegression) return std::log(v / (1 - v));
  return v;
}

void Garden::FromInternal(const std::vector<float> &in, std::vector<float> *out) const {
  out->resize(in.size());
  FromInternal(in.data(), in.size(), out->data());
}

void Garden::FromInternal(const float *in, size_t count, float *out) const {
  if (cfg.objective == kLinearRegression) {
    ParallelFor(count, [&](size_t b, size_t e) { std::memcpy(out + b, in + b, (e - b) * sizeof(float)); });
  } else if (cfg.objective == kLogisticRegression) {  // objective.h:58-69
    ParallelFor(count, [&](size_t b, size_t e) {
      for (size_t i = b; i < e; ++i) out[i] = (float)(1.0 / (1.0 + (double)std::exp(-in[i])));
    });
  } else {  // objective.h:80-113: class-major in, row-major out
    const size_t K = cfg.tree.labels_count;
    const size_t n = count / K;
    ParallelFor(n, [&](size_t b, size_t e) {
      std::vector<double> v(K);
      for (size_t i = b; i < e; ++i) {
        double sum = 0.0;
        for (size_t k = 0; k < K; ++k) {
          v[k] = std::exp((double)in[i + n * k]);
          sum += v[k];
        }
        for (size_t k = 0; k < K; ++k) out[i * K + k] = (float)(v[k] / sum);
      }
    });
  }
}

void Garden::GrowTree(DataMatrix *data, const float *grad) {
  if (cfg.method != kHist && cfg.method != kExact) throw std::runtime_error("unknown method");
  if (grad != nullptr) throw std::runtime_error("user-supplied gradients are not supported");
  if (cfg.objective >= kSoftMaxOneVsAll) {
    if (data->labels.size() != data->rows) throw std::runtime_error("labels are not set");
  } else if (data->y.size() != data->rows) {
    throw std::runtime_error("y is not set");
  }
  // colsample checks of InitGrowingTree, garden.cu:126-140
  const size_t columns = data->columns_dense + data->columns_category;
  if ((int)(cfg.tree.colsample_bytree * columns) == 0)
    throw std::runtime_error("colsample_bytree is too small");
  if ((int)(cfg.tree.colsample_bytree * cfg.tree.colsample_bylevel * columns) == 0)
    throw std::runtime_error("colsample_bytree and colsample_bylevel are too small");
  if (!builder_ && cfg.objective < kSoftMaxOneVsAll) {
    // Gradients are accumulated in fixed point scaled by the largest one; a
    // target that is NaN or infinite has no scale (the reference would carry
    // the NaN into every sum it touches).
    std::atomic<bool> bad{false};
    ParallelFor(data->rows, [&](size_t b, size_t e) {
      bool any = false;
      for (size_t i = b; i < e; ++i) any = any || !std::isfinite(data->y[i]);
      if (any) bad = true;
    });
    if (bad) throw std::runtime_error("y must be finite");
  }
  if (DeviceCount() <= 0) throw std::runtime_error("no HIP device available: training needs an MI355X");
  if (!builder_) {
    // upload_features = false keeps the bins in pinned host memory and streams
    // them (src/core/garden.cu:603-604, hist_tree_grower.cu:335-366)
    QuantiseOnDevice(data, cfg.internal.hist_size, cfg.verbose.data, !cfg.internal.upload_features,
                     cfg.internal.stream_block_rows, cfg.method == kExact, cfg.internal.exact_sort);
    builder_.reset(CreateTreeBuilder(cfg, data));
    builder_->SetInspect(inspect_);
    builder_->EnableTiming(timing_);
    bound_ = data;
  } else if (bound_ != data) {
    throw std::runtime_error("booster is bound to another data matrix");
  }
  builder_->GrowRound(&trees_);
}

void Garden::Predict(const DataMatrix *data, float *out, int n_rounds) const {
  const size_t K = cfg.tree.labels_count;
  SyncTrees();
  const long long use = std::min<long long>(n_rounds, (long long)trees_.size());
  const float init = IntoInternal(cfg.tree.initial_y);
  if (predict_on_device_ && use > 0 && data->rows > 0 && DeviceCount() > 0) {
    if (!predictor_) predictor_.reset(CreateDevicePredictor());
    const float *sums = PredictOnDevice(predictor_.get(), *data, trees_, (size_t)use, K, init);
    FromInternal(sums, data->rows * K, out);
    return;
  }
  std::vector<float> tmp(data->rows * K, init);
  // Every tree over one block of rows before the next block: the block's
  // feature values (column-major, 4096 rows of every column) stay in cache, so
  // the matrix is read once, not once per tree.  Sums per row are added in tree
  // order either way.
  constexpr size_t kBlock = 4096;
  ParallelFor(data->rows, [&](size_t b, size_t e) {
    for (size_t r0 = b; r0 < e; r0 += kBlock) {
      const size_t r1 = std::min(e, r0 + kBlock);
      for (long long t = 0; t < use; ++t) trees_[t].PredictRows(*data, r0, r1, tmp.data());
    }
  });
  FromInternal(tmp.data(), tmp.size(), out);
}

void Garden::UpdateByLastTree(DataMatrix *data) {
  const size_t K = cfg.tree.labels_count;
  if (data->y_hat.empty()) data->y_hat.assign(data->rows * K, IntoInternal(cfg.tree.initial_y));
  if (trees_.size() < K) return;
  SyncTrees();
  for (size_t t = trees_.size() - K; t < trees_.size(); ++t) trees_[t].Predict(*data, data->y_hat.data());
}

void Garden::GetY(const DataMatrix *data, std::vector<float> *out) const {
  FromInternal(data->y_hat, out);
}

// src/core/model_helper.cpp:16-23, json_conversion.h:13-40
const char *Garden::GetModel() {
  using json::Value;
  Value root = Value::MakeObject();
  root["configuration"] = cfg.ToJson();
  Value model = Value::MakeArray();
  SyncTrees();
  for (const RegTree &t : trees_) {
    Value jt = Value::MakeObject();
    Value nodes = Value::MakeArray();
    const size_t internal = ((size_t)1 << (t.depth - 1)) - 1;
    const size_t total = ((size_t)1 << t.depth) - 1;
    for (size_t id = 0; id < total; ++id) {
      Value n = Value::MakeObject();
      n["id"] = Value::MakeInt((int64_t)id);
      const bool leaf = id >= internal;
      n["leaf"] = Value::MakeBool(leaf);
      if (!leaf) {
        n["left"] = Value::MakeInt((int64_t)(2 * id + 1));
        n["right"] = Value::MakeInt((int64_t)(2 * id + 2));
        n["threshold"] = Value::MakeFloat(t.threshold[id]);  // non-finite prints as null
        n["fid"] = Value::MakeInt(t.fid[id]);
      } else {
        n["idx"] = Value::MakeInt((int64_t)(id - internal));
      }
      nodes.push(n);
    }
    jt["nodes"] = nodes;
    Value w = Value::MakeArray();
    for (float x : t.weights) w.push(Value::MakeFloat(x));
    jt["weights"] = w;
    jt["depth"] = Value::MakeInt(t.depth);
    model.push(jt);
  }
  root["model"] = model;
  model_.clear();
  json::Dump(root, model_);
  return model_.c_str();
}

// src/core/model_helper.cpp:25-30, json_conversion.h:26-52, garden.cu:667-677.
// A tree without "depth" takes the booster's depth.
void Garden::Restore(const char *json_model) {
  json::Value j = json::Parse(json_model);
  const json::Value *model = j.find("model");
  if (!model || !model->is_array()) throw std::runtime_error("model: missing \"model\" array");
  std::vector<RegTree> loaded;
  for (const json::Value &jt : *model->a) {
    unsigned depth = cfg.tree.depth;
    if (const json::Value *d = jt.find("depth")) depth = (unsigned)d->number();
    if (depth < 2 || depth >= 32) throw std::runtime_error("model: bad tree depth");
    RegTree t(depth, 0);  // label forced to 0 as in the reference
    const json::Value *nodes = jt.find("nodes");
    const json::Value *weights = jt.find("weights");
    if (!nodes || !nodes->is_array() || !weights || !weights->is_array())
      throw std::runtime_error("model: tree needs \"nodes\" and \"weights\"");
    if (weights->a->size() != t.weights.size()) throw std::runtime_error("model: wrong number of weights");
    for (size_t k = 0; k < t.weights.size(); ++k) t.weights[k] = (float)(*weights->a)[k].number();
    for (const json::Value &n : *nodes->a) {
      const json::Value *id = n.find("id");
      if (!id) throw std::runtime_error("model: node without id");
      const size_t i = (size_t)id->number();
      if (i >= t.fid.size()) continue;  // leaf record
      if (const json::Value *th = n.find("threshold"))
        t.threshold[i] = th->is_null() ? std::numeric_limits<float>::infinity() : (float)th->number();
      if (const json::Value *f = n.find("fid")) t.fid[i] = (unsigned)f->number();
    }
    loaded.push_back(std::move(t));
  }
  SyncTrees();
  for (RegTree &t : loaded) trees_.push_back(std::move(t));
}

}  // namespace arb
