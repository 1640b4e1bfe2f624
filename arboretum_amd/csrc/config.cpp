#include "config.h"

namespace arb {
namespace {

template <typename T>
void GetNum(const json::Value &j, const char *key, T *out) {
  const json::Value *v = j.find(key);
  if (v) *out = (T)v->number();
}
void GetBool(const json::Value &j, const char *key, bool *out) {
  const json::Value *v = j.find(key);
  if (v) *out = v->boolean();
}

}  // namespace

// src/core/param.cpp:47-51 + json_conversion.h from_json overloads: every key
// is optional, unknown keys are ignored.
Configuration Configuration::Parse(const char *text) {
  json::Value j = json::Parse(text);
  if (!j.is_object()) throw std::runtime_error("configuration must be a JSON object");
  Configuration cfg;
  GetNum(j, "method", &cfg.method);
  GetNum(j, "objective", &cfg.objective);
  if (const json::Value *t = j.find("tree")) {
    if (const json::Value *d = t->find("max_depth")) cfg.tree.depth = (unsigned)((int)d->number() + 1);
    GetNum(*t, "min_child_weight", &cfg.tree.min_child_weight);
    GetNum(*t, "min_leaf_size", &cfg.tree.min_leaf_size);
    GetNum(*t, "colsample_bytree", &cfg.tree.colsample_bytree);
    GetNum(*t, "colsample_bylevel", &cfg.tree.colsample_bylevel);
    GetNum(*t, "gamma_absolute", &cfg.tree.gamma_absolute);
    GetNum(*t, "gamma_relative", &cfg.tree.gamma_relative);
    GetNum(*t, "lambda", &cfg.tree.lambda);
    GetNum(*t, "alpha", &cfg.tree.alpha);
    GetNum(*t, "initial_y", &cfg.tree.initial_y);
    GetNum(*t, "eta", &cfg.tree.eta);
    GetNum(*t, "max_leaf_weight", &cfg.tree.max_leaf_weight);
    GetNum(*t, "scale_pos_weight", &cfg.tree.scale_pos_weight);
    GetNum(*t, "labels_count", &cfg.tree.labels_count);
  }
  if (const json::Value *v = j.find("verbose")) {
    GetBool(*v, "gpu", &cfg.verbose.gpu);
    GetBool(*v, "booster", &cfg.verbose.booster);
    GetBool(*v, "data", &cfg.verbose.data);
  }
  if (const json::Value *v = j.find("internals")) {
    GetBool(*v, "double_precision", &cfg.internal.double_precision);
    GetNum(*v, "compute_overlap", &cfg.internal.overlap);
    GetNum(*v, "seed", &cfg.internal.seed);
    GetBool(*v, "use_hist_subtraction_trick", &cfg.internal.use_hist_subtraction_trick);
    GetBool(*v, "upload_features", &cfg.internal.upload_features);
    GetNum(*v, "hist_size", &cfg.internal.hist_size);
    GetNum(*v, "stream_block_rows", &cfg.internal.stream_block_rows);
    GetNum(*v, "stream_resident_bytes", &cfg.internal.stream_resident_bytes);
    if (const json::Value *w = v->find("wide_rows_in_place"))
      cfg.internal.wide_rows_in_place = w->is_number() ? (int)w->number() : (w->boolean() ? 1 : 0);
    if (const json::Value *w = v->find("exact_sort"))
      cfg.internal.exact_sort = w->is_number() ? (int)w->number() : (w->boolean() ? 1 : 0);
  }
  return cfg;
}

// to_json(Configuration), json_conversion.h:62-70,88-105,149-155
json::Value Configuration::ToJson() const {
  using json::Value;
  Value j = Value::MakeObject();
  j["method"] = Value::MakeInt(method);
  j["objective"] = Value::MakeInt(objective);
  Value t = Value::MakeObject();
  t["max_depth"] = Value::MakeInt((int)tree.depth - 1);
  t["min_child_weight"] = Value::MakeFloat(tree.min_child_weight);
  t["min_leaf_size"] = Value::MakeInt(tree.min_leaf_size);
  t["colsample_bytree"] = Value::MakeFloat(tree.colsample_bytree);
  t["colsample_bylevel"] = Value::MakeFloat(tree.colsample_bylevel);
  t["gamma_absolute"] = Value::MakeFloat(tree.gamma_absolute);
  t["gamma_relative"] = Value::MakeFloat(tree.gamma_relative);
  t["lambda"] = Value::MakeFloat(tree.lambda);
  t["alpha"] = Value::MakeFloat(tree.alpha);
  t["initial_y"] = Value::MakeFloat(tree.initial_y);
  t["eta"] = Value::MakeFloat(tree.eta);
  t["max_leaf_weight"] = Value::MakeFloat(tree.max_leaf_weight);
  t["scale_pos_weight"] = Value::MakeFloat(tree.scale_pos_weight);
  t["labels_count"] = Value::MakeInt(tree.labels_count);
  j["tree"] = t;
  Value v = Value::MakeObject();
  v["gpu"] = Value::MakeBool(verbose.gpu);
  v["booster"] = Value::MakeBool(verbose.booster);
  v["data"] = Value::MakeBool(verbose.data);
  j["verbose"] = v;
  Value in = Value::MakeObject();
  in["double_precision"] = Value::MakeBool(internal.double_precision);
  in["compute_overlap"] = Value::MakeInt(internal.overlap);
  in["seed"] = Value::MakeInt(internal.seed);
  in["use_hist_subtraction_trick"] = Value::MakeBool(internal.use_hist_subtraction_trick);
  in["upload_features"] = Value::MakeBool(internal.upload_features);
  in["hist_size"] = Value::MakeInt(internal.hist_size);
  j["internals"] = in;
  return j;
}

}  // namespace arb
