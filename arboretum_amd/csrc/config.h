// Booster configuration and its JSON form.  Keys, defaults and the
// max_depth -> depth + 1 rule follow the reference: src/core/param.h:16-74,
// src/core/json_conversion.h:55-167.
#ifndef ARBORETUM_AMD_CONFIG_H_
#define ARBORETUM_AMD_CONFIG_H_

#include <string>

#include "gain.h"
#include "json_min.h"

namespace arb {

enum Objective {  // param.h:7-14
  kLinearRegression = 0,
  kLogisticRegression = 1,
  kLogisticRegressionNoSigmoid = 2,
  kSoftMaxOneVsAll = 3,
  kSoftMaxOptimal = 4
};
enum Method { kExact = 0, kHist = 1 };

struct TreeParam {  // param.h:20-45
  unsigned depth = 8;  // internal depth = max_depth + 1
  float min_child_weight = 1.0f;
  unsigned min_leaf_size = 1;
  float colsample_bytree = 1.0f;
  float colsample_bylevel = 1.0f;
  float gamma_absolute = 0.0f;
  float gamma_relative = 0.0f;
  float lambda = 1.0f;
  float alpha = 0.0f;
  float initial_y = 0.5f;
  float eta = 0.3f;
  float max_leaf_weight = 0.0f;
  float scale_pos_weight = 1.0f;
  unsigned labels_count = 1;
};

struct Verbose {  // param.h:47-52
  bool gpu = false, booster = false, data = false;
};

struct InternalConfiguration {  // param.h:54-64
  bool double_precision = false;
  unsigned overlap = 2;
  unsigned seed = 0;
  bool use_hist_subtraction_trick = true;
  bool upload_features = true;
  int hist_size = 255;
  // Extension (not a reference key): rows per pinned-host block when the bins
  // are streamed (upload_features = false); 0 = chosen from the matrix size.
  unsigned stream_block_rows = 0;
  // Extension: bytes of a streamed matrix that stay in device memory (whole row blocks, spread
  // evenly over the matrix; only the others are copied at every level).  Negative: as many as
  // fit into 0.9 of the free device memory, the reference's rule for the columns it keeps
  // (src/io/io.cu:496-507); 0: every block is streamed.
  long long stream_resident_bytes = -1;
  // Extension: matrices of more than 32 features keep their rows in place and
  // re-order (row id, gradients) only, where that is the faster way (true, the
  // default: from 48 features on, and for any width whose bins in use fit one
  // LDS histogram); false selects the row-moving passes, the number 2 rows in
  // place for every width above 32 features.
  int wide_rows_in_place = 1;
  // Extension, exact method: features with more than 4096 distinct values are grown over sorted
  // row lists instead of rank histograms (-1, the default); 1: every matrix is; 0: never (such
  // features are an error).
  int exact_sort = -1;
};

struct Configuration {  // param.h:66-74
  int method = kHist;
  int objective = kLinearRegression;
  TreeParam tree;
  Verbose verbose;
  InternalConfiguration internal;

  static Configuration Parse(const char *text);  // throws std::runtime_error
  json::Value ToJson() const;

  GainParams gain_params() const {
    return GainParams{tree.min_leaf_size, tree.min_child_weight, tree.gamma_absolute,
                      tree.gamma_relative, tree.lambda,          tree.alpha,
                      tree.max_leaf_weight};
  }
  // (GRAD_T, SUM_T) dispatch of src/core/garden.cu:538-563
  int sum_kind() const {
    return (objective == kLinearRegression ? 0 : 2) + (internal.double_precision ? 1 : 0);
  }
};

}  // namespace arb
#endif  // ARBORETUM_AMD_CONFIG_H_
