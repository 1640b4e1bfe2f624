// ---------------------------------------------------------------------------
// TEST INFRASTRUCTURE — NOT PART OF THE PRODUCT.
//
// CPU restatement of the histogram tree-growing path of sh1ng/arboretum, used
// only as the checker in tests, in the smoke check and as the timed CPU
// baseline of the benchmark.  The shipped library never links, loads or calls
// anything in this directory.
//
// Every function cites the reference file:line it restates (paths relative to
// the reference tree).  Rows are kept in their ORIGINAL order with a node id
// per row; the reference's physical re-ordering of rows at each level
// (src/core/garden.cu:255-294, src/core/partition.cuh:20-87) does not change
// any value computed here.
//
// Accumulation.  The reference adds (grad, hess) pairs with floating-point
// atomics (src/core/hist_grad_sum.cu:109-215,262-406), so its sums depend on
// the order of addition.  Two accumulation modes exist here:
//   accum = 0  "fixed":  every gradient is rounded once to a 64-bit integer
//              multiple of 2^-shift (|q| <= 2^30, see fix_shift below) and the
//              integers are added; the sum is order independent and is what
//              the GPU library must reproduce bit for bit.
//   accum = 1  "native": sequential accumulation in the reference's SUM_T
//              (float or double), the yardstick for the 1e-5 tolerance.
//
// Parity status of each function (what pins it):
//   quantize_column     pinned: tests/cpp/test_datamatrix.cu:25-197 goldens
//   gain / weight       pinned: tests/cpp/test_hist.cu:119-120,222-226 and the
//                       closed form G^2/(H+lambda) at alpha = 0
//   histogram / trick   pinned: tests/cpp/test_hist_sum.cu closed forms
//   tree growth, leaves, predict, model
//                       pinned: golden models and predictions of
//                       tests/py/test_hist_regregression.py and
//                       tests/py/test_hist_logregression.py
//   softmax grad/hess, softmax link
//                       pinned by the mathematics: the reference's kernel is
//                       empty (src/core/objective.cu:91-100) and holds the
//                       formula only as the comment at objective.cu:60-89, the
//                       link at objective.h:80-113.  Checked against a float64
//                       scipy soft-max, the K = 2 reduction to the logistic
//                       sigmoid, sum-to-zero / range invariants and the central
//                       difference of the log-likelihood.
//   column sampling     pinned (garden.cu:126-165, 249-253): the active ids of
//                       every (tree, level) against literal vectors written by
//                       tests/golden/make_shuffle_vectors.cpp, a program that
//                       holds nothing but the reference's calls on the random
//                       engine; set sizes and split-feature membership; the
//                       two error strings.  (The draw itself is the standard
//                       library's std::shuffle on std::default_random_engine.)
//   exact method        pinned: golden models of tests/py/test_regression.py and
//                       tests/py/test_logresression.py, a plain-Python search over
//                       every distinct value on seeded inputs; the 32-bit ranks of
//                       features with more than 65535 distinct values against the
//                       16-bit ones on the same input (orc_force_wide_ranks)
//   orc_expf            defined here (double polynomial, correctly rounded in
//                       all but rare cases); checked against libm within 1 ulp.
// ---------------------------------------------------------------------------
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <limits>
#include <random>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

// ---------------------------------------------------------------- parameters
struct OrcParams {
  int objective;          // 0 squared, 1 logistic, 4 softmax (param.h:7-14)
  int depth;              // internal depth = max_depth + 1 (json_conversion.h:108-112)
  float min_child_weight;
  unsigned min_leaf_size;
  float gamma_absolute;
  float gamma_relative;
  float lambda;
  float alpha;
  float initial_y;
  float eta;
  float max_leaf_weight;
  int hist_size;
  int double_precision;   // SUM_T = double / double2 when set (garden.cu:538-556)
  int accum;              // 0 fixed-point, 1 native sequential
  int use_trick;          // sibling subtraction (param.h:55)
  int labels_count;
  int threads;            // OpenMP threads for the histogram loop (0 = default)
  float colsample_bytree;
  float colsample_bylevel;
  unsigned seed;
  int method;             // 1 = hist, 0 = exact (param.h:16)
};

// ------------------------------------------------------------------- exp
// exp(x) for float x evaluated in double: x = k*ln2/32 + r, |r| <= ln2/64,
// exp(r) by a degree-7 Taylor polynomial (error < 1e-17 relative), constant
// table of 2^(j/32).  Only +,*,fma-free double operations in a
// fixed order, so any IEEE machine gives the same bits.
static const double kExpTab[32] = {  // 2^(j/32), j = 0..31
    0x1.0000000000000p+0, 0x1.059b0d3158574p+0, 0x1.0b5586cf9890fp+0, 0x1.11301d0125b51p+0,
    0x1.172b83c7d517bp+0, 0x1.1d4873168b9aap+0, 0x1.2387a6e756238p+0, 0x1.29e9df51fdee1p+0,
    0x1.306fe0a31b715p+0, 0x1.371a7373aa9cbp+0, 0x1.3dea64c123422p+0, 0x1.44e086061892dp+0,
    0x1.4bfdad5362a27p+0, 0x1.5342b569d4f82p+0, 0x1.5ab07dd485429p+0, 0x1.6247eb03a5585p+0,
    0x1.6a09e667f3bcdp+0, 0x1.71f75e8ec5f74p+0, 0x1.7a11473eb0187p+0, 0x1.82589994cce13p+0,
    0x1.8ace5422aa0dbp+0, 0x1.93737b0cdc5e5p+0, 0x1.9c49182a3f090p+0, 0x1.a5503b23e255dp+0,
    0x1.ae89f995ad3adp+0, 0x1.b7f76f2fb5e47p+0, 0x1.c199bdd85529cp+0, 0x1.cb720dcef9069p+0,
    0x1.d5818dcfba487p+0, 0x1.dfc97337b9b5fp+0, 0x1.ea4afa2a490dap+0, 0x1.f50765b6e4540p+0};

static inline float orc_expf_impl(float xf) {
  if (xf != xf) return xf;
  if (xf > 88.8f) return std::numeric_limits<float>::infinity();
  if (xf < -104.0f) return 0.0f;
  const double x = (double)xf;
  const double inv = 0x1.71547652b82fep+5;   // 32 / ln 2
  const double c1 = 0x1.62e42fefa39efp-6;    // ln 2 / 32
  double kd = std::nearbyint(x * inv);
  int k = (int)kd;
  double r = x - kd * c1;
  double p = 1.0 / 5040.0;
  p = p * r + 1.0 / 720.0;
  p = p * r + 1.0 / 120.0;
  p = p * r + 1.0 / 24.0;
  p = p * r + 1.0 / 6.0;
  p = p * r + 0.5;
  p = p * r + 1.0;
  p = p * r + 1.0;
  int j = k & 31;
  int m = (k - j) / 32;
  double v = kExpTab[j] * p;
  return (float)std::ldexp(v, m);
}

// Sigmoid: src/core/objective.h:67-69  "1.0 / (1.0 + std::exp(-x))" with a
// float exp and a double divide rounded to float.
static inline float sigmoid_f(float x) {
  return (float)(1.0 / (1.0 + (double)orc_expf_impl(-x)));
}

// ------------------------------------------------------------- quantiser
// src/io/io.cu:349-435 (InitHistInternal), :27-153 (ValueSegmentIterator,
// SegmentLength), :255-270 (ThresholdOutputIterator::operator=), :293-312
// (build_histogram), src/core/cuda_helpers.h:207-222 (lower_bound).
struct QuantResult {
  std::vector<float> thr;  // hist_size entries, +INF where unset
  int size;                // number of real bins = min(unique, hist_size)
};

static QuantResult quantize_thresholds(const float *x, int64_t n, int hist_size) {
  std::vector<float> s(x, x + n);
  // cub radix order for non-negative-sign NaN: after +inf.  NaNs of either
  // sign are placed last here.
  std::sort(s.begin(), s.end(), [](float a, float b) {
    bool an = a != a, bn = b != b;
    if (an || bn) return !an && bn;
    return a < b;
  });
  QuantResult q;
  q.thr.assign(hist_size, std::numeric_limits<float>::infinity());
  unsigned seg = (unsigned)(n / hist_size);  // io.cu:371-372
  if (seg < 1) seg = 1;
  unsigned k = 0;
  for (int64_t i = 1; i < n; ++i) {
    if (s[i] != s[i - 1]) {  // border (io.cu:77); NaN != NaN counts too
      ++k;
      float mid = (float)((double)(float)(s[i] + s[i - 1]) * 0.5);  // io.cu:76
      int slot = (int)std::min<unsigned>(k + 1, (unsigned)(i / seg + 1)) - 2;  // io.cu:257
      if (slot >= 0 && slot < hist_size && mid < q.thr[slot]) q.thr[slot] = mid;
    }
  }
  int unique = 0;  // io.cu:403-408: leading finite thresholds only
  while (unique < hist_size && !std::isinf(q.thr[unique])) ++unique;
  ++unique;
  q.size = std::min(unique, hist_size);
  return q;
}

static inline unsigned bin_of(const float *thr, int size, float x) {
  // values[t] = thr[t] for t < size-1, +INF for t >= size-1 (io.cu:297-302);
  // lower_bound over [0,size) (cuda_helpers.h:207-222): first l with x <= v[l].
  unsigned l = 0, h = (unsigned)size;
  while (l < h) {
    unsigned mid = (l + h) / 2;
    float v = ((int)mid < size - 1) ? thr[mid] : std::numeric_limits<float>::infinity();
    if (x <= v)
      h = mid;
    else
      l = mid + 1;
  }
  return l;
}

// ------------------------------------------------------- gain and weights
// src/core/gain.cu:8-238.  S is the reference's scalar sum type (float or
// double); PAIR selects the (grad,hess) form (float2/double2) against the
// count-as-hessian form (float/double).
struct GainParams {
  unsigned min_leaf_size;
  float hess;  // min_child_weight
  float gamma_absolute, gamma_relative, lambda, alpha, max_leaf_weight;
};

template <typename T>
static inline int sgn(T v) {
  return (T(0) < v) - (v < T(0));  // gain.cu:9-11
}

static inline float threshold_weight(float w, float mlw) {  // gain.cu:25-32
  if (mlw != 0.0f) {
    if (w > mlw) return mlw;
    if (w < -mlw) return -mlw;
  }
  return w;
}

// grad_regularized, gain.cu:19-23: sign(g) * max(0.0, |g| - alpha) computed in
// double and converted back to T.
template <typename S>
static inline S grad_reg(S g, float alpha) {
  S d = std::fabs(g) - (S)alpha;  // float path stays float, double path double
  double m = (double)d > 0.0 ? (double)d : 0.0;
  return (S)(sgn(g) * m);
}

// Weight, count-as-hessian form: gain.cu:34-56
template <typename S>
static inline float weight_cnt(S s, unsigned c, const GainParams &p) {
  float w = 0.0f;
  if (c >= p.min_leaf_size && (float)c >= p.hess) {
    float den = (float)c + p.lambda;
    if (sizeof(S) == 4)
      w = (float)grad_reg<S>(s, p.alpha) / den;
    else
      w = (float)((double)grad_reg<S>(s, p.alpha) / (double)den);
  }
  return threshold_weight(w, p.max_leaf_weight);
}

// Weight, (grad,hess) form: gain.cu:58-76
template <typename S>
static inline float weight_pair(S g, S h, unsigned c, const GainParams &p) {
  float w = 0.0f;
  if (c >= p.min_leaf_size && h >= (S)p.hess) {
    if (sizeof(S) == 4)
      w = (float)grad_reg<S>(g, p.alpha) / ((float)h + p.lambda);
    else
      w = (float)((double)grad_reg<S>(g, p.alpha) / ((double)h + (double)p.lambda));
  }
  return threshold_weight(w, p.max_leaf_weight);
}

// gain(), gain.cu:13-17: -2 * (g*(-w) + 0.5*(h+lambda)*w*w + alpha*|w|), the
// 0.5 literal is double so everything after the first product is double.
template <typename S>
static inline float side_gain_pair(S g, S h, float w, float lambda, float alpha) {
  S a = g * (S)(-w);                 // T1 * float -> T1
  S hl = h + (S)lambda;              // T2 + float -> T2
  double b = 0.5 * (double)hl * (double)w * (double)w;
  float c = alpha * std::fabs(w);
  double r = -2 * (((double)a + b) + (double)c);
  return (float)r;
}
template <typename S>
static inline float side_gain_cnt(S g, uint64_t cnt, float w, float lambda, float alpha) {
  S a = g * (S)(-w);
  float hl = (float)cnt + lambda;    // size_t + float -> float
  double b = 0.5 * (double)hl * (double)w * (double)w;
  float c = alpha * std::fabs(w);
  double r = -2 * (((double)a + b) + (double)c);
  return (float)r;
}

// gain_func (float2 / double2): gain.cu:124-181
template <typename S>
static float gain_pair(S gl, S hl, uint64_t cl, S gt, S ht, uint64_t ct, const GainParams &p) {
  S gr = gt - gl, hr = ht - hl;
  uint64_t cr = ct - cl;
  if (cl >= p.min_leaf_size && cr >= p.min_leaf_size && std::fabs(hl) >= (S)p.hess &&
      std::fabs(hr) >= (S)p.hess) {
    float wl = weight_pair<S>(gl, hl, (unsigned)cl, p);
    float wr = weight_pair<S>(gr, hr, (unsigned)cr, p);
    float wp = weight_pair<S>(gt, ht, (unsigned)ct, p);
    float l = side_gain_pair<S>(gl, hl, wl, p.lambda, p.alpha);
    float r = side_gain_pair<S>(gr, hr, wr, p.lambda, p.alpha);
    float q = side_gain_pair<S>(gt, ht, wp, p.lambda, p.alpha);
    float diff = l + r - q;
    return (float)(diff > p.gamma_absolute && diff > p.gamma_relative * q) * diff;
  }
  return 0.0f;
}

// gain_func (float / double, count is the hessian): gain.cu:183-238
template <typename S>
static float gain_cnt(S gl, uint64_t cl, S gt, uint64_t ct, const GainParams &p) {
  uint64_t cr = ct - cl;
  S gr = gt - gl;
  if (cl >= p.min_leaf_size && cr >= p.min_leaf_size) {
    float wl = weight_cnt<S>(gl, (unsigned)cl, p);
    float wr = weight_cnt<S>(gr, (unsigned)cr, p);
    float wp = weight_cnt<S>(gt, (unsigned)ct, p);
    float l = side_gain_cnt<S>(gl, cl, wl, p.lambda, p.alpha);
    float r = side_gain_cnt<S>(gr, cr, wr, p.lambda, p.alpha);
    float q = side_gain_cnt<S>(gt, ct, wp, p.lambda, p.alpha);
    float diff = l + r - q;
    return (float)(diff > p.gamma_absolute && diff > p.gamma_relative * q) * diff;
  }
  return 0.0f;
}

// One entry point over the four reference instantiations.
// kind: 0 float, 1 double, 2 float2, 3 double2 (garden.cu:538-563).
static float gain_any(int kind, double gl, double hl, uint64_t cl, double gt, double ht,
                      uint64_t ct, const GainParams &p) {
  switch (kind) {
    case 0: return gain_cnt<float>((float)gl, cl, (float)gt, ct, p);
    case 1: return gain_cnt<double>(gl, cl, gt, ct, p);
    case 2: return gain_pair<float>((float)gl, (float)hl, cl, (float)gt, (float)ht, ct, p);
    default: return gain_pair<double>(gl, hl, cl, gt, ht, ct, p);
  }
}
static float weight_any(int kind, double g, double h, unsigned c, const GainParams &p) {
  switch (kind) {
    case 0: return weight_cnt<float>((float)g, c, p);
    case 1: return weight_cnt<double>(g, c, p);
    case 2: return weight_pair<float>((float)g, (float)h, c, p);
    default: return weight_pair<double>(g, h, c, p);
  }
}

// ------------------------------------------------------------ fixed point
// q = rint(v * 2^shift) with shift = 30 - e and |v| <= 2^e for every element,
// so |q| <= 2^30 and any sum over fewer than 2^32 rows fits in int64.
//   logistic: |g| <= 1 -> shift 30; 0 <= h <= 1/4 -> shift 32
//   softmax : |g| <= 1 -> shift 30; 0 <= h <= 1/2 -> shift 31
//   logistic with labels outside [0, 1]: shift of max(|ymin - 1|, |ymax|)
//   squared : e from frexp(max |g|) (max = m * 2^e, 1/2 <= m < 1); h is the count
static inline int fix_shift_from_max(float vmax) {
  if (!(vmax > 0.0f) || std::isinf(vmax)) return 30;
  int e;
  std::frexp(vmax, &e);
  return 30 - e;
}
static inline int64_t to_fixed(float v, int shift) {
  double s = std::ldexp((double)v, shift);
  if (!(std::fabs(s) <= 1073741824.0)) return 0;  // non-finite or out of range
  return (int64_t)std::nearbyint(s);
}
static inline double from_fixed(int64_t q, int shift) { return std::ldexp((double)q, -shift); }

struct Acc {  // one histogram cell / one node total
  int64_t gq = 0, hq = 0;  // fixed mode
  double g = 0, h = 0;     // native mode, value held in SUM_T precision
  uint64_t c = 0;
};

struct TreeOut {
  int depth;                      // internal depth
  std::vector<int> fid;           // 2^(depth-1)-1 internal nodes, heap order
  std::vector<int> quantized;     // split bin or -1
  std::vector<float> threshold;
  std::vector<float> gain;
  std::vector<float> weights;     // 2^(depth-1)
  int label;
};

struct Booster {
  OrcParams p;
  int64_t n = 0;
  int F = 0;
  int slots = 0;  // hist_size + 1 (the extra slot takes NaN when size == hist_size)
  std::vector<float> X;  // row-major copy
  std::vector<std::vector<float>> thr;
  std::vector<int> size;
  std::vector<uint16_t> bins;  // row-major [n][F]
  // exact method with more than 65535 distinct values in a feature: the ranks, instead of `bins`
  std::vector<uint32_t> wide_bins;
  uint32_t bin_at(size_t i, int f) const {
    return wide_bins.empty() ? bins[i * (size_t)F + f] : wide_bins[i * (size_t)F + f];
  }
  std::vector<float> y, yhat, g, h;
  std::vector<uint8_t> labels;
  std::vector<TreeOut> trees;
  // inspection of the last grown tree
  std::vector<uint32_t> leaf;            // per original row
  std::vector<std::vector<Acc>> lvl_hist;  // [level][node*F*slots + f*slots + b]
  std::vector<std::vector<Acc>> lvl_tot;   // [level][node]
  int shift_g = 30, shift_h = 32;
  std::default_random_engine rnd;  // garden.cu:87, seeded with internals.seed
  // inspection: the features a split may use, per grown tree and level, in the
  // order they stand at the front of the shuffled id list
  std::vector<std::vector<std::vector<unsigned>>> active_log;
  uint64_t updates = 0;  // rows*features actually accumulated (work counter)
  int kind() const { return (p.objective == 0 ? 0 : 2) + (p.double_precision ? 1 : 0); }
};

static GainParams gain_params(const OrcParams &p) {
  return GainParams{p.min_leaf_size, p.min_child_weight, p.gamma_absolute, p.gamma_relative,
                    p.lambda,        p.alpha,            p.max_leaf_weight};
}

// IntoInternal, src/core/objective.h:20,55-57
static float into_internal(int objective, float v) {
  if (objective == 1) return std::log(v / (1 - v));
  return v;
}

// ------------------------------------------------------------ objectives
// src/core/objective.cu:28-56 (squared, logistic); softmax after the
// commented formula at objective.cu:60-89.
static void update_grad(Booster &b) {
  const int64_t n = b.n;
  const int K = b.p.labels_count;
  b.g.resize((size_t)n * K);
  b.h.resize((size_t)n * K);
  if (b.p.objective == 0) {
    for (int64_t i = 0; i < n; ++i) {
      b.g[i] = b.y[i] - b.yhat[i];
      b.h[i] = 1.0f;
    }
  } else if (b.p.objective == 1) {
    for (int64_t i = 0; i < n; ++i) {
      float s = sigmoid_f(b.yhat[i]);
      b.g[i] = b.y[i] - s;
      b.h[i] = s * (1.0f - s);
    }
  } else {
    std::vector<double> pr(K);
    for (int64_t i = 0; i < n; ++i) {
      double mx = -1e300, sum = 0;
      for (int k = 0; k < K; ++k) mx = std::max(mx, (double)b.yhat[i + (size_t)k * n]);
      for (int k = 0; k < K; ++k) {
        pr[k] = (double)orc_expf_impl((float)((double)b.yhat[i + (size_t)k * n] - mx));
        sum += pr[k];
      }
      for (int k = 0; k < K; ++k) {
        float pk = (float)(pr[k] / sum);
        float ind = (b.labels[i] == k) ? 1.0f : 0.0f;
        b.g[i + (size_t)k * n] = ind - pk;
        b.h[i + (size_t)k * n] = 2.0f * pk * (1.0f - pk);
      }
    }
  }
}

template <typename S>
static inline void acc_native(Acc &a, float g, float h) {
  a.g = (double)(S)((S)a.g + (S)g);
  a.h = (double)(S)((S)a.h + (S)h);
}

static inline void acc_add(Acc &a, const Booster &b, float g, float h, int64_t gq, int64_t hq) {
  if (b.p.accum == 0) {
    a.gq += gq;
    a.hq += hq;
  } else if (b.p.double_precision) {
    acc_native<double>(a, g, h);
  } else {
    acc_native<float>(a, g, h);
  }
  a.c += 1;
}

// value of an accumulator in the reference's SUM_T, widened to double
static inline void acc_value(const Booster &b, const Acc &a, double &g, double &h) {
  if (b.p.accum == 0) {
    g = from_fixed(a.gq, b.shift_g);
    h = from_fixed(a.hq, b.shift_h);
    if (!b.p.double_precision) {
      g = (double)(float)g;
      h = (double)(float)h;
    }
  } else {
    g = a.g;
    h = a.h;
  }
}

static inline Acc acc_sub(const Booster &b, const Acc &p, const Acc &s) {
  // sibling = parent - smaller child, src/core/hist_grad_sum.cu:6-33
  Acc r;
  r.gq = p.gq - s.gq;
  r.hq = p.hq - s.hq;
  r.c = p.c - s.c;
  if (b.p.double_precision) {
    r.g = p.g - s.g;
    r.h = p.h - s.h;
  } else {
    r.g = (double)((float)p.g - (float)s.g);
    r.h = (double)((float)p.h - (float)s.h);
  }
  return r;
}

// One tree.  src/core/garden.cu:167-197 (level loop), :419-445 (node totals),
// src/core/hist_tree_grower.cu:9-35 (gain scan), :37-102 (candidate choice,
// no-split and empty-node rules), src/core/builder.h:39-49 (tie rule: highest
// bin), :107-123 (bin >= q+1 goes right), src/core/garden.cu:447-503 (node
// records, leaf weights), :45-76 (prediction update).
static void grow_tree(Booster &b, int label) {
  const int64_t n = b.n;
  const int F = b.F, B = b.p.hist_size, SL = b.slots, D = b.p.depth;
  const float *g = b.g.data() + (size_t)label * n;
  const float *h = b.h.data() + (size_t)label * n;
  const GainParams gp = gain_params(b.p);
  const int kind = b.kind();
  const bool pair = b.p.objective != 0;

  if (b.p.objective == 0) {
    float gmax = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
      float a = std::fabs(g[i]);
      if (a > gmax) gmax = a;
    }
    b.shift_g = fix_shift_from_max(gmax);
    b.shift_h = 0;
  } else if (b.p.objective == 1) {
    // g = y - s, 0 <= s <= 1: |g| <= max(|ymin - 1|, |ymax|); 1 for labels in [0, 1]
    float ymin = 0.0f, ymax = 1.0f;
    for (int64_t i = 0; i < n; ++i) {
      ymin = std::min(ymin, b.y[i]);
      ymax = std::max(ymax, b.y[i]);
    }
    const float bound = std::max(std::fabs(ymin - 1.0f), std::fabs(ymax));
    b.shift_g = bound <= 1.0f ? 30 : fix_shift_from_max(bound);
    b.shift_h = 32;
  } else {
    b.shift_g = 30;
    b.shift_h = 31;
  }
  std::vector<int64_t> gq(n), hq(n);
  for (int64_t i = 0; i < n; ++i) {
    gq[i] = to_fixed(g[i], b.shift_g);
    hq[i] = pair ? to_fixed(h[i], b.shift_h) : 0;
  }

  TreeOut t;
  t.depth = D;
  t.label = label;
  const int n_internal = (1 << (D - 1)) - 1;
  t.fid.assign(n_internal, 0);
  t.quantized.assign(n_internal, -1);
  t.threshold.assign(n_internal, std::numeric_limits<float>::infinity());
  t.gain.assign(n_internal, 0.0f);
  t.weights.assign((size_t)1 << (D - 1), 0.0f);

  // column sampling: InitGrowingTree (garden.cu:142-146) shuffles all ids once
  // per tree, InitTreeLevel (:162-165) reshuffles the first
  // int(colsample_bytree * columns) per level, and FindBestSplits (:252-253,
  // 309-310) takes the first unsigned(bylevel * bytree * columns) as active.
  // With both ratios 1.0 every feature is active.
  b.active_log.emplace_back();
  std::vector<unsigned> active_fids(F);
  for (int f = 0; f < F; ++f) active_fids[f] = f;
  std::shuffle(active_fids.begin(), active_fids.end(), b.rnd);
  const int take_tree = (int)(b.p.colsample_bytree * (size_t)F);
  const unsigned take_level = (unsigned)(b.p.colsample_bylevel * b.p.colsample_bytree * (size_t)F);

  std::vector<uint32_t> node(n, 0);
  b.lvl_hist.assign(D - 1, {});
  b.lvl_tot.assign(D - 1, {});

  // root totals (garden.cu:426-439)
  std::vector<Acc> tot(1);
  for (int64_t i = 0; i < n; ++i) acc_add(tot[0], b, g[i], pair ? h[i] : 0.0f, gq[i], hq[i]);

  struct Best {
    float gain = 0;
    int fid = -1;
    int bin = -1;
    Acc left;
  };
  std::vector<Best> best;

  for (int level = 0; level + 1 < D; ++level) {
    const int L = 1 << level;
    std::shuffle(active_fids.begin(), active_fids.begin() + take_tree, b.rnd);
    std::vector<uint8_t> is_active(F, 0);
    for (unsigned j = 0; j < take_level && j < (unsigned)F; ++j) is_active[active_fids[j]] = 1;
    b.active_log.back().emplace_back(active_fids.begin(),
                                     active_fids.begin() + std::min<unsigned>(take_level, (unsigned)F));
    std::vector<Acc> &hist = b.lvl_hist[level];
    hist.assign((size_t)L * F * SL, Acc());
    b.lvl_tot[level] = tot;

    // which nodes are accumulated directly: with the trick only the smaller
    // child of each sibling pair, ties -> left (hist_grad_sum.cu:279-294),
    // valid when the parent level's histogram exists (histogram.cu:46-50).
    const bool trick = b.p.use_trick && level > 0;
    std::vector<uint8_t> direct(L, 1);
    if (trick) {
      for (int nd = 0; nd < L; nd += 2) {
        bool left_small = tot[nd].c <= tot[nd + 1].c;
        direct[nd] = left_small;
        direct[nd + 1] = !left_small;
      }
    }
    uint64_t scanned = 0;
#ifdef _OPENMP
    int nth = b.p.threads > 0 ? b.p.threads : omp_get_max_threads();
#else
    int nth = 1;
#endif
    if (b.p.accum != 0) nth = 1;  // native mode is sequential by definition
    if (nth <= 1) {
      for (int64_t i = 0; i < n; ++i) {
        uint32_t nd = node[i];
        if (!direct[nd]) continue;
        ++scanned;
        Acc *hn = &hist[(size_t)nd * F * SL];
        if (b.wide_bins.empty()) {
          const uint16_t *br = &b.bins[(size_t)i * F];
          for (int f = 0; f < F; ++f) acc_add(hn[(size_t)f * SL + br[f]], b, g[i], pair ? h[i] : 0.0f, gq[i], hq[i]);
        } else {
          const uint32_t *br = &b.wide_bins[(size_t)i * F];
          for (int f = 0; f < F; ++f) acc_add(hn[(size_t)f * SL + br[f]], b, g[i], pair ? h[i] : 0.0f, gq[i], hq[i]);
        }
      }
    } else {
#ifdef _OPENMP
      // integer sums are order independent: one private histogram per thread
      std::vector<std::vector<int64_t>> priv(nth);
#pragma omp parallel num_threads(nth) reduction(+ : scanned)
      {
        int tid = omp_get_thread_num();
        std::vector<int64_t> &pv = priv[tid];
        pv.assign((size_t)L * F * SL * 3, 0);
#pragma omp for schedule(static)
        for (int64_t i = 0; i < n; ++i) {
          uint32_t nd = node[i];
          if (!direct[nd]) continue;
          ++scanned;
          int64_t *hn = &pv[(size_t)nd * F * SL * 3];
          for (int f = 0; f < F; ++f) {
            int64_t *c = hn + ((size_t)f * SL + b.bin_at((size_t)i, f)) * 3;
            c[0] += gq[i];
            c[1] += hq[i];
            c[2] += 1;
          }
        }
      }
      for (int tI = 0; tI < nth; ++tI)
        for (size_t k = 0; k < hist.size(); ++k) {
          hist[k].gq += priv[tI][k * 3];
          hist[k].hq += priv[tI][k * 3 + 1];
          hist[k].c += (uint64_t)priv[tI][k * 3 + 2];
        }
#endif
    }
    b.updates += scanned * (uint64_t)F;
    if (trick) {
      const std::vector<Acc> &ph = b.lvl_hist[level - 1];
      for (int nd = 0; nd < L; ++nd) {
        if (direct[nd]) continue;
        int sib = nd ^ 1, par = nd >> 1;
        for (size_t k = 0; k < (size_t)F * SL; ++k)
          hist[(size_t)nd * F * SL + k] =
              acc_sub(b, ph[(size_t)par * F * SL + k], hist[(size_t)sib * F * SL + k]);
      }
    }

    // split scan
    best.assign(L, Best());
    for (int nd = 0; nd < L; ++nd) {
      if (tot[nd].c == 0) continue;
      double GT, HT;
      acc_value(b, tot[nd], GT, HT);
      for (int f = 0; f < F; ++f) {
        if (!is_active[f]) continue;
        const Acc *hf = &hist[((size_t)nd * F + f) * SL];
        Acc run;
        float cg = 0.0f;
        int cb = -1;
        Acc cl;
        for (int bin = 0; bin < B; ++bin) {
          run.gq += hf[bin].gq;
          run.hq += hf[bin].hq;
          run.c += hf[bin].c;
          if (b.p.double_precision) {
            run.g += hf[bin].g;
            run.h += hf[bin].h;
          } else {
            run.g = (double)((float)run.g + (float)hf[bin].g);
            run.h = (double)((float)run.h + (float)hf[bin].h);
          }
          double GL, HL;
          acc_value(b, run, GL, HL);
          float gn = gain_any(kind, GL, HL, run.c, GT, HT, tot[nd].c, gp);
          // hist_tree_grower.cu:31 (gain > 0) and builder.h:45-46 (>= keeps the
          // later, i.e. higher, bin on equal gain)
          if (gn > 0.0f && gn >= cg) {
            cg = gn;
            cb = bin;
            cl = run;
          }
        }
        // hist_tree_grower.cu:59-60: higher gain, or equal gain and lower fid
        if (cb >= 0 && (best[nd].gain < cg || (best[nd].gain == cg && f < best[nd].fid))) {
          best[nd].gain = cg;
          best[nd].fid = f;
          best[nd].bin = cb;
          best[nd].left = cl;
        }
      }
    }

    // node records (garden.cu:447-485) and children totals
    std::vector<Acc> next((size_t)L * 2);
    const int off = (1 << level) - 1;
    for (int nd = 0; nd < L; ++nd) {
      Best &bs = best[nd];
      if (bs.fid < 0) {  // no split or empty node: everything stays left
        bs.left = tot[nd];
        t.fid[off + nd] = 0;
        t.quantized[off + nd] = -1;
        t.threshold[off + nd] = std::numeric_limits<float>::infinity();
      } else {
        t.fid[off + nd] = bs.fid;
        t.quantized[off + nd] = bs.bin;
        t.gain[off + nd] = bs.gain;
        t.threshold[off + nd] = bs.bin >= (int)b.thr[bs.fid].size()
                                    ? std::numeric_limits<float>::infinity()
                                    : b.thr[bs.fid][bs.bin];
      }
      next[2 * nd] = bs.left;
      next[2 * nd + 1] = acc_sub(b, tot[nd], bs.left);
    }
    // apply (builder.h:107-123): bin >= q+1 -> right
    for (int64_t i = 0; i < n; ++i) {
      uint32_t nd = node[i];
      const Best &bs = best[nd];
      uint32_t right = 0;
      if (bs.fid >= 0) right = b.bin_at((size_t)i, bs.fid) >= (unsigned)(bs.bin + 1);
      node[i] = nd * 2 + right;
    }
    tot.swap(next);
  }

  // leaves (garden.cu:487-503, split.cu:25-35): Weight(sum,count) * eta
  const int NL = 1 << (D - 1);
  for (int l = 0; l < NL; ++l) {
    double G, H;
    acc_value(b, tot[l], G, H);
    if (b.p.accum == 0 && (l & 1)) {
      // right child = parent - left in SUM_T (split.cu:31-35)
      Acc par;
      par.gq = tot[l].gq + tot[l - 1].gq;
      par.hq = tot[l].hq + tot[l - 1].hq;
      double GP, HP, GLf, HLf;
      acc_value(b, par, GP, HP);
      acc_value(b, tot[l - 1], GLf, HLf);
      if (b.p.double_precision) {
        G = GP - GLf;
        H = HP - HLf;
      } else {
        G = (double)((float)GP - (float)GLf);
        H = (double)((float)HP - (float)HLf);
      }
    }
    t.weights[l] = weight_any(kind, G, H, (unsigned)tot[l].c, gp) * b.p.eta;
  }
  // prediction update (garden.cu:45-76)
  b.leaf.assign(node.begin(), node.end());
  float *yh = b.yhat.data() + (size_t)label * n;
  for (int64_t i = 0; i < n; ++i) yh[i] += t.weights[node[i]];
  b.trees.push_back(std::move(t));
}

// RegTree::Predict, src/core/garden.h:70-90: x < threshold -> left (NaN -> right)
static void tree_predict(const TreeOut &t, const float *X, int64_t n, int F, float *out) {
  const int off = (1 << (t.depth - 1)) - 1;
  for (int64_t i = 0; i < n; ++i) {
    unsigned id = 0;
    for (int j = 1; j < t.depth; ++j) {
      bool left = X[(size_t)i * F + t.fid[id]] < t.threshold[id];
      id = left ? 2 * id + 1 : 2 * id + 2;
    }
    out[i + (size_t)t.label * n] += t.weights[id - off];
  }
}

}  // namespace

// ============================================================== C interface
static bool g_force_wide_ranks = false;

extern "C" {

float orc_expf(float x) { return orc_expf_impl(x); }
float orc_sigmoid(float x) { return sigmoid_f(x); }

// Quantise one column.  thr: hist_size floats; bins: n uint16.  Returns size.
int orc_quantize_column(const float *x, int64_t n, int hist_size, float *thr, uint16_t *bins) {
  QuantResult q = quantize_thresholds(x, n, hist_size);
  std::memcpy(thr, q.thr.data(), sizeof(float) * hist_size);
  if (bins)
    for (int64_t i = 0; i < n; ++i) bins[i] = (uint16_t)bin_of(q.thr.data(), q.size, x[i]);
  return q.size;
}

float orc_gain(int kind, double gl, double hl, uint64_t cl, double gt, double ht, uint64_t ct,
               unsigned min_leaf_size, float mcw, float gamma_abs, float gamma_rel, float lambda,
               float alpha, float max_leaf_weight) {
  GainParams p{min_leaf_size, mcw, gamma_abs, gamma_rel, lambda, alpha, max_leaf_weight};
  return gain_any(kind, gl, hl, cl, gt, ht, ct, p);
}

float orc_weight(int kind, double g, double h, unsigned c, unsigned min_leaf_size, float mcw,
                 float lambda, float alpha, float max_leaf_weight) {
  GainParams p{min_leaf_size, mcw, 0, 0, lambda, alpha, max_leaf_weight};
  return weight_any(kind, g, h, c, p);
}

int orc_fix_shift(float vmax) { return fix_shift_from_max(vmax); }
int64_t orc_to_fixed(float v, int shift) { return to_fixed(v, shift); }

// Fixed-point histogram of one row set: bins row-major [n][F] uint8, rows
// selected by sel (NULL = all).  out: F*256 cells of (gq, hq, count) int64.
void orc_hist_fixed_u8(const uint8_t *bins, int64_t n, int F, int stride, const float *g,
                       const float *h, int shift_g, int shift_h, const uint8_t *sel,
                       int64_t *out) {
  std::memset(out, 0, sizeof(int64_t) * 3 * F * 256);
  for (int64_t i = 0; i < n; ++i) {
    if (sel && !sel[i]) continue;
    int64_t gq = to_fixed(g[i], shift_g);
    int64_t hq = h ? to_fixed(h[i], shift_h) : 0;
    for (int f = 0; f < F; ++f) {
      int64_t *c = out + ((size_t)f * 256 + bins[(size_t)i * stride + f]) * 3;
      c[0] += gq;
      c[1] += hq;
      c[2] += 1;
    }
  }
}

void *orc_create(const float *X, int64_t n, int F, const float *y, const uint8_t *labels,
                 const OrcParams *p) {
  Booster *b = new Booster();
  b->p = *p;
  b->n = n;
  b->F = F;
  b->slots = p->hist_size + 1;
  b->X.assign(X, X + (size_t)n * F);
  if (y) b->y.assign(y, y + n);
  if (labels) b->labels.assign(labels, labels + n);
  b->thr.resize(F);
  b->size.resize(F);
  b->bins.resize((size_t)n * F);
  if (p->method == 0) {
    // Exact method.  DataMatrix::InitExact (src/io/io.cu:437-482): every value is replaced by its
    // rank among the column's sorted distinct values (`data_reduced_mapping`).  The grower
    // (src/core/continuous_tree_grower.cu:9-49) sorts each node's rows by rank, takes the
    // exclusive prefix sum of the gradients and evaluates gain_func at every position i where the
    // rank changes (left = the rows before i), keeping the best gain and, on equal gains, the
    // highest position (updateAtomicMax packs (gain, i)); the split value is the rank r at that
    // position, rows with rank >= r go right (builder.h:107-123) and the node's threshold is
    // mapping[r] (garden.cu:463-467).  Left of position i are exactly the rows of rank < r, so
    // the candidates are the prefixes of a histogram over ranks: slot q = r - 1 with "bins <= q
    // left", ties to the highest slot.  That is the histogram scan below with one slot per
    // distinct value and thresholds thr[q] = mapping[q + 1].
    std::vector<std::vector<float>> mapping(F);
    size_t most = 1;
    for (int f = 0; f < F; ++f) {
      std::vector<float> &m = mapping[f];
      m.resize(n);
      for (int64_t i = 0; i < n; ++i) m[i] = X[(size_t)i * F + f];
      std::sort(m.begin(), m.end());
      m.erase(std::unique(m.begin(), m.end()), m.end());
      most = std::max(most, m.size());
    }
    if (most > 65535 || g_force_wide_ranks) {  // ranks beyond 16 bits
      b->bins.clear();
      b->wide_bins.resize((size_t)n * F);
    }
    for (int f = 0; f < F; ++f) {
      const std::vector<float> &m = mapping[f];
      for (int64_t i = 0; i < n; ++i) {
        const size_t r = std::lower_bound(m.begin(), m.end(), X[(size_t)i * F + f]) - m.begin();
        if (b->wide_bins.empty())
          b->bins[(size_t)i * F + f] = (uint16_t)r;
        else
          b->wide_bins[(size_t)i * F + f] = (uint32_t)r;
      }
    }
    b->p.hist_size = (int)most;
    b->slots = (int)most + 1;
    for (int f = 0; f < F; ++f) {
      b->size[f] = (int)mapping[f].size();
      b->thr[f].assign(most, std::numeric_limits<float>::infinity());
      for (size_t k = 0; k + 1 < mapping[f].size(); ++k) b->thr[f][k] = mapping[f][k + 1];
    }
    b->yhat.assign((size_t)n * p->labels_count, into_internal(p->objective, p->initial_y));
    b->rnd.seed(p->seed);
    return b;
  }
  // the columns are independent (io.cu:349-435 handles them one after the other)
#pragma omp parallel for schedule(dynamic, 1) num_threads(p->threads > 0 ? p->threads : omp_get_max_threads())
  for (int f = 0; f < F; ++f) {
    std::vector<float> col(n);
    for (int64_t i = 0; i < n; ++i) col[i] = X[(size_t)i * F + f];
    QuantResult q = quantize_thresholds(col.data(), n, p->hist_size);
    b->thr[f] = q.thr;
    b->size[f] = q.size;
    for (int64_t i = 0; i < n; ++i)
      b->bins[(size_t)i * F + f] = (uint16_t)bin_of(q.thr.data(), q.size, col[i]);
  }
  b->yhat.assign((size_t)n * p->labels_count, into_internal(p->objective, p->initial_y));
  b->rnd.seed(p->seed);
  return b;
}

// Pre-quantised input (bins row-major uint8 [n][F]); thresholds are bin ids.
void *orc_create_binned(const uint8_t *bins, int64_t n, int F, const float *y,
                        const uint8_t *labels, const OrcParams *p) {
  Booster *b = new Booster();
  b->p = *p;
  b->n = n;
  b->F = F;
  b->slots = p->hist_size + 1;
  if (y) b->y.assign(y, y + n);
  if (labels) b->labels.assign(labels, labels + n);
  b->thr.assign(F, std::vector<float>(p->hist_size));
  b->size.assign(F, p->hist_size);
  for (int f = 0; f < F; ++f)
    for (int k = 0; k < p->hist_size; ++k) b->thr[f][k] = (float)k + 0.5f;
  b->bins.resize((size_t)n * F);
  for (size_t k = 0; k < (size_t)n * F; ++k) b->bins[k] = bins[k];
  b->yhat.assign((size_t)n * p->labels_count, into_internal(p->objective, p->initial_y));
  b->rnd.seed(p->seed);
  return b;
}

void orc_free(void *h) { delete static_cast<Booster *>(h); }

// One boosting round = labels_count trees (garden.cu:585-625).  Returns NULL,
// or the message InitGrowingTree throws before anything is drawn
// (garden.cu:127-140): the round then grows nothing.
const char *orc_grow_round(void *hd) {
  Booster &b = *static_cast<Booster *>(hd);
  if ((int)(b.p.colsample_bytree * (size_t)b.F) == 0) return "colsample_bytree is too small";
  if ((int)(b.p.colsample_bytree * b.p.colsample_bylevel * (size_t)b.F) == 0)
    return "colsample_bytree and colsample_bylevel are too small";
  update_grad(b);
  for (int k = 0; k < b.p.labels_count; ++k) grow_tree(b, k);
  return nullptr;
}

// Ids of the features that tree `t` may split on at `level`, in the order they
// stand in the shuffled list.  Returns their number, -1 for a bad index.
int orc_get_active(void *hd, int t, int level, unsigned *out) {
  Booster &b = *static_cast<Booster *>(hd);
  if (t < 0 || t >= (int)b.active_log.size() || level < 0 || level >= (int)b.active_log[t].size())
    return -1;
  const std::vector<unsigned> &a = b.active_log[t][level];
  if (out) std::memcpy(out, a.data(), a.size() * sizeof(unsigned));
  return (int)a.size();
}

// Test switch: exact-mode boosters created from now on keep their ranks in 32 bits whatever the
// number of distinct values (the branch that more than 65535 distinct values take).
void orc_force_wide_ranks(int on) { g_force_wide_ranks = on != 0; }
int orc_hist_size(void *hd) { return static_cast<Booster *>(hd)->p.hist_size; }  // exact: distinct values
int orc_num_trees(void *hd) { return (int)static_cast<Booster *>(hd)->trees.size(); }
uint64_t orc_updates(void *hd) { return static_cast<Booster *>(hd)->updates; }

void orc_get_tree(void *hd, int t, int *fid, int *quantized, float *threshold, float *gain,
                  float *weights) {
  const TreeOut &tr = static_cast<Booster *>(hd)->trees[t];
  size_t ni = tr.fid.size();
  if (fid) std::memcpy(fid, tr.fid.data(), ni * sizeof(int));
  if (quantized) std::memcpy(quantized, tr.quantized.data(), ni * sizeof(int));
  if (threshold) std::memcpy(threshold, tr.threshold.data(), ni * sizeof(float));
  if (gain) std::memcpy(gain, tr.gain.data(), ni * sizeof(float));
  if (weights) std::memcpy(weights, tr.weights.data(), tr.weights.size() * sizeof(float));
}

void orc_get_leaf(void *hd, uint32_t *out) {
  Booster &b = *static_cast<Booster *>(hd);
  std::memcpy(out, b.leaf.data(), b.leaf.size() * sizeof(uint32_t));
}
void orc_get_yhat(void *hd, float *out) {
  Booster &b = *static_cast<Booster *>(hd);
  std::memcpy(out, b.yhat.data(), b.yhat.size() * sizeof(float));
}
void orc_get_grad(void *hd, float *g, float *h) {
  Booster &b = *static_cast<Booster *>(hd);
  std::memcpy(g, b.g.data(), b.g.size() * sizeof(float));
  if (h) std::memcpy(h, b.h.data(), b.h.size() * sizeof(float));
}
void orc_get_bins(void *hd, uint16_t *out) {  // (ranks beyond 16 bits are not handed out: nothing is written)
  Booster &b = *static_cast<Booster *>(hd);
  std::memcpy(out, b.bins.data(), b.bins.size() * sizeof(uint16_t));
}
void orc_get_thresholds(void *hd, int f, float *thr, int *size) {
  Booster &b = *static_cast<Booster *>(hd);
  std::memcpy(thr, b.thr[f].data(), b.thr[f].size() * sizeof(float));
  *size = b.size[f];
}
void orc_get_shifts(void *hd, int *sg, int *sh) {
  Booster &b = *static_cast<Booster *>(hd);
  *sg = b.shift_g;
  *sh = b.shift_h;
}

// Histogram of one level of the last tree.  mode 0: fixed-point integers
// (gq, hq, count) as int64 triples; mode 1: values in SUM_T as doubles
// (g, h, count).  Layout [node][feature][slot], slot count = hist_size + 1.
int orc_get_level_hist(void *hd, int level, int mode, void *out) {
  Booster &b = *static_cast<Booster *>(hd);
  if (level < 0 || level >= (int)b.lvl_hist.size()) return -1;
  const std::vector<Acc> &hs = b.lvl_hist[level];
  for (size_t k = 0; k < hs.size(); ++k) {
    if (mode == 0) {
      int64_t *o = static_cast<int64_t *>(out) + k * 3;
      o[0] = hs[k].gq;
      o[1] = hs[k].hq;
      o[2] = (int64_t)hs[k].c;
    } else {
      double *o = static_cast<double *>(out) + k * 3;
      acc_value(b, hs[k], o[0], o[1]);
      o[2] = (double)hs[k].c;
    }
  }
  return (int)hs.size();
}

// Garden::Predict, src/core/garden.cu:643-657, objective.h FromInternal.
void orc_predict(void *hd, const float *X, int64_t n, int n_rounds, float *out) {
  Booster &b = *static_cast<Booster *>(hd);
  const int K = b.p.labels_count;
  std::vector<float> tmp((size_t)n * K, into_internal(b.p.objective, b.p.initial_y));
  int use = (int)std::min<int64_t>(n_rounds < 0 ? INT32_MAX : n_rounds, (int64_t)b.trees.size());
  for (int t = 0; t < use; ++t) tree_predict(b.trees[t], X, n, b.F, tmp.data());
  if (b.p.objective == 0) {
    std::memcpy(out, tmp.data(), tmp.size() * sizeof(float));
  } else if (b.p.objective == 1) {
    for (size_t i = 0; i < tmp.size(); ++i)
      out[i] = (float)(1.0 / (1.0 + (double)std::exp(-tmp[i])));  // objective.h:67-69 (host)
  } else {
    for (int64_t i = 0; i < n; ++i) {  // objective.h:80-113
      std::vector<double> v(K);
      double s = 0;
      for (int k = 0; k < K; ++k) {
        v[k] = std::exp((double)tmp[i + (size_t)k * n]);
        s += v[k];
      }
      for (int k = 0; k < K; ++k) out[(size_t)i * K + k] = (float)(v[k] / s);
    }
  }
}

}  // extern "C"
