// Split gain, leaf weight and fixed-point helpers shared by host and device
// code.  Arithmetic types follow the reference exactly (src/core/gain.cu:8-238)
// because the chosen (feature, bin) must match bit for bit:
//   * literals 0.5 and 0.0 are double, so the quadratic term and the final
//     product are evaluated in double and rounded once to float;
//   * weights are float, divisions are float for the fp32 sum types and
//     double for the fp64 ones;
//   * no fused multiply-add may be formed (compile with -ffp-contract=off).
#ifndef ARBORETUM_AMD_GAIN_H_
#define ARBORETUM_AMD_GAIN_H_

#include <cmath>
#include <cstdint>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define ARB_HD __host__ __device__ __forceinline__
#else
#define ARB_HD inline
#endif

namespace arb {

// src/core/gain.cuh:11-30
struct GainParams {
  unsigned min_leaf_size;
  float min_child_weight;
  float gamma_absolute;
  float gamma_relative;
  float lambda;
  float alpha;
  float max_leaf_weight;
};

// Sum kinds = the reference's four (GRAD_T, SUM_T) instantiations
// (src/core/garden.cu:538-563): count-as-hessian fp32/fp64, (g,h) fp32/fp64.
enum SumKind { kCntF32 = 0, kCntF64 = 1, kPairF32 = 2, kPairF64 = 3 };

// ----------------------------------------------------------- fixed point
// Every gradient is rounded once to q = rint(v * 2^shift), |q| <= 2^30, and
// histograms add the integers, so sums do not depend on the order of addition.
//   shift = 30 - e with |v| <= 2^e for all rows.
ARB_HD int FixShiftFromMax(float vmax) {
  if (!(vmax > 0.0f) || vmax > 3.4028234663852886e38f) return 30;  // zero, NaN or Inf
  int e;
  (void)frexpf(vmax, &e);  // vmax = m * 2^e, 1/2 <= m < 1
  return 30 - e;
}

// Logistic gradients g = y - s with 0 <= s <= 1 lie in [ymin - 1, ymax] (float
// subtraction is monotonic, so the bounds hold for the rounded values too).
// Labels in [0, 1] give |g| <= 1 and shift 30; any other finite labels get
// the shift of their own bound.
ARB_HD int LogisticGradShift(float ymin, float ymax) {
  const float bound = fmaxf(fabsf(ymin - 1.0f), fabsf(ymax));
  return bound <= 1.0f ? 30 : FixShiftFromMax(bound);
}

ARB_HD long long ToFixed(float v, int shift) {
  // Scaling by a power of two is exact in fp32, and so is rounding the result
  // to an integer (at or above 2^23 it is one already): the value is
  // rint(v * 2^shift) of the real numbers, with no double arithmetic.  A
  // result below the normal range rounds to 0 either way.
  const float s = ldexpf(v, shift);
  if (!(fabsf(s) <= 1073741824.0f)) return 0;  // NaN, Inf or out of range
  return (long long)(int)rintf(s);  // |s| <= 2^30 fits 32 bits
}

// Integer sum -> value in the sum type (float results are float-representable).
template <bool F64>
ARB_HD double FromFixed(long long q, int shift) {
  double v = ldexp((double)q, -shift);
  return F64 ? v : (double)(float)v;
}

// ------------------------------------------------------------- weights
ARB_HD float ClampWeight(float w, float mlw) {  // gain.cu:25-32
  if (mlw != 0.0f) {
    if (w > mlw) return mlw;
    if (w < -mlw) return -mlw;
  }
  return w;
}

// sign(g) * max(0.0, |g| - alpha): gain.cu:19-23
ARB_HD float ShrinkF(float g, float alpha) {
  float d = fabsf(g) - alpha;
  double m = (double)d > 0.0 ? (double)d : 0.0;
  int s = (0.0f < g) - (g < 0.0f);
  return (float)(s * m);
}
ARB_HD double ShrinkD(double g, float alpha) {
  double d = fabs(g) - (double)alpha;
  double m = d > 0.0 ? d : 0.0;
  int s = (0.0 < g) - (g < 0.0);
  return s * m;
}

// Weight(): gain.cu:34-76.  PAIR: hessian is h; else the row count.
// The count is 64 bits wide: a streamed matrix may hold more than 2^32 rows
// (the reference's counts are 32-bit, like its `int` row count).
template <bool PAIR, bool F64>
ARB_HD float LeafWeight(double g, double h, unsigned long long c, const GainParams &p) {
  float w = 0.0f;
  if (PAIR) {
    if (F64) {
      if (c >= p.min_leaf_size && h >= (double)p.min_child_weight)
        w = (float)(ShrinkD(g, p.alpha) / (h + (double)p.lambda));
    } else {
      float hf = (float)h;
      if (c >= p.min_leaf_size && hf >= p.min_child_weight)
        w = ShrinkF((float)g, p.alpha) / (hf + p.lambda);
    }
  } else {
    if (c >= p.min_leaf_size && (float)c >= p.min_child_weight) {
      float den = (float)c + p.lambda;
      if (F64)
        w = (float)(ShrinkD(g, p.alpha) / (double)den);
      else
        w = ShrinkF((float)g, p.alpha) / den;
    }
  }
  return ClampWeight(w, p.max_leaf_weight);
}

// gain(): gain.cu:13-17, -2 * (g*(-w) + 0.5*(h+lambda)*w*w + alpha*|w|)
template <bool PAIR, bool F64>
ARB_HD float SideGain(double g, double h, unsigned long long c, float w, const GainParams &p) {
  double first;   // grad * (-w) in the grad type
  double hl;      // hess + lambda in the hess type
  if (F64)
    first = g * (double)(-w);
  else
    first = (double)((float)g * (-w));
  if (PAIR) {
    if (F64)
      hl = h + (double)p.lambda;
    else
      hl = (double)((float)h + p.lambda);
  } else {
    hl = (double)((float)c + p.lambda);
  }
  double quad = 0.5 * hl * (double)w * (double)w;
  float l1 = p.alpha * fabsf(w);
  return (float)(-2 * ((first + quad) + (double)l1));
}

// gain_func(): gain.cu:124-238.  Sums come in as doubles holding values of
// the sum type; right = total - left is formed in the sum type.
template <bool PAIR, bool F64>
ARB_HD float SplitGain(double gl, double hl, unsigned long long cl, double gt, double ht,
                       unsigned long long ct, const GainParams &p) {
  const unsigned long long cr = ct - cl;
  double gr, hr;
  if (F64) {
    gr = gt - gl;
    hr = ht - hl;
  } else {
    gr = (double)((float)gt - (float)gl);
    hr = (double)((float)ht - (float)hl);
  }
  if (cl < p.min_leaf_size || cr < p.min_leaf_size) return 0.0f;
  if (PAIR) {
    if (F64) {
      if (!(fabs(hl) >= (double)p.min_child_weight && fabs(hr) >= (double)p.min_child_weight))
        return 0.0f;
    } else {
      if (!(fabsf((float)hl) >= p.min_child_weight && fabsf((float)hr) >= p.min_child_weight))
        return 0.0f;
    }
  }
  const float wl = LeafWeight<PAIR, F64>(gl, hl, cl, p);
  const float wr = LeafWeight<PAIR, F64>(gr, hr, cr, p);
  const float wp = LeafWeight<PAIR, F64>(gt, ht, ct, p);
  const float l = SideGain<PAIR, F64>(gl, hl, cl, wl, p);
  const float r = SideGain<PAIR, F64>(gr, hr, cr, wr, p);
  const float q = SideGain<PAIR, F64>(gt, ht, ct, wp, p);
  const float diff = l + r - q;
  return (float)(diff > p.gamma_absolute && diff > p.gamma_relative * q) * diff;
}

ARB_HD float SplitGainKind(int kind, double gl, double hl, unsigned long long cl, double gt,
                           double ht, unsigned long long ct, const GainParams &p) {
  switch (kind) {
    case kCntF32: return SplitGain<false, false>(gl, hl, cl, gt, ht, ct, p);
    case kCntF64: return SplitGain<false, true>(gl, hl, cl, gt, ht, ct, p);
    case kPairF32: return SplitGain<true, false>(gl, hl, cl, gt, ht, ct, p);
    default: return SplitGain<true, true>(gl, hl, cl, gt, ht, ct, p);
  }
}
ARB_HD float LeafWeightKind(int kind, double g, double h, unsigned long long c, const GainParams &p) {
  switch (kind) {
    case kCntF32: return LeafWeight<false, false>(g, h, c, p);
    case kCntF64: return LeafWeight<false, true>(g, h, c, p);
    case kPairF32: return LeafWeight<true, false>(g, h, c, p);
    default: return LeafWeight<true, true>(g, h, c, p);
  }
}

// ------------------------------------------------------------------ exp
// exp of a float evaluated in double with a fixed operation order (range
// reduction by ln2/32, 32-entry table, degree-7 polynomial) so that host and
// device give identical bits.  The table is an array in constant memory: a
// switch over its entries compiles, on the GPU, to a tree of divergent
// branches that costs several times the rest of the function.  The sigmoid
// follows src/core/objective.h:67-69: float exp, double 1/(1+e), rounded to
// float.

// 2^(j/32) rounded to double, j in [0, 32)
ARB_HD const double *Exp2Table() {
  static constexpr double kTable[32] = {
      0x1.0000000000000p+0, 0x1.059b0d3158574p+0, 0x1.0b5586cf9890fp+0, 0x1.11301d0125b51p+0,
      0x1.172b83c7d517bp+0, 0x1.1d4873168b9aap+0, 0x1.2387a6e756238p+0, 0x1.29e9df51fdee1p+0,
      0x1.306fe0a31b715p+0, 0x1.371a7373aa9cbp+0, 0x1.3dea64c123422p+0, 0x1.44e086061892dp+0,
      0x1.4bfdad5362a27p+0, 0x1.5342b569d4f82p+0, 0x1.5ab07dd485429p+0, 0x1.6247eb03a5585p+0,
      0x1.6a09e667f3bcdp+0, 0x1.71f75e8ec5f74p+0, 0x1.7a11473eb0187p+0, 0x1.82589994cce13p+0,
      0x1.8ace5422aa0dbp+0, 0x1.93737b0cdc5e5p+0, 0x1.9c49182a3f090p+0, 0x1.a5503b23e255dp+0,
      0x1.ae89f995ad3adp+0, 0x1.b7f76f2fb5e47p+0, 0x1.c199bdd85529cp+0, 0x1.cb720dcef9069p+0,
      0x1.d5818dcfba487p+0, 0x1.dfc97337b9b5fp+0, 0x1.ea4afa2a490dap+0, 0x1.f50765b6e4540p+0};
  return kTable;
}

// table: the 32 values of Exp2Table, wherever the caller keeps them
ARB_HD float ExpFrom(float xf, const double *table) {
  // Straight-line code: the polynomial runs on the clamped argument and the
  // special cases are selected at the end, so that the evaluations of several
  // rows of a GPU thread interleave (fmaxf drops a NaN: it is put back last).
  const float xc = fminf(fmaxf(xf, -104.0f), 88.8f);
  const double x = (double)xc;
  const double kd = rint(x * 0x1.71547652b82fep+5);   // 32 / ln 2
  const int k = (int)kd;
  const double r = x - kd * 0x1.62e42fefa39efp-6;     // ln 2 / 32
  double p = 1.0 / 5040.0;
  p = p * r + 1.0 / 720.0;
  p = p * r + 1.0 / 120.0;
  p = p * r + 1.0 / 24.0;
  p = p * r + 1.0 / 6.0;
  p = p * r + 0.5;
  p = p * r + 1.0;
  p = p * r + 1.0;
  const int j = k & 31;
  const int m = (k - j) / 32;
  float e = (float)ldexp(table[j] * p, m);
  e = xf > 88.8f ? INFINITY : e;
  e = xf < -104.0f ? 0.0f : e;
  return xf != xf ? xf : e;
}

ARB_HD float ExpF(float xf) { return ExpFrom(xf, Exp2Table()); }

ARB_HD float SigmoidF(float x) { return (float)(1.0 / (1.0 + (double)ExpF(-x))); }
// the same with the caller's copy of the table (a kernel that keeps it in LDS)
ARB_HD float SigmoidFrom(float x, const double *table) {
  return (float)(1.0 / (1.0 + (double)ExpFrom(-x, table)));
}

}  // namespace arb
#endif  // ARBORETUM_AMD_GAIN_H_
