// Gradients of the objectives, root initialisation.
#ifndef ARBORETUM_AMD_KERNELS_OBJECTIVE_H_
#define ARBORETUM_AMD_KERNELS_OBJECTIVE_H_
#include "device_common.h"

namespace arb {
namespace {

// ------------------------------------------------------------- objectives

// squared error: g = y - y_hat (objective.cu:28-38); also max |g| for the
// fixed-point scale
__global__ void k_grad_squared(const float *__restrict__ y, const float *__restrict__ yhat,
                               float *__restrict__ g, size_t n, unsigned *__restrict__ gmax_bits) {
  float m = 0.0f;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const float v = y[i] - yhat[i];
    g[i] = v;
    const float a = fabsf(v);
    if (a > m) m = a;  // NaN never raises the maximum
  }
  m = WaveMaxF(m);
  if ((threadIdx.x & 63) == 0) atomicMax(gmax_bits, __float_as_uint(m));
}

__global__ void k_set_shift(const unsigned *__restrict__ gmax_bits, int *__restrict__ shifts) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    shifts[0] = FixShiftFromMax(__uint_as_float(*gmax_bits));
    shifts[1] = 0;
  }
}

// logistic: s = sigmoid(y_hat), g = y - s, h = s(1-s) (objective.cu:43-56);
// h == nullptr: packed into g (PackGrad)
__global__ void k_grad_logistic(const float *__restrict__ y, const float *__restrict__ yhat,
                                float *__restrict__ g, float *__restrict__ h, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const float s = SigmoidF(yhat[i]);
    if (h != nullptr) {
      g[i] = y[i] - s;
      h[i] = s * (1.0f - s);
    } else {  // 0/1 labels: one float per row
      g[i] = PackGrad(s, y[i]);
    }
  }
}

// soft-max: p = softmax(y_hat[., row]), g_k = [label == k] - p_k,
// h_k = 2 p_k (1 - p_k) (formula in the comment at objective.cu:60-89).
// y_hat, g, h are class-major [K][n].
__global__ void k_grad_softmax(const uint8_t *__restrict__ labels, const float *__restrict__ yhat,
                               float *__restrict__ g, float *__restrict__ h, size_t n, int K) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    double mx = -1e300;
    for (int k = 0; k < K; ++k) mx = fmax(mx, (double)yhat[i + (size_t)k * n]);
    double sum = 0.0;
    for (int k = 0; k < K; ++k) sum += (double)ExpF((float)((double)yhat[i + (size_t)k * n] - mx));
    const int lab = labels[i];
    for (int k = 0; k < K; ++k) {
      const double e = (double)ExpF((float)((double)yhat[i + (size_t)k * n] - mx));
      const float pk = (float)(e / sum);
      g[i + (size_t)k * n] = (lab == k ? 1.0f : 0.0f) - pk;
      h[i + (size_t)k * n] = 2.0f * pk * (1.0f - pk);
    }
  }
}


}  // namespace
}  // namespace arb
#endif  // ARBORETUM_AMD_KERNELS_OBJECTIVE_H_
