// Bin assignment from thresholds, packing of pre-quantised input.
#ifndef ARBORETUM_AMD_KERNELS_QUANTISE_H_
#define ARBORETUM_AMD_KERNELS_QUANTISE_H_
#include "device_common.h"

namespace arb {
namespace {

// --------------------------------------------------------------- quantiser
// bin(x) = first l in [0,size] with x <= v[l], v[t] = thr[t] for t < size-1,
// +INF above (src/core/cuda_helpers.h:207-222, src/io/io.cu:297-302); NaN
// compares false everywhere and lands in bin `size`.
// An id of 256 (a feature of 256 value bins with missing values) is stored as
// byte 255 plus bit f0 + c of hi[r], the ninth-bit word of the row that holds
// the features of this launch (f0: the place in that word of column 0 of this
// launch); without `hi` no id may exceed 255.
__global__ void k_bin_assign(const float *__restrict__ x, int ncols, const float *__restrict__ thr,
                             int thr_stride, const int *__restrict__ sizes,
                             uint32_t *__restrict__ out, size_t n, uint32_t *__restrict__ hi, int f0) {
  __shared__ float s_thr[4][kSlots];
  __shared__ int s_size[4];
  for (int i = threadIdx.x; i < 4 * kSlots; i += blockDim.x) {
    const int c = i >> 8, t = i & 255;
    float v = INFINITY;
    if (c < ncols && t < sizes[c] - 1) v = thr[(size_t)c * thr_stride + t];
    s_thr[c][t] = v;
  }
  if (threadIdx.x < 4) s_size[threadIdx.x] = threadIdx.x < ncols ? sizes[threadIdx.x] : 0;
  __syncthreads();
  for (size_t r = (size_t)blockIdx.x * blockDim.x + threadIdx.x; r < n;
       r += (size_t)gridDim.x * blockDim.x) {
    uint32_t packed = 0, over = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (c < ncols) {
        const float v = x[(size_t)c * n + r];
        unsigned l = 0, h = (unsigned)s_size[c];
        while (l < h) {
          const unsigned mid = (l + h) >> 1;
          if (v <= s_thr[c][mid])
            h = mid;
          else
            l = mid + 1;
        }
        over |= (l > 255u ? 1u : 0u) << c;
        packed |= min(l, 255u) << (8 * c);
      }
    }
    out[r] = packed;
    if (hi != nullptr && over != 0u) hi[r] |= over << f0;  // launches of one matrix run one after the other
  }
}

// The same with 16-bit bins: two features per word, thresholds of both in
// dynamic LDS (2 * thr_stride floats).
__global__ void k_bin_assign_wide(const float *__restrict__ x, int ncols, const float *__restrict__ thr,
                                  int thr_stride, const int *__restrict__ sizes,
                                  uint32_t *__restrict__ out, size_t n) {
  extern __shared__ float s_thr_wide[];
  for (int i = threadIdx.x; i < 2 * thr_stride; i += blockDim.x) {
    const int c = i / thr_stride, t = i % thr_stride;
    float v = INFINITY;
    if (c < ncols && t < sizes[c] - 1) v = thr[(size_t)c * thr_stride + t];
    s_thr_wide[i] = v;
  }
  __syncthreads();
  for (size_t r = (size_t)blockIdx.x * blockDim.x + threadIdx.x; r < n;
       r += (size_t)gridDim.x * blockDim.x) {
    uint32_t packed = 0;
    for (int c = 0; c < ncols; ++c) {
      const float v = x[(size_t)c * n + r];
      unsigned l = 0, h = (unsigned)sizes[c];
      while (l < h) {
        const unsigned mid = (l + h) >> 1;
        if (v <= s_thr_wide[c * thr_stride + mid])
          h = mid;
        else
          l = mid + 1;
      }
      packed |= l << (16 * c);
    }
    out[r] = packed;
  }
}

// row-major uint8 [n][F] -> quads
__global__ void k_pack_prebinned(const uint8_t *__restrict__ in, int F, int Q,
                                 uint32_t *__restrict__ out, size_t stride, size_t n) {
  for (size_t r = (size_t)blockIdx.x * blockDim.x + threadIdx.x; r < n;
       r += (size_t)gridDim.x * blockDim.x) {
    for (int q = 0; q < Q; ++q) {
      uint32_t packed = 0;
      for (int c = 0; c < 4; ++c) {
        const int f = q * 4 + c;
        if (f < F) packed |= (uint32_t)in[r * F + f] << (8 * c);
      }
      out[(size_t)q * stride + r] = packed;
    }
  }
}

// row-major uint16 [n][F] -> words of two 16-bit ids
__global__ void k_pack_prebinned16(const uint16_t *__restrict__ in, int F, int Q,
                                   uint32_t *__restrict__ out, size_t stride, size_t n) {
  for (size_t r = (size_t)blockIdx.x * blockDim.x + threadIdx.x; r < n;
       r += (size_t)gridDim.x * blockDim.x) {
    for (int q = 0; q < Q; ++q) {
      uint32_t packed = in[r * F + 2 * q];
      if (2 * q + 1 < F) packed |= (uint32_t)in[r * F + 2 * q + 1] << 16;
      out[(size_t)q * stride + r] = packed;
    }
  }
}

}  // namespace
}  // namespace arb
#endif  // ARBORETUM_AMD_KERNELS_QUANTISE_H_
