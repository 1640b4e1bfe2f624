// Host-side launch helpers shared by the translation units that run the
// stand-alone histogram kernel.
#ifndef ARBORETUM_AMD_KERNELS_LAUNCH_H_
#define ARBORETUM_AMD_KERNELS_LAUNCH_H_
#include <mutex>
#include <stdexcept>

#include "device_common.h"
#include "kernels_hist.h"

namespace arb {
namespace {

// Raises the dynamic LDS limit of a kernel (needed above 64 KB).
template <typename K>
void AllowLds(K kernel, size_t bytes) {
  HIP_OK(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
}
// The same once per process and call site: `flag` is a static of the caller, one per kernel
// instance.  Safe from several host threads; a later launch pays nothing.
template <typename K>
void AllowLdsOnce(std::once_flag &flag, K kernel, size_t bytes) {
  std::call_once(flag, [&] { AllowLds(kernel, bytes); });
}

template <bool PAIR, int NQ, int HI = 0>
void LaunchHistNQ(hipStream_t st, unsigned grid, const uint32_t *bins, size_t stride, int q0, int F,
                  const float *g, const float *h, const int *shifts, const WorkItem *work,
                  const unsigned *n_work, unsigned long long *slab, int slab_entries, const uint32_t *hi_col) {
  const size_t lds = HistLdsBytes(NQ, PAIR, HI == 1);
  static std::once_flag configured;
  AllowLdsOnce(configured, k_hist<PAIR, NQ, HI>, lds);
  hipLaunchKernelGGL((k_hist<PAIR, NQ, HI>), dim3(grid), dim3(kHistThreads), lds, st, bins, stride, q0, F, g, h,
                     shifts, work, n_work, slab, slab_entries, hi_col);
}

// HI: hi_col holds the ninth-bit words of the features of this launch (k_hist)
template <bool PAIR, int HI = 0>
void LaunchHist(int nq, hipStream_t st, unsigned grid, const uint32_t *bins, size_t stride, int q0, int F,
                const float *g, const float *h, const int *shifts, const WorkItem *work,
                const unsigned *n_work, unsigned long long *slab, int slab_entries,
                const uint32_t *hi_col = nullptr) {
#define ARB_CASE(N) \
  case N: LaunchHistNQ<PAIR, N, HI>(st, grid, bins, stride, q0, F, g, h, shifts, work, n_work, slab, slab_entries, hi_col); break;
  switch (nq) {
    ARB_CASE(1) ARB_CASE(2) ARB_CASE(3) ARB_CASE(4) ARB_CASE(5) ARB_CASE(6) ARB_CASE(7) ARB_CASE(8)
    default: throw std::runtime_error("internal: bad quad count");
  }
#undef ARB_CASE
}

}  // namespace
}  // namespace arb
#endif  // ARBORETUM_AMD_KERNELS_LAUNCH_H_
