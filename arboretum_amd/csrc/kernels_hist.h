// LDS histograms: update order and layout, stand-alone histogram kernels.
#ifndef ARBORETUM_AMD_KERNELS_HIST_H_
#define ARBORETUM_AMD_KERNELS_HIST_H_
#include "device_common.h"

namespace arb {
namespace {

// ---------------------------------------------------------------- histogram
// LDS layout of a histogram of NQ quads (B = ceil(NQ / 4) blocks of 16
// features), in 64-bit words.  Entry (f, bin) of block k = f / 16, f16 = f % 16:
//   one word per entry (squared objective):  bin * 16 B + k * 16 + f16
//   two words per entry (PAIR):              bin * 32 B + k * 32 + f16 for word0,
//                                            16 words (128 bytes) further for word1.
// The 16 lanes of one pass of an LDS atomic, which work on 16 different
// features of their rows, fall on 16 different bank pairs (word % 16 = f16),
// and every update of a row's bin of feature f16 in any block, first or second
// word, uses ONE address register with an immediate offset.
template <int NQ>
struct HistLds {
  static constexpr int blocks = HistBlocks(NQ);
  static constexpr int entries = blocks * kBlockEntries;
};
// Word of word0 of an entry of a histogram of `blocks` blocks, given the
// entry's index in entry order (k * 4096 + bin * 16 + f16); word1 is kWord1
// words further.
constexpr int kWord1 = kBlockFeatures;
template <bool PAIR>
__host__ __device__ __forceinline__ unsigned HistWord(unsigned entry, int blocks) {
  constexpr unsigned per = PAIR ? 2 : 1;
  const unsigned k = entry / kBlockEntries, bin = (entry / kBlockFeatures) % kSlots, f16 = entry % kBlockFeatures;
  return bin * (per * kBlockFeatures * (unsigned)blocks) + k * (per * kBlockFeatures) + f16;
}

// Adds one row per lane (bins of its NQ quads in b) to the LDS histogram.  The
// 28 (or 4*NQ) updates of a row are issued in an order that depends on the
// lane: in step (s, t) of a block, lane l works on quad (s + (l>>2)) % 4 and
// byte (t + l) % 4 of that quad, so the 16 lanes of a pass of the LDS atomic
// touch 16 different features = 16 different bank pairs.  q_first: first quad
// of this launch (a multiple of 4).
// HI: b[NQ] is the ninth-bit word of the row's features 4 q_first .. 4 q_first
// + 31 (bit f set: the id of that feature is 256, its byte 255).  HI = 1: such
// an id falls into the row of entries that follows bin 255 in this bin-major
// layout, so the address arithmetic is the same.  HI = 2 (matrices of several
// groups of quads): such an id is not accumulated at all; no split candidate's
// left side holds it (candidates end at bin 255), so the scan never misses it.
template <bool PAIR, int NQ, int HI = 0>
__device__ __forceinline__ void AccumulateRow(unsigned long long *__restrict__ lds,
                                              const uint32_t (&b)[NQ + (HI != 0 ? 1 : 0)], float gv, float hv, int sg,
                                              int sh, int q_first, int F) {
  using L = HistLds<NQ>;
  const unsigned long long w0 = (1ull << kCountShift) + (unsigned long long)ToFixed(gv, sg);
  unsigned long long w1 = 0;
  if (PAIR) w1 = (unsigned long long)ToFixed(hv, sh);
  const unsigned j = (threadIdx.x >> 2) & 3u, i = threadIdx.x & 3u;
#pragma unroll
  for (int k = 0; k < L::blocks; ++k) {
    // quads of this block; the ones past NQ do not exist
    uint32_t r[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) r[x] = 4 * k + x < NQ ? b[4 * k + x < NQ ? 4 * k + x : 0] : 0u;
#pragma unroll
    for (int s_ = 0; s_ < 4; ++s_) {
      const unsigned qi = ((unsigned)s_ + j) & 3u;  // quad of the block this lane works on
      const uint32_t lo = (j & 1u) ? r[(s_ + 1) & 3] : r[s_];
      const uint32_t hi = (j & 1u) ? r[(s_ + 3) & 3] : r[(s_ + 2) & 3];
      const uint32_t sel = (j & 2u) ? hi : lo;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const unsigned bi = ((unsigned)t + i) & 3u;  // byte of the quad
        unsigned bin = __builtin_amdgcn_ubfe(sel, 8u * bi, 8u);  // one v_bfe_u32
        const unsigned f16 = 4u * qi + bi;
        unsigned ninth = 0;
        if constexpr (HI != 0) ninth = __builtin_amdgcn_ubfe(b[NQ], 16u * (unsigned)k + f16, 1u);
        if constexpr (HI == 1) bin += ninth;
        // Quads past NQ do not exist.  Padding features of the last quad of
        // the matrix (bin 0 in every row) are accumulated like real ones into
        // slots nobody reads: cheaper than a per-update test.
        bool on = true;
        if (4 * k + 3 >= NQ) on = 4u * k + qi < (unsigned)NQ;
        if constexpr (HI == 2) on = on && ninth == 0u;
        if (on) {
          constexpr unsigned per = PAIR ? 2 : 1;
          unsigned long long *cell = &lds[bin * (per * kBlockFeatures * L::blocks) + f16];
          atomicAdd(cell + k * (per * kBlockFeatures), w0);
          if (PAIR) atomicAdd(cell + k * (per * kBlockFeatures) + kWord1, w1);
        }
      }
    }
  }
}

// Writes the LDS histogram to the slab of work item w as it lies in LDS.
// Called by the whole workgroup after its last LDS update.  A slab holds
// slab_entries entries (one or two words each): the histograms of the
// launches (groups of quads) of a level one after the other, each in the
// layout of HistLds for its own number of blocks; q_first is a multiple of 4.
// HI: the image is one row of entries longer (bin 256), and so is the slab:
// slab_entries counts that row too.
template <bool PAIR, int NQ, int HI = 0>
__device__ __forceinline__ void FlushSlab(const unsigned long long *__restrict__ lds,
                                          unsigned long long *__restrict__ slab, unsigned w,
                                          int slab_entries, int q_first) {
  constexpr int words = (int)(HistLdsBytes(NQ, PAIR, HI == 1) / 8);
  constexpr int per = PAIR ? 2 : 1;
  __syncthreads();
  unsigned long long *out =
      slab + ((size_t)w * slab_entries + (size_t)(q_first / kBlockQuads) * kBlockEntries) * per;
  for (int e = threadIdx.x; e < words; e += kHistThreads) out[e] = lds[e];
}

// Histogram of contiguous row ranges: one workgroup per work item, quads
// [q0, q0+NQ).  LDS: NQ*1024 word0 entries, then (PAIR) as many word1 entries.
// PAIR with h == nullptr: g holds packed logistic gradients (PackGrad).
// HI: hi_col is the column of the ninth-bit words of features 4 q0 .. 4 q0 + 31
// (AccumulateRow: 1 = accumulated in a 257th row of entries, 2 = skipped).
template <bool PAIR, int NQ, int HI = 0>
__global__ void __launch_bounds__(kHistThreads)
k_hist(const uint32_t *__restrict__ bins, size_t stride, int q0, int F,
       const float *__restrict__ g, const float *__restrict__ h, const int *__restrict__ shifts,
       const WorkItem *__restrict__ work, const unsigned *__restrict__ n_work,
       unsigned long long *__restrict__ slab, int slab_entries, const uint32_t *__restrict__ hi_col = nullptr) {
  extern __shared__ unsigned long long lds[];
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  constexpr int words = (int)(HistLdsBytes(NQ, PAIR, HI == 1) / 8);
  constexpr int NH = HI != 0 ? 1 : 0;
  for (int i = threadIdx.x; i < words; i += kHistThreads) lds[i] = 0ull;
  __syncthreads();
  const int sg = shifts[0], sh = shifts[1];
  const uint32_t *bq = bins + (size_t)q0 * stride;
  for (unsigned base = it.begin; base < it.end; base += 2 * kHistThreads) {
    const unsigned r0 = base + threadIdx.x, r1 = r0 + kHistThreads;
    const bool v0 = r0 < it.end, v1 = r1 < it.end;
    const unsigned a0 = v0 ? r0 : it.begin, a1 = v1 ? r1 : it.begin;
    uint32_t b0[NQ + NH], b1[NQ + NH];
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      b0[q] = __builtin_nontemporal_load(&bq[(size_t)q * stride + a0]);
      b1[q] = __builtin_nontemporal_load(&bq[(size_t)q * stride + a1]);
    }
    if constexpr (HI != 0) {
      b0[NQ] = __builtin_nontemporal_load(&hi_col[a0]);
      b1[NQ] = __builtin_nontemporal_load(&hi_col[a1]);
    }
    float g0 = g[a0], g1 = g[a1];
    float h0 = 0.0f, h1 = 0.0f;
    if (PAIR) {
      if (h != nullptr) {  // uniform
        h0 = h[a0];
        h1 = h[a1];
      } else {  // packed logistic gradients
        UnpackGrad(g0, &g0, &h0);
        UnpackGrad(g1, &g1, &h1);
      }
    }
    if (v0) AccumulateRow<PAIR, NQ, HI>(lds, b0, g0, h0, sg, sh, q0, F);
    if (v1) AccumulateRow<PAIR, NQ, HI>(lds, b1, g1, h1, sg, sh, q0, F);
  }
  FlushSlab<PAIR, NQ, HI>(lds, slab, w, slab_entries, q0);
}

// Histogram of contiguous row ranges with 16-bit bins: features [f0, f0 + nf)
// (f0 even), `slots` histogram slots per feature, LDS layout f * slots + bin,
// word0 of every entry first, then (PAIR) word1.  The slab of a work item has
// the same feature-major order: word0[slab_entries], word1[slab_entries].
template <bool PAIR>
__global__ void __launch_bounds__(kHistThreads)
k_hist_wide(const uint32_t *__restrict__ bins, size_t stride, int f0, int nf, int slots,
            const float *__restrict__ g, const float *__restrict__ h, const int *__restrict__ shifts,
            const WorkItem *__restrict__ work, const unsigned *__restrict__ n_work,
            unsigned long long *__restrict__ slab, int slab_entries) {
  extern __shared__ unsigned long long lds[];
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const int entries = nf * slots;
  for (int i = threadIdx.x; i < entries * (PAIR ? 2 : 1); i += kHistThreads) lds[i] = 0ull;
  __syncthreads();
  const int sg = shifts[0], sh = shifts[1];
  const int words = (nf + 1) / 2;
  for (unsigned r = it.begin + threadIdx.x; r < it.end; r += kHistThreads) {
    const unsigned long long w0 = (1ull << kCountShift) + (unsigned long long)ToFixed(g[r], sg);
    unsigned long long w1 = 0;
    if (PAIR) w1 = (unsigned long long)ToFixed(h[r], sh);
    for (int k = 0; k < words; ++k) {
      const uint32_t word = bins[(size_t)(f0 / 2 + k) * stride + r];
      const unsigned lo = (unsigned)(2 * k) * slots + (word & 0xffffu);
      atomicAdd(&lds[lo], w0);
      if (PAIR) atomicAdd(&lds[entries + lo], w1);
      if (2 * k + 1 < nf) {
        const unsigned hi = (unsigned)(2 * k + 1) * slots + (word >> 16);
        atomicAdd(&lds[hi], w0);
        if (PAIR) atomicAdd(&lds[entries + hi], w1);
      }
    }
  }
  __syncthreads();
  unsigned long long *out = slab + (size_t)w * slab_entries * (PAIR ? 2 : 1) + (size_t)f0 * slots;
  for (int e = threadIdx.x; e < entries; e += kHistThreads) {
    out[e] = lds[e];
    if (PAIR) out[slab_entries + e] = lds[entries + e];
  }
}

}  // namespace
}  // namespace arb
#endif  // ARBORETUM_AMD_KERNELS_HIST_H_
