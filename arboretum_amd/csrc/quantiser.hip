// Quantile thresholds of one feature column on the GPU: a hand-written LSD
// radix sort of the column followed by the reference's threshold rule.
//
// Replaces cub::DeviceRadixSort::SortKeys + DeviceScan with the
// ValueSegmentIterator / ThresholdOutputIterator pair (src/io/io.cu:349-410,
// 27-153, 255-270):  with s = the sorted column and seg = max(1, n / hist_size),
// the k-th change of value (s[i] != s[i-1], NaN != NaN included) at position i
// writes its midpoint float((s[i] + s[i-1]) * 0.5) to slot
// min(k + 1, i / seg + 1) - 2, lowest midpoint wins; NaN midpoints are never
// stored.  NaNs of either sign sort last.
#include <hip/hip_runtime.h>

#include <cmath>
#include <limits>
#include <stdexcept>
#include <string>
#include <vector>

#include "booster.h"

namespace arb {
namespace {

#define HIP_OK(expr)                                                                        \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if (e_ != hipSuccess)                                                                   \
      throw std::runtime_error(std::string("HIP error: ") + hipGetErrorString(e_) + " in " #expr); \
  } while (0)

constexpr int kSortThreads = 256;
constexpr int kSortRounds = 16;                          // keys per thread
constexpr int kSortTile = kSortThreads * kSortRounds;    // 4096 keys per workgroup
constexpr unsigned kNanKey = 0xffffffffu;

// Order-preserving map float -> uint32; every NaN maps to the largest key.
__device__ __forceinline__ unsigned KeyOf(float v) {
  if (v != v) return kNanKey;
  const unsigned b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float ValueOf(unsigned k) {
  if (k == kNanKey) return __uint_as_float(0x7fc00000u);
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

__global__ void k_rs_keys(const float *__restrict__ x, unsigned *__restrict__ keys, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    keys[i] = KeyOf(x[i]);
}

// Digit counts of one tile: counts[digit * nblk + block].
__global__ void __launch_bounds__(kSortThreads)
k_rs_count(const unsigned *__restrict__ keys, size_t n, int shift, unsigned *__restrict__ counts, unsigned nblk) {
  __shared__ unsigned s_cnt[256];
  s_cnt[threadIdx.x] = 0;
  __syncthreads();
  const size_t base = (size_t)blockIdx.x * kSortTile;
  for (int j = 0; j < kSortRounds; ++j) {
    const size_t i = base + (size_t)j * kSortThreads + threadIdx.x;
    if (i < n) atomicAdd(&s_cnt[(keys[i] >> shift) & 255u], 1u);
  }
  __syncthreads();
  counts[(size_t)threadIdx.x * nblk + blockIdx.x] = s_cnt[threadIdx.x];
}

// In-place exclusive scan of `m` counters.  One workgroup.
__global__ void __launch_bounds__(1024) k_rs_scan(unsigned *__restrict__ v, size_t m) {
  __shared__ unsigned s_part[1024];
  const size_t per = (m + 1023) / 1024;
  const size_t b = min(m, (size_t)threadIdx.x * per), e = min(m, b + per);
  unsigned sum = 0;
  for (size_t i = b; i < e; ++i) sum += v[i];
  s_part[threadIdx.x] = sum;
  __syncthreads();
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    unsigned t[16], tot = 0;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      t[k] = s_part[lane * 16 + k];
      tot += t[k];
    }
    unsigned incl = tot;
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned o = __shfl_up(incl, off);
      if (lane >= off) incl += o;
    }
    unsigned run = incl - tot;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      s_part[lane * 16 + k] = run;
      run += t[k];
    }
  }
  __syncthreads();
  unsigned run = s_part[threadIdx.x];
  for (size_t i = b; i < e; ++i) {
    const unsigned c = v[i];
    v[i] = run;
    run += c;
  }
}

// Exclusive scan of the tile counts of every digit: workgroup d scans
// counts[d * nblk .. (d + 1) * nblk) in place and writes the digit's total.
__global__ void __launch_bounds__(1024)
k_rs_scan_digits(unsigned *__restrict__ counts, unsigned nblk, unsigned *__restrict__ digit_total) {
  __shared__ unsigned s_wave[16];
  __shared__ unsigned s_carry;
  unsigned *v = counts + (size_t)blockIdx.x * nblk;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) s_carry = 0;
  __syncthreads();
  for (unsigned base = 0; base < nblk; base += 1024) {
    const unsigned i = base + threadIdx.x;
    const unsigned c = i < nblk ? v[i] : 0u;
    unsigned incl = c;
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned o = __shfl_up(incl, off);
      if (lane >= off) incl += o;
    }
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    unsigned before = s_carry;
    for (int w = 0; w < wave; ++w) before += s_wave[w];
    if (i < nblk) v[i] = before + incl - c;
    __syncthreads();
    if (threadIdx.x == 1023) s_carry = before + incl;
    __syncthreads();
  }
  if (threadIdx.x == 0) digit_total[blockIdx.x] = s_carry;
}

// Lanes of the wave holding the same 8-bit digit as this lane.
__device__ __forceinline__ unsigned long long DigitPeers(unsigned d, bool valid) {
  unsigned long long peers = __ballot(valid);
#pragma unroll
  for (int b = 0; b < 8; ++b) {
    const unsigned long long m = __ballot((d >> b) & 1u);
    peers &= ((d >> b) & 1u) ? m : ~m;
  }
  return peers;
}

// Stable scatter of one tile by digit; offsets[digit * nblk + block] is the
// first output position of the tile's keys with that digit.
__global__ void __launch_bounds__(kSortThreads)
k_rs_scatter(const unsigned *__restrict__ keys, unsigned *__restrict__ out, size_t n, int shift,
             const unsigned *__restrict__ offsets, unsigned nblk,
             const unsigned *__restrict__ digit_total) {
  __shared__ unsigned s_run[256];                       // keys of each digit already placed
  __shared__ unsigned s_wave[kSortThreads / 64][256];   // per wave counts of the current round
  __shared__ unsigned s_tot[kSortThreads / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  {
    // keys with a smaller digit: exclusive scan of the 256 digit totals (thread = digit)
    const unsigned c = digit_total[threadIdx.x];
    unsigned incl = c;
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned o = __shfl_up(incl, off);
      if (lane >= off) incl += o;
    }
    if (lane == 63) s_tot[wave] = incl;
    __syncthreads();
    unsigned before = 0;
    for (int w = 0; w < wave; ++w) before += s_tot[w];
    s_run[threadIdx.x] = before + incl - c + offsets[(size_t)threadIdx.x * nblk + blockIdx.x];
  }
  for (int w = 0; w < kSortThreads / 64; ++w) s_wave[w][threadIdx.x] = 0;
  __syncthreads();
  const size_t base = (size_t)blockIdx.x * kSortTile;
  for (int j = 0; j < kSortRounds; ++j) {
    const size_t i = base + (size_t)j * kSortThreads + threadIdx.x;
    const bool valid = i < n;
    const unsigned key = valid ? keys[i] : 0u;
    const unsigned d = (key >> shift) & 255u;
    const unsigned long long peers = DigitPeers(d, valid);
    const unsigned rank = (unsigned)__popcll(peers & ((1ull << lane) - 1ull));
    if (valid && rank == 0) s_wave[wave][d] = (unsigned)__popcll(peers);
    __syncthreads();
    if (valid) {
      unsigned pos = s_run[d] + rank;
      for (int w = 0; w < wave; ++w) pos += s_wave[w][d];
      out[pos] = key;
    }
    __syncthreads();
    {
      unsigned t = 0;
      for (int w = 0; w < kSortThreads / 64; ++w) {
        t += s_wave[w][threadIdx.x];
        s_wave[w][threadIdx.x] = 0;
      }
      s_run[threadIdx.x] += t;
    }
    __syncthreads();
  }
}

__device__ __forceinline__ bool IsBorder(const unsigned *__restrict__ keys, size_t i) {
  if (i == 0) return false;
  const float a = ValueOf(keys[i]), b = ValueOf(keys[i - 1]);
  return a != b;  // true for NaN; false for -0.0 against +0.0
}

// Changes of value per tile.
__global__ void __launch_bounds__(kSortThreads)
k_thr_count(const unsigned *__restrict__ keys, size_t n, unsigned *__restrict__ counts) {
  __shared__ unsigned s_cnt[kSortThreads / 64];
  const size_t base = (size_t)blockIdx.x * kSortTile;
  unsigned c = 0;
  for (int j = 0; j < kSortRounds; ++j) {
    const size_t i = base + (size_t)j * kSortThreads + threadIdx.x;
    if (i < n && IsBorder(keys, i)) ++c;
  }
  for (int off = 32; off > 0; off >>= 1) c += __shfl_down(c, off);
  if ((threadIdx.x & 63) == 0) s_cnt[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned t = 0;
    for (int w = 0; w < kSortThreads / 64; ++w) t += s_cnt[w];
    counts[blockIdx.x] = t;
  }
}

// Thresholds as ordered keys: thr[slot] = min over the changes mapped to slot.
// Every wave owns a contiguous quarter of the tile: it counts its changes,
// the workgroup synchronises once, then the wave numbers its changes alone.
__global__ void __launch_bounds__(kSortThreads)
k_thr_emit(const unsigned *__restrict__ keys, size_t n, const unsigned *__restrict__ before, unsigned seg,
           int hist_size, unsigned *__restrict__ thr) {
  constexpr int kWaves = kSortThreads / 64;
  constexpr int kWaveKeys = kSortTile / kWaves;
  __shared__ unsigned s_wave[kWaves];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t wbase = (size_t)blockIdx.x * kSortTile + (size_t)wave * kWaveKeys;
  unsigned mine = 0;
  for (int j = 0; j < kWaveKeys; j += 64) {
    const size_t i = wbase + j + lane;
    mine += (unsigned)__popcll(__ballot(i < n && IsBorder(keys, i)));
  }
  if (lane == 0) s_wave[wave] = mine;
  __syncthreads();
  unsigned run = before[blockIdx.x];  // changes before this wave's keys
  for (int w = 0; w < wave; ++w) run += s_wave[w];
  for (int j = 0; j < kWaveKeys; j += 64) {
    const size_t i = wbase + j + lane;
    const bool border = i < n && IsBorder(keys, i);
    const unsigned long long m = __ballot(border);
    const unsigned long long below = m & ((1ull << lane) - 1ull);
    int slot = -3;
    float mid = 0.0f;
    if (border) {
      const unsigned k = run + (unsigned)__popcll(below) + 1u;  // inclusive count
      const float a = ValueOf(keys[i]), b = ValueOf(keys[i - 1]);
      mid = (float)((double)(float)(a + b) * 0.5);
      const unsigned long long pos_slot = (unsigned long long)(i / seg) + 1ull;
      slot = (int)((long long)min((unsigned long long)k + 1ull, pos_slot) - 2);
    }
    // Slots and midpoints grow with the position (NaN midpoints come last), so
    // the minimum of a slot is at its first change: only the first change of
    // each slot within the wave goes to memory.
    const int prev = below ? 63 - __clzll((long long)below) : lane;
    const int prev_slot = __shfl(slot, prev);
    const bool first = border && (below == 0ull || prev_slot != slot);
    if (first && mid == mid && slot >= 0 && slot < hist_size) {
      const unsigned mk = KeyOf(mid);
      if (mk < thr[slot]) atomicMin(&thr[slot], mk);
    }
    run += (unsigned)__popcll(m);
  }
}

__global__ void k_thr_init(unsigned *thr, int hist_size) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < hist_size) thr[i] = 0xff800000u;  // KeyOf(+INF)
}

__global__ void k_thr_finish(const unsigned *__restrict__ thr, float *__restrict__ out, int hist_size,
                             const unsigned *__restrict__ sorted, size_t n, unsigned *__restrict__ has_nan) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < hist_size) out[i] = ValueOf(thr[i]);
  if (i == 0) *has_nan = sorted[n - 1] == kNanKey ? 1u : 0u;
}

}  // namespace

struct SortWorkspace {
  size_t n = 0;
  unsigned nblk = 0;
  int hist_size = 0;
  unsigned *keys[2] = {nullptr, nullptr};
  unsigned *counts = nullptr, *digit_total = nullptr, *thr = nullptr, *has_nan = nullptr;
  float *thr_f = nullptr;
};

SortWorkspace *CreateSortWorkspace(size_t n, int hist_size) {
  SortWorkspace *ws = new SortWorkspace();
  ws->n = n;
  ws->hist_size = hist_size;
  ws->nblk = (unsigned)((n + kSortTile - 1) / kSortTile);
  HIP_OK(hipMalloc((void **)&ws->keys[0], n * sizeof(unsigned)));
  HIP_OK(hipMalloc((void **)&ws->keys[1], n * sizeof(unsigned)));
  HIP_OK(hipMalloc((void **)&ws->counts, (size_t)256 * ws->nblk * sizeof(unsigned)));
  HIP_OK(hipMalloc((void **)&ws->digit_total, 256 * sizeof(unsigned)));
  HIP_OK(hipMalloc((void **)&ws->thr, (size_t)hist_size * sizeof(unsigned)));
  HIP_OK(hipMalloc((void **)&ws->thr_f, (size_t)hist_size * sizeof(float)));
  HIP_OK(hipMalloc((void **)&ws->has_nan, sizeof(unsigned)));
  return ws;
}

void FreeSortWorkspace(SortWorkspace *ws) {
  if (!ws) return;
  void *p[] = {ws->keys[0], ws->keys[1], ws->counts, ws->digit_total, ws->thr, ws->thr_f, ws->has_nan};
  for (void *q : p)
    if (q) (void)hipFree(q);
  delete ws;
}

// Thresholds of the column d_col (n floats in HBM): `thr` gets hist_size
// entries (+INF where unset), *size the number of real bins (leading finite
// thresholds + 1, capped at hist_size: io.cu:403-410), *has_nan whether a NaN
// is present.
void DeviceThresholds(SortWorkspace *ws, const float *d_col, std::vector<float> *thr, int *size, bool *has_nan) {
  const size_t n = ws->n;
  const unsigned nblk = ws->nblk;
  const int hs = ws->hist_size;
  const int grid_n = (int)std::min<size_t>((n + 255) / 256, 4096);
  hipLaunchKernelGGL(k_rs_keys, dim3(grid_n), dim3(256), 0, 0, d_col, ws->keys[0], n);
  int cur = 0;
  for (int shift = 0; shift < 32; shift += 8) {
    hipLaunchKernelGGL(k_rs_count, dim3(nblk), dim3(kSortThreads), 0, 0, ws->keys[cur], n, shift, ws->counts, nblk);
    hipLaunchKernelGGL(k_rs_scan_digits, dim3(256), dim3(1024), 0, 0, ws->counts, nblk, ws->digit_total);
    hipLaunchKernelGGL(k_rs_scatter, dim3(nblk), dim3(kSortThreads), 0, 0, ws->keys[cur], ws->keys[cur ^ 1], n,
                       shift, ws->counts, nblk, ws->digit_total);
    cur ^= 1;
  }
  unsigned seg = (unsigned)(n / (size_t)hs);
  if (seg < 1) seg = 1;
  hipLaunchKernelGGL(k_thr_init, dim3((hs + 255) / 256), dim3(256), 0, 0, ws->thr, hs);
  hipLaunchKernelGGL(k_thr_count, dim3(nblk), dim3(kSortThreads), 0, 0, ws->keys[cur], n, ws->counts);
  hipLaunchKernelGGL(k_rs_scan, dim3(1), dim3(1024), 0, 0, ws->counts, (size_t)nblk);
  hipLaunchKernelGGL(k_thr_emit, dim3(nblk), dim3(kSortThreads), 0, 0, ws->keys[cur], n, ws->counts, seg, hs, ws->thr);
  hipLaunchKernelGGL(k_thr_finish, dim3((hs + 255) / 256), dim3(256), 0, 0, ws->thr, ws->thr_f, hs, ws->keys[cur], n,
                     ws->has_nan);
  HIP_OK(hipGetLastError());
  thr->resize(hs);
  unsigned nan_flag = 0;
  HIP_OK(hipMemcpy(thr->data(), ws->thr_f, (size_t)hs * sizeof(float), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(&nan_flag, ws->has_nan, sizeof(unsigned), hipMemcpyDeviceToHost));
  int unique = 0;
  while (unique < hs && !std::isinf((*thr)[unique])) ++unique;
  ++unique;
  *size = std::min(unique, hs);
  *has_nan = nan_flag != 0;
}

}  // namespace arb
