// Constants, records and helpers shared by the device kernels of the tree builder.
#ifndef ARBORETUM_AMD_DEVICE_COMMON_H_
#define ARBORETUM_AMD_DEVICE_COMMON_H_
#include <hip/hip_runtime.h>

#include <cstdint>
#include <stdexcept>
#include <string>

#include "gain.h"

namespace arb {
namespace {

#define HIP_OK(expr)                                                                        \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if (e_ != hipSuccess)                                                                   \
      throw std::runtime_error(std::string("HIP error: ") + hipGetErrorString(e_) + " in " #expr); \
  } while (0)

constexpr int kSlots = 256;               // histogram slots per feature (uint8 bins)
constexpr int kMaxWideSlots = 4096;       // histogram slots per feature with 16-bit bins (power of two)
constexpr int kHistThreads = 1024;        // one workgroup per CU, 16 waves
constexpr int kItemWaves = kHistThreads / 64;  // waves per work item in row passes
constexpr unsigned kPartRows = 16384;     // rows per work item of the stand-alone partition
constexpr int kMaxGroupQuads = 8;         // quads per histogram launch (compile-time variants, whole blocks)
constexpr unsigned kMaxHistRows = 64512;  // rows per histogram work item (< 2^16)
constexpr int kCountShift = 47;           // word0 = count << 47 | g
constexpr int kMaxPlanNodes = 4096;       // nodes per level the planner handles
constexpr size_t kLdsBudget = 160 * 1024;
// LDS histograms are laid out bin-major with the features of a bin in blocks
// of 16 (4 quads): in 64-bit words, one word per entry,
//   word(f, bin) = bin * 16 * blocks + (f / 16) * 16 + f % 16
// (twice that with two words per entry, the second word 16 words further; see
// HistLds).  A 64-bit LDS atomic is executed 16 lanes per pass, and two of
// those lanes collide when their addresses share a bank pair (word % 16).
// With this layout the bank pair is f % 16, and the kernels let the 16 lanes
// of a pass work on 16 different features of their rows, so a pass never has a
// bank conflict and never two lanes on one address, whatever the bin
// distribution is (missing values, zeros, a dominant category).  Entries are
// counted in "entry order", (f / 16) * 4096 + bin * 16 + f % 16, wherever a
// histogram is addressed independently of its number of blocks.
constexpr int kBlockFeatures = 16;
constexpr int kBlockQuads = 4;
constexpr int kBlockEntries = kBlockFeatures * kSlots;  // 4096
constexpr int HistBlocks(int nq) { return (nq + kBlockQuads - 1) / kBlockQuads; }
// LDS bytes of a histogram of nq quads; hi: one more row of entries, bin 256
// of every feature (the ninth-bit word, see SplitTest)
constexpr size_t HistLdsBytes(int nq, bool pair, bool hi = false) {
  return (size_t)HistBlocks(nq) * (kBlockEntries + (hi ? kBlockFeatures : 0)) * 8 * (pair ? 2 : 1);
}

// Logistic gradients of 0/1 labels can travel as ONE float per row:
// u = s with the sign bit set when y = 1, s = sigmoid(y_hat) >= 0.  The pair
// (g, h) = (y - s, s (1 - s)) is recomputed where it is used, with the very
// operations of the gradient kernel, so the values are bit-identical; the row
// passes then move four bytes less per row and direction.
__host__ __device__ __forceinline__ float PackGrad(float s, float y) {
  union { float f; uint32_t u; } v;
  v.f = s;
  v.u |= (y != 0.0f) ? 0x80000000u : 0u;
  return v.f;
}
__host__ __device__ __forceinline__ void UnpackGrad(float u, float *g, float *h) {
  union { float f; uint32_t u; } v;
  v.f = u;
  const float y = (v.u >> 31) ? 1.0f : 0.0f;
  v.u &= 0x7fffffffu;
  const float s = v.f;
  *g = y - s;
  *h = s * (1.0f - s);
}

struct NodeSum {
  long long g;
  long long h;
  unsigned long long c;
};

struct SplitRec {
  float gain;
  int fid;   // -1: not split (every row stays left)
  int bin;
  unsigned pad;
  NodeSum left;
};

struct WorkItem {
  unsigned node;
  unsigned begin;  // row range in the current order
  unsigned end;
  unsigned first;  // index of the first work item of this node
};

// How bin ids are packed in the 32-bit words of a row: 8 bits (four features
// per word) or 16 bits (two features per word).
struct BinCode {
  int wshift;  // feature -> word: fid >> wshift
  int bits;
  __host__ __device__ static BinCode Of(int bits) { return BinCode{bits == 8 ? 2 : 1, bits}; }
  __device__ __forceinline__ int Word(int fid) const { return fid >> wshift; }
  __device__ __forceinline__ unsigned Bin(uint32_t word, int fid) const {
    return (word >> (bits * (fid & ((1 << wshift) - 1)))) & ((1u << bits) - 1u);
  }
};

// Bin id 256.  With hist_size 256 a feature that fills all 256 value bins and
// also has missing values needs 257 ids (NaN -> bin `size`,
// src/core/cuda_helpers.h:207-222).  Such an id is stored as byte 255 plus one
// bit in an extra word of the row, a "ninth-bit word": bit f % 32 of word f / 32
// set means the id of feature f is 256.  The words follow the quads of the row
// (columns Q, Q + 1, ... of a matrix of Q quads; one word up to 32 features) and
// move with them.
//
// The test "id > split bin" on one 32-bit word of a row:
//   split bin < 255 (or no ninth bits): the feature's byte against the bin (an
//     id of 256 has byte 255, which is larger than any such bin);
//   split bin 255: only an id of 256 goes right: the feature's ninth bit;
//   node not split: nobody goes right.
struct SplitTest {
  int word;  // column of the row the test reads
  unsigned shift, mask;
  int thr;
  __device__ __forceinline__ bool Right(uint32_t v) const { return (int)((v >> shift) & mask) > thr; }
};
// hi_word: column of the first ninth-bit word, negative when the matrix has none
__device__ __forceinline__ SplitTest MakeSplitTest(const SplitRec &s, BinCode code, int hi_word) {
  if (s.fid < 0) return SplitTest{0, 0u, 0u, 0};
  if (hi_word >= 0 && s.bin >= 255) return SplitTest{hi_word + (s.fid >> 5), (unsigned)(s.fid & 31), 1u, 0};
  return SplitTest{code.Word(s.fid), (unsigned)(code.bits * (s.fid & ((1 << code.wshift) - 1))),
                   (1u << code.bits) - 1u, s.bin};
}

__device__ __forceinline__ float WaveMaxF(float v) {
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_down(v, off));
  return v;
}
__device__ __forceinline__ long long WaveSumLL(long long v) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off);
  return v;
}

__global__ void k_init_root(NodeSum *tot, unsigned *seg_start, unsigned long long n,
                            unsigned *gmax_bits) {  // gmax_bits may be NULL
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    tot[0].g = 0;
    tot[0].h = 0;
    tot[0].c = n;
    seg_start[0] = 0;
    if (gmax_bits) *gmax_bits = 0;
  }
}

__device__ __forceinline__ unsigned RankBelow(unsigned long long m) {
  // number of set bits of m below this lane
  return __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0u));
}

// Rows of a work item are dealt to its waves in chunks of kChunkRows
// consecutive rows, round-robin: wave v takes chunks v, v + kItemWaves, ...  A
// workgroup therefore streams one contiguous block of the item per step (good
// DRAM page locality) while every wave still owns a fixed, countable row set.
constexpr unsigned kChunkRows = 128;
constexpr unsigned kChunkStep = kChunkRows * kItemWaves;

}  // namespace
}  // namespace arb
#endif  // ARBORETUM_AMD_DEVICE_COMMON_H_
