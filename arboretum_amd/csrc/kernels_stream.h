// Kernels for matrices streamed from pinned host memory block by block.
#ifndef ARBORETUM_AMD_KERNELS_STREAM_H_
#define ARBORETUM_AMD_KERNELS_STREAM_H_
#include "device_common.h"
#include "kernels_partition.h"

namespace arb {
namespace {

// ----------------------------------------------------- streamed row blocks
// When the bins do not live in HBM (pinned host blocks copied in at every
// level; the reference streams whole columns, hist_tree_grower.cu:335-366),
// rows are never re-ordered.  A resident node id per row is advanced with the
// parents' splits while its block is on the GPU, the rows of the nodes built
// at this level are gathered node by node into a staging buffer, and the
// ordinary histogram kernel runs on that buffer.

// Is node nd accumulated directly at this level?  With sibling subtraction
// only the smaller child of each pair, ties -> left (hist_grad_sum.cu:279-294).
__device__ __forceinline__ bool NodeIsBuilt(const NodeSum *__restrict__ tot, unsigned nd, int level, int trick) {
  if (level == 0 || !trick) return true;
  const unsigned long long c = tot[nd].c, sib = tot[nd ^ 1u].c;
  return (nd & 1u) ? (c < sib) : (c <= sib);
}

// Advances the node id of every row of the block by the parents' splits and
// counts the rows of every built node (blk_cnt, zero on entry).
__global__ void __launch_bounds__(256)
k_stream_route(const uint32_t *__restrict__ bins, size_t bstride, unsigned rows, int level, int trick,
               const SplitRec *__restrict__ split, const NodeSum *__restrict__ tot,
               unsigned *__restrict__ node_of, unsigned *__restrict__ blk_cnt, int hi_word) {
  __shared__ unsigned s_cnt[kMaxPlanNodes];
  const int L = 1 << level;
  for (int i = threadIdx.x; i < L; i += blockDim.x) s_cnt[i] = 0;
  __syncthreads();
  const int lane = threadIdx.x & 63;
  const unsigned step = gridDim.x * blockDim.x;
  for (unsigned r0 = blockIdx.x * blockDim.x; r0 < rows; r0 += step) {  // whole waves stay together
    const unsigned r = r0 + threadIdx.x;
    unsigned nd = 0;
    bool built = false;
    if (r < rows) {
      if (level > 0) {
        const unsigned parent = node_of[r];
        nd = parent * 2u + (GoesRight(bins, bstride, split[parent], r, BinCode{2, 8}, hi_word) ? 1u : 0u);
      }
      node_of[r] = nd;
      built = NodeIsBuilt(tot, nd, level, trick);
    }
    // one LDS atomic per distinct node of the wave (64 lanes on one address serialise)
    unsigned long long todo = __ballot(built);
    while (todo) {
      const int leader = __ffsll((long long)todo) - 1;
      const unsigned lead_nd = (unsigned)__shfl((int)nd, leader);
      const unsigned long long same = __ballot(built && nd == lead_nd);
      if (lane == leader) atomicAdd(&s_cnt[lead_nd], (unsigned)__popcll(same));
      todo &= ~same;
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < L; i += blockDim.x)
    if (s_cnt[i]) atomicAdd(&blk_cnt[i], s_cnt[i]);
}

// Row ranges of the built nodes inside the staging buffer: exclusive scan of
// blk_cnt; also the cursors of the gather and the totals the planner reads.
// Clears blk_cnt for the next block.  One workgroup.
__global__ void __launch_bounds__(1024)
k_stream_segments(unsigned *__restrict__ blk_cnt, int L, NodeSum *__restrict__ blk_tot,
                  unsigned *__restrict__ blk_seg, unsigned *__restrict__ cursor) {
  __shared__ unsigned s_wave[16];
  __shared__ unsigned s_carry;
  if (threadIdx.x == 0) s_carry = 0;
  __syncthreads();
  for (int base = 0; base < L; base += 1024) {
    const int nd = base + threadIdx.x;
    const unsigned c = nd < L ? blk_cnt[nd] : 0u;
    unsigned incl = c;
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned o = __shfl_up(incl, off);
      if ((threadIdx.x & 63) >= off) incl += o;
    }
    if ((threadIdx.x & 63) == 63) s_wave[threadIdx.x >> 6] = incl;
    __syncthreads();
    unsigned off = s_carry;
    for (int w = 0; w < (int)(threadIdx.x >> 6); ++w) off += s_wave[w];
    const unsigned excl = off + incl - c;
    if (nd < L) {
      blk_seg[nd] = excl;
      cursor[nd] = excl;
      blk_tot[nd].g = 0;
      blk_tot[nd].h = 0;
      blk_tot[nd].c = c;
      blk_cnt[nd] = 0;
    }
    __syncthreads();
    if (threadIdx.x == 1023) s_carry = excl + c;
    __syncthreads();
  }
}

// Copies the rows of the built nodes into the staging buffer, node by node.
// The order inside a node is whatever the atomics give; sums are integers.
// A workgroup takes a tile of kGatherTile consecutive rows and sorts it by node
// in LDS first (rank of every row among the tile's rows of its node, one LDS
// atomic per distinct node of a wave; start of every node inside the tile by a
// scan; one global cursor atomic per node present in the tile), so that the
// tile's rows of one node go to consecutive places of the staging buffer and a
// wave writes runs of them instead of 64 single words: with every lane of a
// wave writing its own row to wherever its node's cursor stood, a store touched
// 64 lines for 256 bytes (measured 1.8 ms per block of 4 M rows x 128
// features, 0.3 TB/s).
// grid ceil(rows / kGatherTile), 1024 threads; LDS: GatherLdsBytes(L).
constexpr unsigned kGatherTile = 8192;
constexpr int kGatherPerThread = kGatherTile / 1024;
inline size_t GatherLdsBytes(int L) { return (size_t)2 * kGatherTile * 4 + (size_t)3 * L * 4 + 64; }

template <bool PAIR>
__global__ void __launch_bounds__(1024)
k_stream_gather(const uint32_t *__restrict__ bins, size_t bstride, int Q, unsigned rows,
                const float *__restrict__ g, const float *__restrict__ h,
                const unsigned *__restrict__ node_of, int level, int trick,
                const NodeSum *__restrict__ tot, unsigned *__restrict__ cursor,
                uint32_t *__restrict__ st_bins, size_t sstride, float *__restrict__ st_g,
                float *__restrict__ st_h) {
  extern __shared__ unsigned s_gather[];
  const int L = 1 << level;
  unsigned *s_src = s_gather;                 // row of the block at every sorted place of the tile
  unsigned *s_dst = s_src + kGatherTile;      // its place in the staging buffer
  unsigned *s_cnt = s_dst + kGatherTile;      // rows of the tile per node
  unsigned *s_start = s_cnt + L;              // first sorted place of every node
  unsigned *s_base = s_start + L;             // first staging place claimed for the tile's rows of every node
  unsigned *s_misc = s_base + L;              // [0..15] wave sums, [16] carry
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const unsigned tile0 = blockIdx.x * kGatherTile;
  for (int i = tid; i < L; i += 1024) s_cnt[i] = 0;
  if (tid == 0) s_misc[16] = 0;
  __syncthreads();
  unsigned nd[kGatherPerThread], rk[kGatherPerThread];
  unsigned built_mask = 0;
#pragma unroll
  for (int k = 0; k < kGatherPerThread; ++k) {
    const unsigned r = tile0 + (unsigned)k * 1024u + (unsigned)tid;  // whole waves stay together
    nd[k] = 0;
    rk[k] = 0;
    bool built = false;
    if (r < rows) {
      nd[k] = node_of[r];
      built = NodeIsBuilt(tot, nd[k], level, trick);
    }
    unsigned long long todo = __ballot(built);
    while (todo) {
      const int leader = __ffsll((long long)todo) - 1;
      const unsigned lead_nd = (unsigned)__shfl((int)nd[k], leader);
      const unsigned long long same = __ballot(built && nd[k] == lead_nd);
      unsigned base = 0;
      if (lane == leader) base = atomicAdd(&s_cnt[lead_nd], (unsigned)__popcll(same));
      base = (unsigned)__shfl((int)base, leader);
      if (built && nd[k] == lead_nd) rk[k] = base + RankBelow(same);
      todo &= ~same;
    }
    built_mask |= built ? 1u << k : 0u;
  }
  __syncthreads();
  // exclusive scan of the counts; claims in the staging buffer
  for (int base = 0; base < L; base += 1024) {
    const int i = base + tid;
    const unsigned c = i < L ? s_cnt[i] : 0u;
    unsigned incl = c;
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned o = __shfl_up(incl, off);
      if (lane >= off) incl += o;
    }
    if (lane == 63) s_misc[wave] = incl;
    __syncthreads();
    unsigned off = s_misc[16];
    for (int w = 0; w < wave; ++w) off += s_misc[w];
    if (i < L) {
      s_start[i] = off + incl - c;
      s_base[i] = c ? atomicAdd(&cursor[i], c) : 0u;
    }
    __syncthreads();
    if (tid == 1023) s_misc[16] = off + incl;
    __syncthreads();
  }
  const unsigned total = s_misc[16];
#pragma unroll
  for (int k = 0; k < kGatherPerThread; ++k) {
    if (built_mask >> k & 1u) {
      const unsigned p = s_start[nd[k]] + rk[k];
      s_src[p] = tile0 + (unsigned)k * 1024u + (unsigned)tid;
      s_dst[p] = s_base[nd[k]] + rk[k];
    }
  }
  __syncthreads();
  for (unsigned p = tid; p < total; p += 1024) {
    const unsigned r = s_src[p], d = s_dst[p];
    int q = 0;
    for (; q + 8 <= Q; q += 8) {  // eight loads in flight
      uint32_t v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = bins[(size_t)(q + j) * bstride + r];
#pragma unroll
      for (int j = 0; j < 8; ++j) __builtin_nontemporal_store(v[j], &st_bins[(size_t)(q + j) * sstride + d]);
    }
    for (; q < Q; ++q) __builtin_nontemporal_store(bins[(size_t)q * bstride + r], &st_bins[(size_t)q * sstride + d]);
    st_g[d] = g[r];
    if (PAIR) st_h[d] = h[r];
  }
}

// sibling = parent - built child for every node that was not built directly
__global__ void k_sibling(long long *__restrict__ hg, long long *__restrict__ hh, unsigned long long *__restrict__ hc,
                          const long long *__restrict__ pg, const long long *__restrict__ ph,
                          const unsigned long long *__restrict__ pc, const NodeSum *__restrict__ tot, int level,
                          int nbin_total) {
  const unsigned nd = blockIdx.y;
  if (NodeIsBuilt(tot, nd, level, 1)) return;
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= nbin_total) return;
  const size_t o = (size_t)nd * nbin_total + e, so = (size_t)(nd ^ 1u) * nbin_total + e,
               po = (size_t)(nd >> 1) * nbin_total + e;
  hg[o] = pg[po] - hg[so];
  hh[o] = ph[po] - hh[so];
  hc[o] = pc[po] - hc[so];
}

}  // namespace
}  // namespace arb
#endif  // ARBORETUM_AMD_KERNELS_STREAM_H_
