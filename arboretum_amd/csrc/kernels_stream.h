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
template <bool PAIR>
__global__ void __launch_bounds__(256)
k_stream_gather(const uint32_t *__restrict__ bins, size_t bstride, int Q, unsigned rows,
                const float *__restrict__ g, const float *__restrict__ h,
                const unsigned *__restrict__ node_of, int level, int trick,
                const NodeSum *__restrict__ tot, unsigned *__restrict__ cursor,
                uint32_t *__restrict__ st_bins, size_t sstride, float *__restrict__ st_g,
                float *__restrict__ st_h) {
  const int lane = threadIdx.x & 63;
  const unsigned step = gridDim.x * blockDim.x;
  for (unsigned r0 = blockIdx.x * blockDim.x; r0 < rows; r0 += step) {  // whole waves stay together
    const unsigned r = r0 + threadIdx.x;
    unsigned nd = 0;
    bool built = false;
    if (r < rows) {
      nd = node_of[r];
      built = NodeIsBuilt(tot, nd, level, trick);
    }
    // one cursor atomic per distinct node of the wave
    unsigned d = 0;
    unsigned long long todo = __ballot(built);
    while (todo) {
      const int leader = __ffsll((long long)todo) - 1;
      const unsigned lead_nd = (unsigned)__shfl((int)nd, leader);
      const unsigned long long same = __ballot(built && nd == lead_nd);
      unsigned base = 0;
      if (lane == leader) base = atomicAdd(&cursor[lead_nd], (unsigned)__popcll(same));
      base = (unsigned)__shfl((int)base, leader);
      if (built && nd == lead_nd) d = base + RankBelow(same);
      todo &= ~same;
    }
    if (built) {
      for (int q = 0; q < Q; ++q) st_bins[(size_t)q * sstride + d] = bins[(size_t)q * bstride + r];
      st_g[d] = g[r];
      if (PAIR) st_h[d] = h[r];
    }
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
