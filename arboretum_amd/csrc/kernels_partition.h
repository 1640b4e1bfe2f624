// Row partition, the fused partition + histogram pass, slab reduction.
#ifndef ARBORETUM_AMD_KERNELS_PARTITION_H_
#define ARBORETUM_AMD_KERNELS_PARTITION_H_
#include "device_common.h"
#include "kernels_hist.h"
#include "kernels_plan.h"
#include "kernels_split.h"

namespace arb {
namespace {

// ---------------------------------------------------------------- partition
__device__ __forceinline__ bool GoesRight(const uint32_t *__restrict__ bins, size_t stride,
                                          const SplitRec &s, unsigned r, BinCode code = BinCode{2, 8},
                                          int hi_word = -1) {
  // builder.h:107-123: bin >= q + 1 goes right
  if (s.fid < 0) return false;
  const SplitTest t = MakeSplitTest(s, code, hi_word);
  return t.Right(bins[(size_t)t.word * stride + r]);
}

// The 128-row chunks of a work item are cut from its begin rounded down to a
// multiple of 64 rows, so that every wave load is one aligned 256-byte
// segment; the rows in front of the begin (fewer than 64, all in the first
// half of wave 0's first chunk; only the first item of a node has any) belong
// to the node before and are masked.  Measured: an item read from an
// unaligned begin takes 15 % longer, and a pass is as slow as its slowest item.
__device__ __forceinline__ unsigned ChunkOrigin(const WorkItem &it) { return it.begin & ~63u; }

// Rows going left, per (work item, wave range).
__global__ void __launch_bounds__(kHistThreads)
k_part_count(const uint32_t *__restrict__ bins, size_t stride, const SplitRec *__restrict__ split,
             const WorkItem *__restrict__ work, const unsigned *__restrict__ n_work,
             unsigned *__restrict__ wave_left, unsigned *__restrict__ item_left, BinCode code, int hi_word) {
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const SplitRec s = split[it.node];
  const SplitTest test = MakeSplitTest(s, code, hi_word);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned cnt = 0;
  // chunks are cut from the item's begin rounded down to 64 rows (ChunkOrigin)
  const unsigned cb = ChunkOrigin(it);
  if (s.fid < 0) {
    for (unsigned base = cb + wave * kChunkRows; base < it.end; base += kChunkStep)
      cnt += lane == 0 ? min(base + kChunkRows, it.end) - max(base, it.begin) : 0u;
  } else {
    const uint32_t *col = bins + (size_t)test.word * stride;
    // eight chunks (16 loads) in flight per wave: the pass is latency-bound
    constexpr int kBatch = 8;
    for (unsigned base = cb + wave * kChunkRows; base < it.end; base += kBatch * kChunkStep) {
      uint32_t v0[kBatch], v1[kBatch];
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const unsigned r0 = base + k * kChunkStep + lane, r1 = r0 + 64;
        v0[k] = col[min(r0, it.end - 1)];
        v1[k] = col[min(r1, it.end - 1)];
      }
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const unsigned r0 = base + k * kChunkStep + lane, r1 = r0 + 64;
        if (r0 >= it.begin && r0 < it.end) cnt += test.Right(v0[k]) ? 0u : 1u;
        if (r1 < it.end) cnt += test.Right(v1[k]) ? 0u : 1u;
      }
    }
  }
  for (int off = 32; off > 0; off >>= 1) cnt += __shfl_down(cnt, off);
  if (lane == 0) wave_left[(size_t)w * kItemWaves + wave] = cnt;
  // per-item total for the offset computation of later items of the node
  __shared__ unsigned s_cnt[kItemWaves];
  if (lane == 0) s_cnt[wave] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned t = 0;
    for (int k = 0; k < kItemWaves; ++k) t += s_cnt[k];
    item_left[w] = t;
  }
}

// Rows going left in the earlier work items of the same node and in the
// earlier waves of this item.  Called by the whole workgroup; s_tmp holds
// kItemWaves + 1 words.
__device__ __forceinline__ unsigned LeftsBefore(const WorkItem &it, unsigned w, int wave,
                                                const unsigned *__restrict__ wave_left,
                                                const unsigned *__restrict__ item_left,
                                                unsigned *s_tmp) {
  unsigned part = 0;
  for (unsigned k = it.first + threadIdx.x; k < w; k += blockDim.x) part += item_left[k];
  for (int off = 32; off > 0; off >>= 1) part += __shfl_down(part, off);
  if ((threadIdx.x & 63) == 0) s_tmp[threadIdx.x >> 6] = part;
  __syncthreads();
  unsigned before = 0;
  for (int k = 0; k < kItemWaves; ++k) before += s_tmp[k];
  for (int k = 0; k < wave; ++k) before += wave_left[(size_t)w * kItemWaves + k];
  __syncthreads();
  return before;
}

// Number of rows of a work item dealt to the waves before `wave`.
__device__ __forceinline__ unsigned RowsOfEarlierWaves(const WorkItem &it, int wave) {
  const unsigned cb = ChunkOrigin(it);
  const unsigned rows = it.end - cb;  // with the masked rows in front
  const unsigned full = rows / kChunkStep, rem = rows % kChunkStep;  // full rounds, rows of the last partial round
  const unsigned dealt = full * kChunkRows * (unsigned)wave + min(rem, kChunkRows * (unsigned)wave);
  return wave == 0 ? 0u : dealt - (it.begin - cb);
}

// Destination offsets of one wave: its rows going left are packed in order
// from the start of the parent's range (after those of earlier items and
// waves), its rows going right from the start of the right child's range.
__device__ __forceinline__ void WaveOffsets(const WorkItem &it, const SplitRec &s, unsigned start,
                                            unsigned lefts_before, int wave, unsigned *lo, unsigned *ro) {
  const unsigned rows_before = (it.begin - start) + RowsOfEarlierWaves(it, wave);
  *lo = start + lefts_before;
  *ro = start + (unsigned)s.left.c + rows_before - lefts_before;
}

// Rows of this wave going left, counted by the wave itself over its own chunks
// (the fused pass does this instead of a separate counting launch).  The chunks
// are read last one first: the lines the pass reads first are then the ones
// most recently brought into the cache.  Wave-uniform result.
// `col` is the column the decision reads: the split feature's quad, or (HI) test.word.
template <int HI>
__device__ __forceinline__ unsigned CountWaveLefts(const WorkItem &it, const SplitRec &s, const SplitTest &test,
                                                  const uint32_t *__restrict__ col, int wave, int lane) {
  const unsigned cb = ChunkOrigin(it);
  const unsigned wb = cb + (unsigned)wave * kChunkRows, we = it.end;
  unsigned cnt = 0;
  if (wb < we) {
    const int nk = (int)((we - wb + kChunkStep - 1) / kChunkStep);  // chunks of this wave
    if (s.fid < 0) {  // not split: every row stays left
      for (int k = 0; k < nk; ++k) {
        const unsigned base = wb + (unsigned)k * kChunkStep;
        cnt += min(base + kChunkRows, we) - max(base, it.begin);
      }
      return cnt;
    }
    const int fs = 8 * (s.fid & 3);
    // (without ninth bits the byte test is spelled out: the fused pass has no register to spare)
    auto right = [&](uint32_t v) {
      if constexpr (HI != 0) return test.Right(v);
      else return (int)((v >> fs) & 255u) > s.bin;
    };
    constexpr int kBatch = 24;  // loads in flight per wave: all of a typical item at once
    for (int k0 = nk - 1; k0 >= 0; k0 -= kBatch) {
      uint32_t v0[kBatch], v1[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const int k = max(k0 - j, 0);
        const unsigned r0 = wb + (unsigned)k * kChunkStep + lane, r1 = r0 + 64;
        v0[j] = col[min(r0, we - 1)];
        v1[j] = col[min(r1, we - 1)];
      }
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const int k = k0 - j;
        const unsigned r0 = wb + (unsigned)max(k, 0) * kChunkStep + lane, r1 = r0 + 64;
        if (k >= 0 && r0 >= it.begin && r0 < we) cnt += right(v0[j]) ? 0u : 1u;
        if (k >= 0 && r1 < we) cnt += right(v1[j]) ? 0u : 1u;
      }
    }
  }
  for (int off = 32; off > 0; off >>= 1) cnt += __shfl_xor(cnt, off);
  return cnt;
}

// Destination offsets of a wave of the fused pass without a counting launch:
// the waves count their rows going left (CountWaveLefts), the workgroup claims
// its share of the two children's row ranges with one atomic add per child on
// the node's pair of cursors (zero at launch), and the waves take their parts
// in wave order.  The order of the work items inside a child's range depends
// on the order of the claims; no result depends on it (all sums are integers).
// The claims of work item w are kept in item_base[2 w], [2 w + 1]: a matrix
// wider than one LDS histogram takes several launches per level, which must
// all send a row to the same place; only the first one claims (cursor set),
// the others read what it claimed (cursor null).
// Called by the whole workgroup; s_tmp holds kItemWaves + 2 words.
// ClaimWithCount: the same from `mine`, the wave's own count of its rows going left.
__device__ __forceinline__ void ClaimWithCount(const WorkItem &it, unsigned w, const SplitRec &s, unsigned start,
                                               unsigned mine, unsigned *__restrict__ cursor,
                                               unsigned *__restrict__ item_base, int wave, int lane,
                                               unsigned *s_tmp, unsigned *lo, unsigned *ro) {
  if (lane == 0) s_tmp[wave] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    if (cursor != nullptr) {
      unsigned lefts = 0;
      for (int k = 0; k < kItemWaves; ++k) lefts += s_tmp[k];
      const unsigned rows = it.end - it.begin;
      item_base[2 * w] = s_tmp[kItemWaves] = atomicAdd(&cursor[2 * it.node], lefts);
      item_base[2 * w + 1] = s_tmp[kItemWaves + 1] = atomicAdd(&cursor[2 * it.node + 1], rows - lefts);
    } else {
      s_tmp[kItemWaves] = item_base[2 * w];
      s_tmp[kItemWaves + 1] = item_base[2 * w + 1];
    }
  }
  __syncthreads();
  unsigned lefts_before = 0;
  for (int k = 0; k < wave; ++k) lefts_before += s_tmp[k];
  const unsigned rows_before = RowsOfEarlierWaves(it, wave);
  *lo = start + s_tmp[kItemWaves] + lefts_before;
  *ro = start + (unsigned)s.left.c + s_tmp[kItemWaves + 1] + rows_before - lefts_before;
}
template <int HI>
__device__ __forceinline__ void ClaimOffsets(const WorkItem &it, unsigned w, const SplitRec &s, const SplitTest &test,
                                             unsigned start,
                                             const uint32_t *__restrict__ col, unsigned *__restrict__ cursor,
                                             unsigned *__restrict__ item_base, int wave, int lane,
                                             unsigned *s_tmp, unsigned *lo, unsigned *ro) {
  ClaimWithCount(it, w, s, start, CountWaveLefts<HI>(it, s, test, col, wave, lane), cursor, item_base, wave, lane,
                 s_tmp, lo, ro);
}

// Destination lane of this lane's row when the rows flagged in the
// wave-uniform mask m are packed, in lane order, into lanes first, first + 1,
// ... (mod 64) of a wave: the flagged rows first, the others behind them, so
// the 64 destinations are a permutation and ds_permute_b32 (every lane sends
// its value to its destination) moves a register in one instruction.
__device__ __forceinline__ int PackedLane(unsigned long long m, unsigned first, int lane) {
  const unsigned below = RankBelow(m);  // flagged rows in the lanes below this one
  const bool mine = (m >> lane) & 1ull;
  const unsigned pos = mine ? below : (unsigned)__popcll(m) + ((unsigned)lane - below);
  return (int)((first + pos) & 63u);
}
// x of every lane to lane `dst` (a permutation of the lanes).
__device__ __forceinline__ uint32_t SendTo(int dst, uint32_t x) {
  return (uint32_t)__builtin_amdgcn_ds_permute(dst << 2, (int)x);
}

// Two rows per lane of a wave's 128-row chunk, as loaded.
template <int NQ>
struct RowSet {
  uint32_t b0[NQ], b1[NQ];
  uint32_t s0, s1;  // word of the split feature when it is not among b0/b1
  float g0, g1, h0, h1;
};

// A wave's register-resident queue of rows on their way to one child's row
// range: lane l holds the row whose destination is base + l, lanes [0, n) are
// occupied, and on a wave's first batch lanes [0, skip) stand for the rows
// before the wave's own range (base is a multiple of 64 rows, so every batch
// is written as one aligned, fully coalesced 256-byte store per array).
// The first batch of a wave is partial when its range does not start on a
// multiple of 64 rows: the other part of that 64-row block is the end of the
// range of the wave before.  Such a first batch is kept (hb, hg: "head") and
// written when the wave is done, next to its last, also partial batch: the two
// halves of a block then reach memory close together, which measured 5 % on
// the fused pass against writing the head when it is complete.  Only kept
// where a row has one gradient word (HeadKept).
template <int NQ>
struct RowQueue {
  uint32_t b[NQ];
  float g, h;
  unsigned n, skip, base;
  uint32_t hb[NQ];
  float hg;
  unsigned hskip, hbase;  // hskip == 64: no head kept
  __device__ __forceinline__ void Init(unsigned first_row) {
#pragma unroll
    for (int q = 0; q < NQ; ++q) b[q] = hb[q] = 0;
    g = h = hg = 0.0f;
    n = skip = first_row & 63u;
    base = first_row - n;
    hskip = 64u;
    hbase = 0u;
  }
};
// (nor with a ninth-bit word: nine more registers per queue do not fit)
template <bool PAIR, bool PACK, int HI = 0>
constexpr bool HeadKept() { return (!PAIR || PACK) && HI == 0; }

// Writes lanes [from, to) of Q to their destination and, for the child whose
// histogram is built, adds them to the LDS histogram.
// HIST: the kernel builds a histogram; GH: the gradients move with the rows;
// PACK: Q.g holds packed logistic gradients (PackGrad), there is no h array.
// NQ quads and, with HI, the ninth-bit word behind them (moved like a quad).
template <bool PAIR, int NQ, bool HIST = true, bool GH = true, bool PACK = false, int HI = 0>
__device__ __forceinline__ void EmitRows(unsigned long long *__restrict__ lds, const RowQueue<NQ + HI> &Q,
                                         unsigned from, unsigned to, bool built,
                                         uint32_t *__restrict__ bins_out, size_t stride,
                                         float *__restrict__ g_out, float *__restrict__ h_out, int lane,
                                         int sg, int sh, int F) {
  if ((unsigned)lane >= from && (unsigned)lane < to) {
    // streaming stores and loads: the pass touches every byte once
    const unsigned d = Q.base + (unsigned)lane;
#pragma unroll
    for (int q = 0; q < NQ + HI; ++q) __builtin_nontemporal_store(Q.b[q], &bins_out[(size_t)q * stride + d]);
    if (GH && g_out != nullptr) {  // a group pass after the first leaves the gradients alone
      __builtin_nontemporal_store(Q.g, &g_out[d]);
      if (PAIR && !PACK) __builtin_nontemporal_store(Q.h, &h_out[d]);
    }
    if (HIST && built) {
      float gv = Q.g, hv = Q.h;
      if (PACK) UnpackGrad(Q.g, &gv, &hv);
      AccumulateRow<PAIR, NQ, HI>(lds, Q.b, gv, hv, sg, sh, 0, F);
    }
  }
}

// The kept first batch of a wave (plain stores: it is about to be completed by
// a neighbour), then what is left in the queue.
template <bool PAIR, int NQ, bool HIST = true, bool GH = true, bool PACK = false, int HI = 0>
__device__ __forceinline__ void FlushQueue(unsigned long long *__restrict__ lds, const RowQueue<NQ + HI> &Q, bool built,
                                           uint32_t *__restrict__ bins_out, size_t stride,
                                           float *__restrict__ g_out, float *__restrict__ h_out, int lane,
                                           int sg, int sh, int F) {
  if (HeadKept<PAIR, PACK, HI>() && (unsigned)lane >= Q.hskip) {
    const unsigned d = Q.hbase + (unsigned)lane;
#pragma unroll
    for (int q = 0; q < NQ + HI; ++q) bins_out[(size_t)q * stride + d] = Q.hb[q];
    if (GH && g_out != nullptr) g_out[d] = Q.hg;
  }
  EmitRows<PAIR, NQ, HIST, GH, PACK, HI>(lds, Q, Q.skip, Q.n, built, bins_out, stride, g_out, h_out, lane, sg, sh, F);
}

// Appends the rows of X flagged in xm (wave-uniform mask, one row per lane) to
// Q in row order with one lane permute (ds_permute_b32) per register; a full queue is emitted
// and the rest of X starts the next batch.
template <bool PAIR, int NQ, bool HIST = true, bool GH = true, bool PACK = false, int HI = 0>
__device__ __forceinline__ void MergeRows(unsigned long long *__restrict__ lds, RowQueue<NQ + HI> &Q,
                                          const uint32_t (&xb)[NQ + HI], float xg, float xh,
                                          unsigned long long xm, bool built,
                                          uint32_t *__restrict__ bins_out, size_t stride,
                                          float *__restrict__ g_out, float *__restrict__ h_out, int lane,
                                          int sg, int sh, int F) {
  const unsigned nx = (unsigned)__popcll(xm);
  if (nx == 0) return;  // wave-uniform
  // lane l receives the k-th flagged row, k = (l - n) mod 64: lanes >= n fill
  // the current batch, lanes < n hold what overflows into the next one
  const unsigned k = ((unsigned)lane - Q.n) & 63u;
  const int dst = PackedLane(xm, Q.n, lane);
  constexpr int NW = NQ + HI;
  uint32_t vb[NW];
#pragma unroll
  for (int q = 0; q < NW; ++q) vb[q] = SendTo(dst, xb[q]);
  const float vg = GH ? __uint_as_float(SendTo(dst, __float_as_uint(xg))) : 0.0f;
  const float vh = GH && PAIR && !PACK ? __uint_as_float(SendTo(dst, __float_as_uint(xh))) : 0.0f;
  if (Q.n + nx >= 64u) {  // wave-uniform: the batch is complete
    const bool fill = (unsigned)lane >= Q.n;
#pragma unroll
    for (int q = 0; q < NW; ++q) Q.b[q] = fill ? vb[q] : Q.b[q];
    Q.g = fill ? vg : Q.g;
    Q.h = fill ? vh : Q.h;
    if (HeadKept<PAIR, PACK, HI>() && Q.skip != 0u) {  // wave-uniform: the wave's first, partial batch
#pragma unroll
      for (int q = 0; q < NW; ++q) Q.hb[q] = Q.b[q];
      Q.hg = Q.g;
      Q.hskip = Q.skip;
      Q.hbase = Q.base;
      if (HIST && built && (unsigned)lane >= Q.skip) {
        float gv = Q.g, hv = 0.0f;
        if (PACK) UnpackGrad(Q.g, &gv, &hv);
        AccumulateRow<PAIR, NQ, HI>(lds, Q.b, gv, hv, sg, sh, 0, F);
      }
    } else {
      EmitRows<PAIR, NQ, HIST, GH, PACK, HI>(lds, Q, Q.skip, 64u, built, bins_out, stride, g_out, h_out, lane, sg, sh, F);
    }
    Q.base += 64u;
    Q.skip = 0u;
#pragma unroll
    for (int q = 0; q < NW; ++q) Q.b[q] = vb[q];
    Q.g = vg;
    Q.h = vh;
    Q.n = Q.n + nx - 64u;
  } else {
    const bool fill = (unsigned)lane >= Q.n && k < nx;
#pragma unroll
    for (int q = 0; q < NW; ++q) Q.b[q] = fill ? vb[q] : Q.b[q];
    Q.g = fill ? vg : Q.g;
    Q.h = fill ? vh : Q.h;
    Q.n += nx;
  }
}

// Fused pass over the rows of the parent nodes of a level: stable partition
// into the children order (WRITE) and histogram of the smaller child of every
// split in LDS.  Each wave owns the 128-row chunks v, v + 16, ... of the item
// and runs without workgroup barriers.  With WRITE the rows of a chunk are
// sorted into two register queues (one per child) with lane permutes; a full
// queue is one aligned 64-row store per array, and the queue of the built
// child is added to the histogram as a full wave (LDS atomic instructions
// cost the same with one active lane as with 64).  Writing each chunk's rows
// directly, as two short unaligned runs per store, costs 40 % more time than
// the copy itself.  On the last level only the quad of the split feature is
// read for every row; the selected rows are queued by row id and read 64 at a
// time.  NQ = all quads of the matrix.
// GROUP: `bins` / `bins_out` point at quad q0 of a wider matrix (q0 a multiple
// of 4); the quad of the split feature is read from `split_bins`, the start of
// the whole matrix, and g_out may be null (the gradients moved with an
// earlier group of the same level).
// PACK (with PAIR): g holds packed logistic gradients (PackGrad); h and h_out
// are not touched.
// HI (not with GROUP): column NQ of the rows is their ninth-bit word (SplitTest);
// it moves with the quads, and ids of 256 are accumulated in a 257th row of
// entries of the LDS histogram and of the slab.
// Without GROUP the splits of the parents are not read from `split` but selected
// here, from the candidates of the split scan (`scan`, LevelScan): no selection
// kernel runs between the split scan of a level and this pass.  (With HI the
// choice is also made at run time, on scan.cand: the register allocation of
// that instance happens to come out with fewer spills that way, 8 bytes per
// lane against 52.)
template <bool PAIR, int NQ, bool WRITE, bool GROUP = false, bool PACK = false, int HI = 0>
__global__ void __launch_bounds__(kHistThreads)
k_part_hist(const uint32_t *__restrict__ bins, uint32_t *__restrict__ bins_out, size_t stride, int F,
            const float *__restrict__ g, float *__restrict__ g_out, const float *__restrict__ h,
            float *__restrict__ h_out, const int *__restrict__ shifts,
            const SplitRec *__restrict__ split, const NodeSum *__restrict__ tot,
            const unsigned *__restrict__ seg_start, const WorkItem *__restrict__ work,
            const unsigned *__restrict__ n_work, unsigned *__restrict__ cursor,
            unsigned *__restrict__ item_base, unsigned long long *__restrict__ slab,
            int slab_entries, const uint32_t *__restrict__ split_bins, int q0, const LevelScan scan) {
  extern __shared__ unsigned long long lds[];
  __shared__ unsigned s_tmp[kItemWaves + 2];
  __shared__ SplitRec s_rec;
  const unsigned w = blockIdx.x;
  const bool own_scan = !GROUP && (HI == 0 || scan.cand != nullptr);  // uniform over the launch
  if (own_scan && w == 0) WriteEmptyNodes(scan, tot, seg_start);
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const SplitRec s = own_scan ? SelectInPass(scan, (int)it.node, tot[it.node], seg_start,
                                             w == scan.node_first[it.node], &s_rec)
                              : split[it.node];
  const unsigned long long cl = s.left.c, cr = tot[it.node].c - cl;
  const bool build_right = cl > cr;  // ties -> left (hist_grad_sum.cu:288-290)
  static_assert(!(HI && GROUP), "ninth bits: one group of quads only");
  constexpr int NW = NQ + HI;  // words of a row
  constexpr int words = (int)(HistLdsBytes(NQ, PAIR, HI != 0) / 8);
  for (int i = threadIdx.x; i < words; i += kHistThreads) lds[i] = 0ull;
  const int sg = shifts[0], sh = shifts[1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const unsigned wb = ChunkOrigin(it) + wave * kChunkRows, we = it.end;
  // which word of a row decides, and how (HI: the ninth-bit word for a split at bin 255; without
  // ninth bits the byte test is spelled out, the pass has no register to spare)
  const SplitTest test = MakeSplitTest(s, BinCode{2, 8}, HI ? NQ : -1);
  const int fq = HI ? test.word : (s.fid < 0 ? 0 : s.fid >> 2), fs = 8 * (s.fid & 3);
  auto goes_right = [&](uint32_t v) {
    if constexpr (HI != 0) return test.Right(v);
    else return s.fid >= 0 && (int)((v >> fs) & 255u) > s.bin;
  };
  unsigned lo = 0, ro = 0;
  if (WRITE)
    ClaimOffsets<HI>(it, w, s, test, seg_start[it.node], split_bins + (size_t)fq * stride, cursor, item_base,
                     wave, lane, s_tmp, &lo, &ro);
  __syncthreads();
  if constexpr (WRITE) {
    // QB: rows of the child whose histogram is built, QO: the other child
    RowQueue<NW> QB, QO;
    QB.Init(build_right ? ro : lo);
    QO.Init(build_right ? lo : ro);
    // Two register sets of 128 rows each: while one is processed the other is
    // in flight.  The loads are unconditional (addresses clamped to the last
    // row of the item) and the sets are never copied, so every wait in the loop
    // is for exactly the set that is needed next.
    const uint32_t *split_col = split_bins + (size_t)fq * stride;
    auto load = [&](RowSet<NW> &R, unsigned base) {
      const unsigned a0 = min(base + lane, we - 1), a1 = min(base + 64 + lane, we - 1);
#pragma unroll
      for (int q = 0; q < NW; ++q) {
        R.b0[q] = __builtin_nontemporal_load(&bins[(size_t)q * stride + a0]);
        R.b1[q] = __builtin_nontemporal_load(&bins[(size_t)q * stride + a1]);
      }
      if (GROUP) {  // the quad of the split feature, wherever it lives
        R.s0 = split_col[a0];
        R.s1 = split_col[a1];
      }
      R.g0 = __builtin_nontemporal_load(&g[a0]);
      R.g1 = __builtin_nontemporal_load(&g[a1]);
      R.h0 = PAIR && !PACK ? __builtin_nontemporal_load(&h[a0]) : 0.0f;
      R.h1 = PAIR && !PACK ? __builtin_nontemporal_load(&h[a1]) : 0.0f;
    };
    auto process = [&](const RowSet<NW> &R, unsigned base) {
      const unsigned r0 = base + lane, r1 = r0 + 64;
      const bool v0 = r0 >= it.begin && r0 < we, v1 = r1 < we;
      uint32_t s0 = 0, s1 = 0;
      if (GROUP) {
        s0 = R.s0;
        s1 = R.s1;
      } else {
#pragma unroll
        for (int q = 0; q < NW; ++q) {
          s0 = q == fq ? R.b0[q] : s0;
          s1 = q == fq ? R.b1[q] : s1;
        }
      }
      const bool right0 = v0 && goes_right(s0);
      const bool right1 = v1 && goes_right(s1);
      const unsigned long long b0 = __ballot(v0 && right0 == build_right), o0 = __ballot(v0 && right0 != build_right);
      const unsigned long long b1 = __ballot(v1 && right1 == build_right), o1 = __ballot(v1 && right1 != build_right);
      MergeRows<PAIR, NQ, true, true, PACK, HI>(lds, QO, R.b0, R.g0, R.h0, o0, false, bins_out, stride, g_out, h_out, lane, sg, sh, F);
      MergeRows<PAIR, NQ, true, true, PACK, HI>(lds, QB, R.b0, R.g0, R.h0, b0, true, bins_out, stride, g_out, h_out, lane, sg, sh, F);
      MergeRows<PAIR, NQ, true, true, PACK, HI>(lds, QO, R.b1, R.g1, R.h1, o1, false, bins_out, stride, g_out, h_out, lane, sg, sh, F);
      MergeRows<PAIR, NQ, true, true, PACK, HI>(lds, QB, R.b1, R.g1, R.h1, b1, true, bins_out, stride, g_out, h_out, lane, sg, sh, F);
    };
    if (wb < we) {
      RowSet<NW> A, B;
      load(A, wb);
      for (unsigned base = wb;; base += 2 * kChunkStep) {
        load(B, base + kChunkStep);
        process(A, base);
        if (base + kChunkStep >= we) break;  // wave-uniform
        load(A, base + 2 * kChunkStep);
        process(B, base + kChunkStep);
        if (base + 2 * kChunkStep >= we) break;
      }
    }
    FlushQueue<PAIR, NQ, true, true, PACK, HI>(lds, QO, false, bins_out, stride, g_out, h_out, lane, sg, sh, F);
    FlushQueue<PAIR, NQ, true, true, PACK, HI>(lds, QB, true, bins_out, stride, g_out, h_out, lane, sg, sh, F);
  } else {
    // Rows selected for the histogram are queued by row id (slot 64 * j + lane
    // of the queue is lane `lane` of q[j]; slots [0, np) are occupied) and read
    // again 64 at a time: LDS atomic instructions cost the same with one active
    // lane as with 64, so only full waves are accumulated.  The second read
    // hits the cache, is requested at the start of a chunk and used at its end,
    // and the wave never waits for its LDS atomics.
    unsigned q0 = it.begin, q1 = it.begin, q2 = it.begin;
    unsigned np = 0;
    uint32_t gb[NW];
    float gg = 0.0f, gh = 0.0f;
    auto gather = [&](bool valid) {  // requests the rows of queue slots [0, 64)
      const unsigned a = valid ? q0 : it.begin;
#pragma unroll
      for (int q = 0; q < NW; ++q) gb[q] = bins[(size_t)q * stride + a];
      gg = g[a];
      gh = PAIR && !PACK ? h[a] : 0.0f;
      q0 = q1;
      q1 = q2;
    };
    // m: wave-uniform mask of the selected rows among base + [0, 64); np < 128
    auto enqueue = [&](unsigned base, unsigned long long m) {
      const unsigned nx = (unsigned)__popcll(m);
      if (nx == 0) return;
      const unsigned r = np & 63u, j = np >> 6;
      const unsigned k = ((unsigned)lane - r) & 63u;  // slot np + k
      const unsigned id = SendTo(PackedLane(m, r, lane), base + (unsigned)lane);
      const bool here = (unsigned)lane >= r && k < nx;   // lands in q[j]
      const bool next = (unsigned)lane < r && k < nx;    // lands in q[j + 1]
      q0 = (j == 0 && here) ? id : q0;
      q1 = ((j == 1 && here) || (j == 0 && next)) ? id : q1;
      q2 = (j == 1 && next) ? id : q2;
      np += nx;
    };
    // after a chunk: at most 127 rows stay queued
    auto drain = [&](unsigned limit) {
      while (np > limit) {
        const unsigned take = min(np, 64u);
        const bool valid = (unsigned)lane < take;
        gather(valid);
        if (PACK) UnpackGrad(gg, &gg, &gh);
        if (valid) AccumulateRow<PAIR, NQ, HI>(lds, gb, gg, gh, sg, sh, 0, F);
        np -= take;
      }
    };
    if (wb < we) {
      // last level: only the quad of the split feature decides; the selected
      // rows are read when they are accumulated
      const uint32_t *col = split_bins + (size_t)fq * stride;
      auto step = [&](uint32_t s0, uint32_t s1, uint32_t &n0, uint32_t &n1, unsigned base) {
        const bool full = np >= 64u;  // wave-uniform
        if (full) {
          gather(true);
          np -= 64u;
        }
        n0 = col[min(base + kChunkStep + lane, we - 1)];
        n1 = col[min(base + kChunkStep + 64 + lane, we - 1)];
        const unsigned r0 = base + lane, r1 = r0 + 64;
        const bool v0 = r0 >= it.begin && r0 < we, v1 = r1 < we;
        const bool right0 = v0 && goes_right(s0);
        const bool right1 = v1 && goes_right(s1);
        enqueue(base, __ballot(v0 && right0 == build_right));
        enqueue(base + 64, __ballot(v1 && right1 == build_right));
        if (full) {
          if (PACK) UnpackGrad(gg, &gg, &gh);
          AccumulateRow<PAIR, NQ, HI>(lds, gb, gg, gh, sg, sh, 0, F);
        }
        drain(127u);
      };
      uint32_t a0 = col[min(wb + lane, we - 1)], a1 = col[min(wb + 64 + lane, we - 1)], b0, b1;
      for (unsigned base = wb;; base += 2 * kChunkStep) {
        step(a0, a1, b0, b1, base);
        if (base + kChunkStep >= we) break;  // wave-uniform
        step(b0, b1, a0, a1, base + kChunkStep);
        if (base + 2 * kChunkStep >= we) break;
      }
    }
    drain(0u);
  }
  FlushSlab<PAIR, NQ, HI>(lds, slab, w, slab_entries, q0);
}

// Stable partition alone (matrices too wide for the fused pass, 16-bit bins):
// words [q0, q0 + NQ) of every row, and with GH the gradients, go to the
// children order through the two register queues of the fused pass.  One launch
// per group of words; every launch reads the word of the split feature again.
template <bool PAIR, int NQ, bool GH>
__global__ void __launch_bounds__(kHistThreads)
k_part_rows(const uint32_t *__restrict__ bins, uint32_t *__restrict__ bins_out, size_t stride, int q0,
            const float *__restrict__ g, float *__restrict__ g_out, const float *__restrict__ h,
            float *__restrict__ h_out, const SplitRec *__restrict__ split,
            const unsigned *__restrict__ seg_start, const WorkItem *__restrict__ work,
            const unsigned *__restrict__ n_work, const unsigned *__restrict__ wave_left,
            const unsigned *__restrict__ item_left, BinCode code, int hi_word) {
  __shared__ unsigned s_tmp[kItemWaves + 1];
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const SplitRec s = split[it.node];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const unsigned wb = ChunkOrigin(it) + wave * kChunkRows, we = it.end;
  unsigned lo, ro;
  const unsigned before = LeftsBefore(it, w, wave, wave_left, item_left, s_tmp);
  WaveOffsets(it, s, seg_start[it.node], before, wave, &lo, &ro);
  if (wb >= we) return;
  const uint32_t *group = bins + (size_t)q0 * stride;
  uint32_t *group_out = bins_out + (size_t)q0 * stride;
  const SplitTest test = MakeSplitTest(s, code, hi_word);
  const uint32_t *split_col = bins + (size_t)test.word * stride;
  RowQueue<NQ> QL, QR;
  QL.Init(lo);
  QR.Init(ro);
  struct Rows {
    RowSet<NQ> r;
    uint32_t s0, s1;  // word of the split feature
  };
  auto load = [&](Rows &R, unsigned base) {
    const unsigned a0 = min(base + lane, we - 1), a1 = min(base + 64 + lane, we - 1);
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      R.r.b0[q] = __builtin_nontemporal_load(&group[(size_t)q * stride + a0]);
      R.r.b1[q] = __builtin_nontemporal_load(&group[(size_t)q * stride + a1]);
    }
    R.s0 = split_col[a0];
    R.s1 = split_col[a1];
    R.r.g0 = GH ? __builtin_nontemporal_load(&g[a0]) : 0.0f;
    R.r.g1 = GH ? __builtin_nontemporal_load(&g[a1]) : 0.0f;
    R.r.h0 = GH && PAIR ? __builtin_nontemporal_load(&h[a0]) : 0.0f;
    R.r.h1 = GH && PAIR ? __builtin_nontemporal_load(&h[a1]) : 0.0f;
  };
  auto process = [&](const Rows &R, unsigned base) {
    const unsigned r0 = base + lane, r1 = r0 + 64;
    const bool v0 = r0 >= it.begin && r0 < we, v1 = r1 < we;
    const bool right0 = v0 && test.Right(R.s0);
    const bool right1 = v1 && test.Right(R.s1);
    const unsigned long long lm0 = __ballot(v0 && !right0), rm0 = __ballot(right0);
    const unsigned long long lm1 = __ballot(v1 && !right1), rm1 = __ballot(right1);
    MergeRows<PAIR, NQ, false, GH>(nullptr, QL, R.r.b0, R.r.g0, R.r.h0, lm0, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
    MergeRows<PAIR, NQ, false, GH>(nullptr, QR, R.r.b0, R.r.g0, R.r.h0, rm0, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
    MergeRows<PAIR, NQ, false, GH>(nullptr, QL, R.r.b1, R.r.g1, R.r.h1, lm1, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
    MergeRows<PAIR, NQ, false, GH>(nullptr, QR, R.r.b1, R.r.g1, R.r.h1, rm1, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
  };
  Rows A, B;
  load(A, wb);
  for (unsigned base = wb;; base += 2 * kChunkStep) {
    load(B, base + kChunkStep);
    process(A, base);
    if (base + kChunkStep >= we) break;  // wave-uniform
    load(A, base + 2 * kChunkStep);
    process(B, base + kChunkStep);
    if (base + 2 * kChunkStep >= we) break;
  }
  FlushQueue<PAIR, NQ, false, GH>(nullptr, QL, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
  FlushQueue<PAIR, NQ, false, GH>(nullptr, QR, false, group_out, stride, g_out, h_out, lane, 0, 0, 0);
}

// Adds the slabs of every directly built node of a level (on top of the stored
// histogram when `accumulate`) and, with `trick`, derives its sibling as
// parent - node.  Slabs are in LDS order (HistLds; `entry` below counts
// k * 4096 + bin * 16 + f16 over all blocks of the matrix); the histograms
// written here are feature-major: hist[node][f * 256 + bin].
// grid (slab_entries/64, L), 1024 threads = 64 entries x 16 slab lanes.
//   by_parent = 0: slabs belong to work items of the node itself
//               (node_items == 0xffffffff marks a derived node);
//   by_parent = 1: slabs belong to work items of the parent (fused pass); the
//               built child is the smaller one, ties -> left.
// hi_base > 0: the slabs hold one more row of entries, bin 256 of every feature
// (matrices with a ninth-bit word); one more block of the grid (the last one)
// reduces it into cell hi_base + f of the node's histogram, behind the 256-bin
// histograms of the features.
// Work plan of the next fused pass, made by one more block of the slab reduction (the ranges of
// the nodes are known since their parents were split): work == null, none.  node_first /
// node_items must be other arrays than the ones this reduction reads.
struct NextPlan {
  const NodeSum *tot = nullptr;
  const unsigned *seg_start = nullptr;
  int L = 0;
  unsigned rows_per_item = 0;
  WorkItem *work = nullptr;
  unsigned *n_work = nullptr, *node_first = nullptr, *node_items = nullptr;
  unsigned max_items = 0;
  unsigned *overflow = nullptr, *cursor = nullptr;
};

// CNT: type of the row counts of the node histograms.  The tree builder keeps
// 64-bit counts: a streamed matrix may hold 2^32 rows and more, all of which can
// sit in one cell (a constant feature, the bin of the missing values).
template <bool PAIR, int LANES, typename CNT = unsigned>
__global__ void __launch_bounds__(1024)
k_hist_reduce(const unsigned long long *__restrict__ slab, int slab_entries, int nbin_total,
              const unsigned *__restrict__ node_first, const unsigned *__restrict__ node_items,
              int by_parent, const SplitRec *__restrict__ parent_split,
              const NodeSum *__restrict__ parent_tot, long long *__restrict__ hg,
              long long *__restrict__ hh, CNT *__restrict__ hc,
              const long long *__restrict__ pg, const long long *__restrict__ ph,
              const CNT *__restrict__ pc, int trick, int accumulate, int plain, int group_blocks,
              int lds_slots = kSlots, int lay_blocks = 0, int hi_base = 0, const NextPlan plan = NextPlan{}) {
  // one more block in the grid's x direction (for node 0 only) cuts the row ranges of this
  // level's nodes into the work items of the fused pass that follows
  if (plan.work != nullptr && blockIdx.x + 1 == gridDim.x) {
    if (blockIdx.y == 0)
      PlanBody(plan.tot, plan.seg_start, plan.L, 0, plan.rows_per_item, plan.work, plan.n_work, plan.node_first,
               plan.node_items, nullptr, nullptr, plan.max_items, plan.overflow, plan.cursor);
    return;
  }
  // LANES threads share the slabs of one entry; a block covers 1024 / LANES
  // consecutive entries (with 4 lanes: 16 bins x 16 features, so the
  // feature-major output is written in runs of 16 bins)
  constexpr int kEntries = 1024 / LANES;
  __shared__ long long s_g[LANES][kEntries];
  __shared__ long long s_h[LANES][kEntries];
  __shared__ unsigned s_c[LANES][kEntries];  // (the slabs of one call hold fewer than 2^32 rows)
  const int nd = blockIdx.y;
  unsigned items, first;
  if (by_parent) {
    const int p = nd >> 1;
    const unsigned long long cl = parent_split[p].left.c, cr = parent_tot[p].c - cl;
    const bool build_right = cl > cr;
    if (((nd & 1) != 0) != build_right) return;  // derived from its sibling
    items = node_items[p];
    first = node_first[p];
  } else {
    items = node_items[nd];
    first = node_first[nd];
    if (items == 0xffffffffu) return;  // derived from its sibling
  }
  const int e = threadIdx.x % kEntries, lane = threadIdx.x / kEntries;
  // slab order; with fewer than 256 bins per feature in the slabs only the first lds_slots * 16
  // entries of every 16-feature block hold anything, and the grid covers only those
  const int per_block = plain ? 1 : (lds_slots * kBlockFeatures + kEntries - 1) / kEntries;
  // the block behind those of the 256 bins takes the row of bin 256: entry e is feature e
  const bool hi_row = hi_base > 0 && (int)blockIdx.x == slab_entries / kBlockEntries * per_block;
  const int entry = hi_row ? e
                    : plain ? (int)blockIdx.x * kEntries + e
                            : ((int)blockIdx.x / per_block) * kBlockEntries + ((int)blockIdx.x % per_block) * kEntries + e;
  // plain: the slabs are feature-major already (16-bit bins)
  const int f = hi_row ? e : (entry / kBlockEntries) * kBlockFeatures + (entry & (kBlockFeatures - 1));
  const int bin = (entry / kBlockFeatures) & (kSlots - 1);
  // the last 16-feature block may have fewer than 16 features
  // lds_slots < 256: the slabs hold that many bins per feature only (the rest are empty)
  const int hist_cells = hi_base > 0 ? hi_base : nbin_total;  // cells of the 256-bin histograms
  const bool live = hi_row ? f < hist_cells / kSlots : (plain ? entry < nbin_total : f * kSlots < hist_cells);
  const bool stored = plain || hi_row || bin < lds_slots;
  // lay_blocks > 0: the slabs are laid out for that many 16-feature blocks (a power of two of
  // bytes between bins), of which the matrix has slab_entries / 4096
  const size_t slab_words = plain ? (size_t)slab_entries * (PAIR ? 2 : 1)
                            : lay_blocks > 0 ? (size_t)lay_blocks * kBlockFeatures * (size_t)lds_slots * (PAIR ? 2 : 1)
                                             : (size_t)slab_entries / kSlots * (size_t)(lds_slots + (hi_base > 0 ? 1 : 0)) * (PAIR ? 2 : 1);
  long long ag = 0, ah = 0;
  unsigned ac = 0;
  if (live) {
    // plain slabs: word0 of every entry, then word1 of every entry; others: the
    // launches of the level (groups of group_blocks blocks, the last one maybe
    // shorter) one after the other, each in its LDS layout
    unsigned i0 = (unsigned)entry, i1 = (unsigned)(slab_entries + entry);
    if (hi_row) {
      // behind the image of the 256 bins, laid out like one more bin
      i0 = (unsigned)slab_entries * (PAIR ? 2u : 1u) + (unsigned)(f / kBlockFeatures) * (PAIR ? 2u : 1u) * kBlockFeatures +
           (unsigned)(f % kBlockFeatures);
      i1 = i0 + kWord1;
    } else if (!plain) {
      const int block = entry / kBlockEntries, group = block / group_blocks;
      const int blocks_here = min(group_blocks, slab_entries / kBlockEntries - group * group_blocks);
      const unsigned in_group = (unsigned)(entry - group * group_blocks * kBlockEntries);
      i0 = (unsigned)(group * group_blocks * kBlockEntries) * (PAIR ? 2u : 1u) +
           HistWord<PAIR>(in_group, lay_blocks > 0 ? lay_blocks : blocks_here);
      i1 = i0 + kWord1;
    }
    for (unsigned s = lane; s < items && stored; s += LANES) {
      const unsigned long long *p = slab + (size_t)(first + s) * slab_words;
      const unsigned long long w0 = p[i0];
      const long long gq = ((long long)(w0 << (64 - kCountShift))) >> (64 - kCountShift);
      ag += gq;
      ac += (unsigned)((w0 - (unsigned long long)gq) >> kCountShift);
      if (PAIR) ah += (long long)p[i1];
    }
  }
  s_g[lane][e] = ag;
  s_h[lane][e] = ah;
  s_c[lane][e] = ac;
  __syncthreads();
  // cells of bins the slabs do not hold are zero in every node histogram, once and for all
  if (lane == 0 && live && stored) {
    for (int k = 1; k < LANES; ++k) {
      ag += s_g[k][e];
      ah += s_h[k][e];
      ac += s_c[k][e];
    }
    const size_t cell = hi_row ? (size_t)hi_base + f : plain ? (size_t)entry : (size_t)f * kSlots + bin;
    const size_t o = (size_t)nd * nbin_total + cell;
    // without hessians (count as hessian) the caller may pass no hh / ph arrays
    const bool with_h = PAIR || hh != nullptr;
    CNT cnt = ac;
    if (accumulate) {  // streamed matrices: one call per row block
      ag += hg[o];
      if (with_h) ah += hh[o];
      cnt += hc[o];
    }
    hg[o] = ag;
    if (with_h) hh[o] = ah;
    hc[o] = cnt;
    if (trick) {
      const size_t po = (size_t)(nd >> 1) * nbin_total + cell;
      const size_t so = (size_t)(nd ^ 1) * nbin_total + cell;
      hg[so] = pg[po] - ag;
      if (with_h) hh[so] = ph[po] - ah;
      hc[so] = pc[po] - cnt;
    }
  }
}

// Root totals = sum over the slots of feature 0 of the root histogram (every
// row, NaN included, sits in exactly one slot).  Replaces the reduction over
// the gradient array of garden.cu:432-435.  One wave.
// hi_cell > 0: the cell of feature 0's bin 256 (matrices with a ninth-bit word).
__global__ void __launch_bounds__(64)
k_root_from_hist(const long long *__restrict__ hg, const long long *__restrict__ hh,
                 NodeSum *__restrict__ tot, int slots, int hi_cell = 0) {
  long long a = 0, b = 0;
  for (int i = threadIdx.x; i < slots; i += 64) {
    a += hg[i];
    b += hh[i];
  }
  if (hi_cell > 0 && threadIdx.x == 0) {
    a += hg[hi_cell];
    b += hh[hi_cell];
  }
  a = WaveSumLL(a);
  b = WaveSumLL(b);
  if (threadIdx.x == 0) {
    tot[0].g = a;
    tot[0].h = b;
  }
}

}  // namespace
}  // namespace arb
#endif  // ARBORETUM_AMD_KERNELS_PARTITION_H_
