// Kernels for matrices too wide for the fused pass (more than 32 features):
// the rows stay where they are and only (row id, gradients) are re-ordered.
//
// Moving a row of F bin bytes at every level costs 2 F bytes per row and
// level; from a few dozen features on that dominates everything else.  A row
// kept as one contiguous record of at least 128 bytes can be gathered through
// an index list at the rate of a stream (each record fills whole memory
// lines), so for wide matrices the bins are stored a second time row-major
// ("records"), the node order of a level is a list of row ids with the rows'
// gradients beside it, a level's partition moves 12 bytes per row, and the
// histogram kernel gathers the records of the smaller children.
#ifndef ARBORETUM_AMD_KERNELS_INDEXED_H_
#define ARBORETUM_AMD_KERNELS_INDEXED_H_
#include "device_common.h"
#include "kernels_hist.h"
#include "kernels_partition.h"

namespace arb {
namespace {

// Quad columns [Q][stride] -> records [rows][RS] (RS words per row, the words
// past Q zero); the first id_quads of them hold bin ids, four bytes each, whose
// largest is reported (atomic max on *largest_id).  A workgroup transposes 64 rows through LDS: the reads are
// coalesced along the rows, the writes along the record.
__global__ void __launch_bounds__(256)
k_to_records(const uint32_t *__restrict__ bins, size_t stride, int Q, uint32_t *__restrict__ rec, int RS,
             size_t n, int id_quads, unsigned *__restrict__ largest_id) {
  extern __shared__ uint32_t s_tile[];  // [64][RS + 1]
  const size_t r0 = (size_t)blockIdx.x * 64;
  const int lane = threadIdx.x & 63, part = threadIdx.x >> 6;  // 4 parts
  unsigned top = 0;  // the largest bin id (byte) among the words this thread moves
  for (int q = part; q < RS; q += 4) {
    uint32_t v = 0;
    if (q < Q && r0 + lane < n) v = bins[(size_t)q * stride + r0 + lane];
    if (q < id_quads) top = max(max(top, v & 255u), max(max((v >> 8) & 255u, (v >> 16) & 255u), v >> 24));
    s_tile[lane * (RS + 1) + q] = v;
  }
  // (the histogram kernel over the records trusts the ids to be below its number of slots: the
  // caller compares what was seen here with the bound it sizes the histogram by)
  for (int off = 32; off > 0; off >>= 1) top = max(top, (unsigned)__shfl_down((int)top, off));
  if (lane == 0 && top != 0) atomicMax(largest_id, top);
  __syncthreads();
  const size_t rows = min((size_t)64, n - r0);
  for (size_t e = threadIdx.x; e < rows * RS; e += 256) {
    const size_t r = e / RS, q = e % RS;
    rec[(r0 + r) * RS + q] = s_tile[r * (RS + 1) + q];
  }
}

// Quad columns [Q][stride] -> byte columns [4 Q][stride8]: one byte per row and feature, so that
// a 64-byte fetch of a feature's column holds 64 rows instead of 16.
__global__ void __launch_bounds__(256)
k_to_byte_columns(const uint32_t *__restrict__ bins, size_t stride, int Q, uint8_t *__restrict__ bytes,
                  size_t stride8, size_t n) {
  const size_t r = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= n) return;
  for (int q = 0; q < Q; ++q) {
    const uint32_t v = bins[(size_t)q * stride + r];
#pragma unroll
    for (int b = 0; b < 4; ++b) bytes[(size_t)(4 * q + b) * stride8 + r] = (uint8_t)(v >> (8 * b));
  }
}

// Ninth-bit words [H][stride] (bit f % 32 of word f / 32: the id of feature f is 256) -> bit
// columns [F][strideb]: bit r % 8 of byte r / 8 of feature f's column, so that the partition can
// gather the bit of one feature of a row with one byte fetch.
__global__ void __launch_bounds__(256)
k_to_hi_bits(const uint32_t *__restrict__ hi, size_t stride, int F, uint8_t *__restrict__ bits, size_t strideb,
             size_t n) {
  const size_t j = (size_t)blockIdx.x * 256 + threadIdx.x;  // byte of every column: rows 8 j .. 8 j + 7
  if (j * 8 >= n) return;
  for (int w = 0; w * 32 < F; ++w) {
    uint32_t v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = j * 8 + k < n ? hi[(size_t)w * stride + j * 8 + k] : 0u;
    for (int b = 0; b < 32 && w * 32 + b < F; ++b) {
      unsigned byte = 0;
#pragma unroll
      for (int k = 0; k < 8; ++k) byte |= ((v[k] >> b) & 1u) << k;
      bits[(size_t)(w * 32 + b) * strideb + j] = (uint8_t)byte;
    }
  }
}

// Sum of the fixed-point gradients of all rows: the totals of the root when no feature's
// histogram holds every row (ids of 256 are left out of the histograms of matrices with several
// ninth-bit words).  tot[0].g / .h must be zero at launch; integer sums, any order.
__global__ void __launch_bounds__(256)
k_sum_grad(const float *__restrict__ g, const float *__restrict__ h, size_t n, const int *__restrict__ shifts,
           NodeSum *__restrict__ tot) {
  const int sg = shifts[0], sh = shifts[1];
  long long a = 0, b = 0;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    a += ToFixed(g[i], sg);
    if (h != nullptr) b += ToFixed(h[i], sh);
  }
  a = WaveSumLL(a);
  b = WaveSumLL(b);
  if ((threadIdx.x & 63) == 0) {
    atomicAdd(reinterpret_cast<unsigned long long *>(&tot[0].g), (unsigned long long)a);
    if (h != nullptr) atomicAdd(reinterpret_cast<unsigned long long *>(&tot[0].h), (unsigned long long)b);
  }
}

// Partition of (row id, gradients) of the parents of a level into the children order, one launch
// per level, rows in place.  ids: the row at each position (null: position = row, the first
// level).  Each wave first decides its own rows: the split feature's bin of a row is read from
// the byte columns, not from the records (the ids of a node ascend, so the reads of a node walk
// one column forwards, and the deeper the level, the fewer rows of a node share a 64-byte fetch:
// with a byte per row that happens two levels later than with a word per row).  A work item
// holds at most kPartRows rows, eight 128-row chunks per wave, so the sixteen decisions of a
// lane stay in the bits of one register; the workgroup then claims its share of the two
// children's ranges on the node's cursors (ClaimWithCount: zero at launch, the planner clears
// them) and the waves move their rows through the register queues of the row passes: the bin
// is gathered once, and no decision array or counting launch exists.  Within a child the work
// items lie in the order of their claims; no result depends on it (integer sums).
// hibits (may be null): bit columns of the ninth bits (k_to_hi_bits); a split at bin 255 sends
// right exactly the rows whose id is 256.
constexpr int kIxChunks = (int)(kPartRows / kChunkStep);  // chunks of a wave in one work item
static_assert(kIxChunks * 2 <= 32, "a lane's decisions of one work item must fit one register");
template <bool PAIR>
__global__ void __launch_bounds__(kHistThreads)
k_ix_part(const uint8_t *__restrict__ bytes, size_t stride8, const unsigned *__restrict__ ids,
          unsigned *__restrict__ ids_out, const float *__restrict__ g, float *__restrict__ g_out,
          const float *__restrict__ h, float *__restrict__ h_out, const SplitRec *__restrict__ split,
          const unsigned *__restrict__ seg_start, const WorkItem *__restrict__ work,
          const unsigned *__restrict__ n_work, unsigned *__restrict__ cursor, unsigned *__restrict__ item_base,
          const uint8_t *__restrict__ hibits, size_t strideb) {
  __shared__ unsigned s_tmp[kItemWaves + 2];
  const unsigned w = blockIdx.x;
  if (w >= *n_work) return;
  const WorkItem it = work[w];
  const SplitRec s = split[it.node];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const unsigned wb = ChunkOrigin(it) + wave * kChunkRows, we = it.end;
  const bool by_bit = hibits != nullptr && s.bin >= 255;  // uniform: only an id of 256 goes right
  const uint8_t *col = by_bit ? hibits + (size_t)s.fid * strideb : bytes + (size_t)(s.fid < 0 ? 0 : s.fid) * stride8;
  // decisions of this lane's rows: bit 2 k + half = row (chunk k, half) goes right
  unsigned right_bits = 0, lefts = 0;
  if (s.fid >= 0) {
    constexpr int kBatch = 4;  // 8 ids, then 8 gathers in flight per lane
#pragma unroll
    for (int k0 = 0; k0 < kIxChunks; k0 += kBatch) {
      if (wb + (unsigned)k0 * kChunkStep < we) {  // wave-uniform
        unsigned id[2 * kBatch], bin[2 * kBatch];
#pragma unroll
        for (int k = 0; k < 2 * kBatch; ++k) {
          const unsigned r = wb + (unsigned)(k0 + (k >> 1)) * kChunkStep + (k & 1) * 64 + lane;
          const unsigned a = min(r, we - 1);
          id[k] = ids ? ids[a] : a;
        }
#pragma unroll
        for (int k = 0; k < 2 * kBatch; ++k) bin[k] = by_bit ? (col[id[k] >> 3] >> (id[k] & 7u)) & 1u : col[id[k]];
#pragma unroll
        for (int k = 0; k < 2 * kBatch; ++k) {
          const unsigned r = wb + (unsigned)(k0 + (k >> 1)) * kChunkStep + (k & 1) * 64 + lane;
          const bool valid = r >= it.begin && r < we;
          const bool right = by_bit ? bin[k] != 0u : (int)bin[k] > s.bin;  // builder.h:107-123
          right_bits |= (valid && right ? 1u : 0u) << (2 * k0 + k);
          lefts += valid && !right ? 1u : 0u;
        }
      }
    }
  } else {  // not split: every row stays left
#pragma unroll
    for (int k = 0; k < 2 * kIxChunks; ++k) {
      const unsigned r = wb + (unsigned)(k >> 1) * kChunkStep + (k & 1) * 64 + lane;
      lefts += r >= it.begin && r < we ? 1u : 0u;
    }
  }
  for (int off = 32; off > 0; off >>= 1) lefts += __shfl_xor(lefts, off);
  unsigned lo, ro;
  ClaimWithCount(it, w, s, seg_start[it.node], lefts, cursor, item_base, wave, lane, s_tmp, &lo, &ro);
  if (wb >= we) return;
  RowQueue<1> QL, QR;
  QL.Init(lo);
  QR.Init(ro);
  auto load = [&](RowSet<1> &R, unsigned base) {
    const unsigned a0 = min(base + lane, we - 1), a1 = min(base + 64 + lane, we - 1);
    R.b0[0] = ids ? ids[a0] : a0;
    R.b1[0] = ids ? ids[a1] : a1;
    R.g0 = g[a0];
    R.g1 = g[a1];
    R.h0 = PAIR ? h[a0] : 0.0f;
    R.h1 = PAIR ? h[a1] : 0.0f;
  };
  auto process = [&](const RowSet<1> &R, unsigned base, unsigned chunk) {
    const unsigned r0 = base + lane, r1 = r0 + 64;
    const bool v0 = r0 >= it.begin && r0 < we, v1 = r1 < we;
    const bool right0 = (right_bits >> (2u * chunk)) & 1u, right1 = (right_bits >> (2u * chunk + 1u)) & 1u;
    const unsigned long long lm0 = __ballot(v0 && !right0), rm0 = __ballot(v0 && right0);
    const unsigned long long lm1 = __ballot(v1 && !right1), rm1 = __ballot(v1 && right1);
    uint32_t *out = ids_out;
    MergeRows<PAIR, 1, false, true>(nullptr, QL, R.b0, R.g0, R.h0, lm0, false, out, 0, g_out, h_out, lane, 0, 0, 0);
    MergeRows<PAIR, 1, false, true>(nullptr, QR, R.b0, R.g0, R.h0, rm0, false, out, 0, g_out, h_out, lane, 0, 0, 0);
    MergeRows<PAIR, 1, false, true>(nullptr, QL, R.b1, R.g1, R.h1, lm1, false, out, 0, g_out, h_out, lane, 0, 0, 0);
    MergeRows<PAIR, 1, false, true>(nullptr, QR, R.b1, R.g1, R.h1, rm1, false, out, 0, g_out, h_out, lane, 0, 0, 0);
  };
  RowSet<1> A, B;
  load(A, wb);
  unsigned chunk = 0;
  for (unsigned base = wb;; base += 2 * kChunkStep, chunk += 2) {
    load(B, base + kChunkStep);
    process(A, base, chunk);
    if (base + kChunkStep >= we) break;  // wave-uniform
    load(A, base + 2 * kChunkStep);
    process(B, base + kChunkStep, chunk + 1);
    if (base + 2 * kChunkStep >= we) break;
  }
  FlushQueue<PAIR, 1, false, true>(nullptr, QL, false, ids_out, 0, g_out, h_out, lane, 0, 0, 0);
  FlushQueue<PAIR, 1, false, true>(nullptr, QR, false, ids_out, 0, g_out, h_out, lane, 0, 0, 0);
}

// Histogram over records, every feature in one LDS histogram of `slots` bins
// per feature (possible when features x slots is small enough: 200 features of
// 65 bins with one word per cell take 108 KB): the record of a row is read
// once, whole.  The row at position p of a work item is ids[p] (null: p itself),
// its gradients are g[p], h[p].
//
// A lane owns one 16-byte piece of a record, i.e. one 16-feature block of one
// row: the (row, piece) pairs of a work item are dealt to the lanes in row-major
// order, so consecutive lanes read consecutive pieces and a wave's load covers
// whole records as contiguous runs, with every lane busy whatever the number of
// pieces per record.  One row per lane would touch 64 records 16 bytes at a time
// and come back to each of them once per piece, with far more data in flight
// than the caches hold.  The 16 updates of a lane go to features (t + lane) % 16
// of its block in step t, so the 16 lanes of a pass of the LDS atomic unit still
// hit 16 different bank pairs, whatever rows and blocks they own.
//
// A workgroup covers the pieces [piece0, piece0 + npieces) of the records of its work item: all
// of them when the whole histogram fits the LDS at `slots` bins per feature (one group; the slab
// of a work item is the LDS image, item_words its size), else one of `ngroups` groups of
// group_pieces 16-feature blocks at 256 bins per feature; the slab of a work item then holds
// the images of the groups one after the other, as the histogram kernels of row-moving
// matrices write them (item_words = words of all groups).  The grid is ngroups times the number
// of work items rounded up to a multiple of eight.
//
// LDS layout (bin-major, as the other histograms): word0 of (feature f, bin) at
// bin * bin_stride + (f / 16) * (PAIR ? 32 : 16) + f % 16, bin_stride = blocks *
// (PAIR ? 32 : 16), word1 16 words further.  The slab of a work item is
// the LDS image: blocks * 16 * slots entries of one or two words.
// POW2: a power of two of bytes between the bins of the LDS image (stride_shift): the offset of
// a cell is a shift and an add instead of a multiply and an add.  Every bin id is below `slots`:
// the caller sizes the histogram by the largest id the records hold (k_to_records reports it).
// lay_blocks: 16-feature blocks the image is laid out for (0: the pieces of the workgroup's
// group); more than the matrix has makes the stride a power of two.
// HI: words Q, Q + 1, ... of a record are the row's ninth-bit words; a feature whose bit is set
// (id 256) is not accumulated (AccumulateRow, HI = 2).
template <bool PAIR, bool POW2 = false, bool HI = false>
__global__ void __launch_bounds__(kHistThreads)
k_hist_rec(const uint32_t *__restrict__ rec, int RS, const unsigned *__restrict__ ids, int Q, int slots,
           const float *__restrict__ g, const float *__restrict__ h, const int *__restrict__ shifts,
           const WorkItem *__restrict__ work, const unsigned *__restrict__ n_work,
           unsigned long long *__restrict__ slab, int group_pieces, int total_pieces, int ngroups,
           size_t item_words, int lay_blocks) {
  extern __shared__ unsigned long long lds[];
  // Workgroup -> (work item, group of pieces): workgroups are dealt to the eight XCDs in turn
  // (workgroup b runs on XCD b % 8), and the groups of one work item read the same records, so
  // they are given ids that differ by 8: they start together on the same XCD, and what the first
  // of them fetches the others find in that XCD's L2.
  const unsigned xcd = blockIdx.x & 7u, turn = blockIdx.x >> 3;
  const unsigned w = (turn / (unsigned)ngroups) * 8u + xcd;
  if (w >= *n_work) return;
  const int piece0 = (int)(turn % (unsigned)ngroups) * group_pieces;
  const int npieces = min(group_pieces, total_pieces - piece0);
  const WorkItem it = work[w];
  constexpr unsigned per = PAIR ? 2 : 1;
  const unsigned blocks = (unsigned)npieces;
  const unsigned bin_stride = (lay_blocks > 0 ? (unsigned)lay_blocks : blocks) * per * kBlockFeatures;
  const unsigned words = (unsigned)slots * bin_stride;
  for (unsigned i = threadIdx.x; i < words; i += kHistThreads) lds[i] = 0ull;
  __syncthreads();
  const int sg = shifts[0], sh = shifts[1];
  const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const unsigned j = (lane >> 2) & 3u, i4 = lane & 3u;
  // The (row, piece) pairs of the work item, row-major, are dealt out 64 at a time: wave v takes
  // pairs [1024 G + 64 v, + 64) of group G, its lane l the pair 1024 G + 64 v + l.  Every lane has
  // work until the item runs out, however many pieces a record has.
  const unsigned n_rows = it.end - it.begin;
  const unsigned n_pairs = n_rows * blocks;                  // at most 64512 x 64 < 2^22
  const unsigned inv_blocks = (unsigned)(((1ull << 32) + blocks - 1u) / blocks);  // exact quotients below 2^22
  constexpr int kSteps = 4;                       // groups per wave and step
  constexpr unsigned kGroupPairs = kItemWaves * 64u;
  constexpr unsigned kStepPairs = kSteps * kGroupPairs;
  // One step of a wave: the row ids of its kSteps groups, then their record pieces and
  // gradients, then the updates.  The three stages of consecutive steps overlap: while the
  // updates of a step run, the records of the next one and the row ids of the one after are in
  // flight.  Loads are issued for steps that begin inside the work item only, and every address
  // is clamped to a row of the item and a piece of a record.
  struct RowIds { unsigned id[kSteps]; };
  struct Pieces {
    uint4 q[kSteps];
    float gv[kSteps], hv[kSteps];
    unsigned piece[kSteps];
    unsigned ninth[kSteps];  // HI: the ninth bits of the piece's 16 features
    bool v[kSteps];
  };
  // position in the item's row range and piece of this lane's pair in group k of the step at `first`
  auto locate = [&](unsigned first, int k, unsigned *piece, bool *valid) {
    const unsigned pair = first + (unsigned)k * kGroupPairs + wave * 64u + lane;
    *valid = pair < n_pairs;
    const unsigned pr = *valid ? pair : 0u;
    const unsigned rel = min(blocks == 1u ? pr : __umulhi(pr, inv_blocks), n_rows - 1u);   // pair / blocks
    *piece = min(pr - rel * blocks, blocks - 1u);
    return it.begin + rel;
  };
  auto load_ids = [&](unsigned first, RowIds &I) {
#pragma unroll
    for (int k = 0; k < kSteps; ++k) {
      unsigned piece;
      bool valid;
      const unsigned a = locate(first, k, &piece, &valid);
      I.id[k] = ids ? ids[a] : a;
    }
  };
  auto load_pieces = [&](unsigned first, const RowIds &I, Pieces &R) {
#pragma unroll
    for (int k = 0; k < kSteps; ++k) {
      const unsigned a = locate(first, k, &R.piece[k], &R.v[k]);
      R.q[k] = *reinterpret_cast<const uint4 *>(rec + (size_t)I.id[k] * RS + 4u * ((unsigned)piece0 + R.piece[k]));
      if (HI) {
        const unsigned p = (unsigned)piece0 + R.piece[k];
        R.ninth[k] = (rec[(size_t)I.id[k] * RS + (unsigned)Q + (p >> 1)] >> (16u * (p & 1u))) & 0xffffu;
      } else {
        R.ninth[k] = 0u;
      }
      R.gv[k] = g[a];
      R.hv[k] = PAIR ? h[a] : 0.0f;
    }
  };
  unsigned char *lds_b = reinterpret_cast<unsigned char *>(lds);
  const unsigned bin_stride_b = bin_stride * 8u;    // at most 64 x 2 x 16 x 8 = 16 KB
  const unsigned stride_shift = 31u - (unsigned)__clz((int)bin_stride_b);   // POW2: bin_stride_b = 1 << stride_shift
  auto accumulate = [&](const Pieces &R) {
#pragma unroll
    for (int k = 0; k < kSteps; ++k) {
      if (!R.v[k]) continue;
      // byte offsets into the histogram; the products fit 24 bits (v_mad_u32_u24 is a
      // full-rate instruction, a 32-bit multiply takes four times as long)
      const unsigned piece_b = R.piece[k] * (per * kBlockFeatures * 8u);
      const unsigned piece = R.piece[k];
      const unsigned long long w0 = (1ull << kCountShift) + (unsigned long long)ToFixed(R.gv[k], sg);
      const unsigned long long w1 = PAIR ? (unsigned long long)ToFixed(R.hv[k], sh) : 0ull;
#pragma unroll
      for (int s_ = 0; s_ < 4; ++s_) {
        const unsigned qi = ((unsigned)s_ + j) & 3u;   // quad of the block this lane works on
        const uint32_t ra = s_ == 0 ? R.q[k].x : s_ == 1 ? R.q[k].y : s_ == 2 ? R.q[k].z : R.q[k].w;
        const uint32_t rb = s_ == 0 ? R.q[k].y : s_ == 1 ? R.q[k].z : s_ == 2 ? R.q[k].w : R.q[k].x;
        const uint32_t rc = s_ == 0 ? R.q[k].z : s_ == 1 ? R.q[k].w : s_ == 2 ? R.q[k].x : R.q[k].y;
        const uint32_t rd = s_ == 0 ? R.q[k].w : s_ == 1 ? R.q[k].x : s_ == 2 ? R.q[k].y : R.q[k].z;
        const uint32_t lo = (j & 1u) ? rb : ra, hi = (j & 1u) ? rd : rc;
        // the quad, turned so that the byte of step t sits at byte t whatever the lane: the byte
        // is then picked by a constant (an operand modifier of the shift below, not an instruction)
        const uint32_t sel = __builtin_amdgcn_alignbit((j & 2u) ? hi : lo, (j & 2u) ? hi : lo, 8u * i4);
        if (4u * ((unsigned)piece0 + piece) + qi < (unsigned)Q) {   // quads past the matrix do not exist
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const unsigned bi = ((unsigned)t + i4) & 3u;
            unsigned off;
            const unsigned bin = (sel >> (8 * t)) & 255u;
            if (POW2) off = (bin << stride_shift) + (piece_b + (4u * qi + bi) * 8u);
            else off = __umul24(bin, bin_stride_b) + (piece_b + (4u * qi + bi) * 8u);
            unsigned long long *cell = reinterpret_cast<unsigned long long *>(lds_b + off);
            if (HI && ((R.ninth[k] >> (4u * qi + bi)) & 1u)) continue;  // id 256: in no candidate's left side
            atomicAdd(cell, w0);
            if (PAIR) atomicAdd(cell + kWord1, w1);
          }
        }
      }
    }
  };
  if (n_pairs != 0) {                             // uniform over the workgroup, as every branch below
    RowIds I;
    Pieces R;
    load_ids(0u, I);
    load_pieces(0u, I, R);
    unsigned next = kStepPairs;
    if (next < n_pairs) load_ids(next, I);
    for (;;) {
      const bool more = next < n_pairs;
      Pieces N;
      if (more) {
        load_pieces(next, I, N);
        if (next + kStepPairs < n_pairs) load_ids(next + kStepPairs, I);
      }
      accumulate(R);
      if (!more) break;
      R = N;
      next += kStepPairs;
    }
  }
  __syncthreads();
  unsigned long long *out = slab + (size_t)w * item_words + (size_t)piece0 * (kBlockEntries * per);
  for (unsigned e = threadIdx.x; e < words; e += kHistThreads) out[e] = lds[e];
}

}  // namespace
}  // namespace arb
#endif  // ARBORETUM_AMD_KERNELS_INDEXED_H_
