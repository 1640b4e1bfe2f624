/*
 * Entry points of libarboretum.so that have no counterpart in the reference's
 * wrapper (python-wrapper/arboretum_wrapper.h).  They exist for three callers:
 * parity tests (inspection of the device-side state), the benchmark (device
 * timings and work counters) and data that is already quantised (the
 * reference's ABI only takes fp32 rows and an `int` row count).
 * Same convention as arboretum_wrapper.h: NULL on success, else a message.
 */
#ifndef ARBORETUM_EXT_H_
#define ARBORETUM_EXT_H_

#include "arboretum_wrapper.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Number of HIP devices visible (0 on a CPU-only host). */
const char *ADeviceCount(int *out);

/* Runs one plain device-to-device copy kernel (k_copy_probe) of `bytes` bytes:
 * a dispatch of exactly known HBM traffic, against which the FETCH_SIZE /
 * WRITE_SIZE counters of a profile are scaled. */
const char *ADeviceCopyProbe(unsigned long long bytes);

/* Data matrix from bin ids: `bins` row-major uint8 [nrow][ncol], copied.
 * Thresholds are reported as bin + 0.5 and prediction walks the bin ids.
 * Counterpart of the reference's quantised columns (src/io/io.h:65-76), which
 * it can only produce itself from fp32 input. */
const char *ACreateFromQuantized(const unsigned char *bins, long long nrow, int ncol,
                                 VoidPointer *out);

/* Data matrix over bin ids that stay where the caller keeps them: for matrices
 * beyond HBM and beyond the reference's `int nrow` (python-wrapper/
 * arboretum_wrapper.h:6-10 takes one fp32 array and an int row count).  The
 * rows live in `nblocks` caller-owned host blocks of `block_rows` rows (a
 * multiple of 64, below 2^31; the last block may hold fewer: nrow in all, a
 * 64-bit count below 2^33, the limit of the 64-bit integer gradient sums; row
 * counts per histogram cell are 64-bit as well); nothing is copied and nothing
 * is freed with the matrix.
 * Block layout (what the GPU streams as it is): 32-bit words
 * [Q][block_rows], Q = ceil(ncol / 4), word q * block_rows + r = bin ids of
 * features 4 q .. 4 q + 3 of the block's row r, one byte each, lowest byte
 * first.  Allocate the blocks with hipHostMalloc for the full host-to-device
 * rate.  Training needs `internals.upload_features: false` (the blocks are
 * streamed once per tree level); several descriptors may name the same block.
 * Thresholds are reported as bin + 0.5, as for ACreateFromQuantized. */
const char *ACreateFromQuantizedBlocks(const unsigned *const *blocks, int nblocks, long long block_rows,
                                       long long nrow, int ncol, VoidPointer *out);

/* Runs the quantiser now (the reference defers it to the first AGrowTree,
 * src/core/garden.cu:586-589).  Needs a GPU. */
const char *AQuantize(VoidPointer data, int hist_size);

/* Quantiser output: bins as row-major uint8 [nrow][ncol]; thresholds of one
 * feature (hist_size floats, +INF where unset) and its number of real bins
 * (DataMatrix::data_reduced_mapping / reduced_size, src/io/io.h:24,32). */
const char *AGetBins(VoidPointer data, unsigned char *out);
const char *AGetThresholds(VoidPointer data, int fid, float *thr, int *size);
/* Bin ids take 8 bits unless a feature has more than 256 of them (hist_size
 * above 255 on a column with that many distinct values): then 16 bits, as the
 * reference switches BIN_T by hist_size (src/core/garden.cu:506-569).  The one
 * id past a byte that hist_size 256 produces (256 value bins plus the bin of
 * the missing values, src/core/cuda_helpers.h:207-222) is kept beside 8-bit ids
 * as a ninth bit per feature when the matrix has at most 32 features: the
 * layout then reports 8 bits and 257 slots.
 * AGetBinLayout: bits per bin id (8 or 16) and histogram slots per feature;
 * AGetBins16: the bins as row-major uint16 [nrow][ncol] (AGetBins is for 8 bits
 * and 256 slots). */
const char *AGetBinLayout(VoidPointer data, int *bits, int *slots);
const char *AGetBins16(VoidPointer data, unsigned short *out);

/* Where APredict walks the trees (src/core/garden.cu:643-657 does it on the
 * host): on != 0 (default) uses the GPU when a device is present, 0 the host
 * walk.  Both give the same bits. */
const char *AGardenPredictOnDevice(VoidPointer garden, int on);

/* Inspection of the booster; valid after AGrowTree. */
const char *AGardenSetInspect(VoidPointer garden, int on);      /* keep per-level histograms */
const char *AGardenNumTrees(VoidPointer garden, int *out);
/* Tree t: fid/bin/threshold/gain of the 2^(depth-1)-1 internal nodes in heap
 * order (bin -1 = not split), 2^(depth-1) leaf weights.  Any pointer may be
 * NULL.  depth is the tree's own (AGardenGetTreeDepth: max_depth + 1 for a
 * grown tree, the model's "depth" for a loaded one); size the arrays from it. */
const char *AGardenGetTreeDepth(VoidPointer garden, int t, int *depth);
const char *AGardenGetTree(VoidPointer garden, int t, int *fid, int *bin, float *threshold,
                           float *gain, float *weights);
/* Leaf index of every training row in the last tree, original row order
 * (the reference's row2Node, src/core/garden.cu:56,67). */
const char *AGardenGetLeaves(VoidPointer garden, unsigned *out);
/* Device-side y_hat (internal scale) and gradients, class-major [labels][nrow]. */
const char *AGardenGetTrainYHat(VoidPointer garden, float *out);
const char *AGardenGetGrad(VoidPointer garden, float *g, float *h);
/* Fixed-point histogram of one level of the last tree (needs inspect on):
 * int64 [nodes][ncol][256][3] = (sum g_q, sum h_q, count); *cells = nodes*ncol*256. */
const char *AGardenGetLevelHist(VoidPointer garden, int level, long long *out, int *cells);
/* Binary exponents of the fixed-point scale: value = q * 2^-shift. */
const char *AGardenGetShifts(VoidPointer garden, int *shift_g, int *shift_h);

/* Device timings (HIP events on the builder's stream), accumulated since the
 * call that enabled them; `out` holds 16 doubles.  out[0..7] = milliseconds
 * in: gradients, root histogram kernel, deeper-level histogram kernels (the
 * fused partition + histogram kernel where it applies), slab reduce, split
 * scan, partition bookkeeping (left counts, offset scan, stand-alone
 * partition), leaf pass, planning; out[8] = root histogram launches, out[9] =
 * rows read by them, out[10] = deeper-level histogram launches, out[11] =
 * milliseconds in the fused kernel of the last level (it moves no rows),
 * out[12] = its launches.  `on`: 0 = off, 1 = every phase (about 35 event
 * records per tree), 2 = only the deeper-level histogram kernels (out[2] and
 * out[10]; a third of the records), 3 = those on every fourth tree only (for
 * timed runs: the records themselves cost time). */
const char *AGardenEnableTiming(VoidPointer garden, int on);
const char *AGardenGetTimings(VoidPointer garden, double *out);
/* Rows accumulated into histograms so far (x ncol = histogram updates). */
const char *AGardenRowsScanned(VoidPointer garden, unsigned long long *out);
/* The same per tree level: out[32], out[l] = rows accumulated at level l (the
 * root is level 0; levels past 31 share the last entry). */
const char *AGardenRowsScannedByLevel(VoidPointer garden, unsigned long long *out);
/* Streamed matrix (internals.upload_features false): row blocks that stay in
 * device memory and row blocks in all.  As many blocks as fit into 0.9 of the
 * free device memory are kept, spread evenly over the matrix, and only the
 * others are copied at every level: the reference's rule for the columns it
 * keeps (src/io/io.cu:496-507; pipeline src/core/garden.cu:296-347), with row
 * blocks as the unit.  internals.stream_resident_bytes (an extension key) caps
 * the bytes kept; 0 streams every block.  0 of 0 for a resident matrix. */
const char *AGardenStreamResidency(VoidPointer garden, unsigned long long *resident, unsigned long long *blocks);
/* Waits for all device work of the booster. */
const char *AGardenSynchronize(VoidPointer garden);

/* Histogram sums of node segments on the device, for data that already lives
 * there: the counterpart of HistTreeGrower::HistSum
 * (src/core/hist_tree_grower.h:17-23, hist_tree_grower.cu:200-301; called
 * directly by tests/cpp/test_hist_sum.cu), which takes one feature column per
 * call; this one takes every feature of a quad-packed matrix.  EVERY POINTER
 * IS A DEVICE POINTER.  Argument order follows the reference: outputs,
 * parents, gradients, node offsets, bins, sizes, trick.
 *   bins       [Q][stride] 32-bit words, Q = ceil(ncol / 4); byte k of word q
 *              of a row is the 8-bit bin id of feature 4 q + k; rows in node
 *              order (stride >= nrow, in words)
 *   grad/hess  [nrow] floats; hess NULL: the row count is the hessian
 *              (squared error) and sum_h / parent_h may be NULL
 *   node_size  nodes + 1 non-decreasing row offsets (the reference's
 *              node_size): node k owns rows [node_size[k], node_size[k + 1])
 *   use_trick  nodes are sibling pairs (2 k, 2 k + 1): only the smaller one
 *              (ties -> left, hist_grad_sum.cu:279-294) is accumulated, the
 *              other is parent[k] - it
 *   shift_g/h  sums are exact integers: every value is rounded once to
 *              rint(v * 2^shift) (|v * 2^shift| <= 2^30 required) and the
 *              integers are added, so the result does not depend on the order
 *   sum_g, sum_h, bin_count
 *              [nodes][4 Q][256]: cell (node, feature, bin)
 * Allocates its work memory with hipMalloc, runs on `stream` (a hipStream_t,
 * NULL = default stream) and waits for the result. */
const char *AHistSum(long long *sum_g, long long *sum_h, unsigned *bin_count, const long long *parent_g,
                     const long long *parent_h, const unsigned *parent_c, const float *grad, const float *hess,
                     const unsigned *node_size, const unsigned *bins, unsigned long long stride, long long nrow,
                     int ncol, int nodes, int use_trick, int shift_g, int shift_h, void *stream);

/* The work plan AHistSum makes for nrow rows in `nodes` segments, host arithmetic
 * only: rows per work item (about 512 items where items of at most 64512 rows
 * allow it, else items of that many rows) and the work items it sizes its
 * work memory for (one slab of 64 KB per 16 features, 128 KB with hessians,
 * each). */
const char *AHistSumPlan(long long nrow, int nodes, unsigned *rows_per_item, unsigned *work_items);

/* AHistSum for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  Same arguments and results as AHistSum; the
 * work plan and the per-work-item histograms live in a static device array of
 * 32 MB + 192 KB that every GPU running this library holds until the process
 * ends.  The call makes no hipMalloc / hipFree and no allocating library
 * call; it enqueues its kernels on `stream` and returns WITHOUT waiting.
 *   status   device word, may be NULL: written by the kernels, 0 = done,
 *            1 = node_size is not non-decreasing within [0, nrow] (such nodes
 *            are skipped), 2 = internal planning error
 * Limits (an error string is returned beyond them, before anything runs): the
 * array holds min(1024, 32 MB / slab) work items, slab = 64 KB per 16 features
 * (128 KB with hessians); a work item covers at most 64512 rows and every node
 * needs two spare items, so e.g. 28 features with hessians and 64 nodes allow
 * 8.1 M rows.  All calls on one GPU share the array: calls that overlap in
 * time on one GPU (two streams, two threads) race; calls on one stream, one
 * after the other, are safe, and nothing has to be cleared between them.
 * The FIRST call on a device, and the first call for a feature count (in steps
 * of 4 up to 32) and hessian choice, also resolves the array's device address
 * (hipGetSymbolAddress) and raises the LDS limit of the kernels it uses
 * (hipFuncSetAttribute): calls outside any stream, made once per process.  A
 * caller under graph capture makes one call of the shape it will capture
 * beforehand. */
const char *AHistSumNoAlloc(long long *sum_g, long long *sum_h, unsigned *bin_count, const long long *parent_g,
                            const long long *parent_h, const unsigned *parent_c, const float *grad,
                            const float *hess, const unsigned *node_size, const unsigned *bins,
                            unsigned long long stride, long long nrow, int ncol, int nodes, int use_trick,
                            int shift_g, int shift_h, void *stream, unsigned *status);

#ifdef __cplusplus
}
#endif
#endif /* ARBORETUM_EXT_H_ */
