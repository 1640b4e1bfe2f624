// Batch prediction on the GPU: the tree walks of RegTree::Predict /
// Garden::Predict (src/core/garden.h:70-90, src/core/garden.cu:643-657) for a
// float matrix (or a pre-quantised one, whose bin ids are compared as floats
// like the host walk does), every tree over a block of rows while the next
// block is staged.  The arithmetic is the host walk's: `x < threshold` goes left (NaN
// right), the leaf weights of one label are added in tree order in fp32, so
// the sums are bit-identical to the host path.  The link function stays with
// the caller.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>
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

constexpr int kPredictThreads = 1024;          // rows per workgroup, one row per thread
constexpr size_t kTreeLdsBytes = 64 * 1024;    // trees staged in LDS at a time: two workgroups per CU
constexpr size_t kStageBytes = 32u << 20;      // one pinned staging buffer
constexpr size_t kCacheBytes = (size_t)8 << 30;  // largest float matrix kept on the device between calls

struct TreeRef {
  unsigned node_off;  // first internal node in the flattened node array
  unsigned leaf_off;  // first leaf weight
  unsigned depth;     // internal depth: depth - 1 comparisons
  unsigned label;
};

// Consecutive trees [t0, t1) whose nodes and leaves fit the LDS budget
// together, or a single tree that does not (in_lds = 0, read from global).
struct Chunk {
  unsigned t0, t1, in_lds, n_nodes, n_leaves;
};

// Where a row's feature values come from.
enum Source {
  kFloatCols = 0,  // float columns [F][ld]
  kByteRows = 1,   // pre-quantised rows [rows][ld = F] of uint8 bin ids
  kQuadCols = 2    // pre-quantised quad columns [Q][ld]: four uint8 bin ids per word
};

template <int SRC>
__device__ __forceinline__ float Fetch(const void *__restrict__ base, size_t ld, unsigned r, unsigned f) {
  if (SRC == kFloatCols) return static_cast<const float *>(base)[(size_t)f * ld + r];
  if (SRC == kByteRows) return (float)static_cast<const uint8_t *>(base)[(size_t)r * ld + f];
  return (float)((static_cast<const uint32_t *>(base)[(size_t)(f >> 2) * ld + r] >> (8u * (f & 3u))) & 255u);
}

// Walks trees [t0, t1) for row r of `base`.  acc holds the running sum of
// label *cur.
template <int SRC>
__device__ __forceinline__ void WalkTrees(const uint2 *nd, const float *lf, unsigned node_base, unsigned leaf_base,
                                          const TreeRef *__restrict__ refs, unsigned t0, unsigned t1,
                                          const void *__restrict__ base, size_t ld, unsigned r,
                                          float *__restrict__ out, size_t out_ld, bool live, int *cur, float *acc) {
  for (unsigned t = t0; t < t1; ++t) {
    const TreeRef ref = refs[t];
    if ((int)ref.label != *cur) {
      if (*cur >= 0 && live) out[(size_t)*cur * out_ld] = *acc;
      *cur = (int)ref.label;
      *acc = out[(size_t)ref.label * out_ld];
    }
    const uint2 *tn = nd + (ref.node_off - node_base);
    unsigned id = 0;
    for (unsigned j = 1; j < ref.depth; ++j) {
      const uint2 n = tn[id];
      const float v = Fetch<SRC>(base, ld, r, n.x);
      id = 2 * id + 2 - (unsigned)(v < __uint_as_float(n.y));
    }
    *acc += lf[ref.leaf_off - leaf_base + (id - ((1u << (ref.depth - 1)) - 1))];
  }
}

// base: this block's rows as SRC says; out: [labels][out_ld], already offset
// to the block's first row.  grid ceil(rows / 1024).
template <int SRC>
__global__ void __launch_bounds__(kPredictThreads)
k_predict(const void *__restrict__ base, size_t ld, unsigned rows, const uint2 *__restrict__ nodes,
          const float *__restrict__ leaves, const TreeRef *__restrict__ refs, const Chunk *__restrict__ chunks,
          int n_chunks, float *__restrict__ out, size_t out_ld) {
  extern __shared__ unsigned char smem[];
  const unsigned i = blockIdx.x * kPredictThreads + threadIdx.x;
  const bool live = i < rows;
  const unsigned r = live ? i : rows - 1;
  float *o = out + r;
  int cur = -1;
  float acc = 0.0f;
  for (int c = 0; c < n_chunks; ++c) {
    const Chunk ch = chunks[c];
    const unsigned node_base = refs[ch.t0].node_off, leaf_base = refs[ch.t0].leaf_off;
    if (ch.in_lds) {
      uint2 *s_nd = (uint2 *)smem;
      float *s_lf = (float *)(smem + (size_t)ch.n_nodes * sizeof(uint2));
      __syncthreads();  // the previous chunk's trees are no longer read
      for (unsigned k = threadIdx.x; k < ch.n_nodes; k += kPredictThreads) s_nd[k] = nodes[node_base + k];
      for (unsigned k = threadIdx.x; k < ch.n_leaves; k += kPredictThreads) s_lf[k] = leaves[leaf_base + k];
      __syncthreads();
      WalkTrees<SRC>(s_nd, s_lf, node_base, leaf_base, refs, ch.t0, ch.t1, base, ld, r, o, out_ld, live, &cur, &acc);
    } else {
      WalkTrees<SRC>(nodes + node_base, leaves + leaf_base, node_base, leaf_base, refs, ch.t0, ch.t1, base, ld, r, o,
                     out_ld, live, &cur, &acc);
    }
  }
  if (cur >= 0 && live) o[(size_t)cur * out_ld] = acc;
}

__global__ void __launch_bounds__(256) k_predict_fill(float *__restrict__ p, size_t n, float v) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = v;
}

template <typename T>
struct DevBuf {
  T *p = nullptr;
  size_t n = 0;
  ~DevBuf() { if (p) (void)hipFree(p); }
  void Reserve(size_t want) {
    if (want <= n) return;
    if (p) HIP_OK(hipFree(p));
    p = nullptr;
    n = 0;
    HIP_OK(hipMalloc((void **)&p, want * sizeof(T)));
    n = want;
  }
  // blocking: the vector may be gone when the call returns
  void Upload(const std::vector<T> &v) {
    Reserve(std::max<size_t>(v.size(), 1));
    if (!v.empty()) HIP_OK(hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
  }
};

}  // namespace

// Buffers kept between calls: staging and device blocks are sized once, and
// the columns of the last matrix (up to kCacheBytes) stay on the device, so
// that predicting on it again (an evaluation set, once per boosting round)
// copies nothing.
struct DevicePredictor {
  hipStream_t stream = nullptr;
  hipEvent_t copied[2] = {nullptr, nullptr};
  float *stage[2] = {nullptr, nullptr};
  size_t stage_floats = 0;
  DevBuf<float> block, out, leaves, cache;
  float *result = nullptr;  // pinned; the sums of the last call
  size_t result_floats = 0;
  uint64_t cached_uid = 0;  // matrix whose columns `cache` holds as [F][cache_ld]
  size_t cache_ld = 0;
  DevBuf<uint2> nodes;
  DevBuf<TreeRef> refs;
  DevBuf<Chunk> chunks;

  ~DevicePredictor() {
    for (int k = 0; k < 2; ++k) {
      if (stage[k]) (void)hipHostFree(stage[k]);
      if (copied[k]) (void)hipEventDestroy(copied[k]);
    }
    if (result) (void)hipHostFree(result);
    if (stream) (void)hipStreamDestroy(stream);
  }

  const float *Run(const DataMatrix &data, const std::vector<RegTree> &trees, size_t use, size_t labels, float init) {
    const size_t n = data.rows, F = data.columns_dense;
    if (n == 0 || F == 0) throw std::runtime_error("empty data matrix");
    // only the block-wise walk of a streamed matrix indexes rows with 64 bits
    if (n >= (1ull << 31) && !(data.is_prebinned && data.prebinned.empty() && !data.stream_blocks.empty()))
      throw std::runtime_error("too many rows");
    if (!stream) {
      HIP_OK(hipStreamCreate(&stream));
      for (int k = 0; k < 2; ++k) HIP_OK(hipEventCreateWithFlags(&copied[k], hipEventDisableTiming));
    }
    // ---- the model, flattened in tree order
    std::vector<uint2> h_nodes;
    std::vector<float> h_leaves;
    std::vector<TreeRef> h_refs;
    std::vector<Chunk> h_chunks;
    for (size_t t = 0; t < use; ++t) {
      const RegTree &tr = trees[t];
      if (tr.label >= labels) throw std::runtime_error("tree label out of range");
      if (h_nodes.size() + tr.fid.size() >= (1ull << 32) || h_leaves.size() + tr.weights.size() >= (1ull << 32))
        throw std::runtime_error("model too large for device prediction");
      TreeRef ref;
      ref.node_off = (unsigned)h_nodes.size();
      ref.leaf_off = (unsigned)h_leaves.size();
      ref.depth = tr.depth;
      ref.label = tr.label;
      h_refs.push_back(ref);
      for (size_t k = 0; k < tr.fid.size(); ++k) {
        uint2 nd;
        float thr = tr.threshold[k];
        nd.x = tr.fid[k];
        if (tr.fid[k] >= F) {  // a feature the matrix does not have reads as NaN: always right
          nd.x = 0;
          thr = -std::numeric_limits<float>::infinity();
        }
        std::memcpy(&nd.y, &thr, sizeof(float));
        h_nodes.push_back(nd);
      }
      h_leaves.insert(h_leaves.end(), tr.weights.begin(), tr.weights.end());
      const size_t bytes = tr.fid.size() * sizeof(uint2) + tr.weights.size() * sizeof(float);
      const bool fits = bytes <= kTreeLdsBytes;
      bool joined = false;
      if (fits && !h_chunks.empty() && h_chunks.back().in_lds) {
        Chunk &c = h_chunks.back();
        const size_t total = (c.n_nodes + tr.fid.size()) * sizeof(uint2) + (c.n_leaves + tr.weights.size()) * sizeof(float);
        if (total <= kTreeLdsBytes) {
          c.t1 = (unsigned)t + 1;
          c.n_nodes += (unsigned)tr.fid.size();
          c.n_leaves += (unsigned)tr.weights.size();
          joined = true;
        }
      }
      if (!joined) {
        Chunk c;
        c.t0 = (unsigned)t;
        c.t1 = (unsigned)t + 1;
        c.in_lds = fits ? 1u : 0u;
        c.n_nodes = (unsigned)tr.fid.size();
        c.n_leaves = (unsigned)tr.weights.size();
        h_chunks.push_back(c);
      }
    }
    nodes.Upload(h_nodes);
    leaves.Upload(h_leaves);
    refs.Upload(h_refs);
    chunks.Upload(h_chunks);
    out.Reserve(labels * n);
    hipLaunchKernelGGL(k_predict_fill, dim3((unsigned)((labels * n + 255) / 256)), dim3(256), 0, stream, out.p,
                       labels * n, init);
    HIP_OK(hipGetLastError());
    auto walk = [&](int src, const void *base, size_t ld, size_t r0, size_t rows) {
      if (use == 0) return;
      const dim3 grid((unsigned)((rows + kPredictThreads - 1) / kPredictThreads)), block_dim(kPredictThreads);
#define ARB_WALK(S)                                                                                         \
  hipLaunchKernelGGL((k_predict<S>), grid, block_dim, kTreeLdsBytes, stream, base, ld, (unsigned)rows, nodes.p, \
                     leaves.p, refs.p, chunks.p, (int)h_chunks.size(), out.p + r0, n)
      if (src == kFloatCols) ARB_WALK(kFloatCols);
      else if (src == kByteRows) ARB_WALK(kByteRows);
      else ARB_WALK(kQuadCols);
#undef ARB_WALK
      HIP_OK(hipGetLastError());
    };
    auto reserve_stage = [&](size_t floats) {
      if (floats <= stage_floats) return;
      for (int k = 0; k < 2; ++k) {
        if (stage[k]) HIP_OK(hipHostFree(stage[k]));
        stage[k] = nullptr;
      }
      stage_floats = 0;
      for (int k = 0; k < 2; ++k) HIP_OK(hipHostMalloc((void **)&stage[k], floats * sizeof(float), hipHostMallocDefault));
      stage_floats = floats;
    };
    if (data.is_prebinned) {
      cached_uid = 0;
      if (!data.prebinned.empty()) {
        // row-major bytes on the host: blocks of whole rows through the staging buffers
        const size_t block_rows =
            std::min(std::max<size_t>(kStageBytes / F / kPredictThreads, 1) * kPredictThreads, (n + 63) / 64 * 64);
        const size_t floats = (block_rows * F + 3) / 4;
        reserve_stage(floats);
        block.Reserve(floats);
        const size_t nblocks = (n + block_rows - 1) / block_rows;
        for (size_t b = 0; b < nblocks; ++b) {
          const int buf = (int)(b & 1);
          const size_t r0 = b * block_rows, rows = std::min(block_rows, n - r0);
          if (b >= 2) HIP_OK(hipEventSynchronize(copied[buf]));
          uint8_t *dst = reinterpret_cast<uint8_t *>(stage[buf]);
          const uint8_t *src = data.prebinned.data() + r0 * F;
          ParallelFor(rows * F, [&](size_t lo, size_t hi) { std::memcpy(dst + lo, src + lo, hi - lo); });
          HIP_OK(hipMemcpyAsync(block.p, dst, rows * F, hipMemcpyHostToDevice, stream));
          HIP_OK(hipEventRecord(copied[buf], stream));
          walk(kByteRows, block.p, F, r0, rows);
        }
      } else if (!data.stream_blocks.empty()) {
        // streamed matrix: its pinned blocks of quad columns go up as they are
        const size_t br = data.stream_block_rows, Q = (F + 3) / 4;
        block.Reserve(Q * br);
        for (size_t b = 0; b < data.stream_blocks.size(); ++b) {
          const size_t r0 = b * br;
          if (r0 >= n) break;
          const size_t rows = std::min(br, n - r0);
          HIP_OK(hipMemcpyAsync(block.p, data.stream_blocks[b], Q * br * sizeof(uint32_t), hipMemcpyHostToDevice,
                                stream));
          walk(kQuadCols, block.p, br, r0, rows);
        }
      } else {
        throw std::runtime_error("pre-quantised matrix without bins");
      }
    } else {
      const size_t ld_all = (n + 63) / 64 * 64;
      const bool cacheable = F * ld_all * sizeof(float) <= kCacheBytes;
      if (cacheable && cached_uid == data.uid && cache_ld == ld_all) {
        walk(kFloatCols, cache.p, cache_ld, 0, n);  // the columns are on the device already
      } else {
        // ---- row blocks: [F][block_rows] floats, about kStageBytes each
        size_t block_rows = std::max<size_t>(kStageBytes / (F * sizeof(float)) / kPredictThreads, 1) * kPredictThreads;
        block_rows = std::min(block_rows, ld_all);
        const size_t floats = F * block_rows;
        reserve_stage(floats);
        block.Reserve(floats);
        cached_uid = 0;
        if (cacheable) cache.Reserve(F * ld_all);
        const size_t nblocks = (n + block_rows - 1) / block_rows;
        for (size_t b = 0; b < nblocks; ++b) {
          const int buf = (int)(b & 1);
          const size_t r0 = b * block_rows, rows = std::min(block_rows, n - r0);
          if (b >= 2) HIP_OK(hipEventSynchronize(copied[buf]));  // the copy out of this staging buffer is done
          float *dst = stage[buf];
          ParallelFor(rows, [&](size_t lo, size_t hi) {
            for (size_t f = 0; f < F; ++f)
              std::memcpy(dst + f * block_rows + lo, data.data[f].data() + r0 + lo, (hi - lo) * sizeof(float));
          });
          HIP_OK(hipMemcpyAsync(block.p, dst, floats * sizeof(float), hipMemcpyHostToDevice, stream));
          HIP_OK(hipEventRecord(copied[buf], stream));
          walk(kFloatCols, block.p, block_rows, r0, rows);
          if (cacheable)  // rows [r0, r0 + rows) of every column into their place in the whole matrix
            HIP_OK(hipMemcpy2DAsync(cache.p + r0, ld_all * sizeof(float), block.p, block_rows * sizeof(float),
                                    rows * sizeof(float), F, hipMemcpyDeviceToDevice, stream));
        }
        if (cacheable) {
          cached_uid = data.uid;
          cache_ld = ld_all;
        }
      }
    }
    if (labels * n > result_floats) {
      if (result) HIP_OK(hipHostFree(result));
      result = nullptr;
      result_floats = 0;
      HIP_OK(hipHostMalloc((void **)&result, labels * n * sizeof(float), hipHostMallocDefault));
      result_floats = labels * n;
    }
    HIP_OK(hipMemcpyAsync(result, out.p, labels * n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    return result;
  }
};

DevicePredictor *CreateDevicePredictor() { return new DevicePredictor(); }
void FreeDevicePredictor(DevicePredictor *p) { delete p; }
const float *PredictOnDevice(DevicePredictor *p, const DataMatrix &data, const std::vector<RegTree> &trees,
                             size_t use, size_t labels, float init) {
  return p->Run(data, trees, use, labels, init);
}

}  // namespace arb
