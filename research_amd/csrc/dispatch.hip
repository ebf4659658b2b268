// Token dispatch: per-expert histogram, exclusive prefix sum, the stable
// permutation of assignments into expert-contiguous order with its inverse, and
// the row gather into expert-major order.
//
// Follows local_dispatch of the reference at ep_size == 1 (moe.py:583-602):
//   source_order = argsort(ids, stable)      inverse = argsort(source_order)
//   group_sizes  = histogram(ids)            offsets = cumsum(group_sizes) - group_sizes
//   packed_x[j]  = x[source_order[j] / K]
//
// The permutation is a counting sort whose positions come from an exclusive scan
// over (expert-major, chunk-minor) partial histograms, so it is stable and
// deterministic: no atomics decide a position.  The scan is a launch of its own
// only for very large batches; otherwise every workgroup of the rank pass sums
// the histograms it needs itself.
#include "common.hpp"
#include "dispatch_small.hpp"

#include <mutex>

namespace jtmoe {
namespace {

constexpr int kDispThreads = 256;
constexpr int kDispWaves = kDispThreads / kWave;
constexpr int kDispIters = 4;
constexpr int kDispChunk = kDispThreads * kDispIters;  // assignments per workgroup

inline int dispatch_chunks(int64_t A) { return (int)((A + kDispChunk - 1) / kDispChunk); }

// pass 1: partial[e * nchunks + chunk] = #{a in chunk : ids[a] == e}
// (kChunkMajor: partial[chunk * E + e], the layout the rank pass reads when it does the scan itself)
// kStats: also partial_imp[same index] = the sum of the route weights of those assignments,
// in 32.32 fixed point (the importance of _router_stats, moe.py:804, summed here instead of in the
// router when the layer runs both)
template <bool kStats, typename WT, bool kChunkMajor>
__global__ __launch_bounds__(kDispThreads) void dispatch_hist_kernel(const int32_t* __restrict__ ids,
                                                                     const WT* __restrict__ weights, int A, int E,
                                                                     int nchunks, int* __restrict__ partial,
                                                                     unsigned long long* __restrict__ partial_imp) {
  extern __shared__ __align__(8) unsigned char hist_raw[];
  unsigned long long* const imp = reinterpret_cast<unsigned long long*>(hist_raw);  // [E], kStats only
  int* const hist = reinterpret_cast<int*>(hist_raw + (kStats ? (size_t)E * 8 : 0));
  for (int e = threadIdx.x; e < E; e += kDispThreads) {
    hist[e] = 0;
    if (kStats) imp[e] = 0ull;
  }
  __syncthreads();
  const int base = blockIdx.x * kDispChunk;
#pragma unroll
  for (int it = 0; it < kDispIters; ++it) {
    const int a = base + it * kDispThreads + threadIdx.x;
    if (a < A) {
      const int id = ids[a];
      if (id >= 0 && id < E) {
        atomicAdd(&hist[id], 1);
        if (kStats) atomicAdd(&imp[id], importance_term(Elem<WT>::load(weights + a)));
      }
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += kDispThreads) {
    const size_t o = kChunkMajor ? (size_t)blockIdx.x * E + e : (size_t)e * nchunks + blockIdx.x;
    partial[o] = hist[e];
    if (kStats) partial_imp[o] = imp[e];
  }
}

// pass 2 (one workgroup of 16 waves): in-place exclusive scan of partial[0 .. E*nchunks), then
// group_sizes / offsets per expert.  Wave w owns one contiguous segment, which it reads twice with
// whole-line accesses (64 consecutive ints per step, four steps in flight): once for the segment
// total, once more to write the running sums.
// kStats: expert_counts / importance of the layer from the same partial sums.
constexpr int kScanThreads = 1024;
constexpr int kScanWaves = kScanThreads / kWave;
template <bool kStats>
__global__ __launch_bounds__(kScanThreads) void dispatch_scan_kernel(int* __restrict__ partial,
                                                                     const unsigned long long* __restrict__ partial_imp,
                                                                     int E, int nchunks,
                                                                     int32_t* __restrict__ group_sizes,
                                                                     int32_t* __restrict__ offsets,
                                                                     float* __restrict__ expert_counts,
                                                                     float* __restrict__ importance) {
  __shared__ int wave_total[kScanWaves];
  const int n = E * nchunks;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int seg = (n + kScanWaves * kWave - 1) / (kScanWaves * kWave) * kWave;
  const int lo = min(n, wave * seg), hi = min(n, lo + seg);
  int sum = 0;
  for (int i = lo + lane; i < hi; i += kWave) sum += partial[i];
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) sum += __shfl_xor(sum, d);
  if (lane == 0) wave_total[wave] = sum;
  __syncthreads();
  int carry = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kScanWaves; ++w) {
    const int v = wave_total[w];
    if (w < wave) carry += v;
    total += v;
  }
  for (int i0 = lo; i0 < hi; i0 += 4 * kWave) {
    int v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = i0 + j * kWave + lane;
      v[j] = i < hi ? partial[i] : 0;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = i0 + j * kWave + lane;
      int incl = v[j];
#pragma unroll
      for (int d = 1; d < kWave; d <<= 1) {
        const int up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
      }
      if (i < hi) partial[i] = carry + incl - v[j];
      carry += __shfl(incl, kWave - 1);
    }
  }
  __syncthreads();  // the running sums written above are read by other threads of the workgroup below
  for (int e = threadIdx.x; e < E; e += kScanThreads) {
    const int start = partial[(size_t)e * nchunks];
    const int next = (e + 1 < E) ? partial[(size_t)(e + 1) * nchunks] : total;
    offsets[e] = start;
    group_sizes[e] = next - start;
    if (kStats) expert_counts[e] = (float)(next - start);
  }
  if (kStats) {
    // a wave per expert, four experts in flight
    for (int e0 = wave; e0 < E; e0 += 4 * kScanWaves) {
      unsigned long long acc[4] = {0ull, 0ull, 0ull, 0ull};
      for (int c = lane; c < nchunks; c += kWave)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int e = e0 + j * kScanWaves;
          if (e < E) acc[j] += partial_imp[(size_t)e * nchunks + c];
        }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int d = kWave / 2; d > 0; d >>= 1) acc[j] += __shfl_xor(acc[j], d);
        const int e = e0 + j * kScanWaves;
        if (lane == 0 && e < E) importance[e] = (float)((double)acc[j] * (1.0 / 4294967296.0));
      }
    }
  }
}

// Up to this many chunks the rank pass works out its bases itself from the chunk-major partial
// histograms (every workgroup reads all of them, nchunks * E ints) and the scan launch is left out;
// beyond it that read, which grows with the square of the batch, costs more than the launch.
constexpr int kDirectMaxChunks = 256;

// LDS of the rank pass: imp[E] of 8 bytes (kDirect && kStats), cursor[E], wavehist[kDispWaves][E],
// and for kDirect tot[kDispThreads], pre[kDispThreads], wave_s[kDispWaves]
inline size_t rank_smem_bytes(int E, bool direct, bool stats) {
  size_t n = (size_t)E * (1 + kDispWaves) * sizeof(int);
  if (direct) n += ((size_t)2 * kDispThreads + kDispWaves) * sizeof(int);
  if (direct && stats) n += (size_t)E * 8;
  return n;
}

// cursor[e] = (assignments of the experts before e) + (assignments of e in the chunks before this
// one), from partial[chunk * E + e].  Workgroup 0 also writes the per-expert outputs of the call:
// offsets, group_sizes and (kStats) expert_counts / importance.
template <bool kStats>
__device__ __forceinline__ void chunk_bases(const int* __restrict__ partial,
                                            const unsigned long long* __restrict__ partial_imp, int E, int nchunks,
                                            int* cursor, int* tmp, unsigned long long* imp_s,
                                            int32_t* __restrict__ group_sizes, int32_t* __restrict__ offsets,
                                            float* __restrict__ expert_counts, float* __restrict__ importance) {
  static_assert(JTMOE_MAX_EXPERTS <= kDispThreads, "one thread per expert in the scan over the experts");
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  int* const tot_s = tmp;                  // [kDispThreads]
  int* const pre_s = tmp + kDispThreads;   // [kDispThreads]
  int* const wave_s = pre_s + kDispThreads;
  const bool first = blockIdx.x == 0;
  if (kStats && first) {
    for (int e = tid; e < E; e += kDispThreads) imp_s[e] = 0ull;
    __syncthreads();
  }
  // G groups of E threads share out the chunks: chunk c goes to group c % G
  const int G = kDispThreads / E;
  const int g = tid / E, e = tid - g * E;
  if (g < G) {
    int tot = 0, pre = 0;
    unsigned long long acc = 0ull;
    // 16 loads in flight at a time: the table is in the L2, what costs is the round trip
    constexpr int kBatch = 16;
    for (int c0 = g; c0 < nchunks; c0 += kBatch * G) {
      int v[kBatch];
      unsigned long long w[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const int c = c0 + j * G;
        v[j] = c < nchunks ? partial[(size_t)c * E + e] : 0;
        if (kStats && first) w[j] = c < nchunks ? partial_imp[(size_t)c * E + e] : 0ull;
      }
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const int c = c0 + j * G;
        tot += v[j];
        pre += c < (int)blockIdx.x ? v[j] : 0;
        if (kStats && first) acc += w[j];
      }
    }
    tot_s[tid] = tot;
    pre_s[tid] = pre;
    if (kStats && first) atomicAdd(&imp_s[e], acc);
  }
  __syncthreads();
  // thread e owns expert e: its total over the groups, then an exclusive scan over the experts
  int total = 0, before = 0;
  if (tid < E)
    for (int gg = 0; gg < G; ++gg) {
      total += tot_s[gg * E + tid];
      before += pre_s[gg * E + tid];
    }
  int incl = total;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int v = __shfl_up(incl, d);
    if (lane >= d) incl += v;
  }
  if (lane == kWave - 1) wave_s[wave] = incl;
  __syncthreads();
  int start = incl - total;
  for (int w = 0; w < wave; ++w) start += wave_s[w];
  if (tid < E) {
    cursor[tid] = start + before;
    if (first) {
      offsets[tid] = start;
      group_sizes[tid] = total;
      if (kStats) {
        expert_counts[tid] = (float)total;
        importance[tid] = (float)((double)imp_s[tid] * (1.0 / 4294967296.0));
      }
    }
  }
}

// pass 3: stable rank of every assignment inside its chunk + the chunk's base.
// kDirect: the bases come from chunk_bases (no scan launch before this one); otherwise base_g holds
// the scanned expert-major table.
template <bool kDirect, bool kStats>
__global__ __launch_bounds__(kDispThreads) void dispatch_rank_kernel(const int32_t* __restrict__ ids, int A, int E,
                                                                     int nchunks, const int* __restrict__ base_g,
                                                                     const unsigned long long* __restrict__ partial_imp,
                                                                     int32_t* __restrict__ source_order,
                                                                     int32_t* __restrict__ inverse,
                                                                     int32_t* __restrict__ group_sizes,
                                                                     int32_t* __restrict__ offsets,
                                                                     float* __restrict__ expert_counts,
                                                                     float* __restrict__ importance) {
  extern __shared__ __align__(8) unsigned char rank_raw[];
  unsigned long long* const imp_s = reinterpret_cast<unsigned long long*>(rank_raw);  // [E], kDirect && kStats
  int* const smem = reinterpret_cast<int*>(rank_raw + ((kDirect && kStats) ? (size_t)E * 8 : 0));
  int* cursor = smem;         // [E] next free packed row of expert e for this chunk
  int* wavehist = smem + E;   // [kDispWaves][E]
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  for (int i = tid; i < kDispWaves * E; i += kDispThreads) wavehist[i] = 0;
  if (kDirect) {
    chunk_bases<kStats>(base_g, partial_imp, E, nchunks, cursor, wavehist + kDispWaves * E, imp_s, group_sizes,
                        offsets, expert_counts, importance);
  } else {
    for (int e = tid; e < E; e += kDispThreads) cursor[e] = base_g[(size_t)e * nchunks + blockIdx.x];
  }
  __syncthreads();
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  const int base = blockIdx.x * kDispChunk;
  for (int it = 0; it < kDispIters; ++it) {
    const int a = base + it * kDispThreads + tid;
    int id = -1;
    if (a < A) {
      id = ids[a];
      if (id < 0 || id >= E) id = -1;
    }
    const bool valid = id >= 0;
    // lanes of this wave holding the same expert id
    unsigned long long peers = __ballot(valid);
    for (int b = 0; b < nbits; ++b) {
      const bool bit = (id >> b) & 1;
      const unsigned long long m = __ballot(valid && bit);
      peers &= bit ? m : ~m;
    }
    const unsigned long long lt = (1ull << lane) - 1ull;
    const int rank = __popcll(peers & lt);
    if (valid && rank == 0) wavehist[wave * E + id] = __popcll(peers);
    __syncthreads();
    if (valid) {
      int pos = cursor[id] + rank;
      for (int w = 0; w < wave; ++w) pos += wavehist[w * E + id];
      inverse[a] = pos;
      source_order[pos] = a;
    } else if (a < A) {
      inverse[a] = -1;
    }
    __syncthreads();
    for (int e = tid; e < E; e += kDispThreads) {
      int add = 0;
#pragma unroll
      for (int w = 0; w < kDispWaves; ++w) {
        add += wavehist[w * E + e];
        wavehist[w * E + e] = 0;
      }
      cursor[e] += add;
    }
    __syncthreads();
  }
}

// Small batches: the three passes in one workgroup of 1024 threads (dispatch_small.hpp).  At a few
// hundred assignments the three launches above are idle most of their time; this is one launch with
// the same results.
constexpr int kSmallThreads = 1024;
template <bool kStats, typename WT>
__global__ __launch_bounds__(kSmallThreads) void dispatch_small_kernel(const int32_t* __restrict__ ids,
                                                                      const WT* __restrict__ weights, int A, int E,
                                                                      int32_t* __restrict__ group_sizes,
                                                                      int32_t* __restrict__ offsets,
                                                                      int32_t* __restrict__ source_order,
                                                                      int32_t* __restrict__ inverse,
                                                                      float* __restrict__ expert_counts,
                                                                      float* __restrict__ importance) {
  extern __shared__ __align__(8) unsigned char small_raw[];
  dispatch_small_body<kSmallThreads, kStats, WT>(ids, weights, A, E, group_sizes, offsets, source_order, inverse,
                                                 expert_counts, importance, small_raw);
}

// pass 4: token-major row scatter; each token row is read once and written to
// its K packed positions.  V is the vector type moved per lane.
template <typename V>
__global__ __launch_bounds__(256) void dispatch_rows_kernel(const V* __restrict__ x, const int32_t* __restrict__ inverse,
                                                            int tokens, int K, int A, int row_vecs,
                                                            V* __restrict__ packed_x) {
  const int rows_per_block = blockDim.y;
  const int t = blockIdx.x * rows_per_block + threadIdx.y;
  if (t >= tokens) return;
  const V* src = x + (size_t)t * row_vecs;
  for (int v0 = threadIdx.x; v0 < row_vecs; v0 += blockDim.x * 4) {
    V r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int v = v0 + j * blockDim.x;
      if (v < row_vecs) r[j] = load_stream(&src[v]);
    }
    for (int s = 0; s < K; ++s) {
      const int pos = inverse[(size_t)t * K + s];
      if (pos < 0 || pos >= A) continue;
      V* dst = packed_x + (size_t)pos * row_vecs;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int v = v0 + j * blockDim.x;
        if (v < row_vecs) store_stream(&dst[v], r[j]);
      }
    }
  }
}

}  // namespace

// packed[inverse[t*K + s]] = x[t] for every token t and slot s (rows of H elements)
void launch_dispatch_rows(const void* x, const int32_t* inverse, int64_t T, int64_t K, int64_t H, int dtype,
                          void* packed_x, hipStream_t s) {
  if (T == 0) return;
  const int64_t A = T * K;
  const size_t row_bytes = (size_t)H * dtype_bytes(dtype);
  const bool vec16 = row_bytes % 16 == 0 && aligned16(x) && aligned16(packed_x);
  if (vec16) {
    const int row_vecs = (int)(row_bytes / 16);
    // one 16-byte vector per lane where the row has that many: a 4 KB row is then moved by a whole
    // workgroup of four waves, each writing a 1 KB quarter of every destination row (measured against
    // one wave per row with four vectors per lane at 16384 x 4 KB rows, top-8: 113 vs 124 us)
    int bx = 64;
    while (bx < 256 && bx < row_vecs) bx *= 2;
    dim3 block(bx, 256 / bx);
    const int grid = (int)((T + block.y - 1) / block.y);
    dispatch_rows_kernel<uint4><<<grid, block, 0, s>>>(static_cast<const uint4*>(x), inverse, (int)T, (int)K, (int)A,
                                                       row_vecs, static_cast<uint4*>(packed_x));
  } else if (dtype == JTMOE_BF16) {
    dim3 block(64, 4);
    const int grid = (int)((T + block.y - 1) / block.y);
    dispatch_rows_kernel<uint16_t><<<grid, block, 0, s>>>(static_cast<const uint16_t*>(x), inverse, (int)T, (int)K,
                                                          (int)A, (int)H, static_cast<uint16_t*>(packed_x));
  } else {
    dim3 block(64, 4);
    const int grid = (int)((T + block.y - 1) / block.y);
    dispatch_rows_kernel<uint32_t><<<grid, block, 0, s>>>(static_cast<const uint32_t*>(x), inverse, (int)T, (int)K,
                                                          (int)A, (int)H, static_cast<uint32_t*>(packed_x));
  }
}

}  // namespace jtmoe

using namespace jtmoe;

extern "C" size_t jtmoe_dispatch_workspace_bytes(int64_t A, int64_t E) {
  if (A < 0 || E <= 0) return 0;
  const size_t chunks = (size_t)dispatch_chunks(A > 0 ? A : 1);
  return align_up(chunks * (size_t)E * sizeof(int), 256);
}

namespace jtmoe {
namespace {

// Scratch of jtmoe_dispatch_static: the partial histograms [E][chunks] of the largest problem it
// accepts.  Host code must not pass this name to a kernel (on the host it is a stand-in, not a device
// address): the address on each device comes from hipGetSymbolAddress, once per device.
constexpr size_t kStaticScratchBytes = JTMOE_DISPATCH_STATIC_MAX_BYTES;  // per GPU, held until the process ends
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices];  // per device, null until looked up

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_scratch(void** out) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices)
    return fail(JTMOE_ELAUNCH, "dispatch_static: no current device (or its index is beyond %d)", kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    void* ptr = nullptr;
    const hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr)
      return fail(JTMOE_ELAUNCH, "dispatch_static: hipGetSymbolAddress failed: %s", hipGetErrorString(err));
    g_scratch_ptr[device] = ptr;
  }
  *out = g_scratch_ptr[device];
  return JTMOE_OK;
}

// Argument checks shared by the two entry points (everything but the scratch).
int dispatch_validate(const char* who, const int32_t* expert_ids, const void* x, int64_t T, int64_t H, int64_t E,
                      int64_t K, int dtype, const int32_t* group_sizes, const int32_t* offsets,
                      const int32_t* source_order, const int32_t* inverse, const void* packed_x) {
  JT_REQUIRE(dtype_ok(dtype), "%s: unknown dtype %d", who, dtype);
  JT_REQUIRE(T >= 0 && K > 0 && E > 0, "%s: T=%lld K=%lld E=%lld out of range", who, (long long)T, (long long)K,
             (long long)E);
  if (E > JTMOE_MAX_EXPERTS) return fail(JTMOE_EUNSUPPORTED, "%s: E=%lld exceeds %d", who, (long long)E, JTMOE_MAX_EXPERTS);
  JT_REQUIRE(T < ((int64_t)1 << 31) && T * K < ((int64_t)1 << 31), "%s: T*K exceeds int32", who);
  JT_REQUIRE(group_sizes && offsets, "%s: null pointer argument", who);
  JT_REQUIRE(T * K == 0 || (expert_ids && source_order && inverse), "%s: null pointer argument", who);
  JT_REQUIRE(x == nullptr || (H > 0 && packed_x != nullptr), "%s: x given without H or packed_x", who);
  JT_REQUIRE(x == nullptr || H * (int64_t)dtype_bytes(dtype) < ((int64_t)1 << 31), "%s: row too long", who);
  return JTMOE_OK;
}

// Where the fixed-point weight sums [E][chunks] of the layer's statistics start inside the scratch.
inline size_t partial_imp_offset(int64_t A, int64_t E) { return jtmoe_dispatch_workspace_bytes(A, E); }

// The launches of a validated dispatch; `partial` holds jtmoe_dispatch_workspace_bytes(A, E) bytes
// (dispatch_layer_workspace_bytes(A, E) when `weights` is given).
// Every entry of partial that is read has been written by the histogram pass of the same call, so
// the scratch needs no clearing between calls.
// stats (weights of element type = dtype): also expert_counts[E] and importance[E], the statistics
// that jtmoe_router would have produced for these ids and weights.
template <typename WT>
int dispatch_launch_t(const int32_t* expert_ids, const WT* weights, bool stats, const void* x, int64_t T, int64_t H,
                      int64_t E, int64_t K, int dtype, int32_t* group_sizes, int32_t* offsets, int32_t* source_order,
                      int32_t* inverse, void* packed_x, float* expert_counts, float* importance, int* partial,
                      hipStream_t s) {
  const int64_t A = T * K;
  if (A > 0 && A <= kSmallMaxAssignments && E <= kSmallMaxExperts) {
    const size_t smem = dispatch_small_smem_bytes((int)E, kSmallThreads, stats);
    if (stats)
      dispatch_small_kernel<true, WT><<<1, kSmallThreads, smem, s>>>(expert_ids, weights, (int)A, (int)E, group_sizes,
                                                                     offsets, source_order, inverse, expert_counts,
                                                                     importance);
    else
      dispatch_small_kernel<false, WT><<<1, kSmallThreads, smem, s>>>(expert_ids, nullptr, (int)A, (int)E, group_sizes,
                                                                      offsets, source_order, inverse, nullptr, nullptr);
    stage_mark(kStageDispatchMeta, s);
    if (x != nullptr) launch_dispatch_rows(x, inverse, T, K, H, dtype, packed_x, s);
    stage_mark(kStageDispatchRows, s);
    return check_launch("dispatch");
  }
  const int nchunks = dispatch_chunks(A > 0 ? A : 1);
  unsigned long long* const partial_imp =
      stats ? reinterpret_cast<unsigned long long*>(reinterpret_cast<unsigned char*>(partial) + partial_imp_offset(A, E))
            : nullptr;
  // two launches (histogram, rank with its own scan) up to kDirectMaxChunks chunks, three beyond
  const bool direct = A > 0 && nchunks <= kDirectMaxChunks;
  const size_t hist_smem = (size_t)E * (stats ? 12 : 4);
#define JT_HIST(STATS, DIRECT)                                                                             \
  dispatch_hist_kernel<STATS, WT, DIRECT><<<nchunks, kDispThreads, hist_smem, s>>>(expert_ids, weights, (int)A, \
                                                                                   (int)E, nchunks, partial,    \
                                                                                   partial_imp)
#define JT_RANK(DIRECT, STATS)                                                                                  \
  dispatch_rank_kernel<DIRECT, STATS><<<nchunks, kDispThreads, rank_smem_bytes((int)E, DIRECT, STATS), s>>>(    \
      expert_ids, (int)A, (int)E, nchunks, partial, partial_imp, source_order, inverse, group_sizes, offsets,   \
      expert_counts, importance)
  if (direct) {
    if (stats) {
      JT_HIST(true, true);
      JT_RANK(true, true);
    } else {
      JT_HIST(false, true);
      JT_RANK(true, false);
    }
  } else {
    if (stats) {
      JT_HIST(true, false);
      dispatch_scan_kernel<true><<<1, kScanThreads, 0, s>>>(partial, partial_imp, (int)E, nchunks, group_sizes, offsets,
                                                            expert_counts, importance);
    } else {
      JT_HIST(false, false);
      dispatch_scan_kernel<false><<<1, kScanThreads, 0, s>>>(partial, nullptr, (int)E, nchunks, group_sizes, offsets,
                                                             nullptr, nullptr);
    }
    if (A > 0) JT_RANK(false, false);
  }
#undef JT_HIST
#undef JT_RANK
  if (A > 0) {
    stage_mark(kStageDispatchMeta, s);
    if (x != nullptr) launch_dispatch_rows(x, inverse, T, K, H, dtype, packed_x, s);
  }
  if (A == 0) stage_mark(kStageDispatchMeta, s);
  stage_mark(kStageDispatchRows, s);
  return check_launch("dispatch");
}

int dispatch_launch(const int32_t* expert_ids, const void* x, int64_t T, int64_t H, int64_t E, int64_t K, int dtype,
                    int32_t* group_sizes, int32_t* offsets, int32_t* source_order, int32_t* inverse, void* packed_x,
                    int* partial, hipStream_t s) {
  return dispatch_launch_t<float>(expert_ids, nullptr, false, x, T, H, E, K, dtype, group_sizes, offsets, source_order,
                                  inverse, packed_x, nullptr, nullptr, partial, s);
}

}  // namespace

size_t dispatch_layer_workspace_bytes(int64_t A, int64_t E) {
  if (A < 0 || E <= 0) return 0;
  const size_t chunks = (size_t)dispatch_chunks(A > 0 ? A : 1);
  return jtmoe_dispatch_workspace_bytes(A, E) + align_up(chunks * (size_t)E * sizeof(unsigned long long), 256);
}

int dispatch_for_layer(const int32_t* expert_ids, const void* weights, const void* x, int64_t T, int64_t H, int64_t E,
                       int64_t K, int dtype, int32_t* group_sizes, int32_t* offsets, int32_t* source_order,
                       int32_t* inverse, void* packed_x, float* expert_counts, float* importance, void* workspace,
                       bool want_stats, bool plan_done, hipStream_t s) {
  const int rc = dispatch_validate("dispatch", expert_ids, x, T, H, E, K, dtype, group_sizes, offsets, source_order,
                                   inverse, packed_x);
  if (rc) return rc;
  JT_REQUIRE(workspace != nullptr, "dispatch: null pointer argument");
  JT_REQUIRE(!want_stats || (expert_counts && importance && (weights || T == 0)), "dispatch: null pointer argument");
  if (plan_done) {  // the router's finishing workgroup has written the plan
    stage_mark(kStageDispatchMeta, s);
    if (x != nullptr && T > 0) launch_dispatch_rows(x, inverse, T, K, H, dtype, packed_x, s);
    stage_mark(kStageDispatchRows, s);
    return check_launch("dispatch");
  }
  if (dtype == JTMOE_BF16)
    return dispatch_launch_t<bf16_raw>(expert_ids, static_cast<const bf16_raw*>(weights), want_stats, x, T, H, E, K,
                                       dtype, group_sizes, offsets, source_order, inverse, packed_x, expert_counts,
                                       importance, static_cast<int*>(workspace), s);
  return dispatch_launch_t<float>(expert_ids, static_cast<const float*>(weights), want_stats, x, T, H, E, K, dtype,
                                  group_sizes, offsets, source_order, inverse, packed_x, expert_counts, importance,
                                  static_cast<int*>(workspace), s);
}

}  // namespace jtmoe

extern "C" int jtmoe_dispatch(const int32_t* expert_ids, const void* x, int64_t T, int64_t H, int64_t E, int64_t K,
                              int dtype, int32_t* group_sizes, int32_t* offsets, int32_t* source_order,
                              int32_t* inverse, void* packed_x, void* workspace, size_t workspace_bytes,
                              void* stream) {
  clear_error();
  const int rc = dispatch_validate("dispatch", expert_ids, x, T, H, E, K, dtype, group_sizes, offsets, source_order,
                                   inverse, packed_x);
  if (rc) return rc;
  JT_REQUIRE(workspace != nullptr, "dispatch: null pointer argument");
  if (workspace_bytes < jtmoe_dispatch_workspace_bytes(T * K, E))
    return fail(JTMOE_EWORKSPACE, "dispatch: workspace %zu < %zu bytes", workspace_bytes,
                jtmoe_dispatch_workspace_bytes(T * K, E));
  return dispatch_launch(expert_ids, x, T, H, E, K, dtype, group_sizes, offsets, source_order, inverse, packed_x,
                         static_cast<int*>(workspace), as_stream(stream));
}

extern "C" int jtmoe_dispatch_static(const int32_t* expert_ids, const void* x, int64_t T, int64_t H, int64_t E,
                                     int64_t K, int dtype, int32_t* group_sizes, int32_t* offsets,
                                     int32_t* source_order, int32_t* inverse, void* packed_x, void* stream) {
  clear_error();
  int rc = dispatch_validate("dispatch_static", expert_ids, x, T, H, E, K, dtype, group_sizes, offsets, source_order,
                             inverse, packed_x);
  if (rc) return rc;
  const size_t need = jtmoe_dispatch_workspace_bytes(T * K, E);
  if (need > kStaticScratchBytes)
    return fail(JTMOE_EUNSUPPORTED,
                "dispatch_static: T*K=%lld assignments over E=%lld experts need %zu bytes of scratch, the built-in "
                "buffer holds %zu (ceil(T*K/1024)*E <= 262144); use jtmoe_dispatch with a workspace",
                (long long)(T * K), (long long)E, need, kStaticScratchBytes);
  void* ptr = nullptr;
  rc = static_scratch(&ptr);
  if (rc) return rc;
  return dispatch_launch(expert_ids, x, T, H, E, K, dtype, group_sizes, offsets, source_order, inverse, packed_x,
                         static_cast<int*>(ptr), as_stream(stream));
}
