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
// deterministic: no atomics decide a position.
#include "common.hpp"

#include <mutex>

namespace jtmoe {
namespace {

constexpr int kDispThreads = 256;
constexpr int kDispWaves = kDispThreads / kWave;
constexpr int kDispIters = 4;
constexpr int kDispChunk = kDispThreads * kDispIters;  // assignments per workgroup

inline int dispatch_chunks(int64_t A) { return (int)((A + kDispChunk - 1) / kDispChunk); }

// pass 1: partial[e * nchunks + chunk] = #{a in chunk : ids[a] == e}
__global__ __launch_bounds__(kDispThreads) void dispatch_hist_kernel(const int32_t* __restrict__ ids, int A, int E,
                                                                     int nchunks, int* __restrict__ partial) {
  extern __shared__ int hist[];
  for (int e = threadIdx.x; e < E; e += kDispThreads) hist[e] = 0;
  __syncthreads();
  const int base = blockIdx.x * kDispChunk;
#pragma unroll
  for (int it = 0; it < kDispIters; ++it) {
    const int a = base + it * kDispThreads + threadIdx.x;
    if (a < A) {
      const int id = ids[a];
      if (id >= 0 && id < E) atomicAdd(&hist[id], 1);
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += kDispThreads) partial[(size_t)e * nchunks + blockIdx.x] = hist[e];
}

// pass 2 (one workgroup): in-place exclusive scan of partial[0 .. E*nchunks),
// then group_sizes / offsets per expert.
constexpr int kScanThreads = 1024;
__global__ __launch_bounds__(kScanThreads) void dispatch_scan_kernel(int* __restrict__ partial, int E, int nchunks,
                                                                     int32_t* __restrict__ group_sizes,
                                                                     int32_t* __restrict__ offsets) {
  __shared__ int wave_sums[kScanThreads / kWave];
  __shared__ int total_s;
  const int n = E * nchunks;
  const int per = (n + kScanThreads - 1) / kScanThreads;
  const int lo = min(n, (int)threadIdx.x * per), hi = min(n, lo + per);
  int local = 0;
  for (int i = lo; i < hi; ++i) local += partial[i];
  // inclusive scan of the 1024 thread sums: inside each wave with shuffles, then over the 16 wave
  // totals (by every wave for itself), two barriers in all
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  int incl = local;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int v = __shfl_up(incl, d);
    if (lane >= d) incl += v;
  }
  if (lane == kWave - 1) wave_sums[wave] = incl;
  __syncthreads();
  int before = 0;
  for (int w = 0; w < wave; ++w) before += wave_sums[w];
  incl += before;
  int run = incl - local;
  if (threadIdx.x == kScanThreads - 1) total_s = incl;
  for (int i = lo; i < hi; ++i) {
    const int v = partial[i];
    partial[i] = run;
    run += v;
  }
  __syncthreads();
  const int total = total_s;
  for (int e = threadIdx.x; e < E; e += kScanThreads) {
    const int start = partial[(size_t)e * nchunks];
    const int next = (e + 1 < E) ? partial[(size_t)(e + 1) * nchunks] : total;
    offsets[e] = start;
    group_sizes[e] = next - start;
  }
}

// pass 3: stable rank of every assignment inside its chunk + the chunk's base.
__global__ __launch_bounds__(kDispThreads) void dispatch_rank_kernel(const int32_t* __restrict__ ids, int A, int E,
                                                                     int nchunks, const int* __restrict__ base_g,
                                                                     int32_t* __restrict__ source_order,
                                                                     int32_t* __restrict__ inverse) {
  extern __shared__ int smem[];
  int* cursor = smem;         // [E] next free packed row of expert e for this chunk
  int* wavehist = smem + E;   // [kDispWaves][E]
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  for (int e = tid; e < E; e += kDispThreads) cursor[e] = base_g[(size_t)e * nchunks + blockIdx.x];
  for (int i = tid; i < kDispWaves * E; i += kDispThreads) wavehist[i] = 0;
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

// Small batches: the three passes in one workgroup of 1024 threads (histogram in LDS, scan over the
// experts with wave shuffles, then the same ballot ranking with 16 waves per round of 1024
// assignments).  At a few hundred assignments the three launches above are idle most of their
// time; this is one launch with the same results.
constexpr int kSmallThreads = 1024;
constexpr int kSmallWaves = kSmallThreads / kWave;
constexpr int kSmallMaxAssignments = 8192;
constexpr int kSmallMaxExperts = JTMOE_MAX_EXPERTS;  // one thread per expert in the scan
__global__ __launch_bounds__(kSmallThreads) void dispatch_small_kernel(const int32_t* __restrict__ ids, int A, int E,
                                                                      int32_t* __restrict__ group_sizes,
                                                                      int32_t* __restrict__ offsets,
                                                                      int32_t* __restrict__ source_order,
                                                                      int32_t* __restrict__ inverse) {
  extern __shared__ int smem[];
  int* cursor = smem;        // [E] histogram, then the next free packed row of expert e
  int* wavehist = smem + E;  // [kSmallWaves][E]
  __shared__ int wave_sums[kSmallWaves];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  for (int e = tid; e < E; e += kSmallThreads) cursor[e] = 0;
  for (int i = tid; i < kSmallWaves * E; i += kSmallThreads) wavehist[i] = 0;
  __syncthreads();
  for (int a = tid; a < A; a += kSmallThreads) {
    const int id = ids[a];
    if (id >= 0 && id < E) atomicAdd(&cursor[id], 1);
  }
  __syncthreads();
  // exclusive scan over the experts: thread e owns expert e (E <= 1024 threads)
  const int count = tid < E ? cursor[tid] : 0;
  int incl = count;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int v = __shfl_up(incl, d);
    if (lane >= d) incl += v;
  }
  if (lane == kWave - 1) wave_sums[wave] = incl;
  __syncthreads();
  int before = 0;
  for (int w = 0; w < wave; ++w) before += wave_sums[w];
  const int start = incl + before - count;
  if (tid < E) {
    offsets[tid] = start;
    group_sizes[tid] = count;
    cursor[tid] = start;
  }
  __syncthreads();
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  for (int base = 0; base < A; base += kSmallThreads) {
    const int a = base + tid;
    int id = -1;
    if (a < A) {
      id = ids[a];
      if (id < 0 || id >= E) id = -1;
    }
    const bool valid = id >= 0;
    unsigned long long peers = __ballot(valid);  // lanes of this wave holding the same expert id
    for (int b = 0; b < nbits; ++b) {
      const bool bit = (id >> b) & 1;
      const unsigned long long m = __ballot(valid && bit);
      peers &= bit ? m : ~m;
    }
    const int rank = __popcll(peers & ((1ull << lane) - 1ull));
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
    for (int e = tid; e < E; e += kSmallThreads) {
      int add = 0;
#pragma unroll
      for (int w = 0; w < kSmallWaves; ++w) {
        add += wavehist[w * E + e];
        wavehist[w * E + e] = 0;
      }
      cursor[e] += add;
    }
    __syncthreads();
  }
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
    // one wave per row for short rows, up to 256 lanes for long ones
    int bx = 64;
    while (bx < 256 && bx * 4 < row_vecs) bx *= 2;
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

// The launches of a validated dispatch; `partial` holds jtmoe_dispatch_workspace_bytes(A, E) bytes.
// Every entry of partial that is read has been written by the histogram pass of the same call, so
// the scratch needs no clearing between calls.
int dispatch_launch(const int32_t* expert_ids, const void* x, int64_t T, int64_t H, int64_t E, int64_t K, int dtype,
                    int32_t* group_sizes, int32_t* offsets, int32_t* source_order, int32_t* inverse, void* packed_x,
                    int* partial, hipStream_t s) {
  const int64_t A = T * K;
  if (A > 0 && A <= kSmallMaxAssignments && E <= kSmallMaxExperts) {
    dispatch_small_kernel<<<1, kSmallThreads, (size_t)E * (1 + kSmallWaves) * sizeof(int), s>>>(
        expert_ids, (int)A, (int)E, group_sizes, offsets, source_order, inverse);
    stage_mark(kStageDispatchMeta, s);
    if (x != nullptr) launch_dispatch_rows(x, inverse, T, K, H, dtype, packed_x, s);
    stage_mark(kStageDispatchRows, s);
    return check_launch("dispatch");
  }
  const int nchunks = dispatch_chunks(A > 0 ? A : 1);
  dispatch_hist_kernel<<<nchunks, kDispThreads, (size_t)E * sizeof(int), s>>>(expert_ids, (int)A, (int)E, nchunks,
                                                                              partial);
  dispatch_scan_kernel<<<1, kScanThreads, 0, s>>>(partial, (int)E, nchunks, group_sizes, offsets);
  if (A > 0) {
    dispatch_rank_kernel<<<nchunks, kDispThreads, (size_t)E * (1 + kDispWaves) * sizeof(int), s>>>(
        expert_ids, (int)A, (int)E, nchunks, partial, source_order, inverse);
    stage_mark(kStageDispatchMeta, s);
    if (x != nullptr) launch_dispatch_rows(x, inverse, T, K, H, dtype, packed_x, s);
  }
  if (A == 0) stage_mark(kStageDispatchMeta, s);
  stage_mark(kStageDispatchRows, s);
  return check_launch("dispatch");
}

}  // namespace
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
