// The dispatch plan of a small batch, computed by ONE workgroup: histogram of the expert ids in LDS,
// exclusive scan over the experts, then the stable rank of every assignment (ballots inside a wave,
// a per-wave table across the waves).  Same results as the three-pass plan of dispatch.hip
// (local_dispatch of the reference at ep_size == 1, moe.py:583-602).
//
// The body is a device function so that two kernels can end in it: the stand-alone small dispatch,
// and the last workgroup of the small-batch router, which then goes on from the ids it still holds
// in LDS instead of a second launch reading them back.
#pragma once

#include "common.hpp"

namespace jtmoe {

constexpr int kSmallMaxAssignments = 8192;
constexpr int kSmallMaxExperts = JTMOE_MAX_EXPERTS;
constexpr float kImportanceScale = 4294967296.0f;  // importance is summed in 32.32 fixed point: any order, same sum
// A route weight as a 32.32 fixed-point term.  Route weights are finite, non-negative and far below 2^32
// (at most route_scale); anything else (a NaN from non-finite logits, a negative or huge value handed
// to the dispatcher by a caller) would make the float -> integer conversion undefined, so NaN and
// negative values count as 0 and the rest is clamped to the largest float below 2^32.
__device__ __forceinline__ unsigned long long importance_term(float w) {
  w = fminf(fmaxf(w, 0.0f), 4294967040.0f);  // fmaxf(NaN, 0) = 0
  return (unsigned long long)(w * kImportanceScale);
}

// LDS of the body: cursor[E], wavehist[waves][E], wave_sums[waves] ints, then (kStats) imp[E] of 8 bytes
__host__ __device__ inline size_t dispatch_small_smem_bytes(int E, int threads, bool stats) {
  const int waves = threads / kWave;
  size_t n = ((size_t)E * (1 + waves) + waves) * sizeof(int);
  n = (n + 7) / 8 * 8;
  if (stats) n += (size_t)E * 8;
  return n;
}

// ids: A expert ids in assignment order (global memory or LDS); ids outside [0, E) are dropped.
// kStats: also expert_counts[e] = number of assignments of e (as float) and importance[e] = the sum
// of their route weights (the two vectors of _router_stats, moe.py:802-805).
// Requires blockDim.x == kThreads and, for the scan, E <= kThreads.  Ends without a barrier.
template <int kThreads, bool kStats, typename WT>
__device__ __forceinline__ void dispatch_small_body(const int32_t* ids, const WT* weights, int A, int E,
                                                    int32_t* __restrict__ group_sizes, int32_t* __restrict__ offsets,
                                                    int32_t* __restrict__ source_order, int32_t* __restrict__ inverse,
                                                    float* __restrict__ expert_counts, float* __restrict__ importance,
                                                    unsigned char* smem_raw) {
  constexpr int kWaves = kThreads / kWave;
  int* const cursor = reinterpret_cast<int*>(smem_raw);  // [E] histogram, then the next free packed row of expert e
  int* const wavehist = cursor + E;                      // [kWaves][E]
  int* const wave_sums = wavehist + kWaves * E;          // [kWaves]
  unsigned long long* const imp =
      reinterpret_cast<unsigned long long*>(smem_raw + (((size_t)E * (1 + kWaves) + kWaves) * sizeof(int) + 7) / 8 * 8);
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  for (int e = tid; e < E; e += kThreads) {
    cursor[e] = 0;
    if (kStats) imp[e] = 0ull;
  }
  for (int i = tid; i < kWaves * E; i += kThreads) wavehist[i] = 0;
  __syncthreads();
  for (int a = tid; a < A; a += kThreads) {
    const int id = ids[a];
    if (id >= 0 && id < E) {
      atomicAdd(&cursor[id], 1);
      if (kStats) atomicAdd(&imp[id], importance_term(Elem<WT>::load(weights + a)));
    }
  }
  __syncthreads();
  // exclusive scan over the experts: thread e owns expert e
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
    if (kStats) {
      expert_counts[tid] = (float)count;
      importance[tid] = (float)((double)imp[tid] * (1.0 / 4294967296.0));
    }
  }
  __syncthreads();
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  for (int base = 0; base < A; base += kThreads) {
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
    if (base + kThreads >= A) break;  // last round: the tables are not needed again
    __syncthreads();
    for (int e = tid; e < E; e += kThreads) {
      int add = 0;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        add += wavehist[w * E + e];
        wavehist[w * E + e] = 0;
      }
      cursor[e] += add;
    }
    __syncthreads();
  }
}

}  // namespace jtmoe
