// Router: logits -> sigmoid -> (+bias) top-k -> renormalised weights, plus the
// per-expert counts / importance of the router statistics.
//
// Follows SigmoidTopKRouter.__call__ (reference moe.py:131-147) and the two
// vector outputs of _router_stats (moe.py:802-805).  The _sf entry points take the
// score function as an attribute: the reference's sigmoid, or a softmax over the
// experts (which the reference does not have) in front of the same selection.
//
// This file is compiled with floating-point contraction OFF and correctly
// rounded fp32 division: everything after the logits is a fixed sequence of
// IEEE-754 single operations, so the routing decision is a pure function of the
// logits and can be reproduced bit for bit on a CPU.
#include "common.hpp"
#include "dispatch_small.hpp"
#include "grouped_gemm_dma.hpp"

#include <atomic>
#include <chrono>
#include <random>

#include <mutex>

namespace jtmoe {
namespace {

// A workgroup of NW waves routes 16*NW tokens with 64*NW threads (4 lanes per token in the
// selection phase).

// ---- fully specified fp32 sigmoid ------------------------------------------
__device__ __forceinline__ float exp_fixed(float x) {
#pragma clang fp contract(off)
  const float n = rintf(x * 1.4426950408889634f);
  float r = x - n * 0.693145751953125f;
  r = r - n * 1.428606765330187e-06f;
  float p = 1.9875691500e-4f;
  p = p * r;
  p = p + 1.3981999507e-3f;
  p = p * r;
  p = p + 8.3334519073e-3f;
  p = p * r;
  p = p + 4.1665795894e-2f;
  p = p * r;
  p = p + 1.6666665459e-1f;
  p = p * r;
  p = p + 5.0000001201e-1f;
  const float rr = r * r;
  p = p * rr;
  p = p + r;
  p = p + 1.0f;
  return ldexpf(p, (int)n);
}

__device__ __forceinline__ float sigmoid_fixed(float z) {
#pragma clang fp contract(off)
  if (z != z) return z;  // fmaxf / fminf below would turn a NaN into a finite score
  float t = -z;
  t = fmaxf(t, -86.0f);
  t = fminf(t, 86.0f);
  const float e = exp_fixed(t);
  return 1.0f / (1.0f + e);
}

// ---- scratch ----------------------------------------------------------------
struct RouterScratch {
  unsigned long long* imp;  // [E] 32.32 fixed point
  int* cnt;                 // [E]
};

__host__ __device__ inline RouterScratch router_scratch(void* ws, int E) {
  RouterScratch s;  // ws == null: a call that leaves the statistics to the dispatch behind it
  s.imp = reinterpret_cast<unsigned long long*>(ws);
  s.cnt = ws ? reinterpret_cast<int*>(s.imp + E) : nullptr;
  return s;
}

inline size_t router_scratch_bytes(int64_t E) { return align_up((size_t)E * 12, 256); }
// the partial sums of the small-batch kernels start behind the scratch; the arrival word of the decode
// launch behind them
inline size_t router_arrivals_offset(int64_t E);

__global__ void router_zero_kernel(void* ws, int E) {
  RouterScratch s = router_scratch(ws, E);
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    s.imp[e] = 0ull;
    s.cnt[e] = 0;
  }
}

__global__ void router_finalize_kernel(const void* ws, int E, float* counts, float* importance) {
  RouterScratch s = router_scratch(const_cast<void*>(ws), E);
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    counts[e] = (float)s.cnt[e];
    importance[e] = (float)((double)s.imp[e] * (1.0 / 4294967296.0));
  }
}

// ---- LDS layout of one workgroup ----------------------------------------------
struct RouterSmem {
  float* tile;       // [kRouterTokens][E+1] logits, then scores
  float* bias;       // [E]
  int* top_id;       // [kRouterTokens][K]
  int* cnt;          // [E]
  unsigned long long* imp;  // [E]
};

__host__ __device__ inline size_t router_smem_bytes(int E, int K, int kRouterTokens) {
  size_t n = 0;
  n += (size_t)E * 8;                        // imp (first: 8-byte aligned)
  n += (size_t)kRouterTokens * (E + 1) * 4;  // tile
  n += (size_t)E * 4;                        // bias
  n += (size_t)kRouterTokens * K * 4;        // top_id
  n += (size_t)E * 4;                        // cnt
  return n;
}

__device__ __forceinline__ RouterSmem router_smem(unsigned char* base, int E, int K, int kRouterTokens) {
  RouterSmem s;
  s.imp = reinterpret_cast<unsigned long long*>(base);
  s.tile = reinterpret_cast<float*>(s.imp + E);
  s.bias = s.tile + kRouterTokens * (E + 1);
  s.top_id = reinterpret_cast<int*>(s.bias + E);
  s.cnt = s.top_id + kRouterTokens * K;
  return s;
}

// Exchange inside an aligned group of four lanes (lane ^ 1 and lane ^ 2) as a DPP register move
// instead of a trip through the LDS crossbar.
template <int kXor>
__device__ __forceinline__ int quad_xor_i32(int v) {
  static_assert(kXor == 1 || kXor == 2, "quad exchange");
  return kXor == 1 ? __builtin_amdgcn_mov_dpp(v, 0xB1, 0xf, 0xf, true)   // quad_perm [1,0,3,2]
                   : __builtin_amdgcn_mov_dpp(v, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
}
template <int kXor>
__device__ __forceinline__ float quad_xor_f32(float v) {
  return __builtin_bit_cast(float, quad_xor_i32<kXor>(__builtin_bit_cast(int, v)));
}

// Order-preserving map of a float onto a signed integer: a > b as floats <=> key(a) > key(b)
// (-0 is canonicalised to +0 first, so equal floats have equal keys).  Every NaN gets one key below
// -infinity's: a NaN score is chosen last, among NaNs the lower index first -- the order a stable
// descending sort gives (NumPy sorts NaN to the end), and one that keeps the chosen index in range.
// No float maps to INT_MIN, which therefore serves as "already taken".
constexpr int kTakenKey = (int)0x80000000u;
constexpr int kNanKey = kTakenKey + 1;
__device__ __forceinline__ int order_key(float v) {
  const int bits = __builtin_bit_cast(int, v + 0.0f);
  return v != v ? kNanKey : bits ^ ((bits >> 31) & 0x7fffffff);
}

// K rounds of "largest remaining score + bias, lower index on ties" for one token, by its four
// lanes: lane q owns experts [e_begin, e_begin + EQ) and keeps their keys in registers; a taken
// expert's key becomes kTakenKey, below every real value.  A round: the largest key of the token (a run
// of max operations in the lane, two exchanges inside the quad), the lowest index that holds it (the
// lane's own, scanned downwards so that the lowest wins, then the minimum over the quad), and the key at
// that index retired -- no branch, and nothing that waits for the LDS.
constexpr int kNoExpert = 0x7fffffff;
template <int kXor>
__device__ __forceinline__ int quad_max_i32(int v) {
  const int o = quad_xor_i32<kXor>(v);
  return o > v ? o : v;
}
template <int kXor>
__device__ __forceinline__ int quad_min_i32(int v) {
  const int o = quad_xor_i32<kXor>(v);
  return o < v ? o : v;
}
template <int EQ>
__device__ __forceinline__ void select_from_registers(const RouterSmem& sm, const float* row, int e_begin, bool row_ok,
                                                      int t, int q, int K) {
#pragma clang fp contract(off)
  int key[EQ];
#pragma unroll
  for (int j = 0; j < EQ; ++j) key[j] = row_ok ? order_key(row[e_begin + j] + sm.bias[e_begin + j]) : kTakenKey;
  for (int r = 0; r < K; ++r) {
    int best_k = key[0];
#pragma unroll
    for (int j = 1; j < EQ; ++j) best_k = key[j] > best_k ? key[j] : best_k;
    best_k = quad_max_i32<1>(best_k);
    best_k = quad_max_i32<2>(best_k);
    int best_e = kNoExpert;
#pragma unroll
    for (int j = EQ - 1; j >= 0; --j) best_e = key[j] == best_k ? e_begin + j : best_e;
    best_e = quad_min_i32<1>(best_e);
    best_e = quad_min_i32<2>(best_e);
    const int own = best_e - e_begin;
#pragma unroll
    for (int j = 0; j < EQ; ++j) key[j] = j == own ? kTakenKey : key[j];
    if (row_ok && q == 0) sm.top_id[t * K + r] = best_e;
  }
}

// The same selection (same keys, same comparisons) for any expert count: the lane re-reads its quarter
// from LDS in every round.
__device__ __forceinline__ void select_from_lds(const RouterSmem& sm, const float* row, int e_begin, int eq, int E,
                                                bool row_ok, int t, int q, int K) {
#pragma clang fp contract(off)
  unsigned long long taken = 0ull;
  for (int r = 0; r < K; ++r) {
    int best_k = kTakenKey, best_e = -1;
    if (row_ok) {
      for (int j = 0; j < eq; ++j) {
        const int e = e_begin + j;
        if (e < E && !((taken >> j) & 1ull)) {
          const int k = order_key(row[e] + sm.bias[e]);
          if (k > best_k) {  // strictly: the lower index keeps a tie
            best_k = k;
            best_e = e;
          }
        }
      }
    }
#pragma unroll
    for (int m = 1; m <= 2; m <<= 1) {
      const int ok = __shfl_xor(best_k, m, 4);
      const int oe = __shfl_xor(best_e, m, 4);
      const bool take = oe >= 0 && (best_e < 0 || ok > best_k || (ok == best_k && oe < best_e));
      if (take) {
        best_k = ok;
        best_e = oe;
      }
    }
    if (row_ok) {
      const int j = best_e - e_begin;
      if (j >= 0 && j < eq) taken |= 1ull << j;
      if (q == 0) sm.top_id[t * K + r] = best_e;
    }
  }
}

// Everything after the logits tile is in LDS.  `T` is the output element type of
// the weights.
template <typename T, int kRouterTokens, int kRouterThreads>
__device__ void router_epilogue(const RouterSmem& sm, const float* __restrict__ bias_g, int t0, int tokens,
                                int E, int K, float route_scale, int32_t* __restrict__ ids_out,
                                T* __restrict__ weights_out, float* __restrict__ scores_out,
                                float* __restrict__ logits_out, RouterScratch g, int score_func,
                                float* __restrict__ counts_final = nullptr,
                                float* __restrict__ importance_final = nullptr) {
#pragma clang fp contract(off)
  const int tid = threadIdx.x;
  const int stride = E + 1;
  const int nrows = min(kRouterTokens, tokens - t0);
  const bool softmax = score_func == JTMOE_SCORE_SOFTMAX;

  for (int e = tid; e < E; e += kRouterThreads) {
    sm.bias[e] = bias_g ? bias_g[e] : 0.0f;
    sm.cnt[e] = 0;
    sm.imp[e] = 0ull;
  }
  if (softmax) {
    // Softmax over the experts of every token, in place, by the token's four lanes (lane q owns the
    // run of ceil(E/4) consecutive experts that it owns in the selection below):
    // m = max z;  p_e = exp(max(z_e - m, -86));  the four run sums, each added in index order, are
    // combined as (s0 + s1) + (s2 + s3);  score_e = p_e / sum.  A fixed sequence of fp32 operations.
    if (logits_out)
      for (int idx = tid; idx < nrows * E; idx += kRouterThreads) {
        const int t = idx / E, e = idx - t * E;
        logits_out[(size_t)(t0 + t) * E + e] = sm.tile[t * stride + e];
      }
    __syncthreads();
    const int t = tid >> 2, q = tid & 3;
    const int eq = (E + 3) >> 2;
    const int e_lo = q * eq, e_hi = min(E, e_lo + eq);
    const bool row_ok = t < nrows;
    float* const row = sm.tile + t * stride;
    float m = -INFINITY;
    if (row_ok)
      for (int e = e_lo; e < e_hi; ++e) m = fmaxf(m, row[e]);
    m = fmaxf(m, quad_xor_f32<1>(m));
    m = fmaxf(m, quad_xor_f32<2>(m));
    float part = 0.0f;
    if (row_ok)
      for (int e = e_lo; e < e_hi; ++e) {
        float d = row[e] - m;
        d = fmaxf(d, -86.0f);
        const float p = exp_fixed(d);
        row[e] = p;
        part = part + p;
      }
    const float pair = part + quad_xor_f32<1>(part);
    const float total = pair + quad_xor_f32<2>(pair);
    if (row_ok)
      for (int e = e_lo; e < e_hi; ++e) row[e] = row[e] / total;
    __syncthreads();
  }
  // logits -> scores (in place), both written out row-major
  for (int idx = tid; idx < nrows * E; idx += kRouterThreads) {
    const int t = idx / E, e = idx - t * E;
    const float z = sm.tile[t * stride + e];
    if (logits_out && !softmax) logits_out[(size_t)(t0 + t) * E + e] = z;
    const float s = softmax ? z : sigmoid_fixed(z);
    sm.tile[t * stride + e] = s;
    scores_out[(size_t)(t0 + t) * E + e] = s;
  }
  __syncthreads();

  // selection: 4 lanes per token, each owning a contiguous quarter of the experts
  // (sixteen lanes per token, where a workgroup has them to spare, measured no faster: a round costs
  // its chain of dependent steps, not its compares)
  const int t = tid >> 2, q = tid & 3;
  const int eq = (E + 3) >> 2;
  const int e_begin = q * eq;
  const bool row_ok = t < nrows;
  const float* row = sm.tile + t * stride;
  // For the usual expert counts the lane keeps its quarter (score + bias) in registers, so that a
  // round is a run of compares instead of a chain of LDS reads; same scan order, same comparisons.
  if (E == 64 || E == 128 || E == 32 || E == 256 || E == 16) {
    switch (E) {
      case 16: select_from_registers<4>(sm, row, e_begin, row_ok, t, q, K); break;
      case 32: select_from_registers<8>(sm, row, e_begin, row_ok, t, q, K); break;
      case 64: select_from_registers<16>(sm, row, e_begin, row_ok, t, q, K); break;
      case 128: select_from_registers<32>(sm, row, e_begin, row_ok, t, q, K); break;
      default: select_from_registers<64>(sm, row, e_begin, row_ok, t, q, K); break;
    }
  } else {
    select_from_lds(sm, row, e_begin, eq, E, row_ok, t, q, K);
  }
  __syncthreads();  // the selection of a token was written by its lane 0 and is read by all its lanes
  // renormalise: the lanes of a token share out its K slots; each adds up the denominator itself, in
  // slot order
  if (row_ok) {
    float denom = row[sm.top_id[t * K]];
    for (int r = 1; r < K; ++r) denom = denom + row[sm.top_id[t * K + r]];
    denom = denom + 1e-20f;
    for (int r = q; r < K; r += 4) {
      const int e = sm.top_id[t * K + r];
      float w = row[e] / denom;
      w = w * route_scale;
      w = Elem<T>::round(w);
      const size_t o = (size_t)(t0 + t) * K + r;
      ids_out[o] = e;
      Elem<T>::store(weights_out + o, w);
      atomicAdd(&sm.cnt[e], 1);
      atomicAdd(&sm.imp[e], importance_term(w));
    }
  }
  __syncthreads();
  if (counts_final != nullptr) {
    // the only workgroup of the call: its sums are the statistics (same conversion as router_finalize_kernel)
    for (int e = tid; e < E; e += kRouterThreads) {
      counts_final[e] = (float)sm.cnt[e];
      importance_final[e] = (float)((double)sm.imp[e] * (1.0 / 4294967296.0));
    }
    return;
  }
  if (g.cnt == nullptr) return;
  for (int e = tid; e < E; e += kRouterThreads) {
    const int c = sm.cnt[e];
    if (c) {
      atomicAdd(&g.cnt[e], c);
      atomicAdd(&g.imp[e], sm.imp[e]);
    }
  }
}

// Generic projection: any H, E; fp32 accumulation in k order.
template <typename T, bool kFromLogits>
__global__ __launch_bounds__(256) void router_kernel(
    const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ logits_in,
    const float* __restrict__ bias, int tokens, int H, int E, int K, float route_scale,
    int32_t* __restrict__ ids, T* __restrict__ weights, float* __restrict__ scores,
    float* __restrict__ logits_out, void* ws, int score_func) {
  constexpr int kRouterTokens = 64, kRouterThreads = 256;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  RouterSmem sm = router_smem(smem_raw, E, K, kRouterTokens);
  const int t0 = blockIdx.x * kRouterTokens;
  const int nrows = min(kRouterTokens, tokens - t0);
  const int stride = E + 1;
  for (int idx = threadIdx.x; idx < nrows * E; idx += kRouterThreads) {
    const int t = idx / E, e = idx - t * E;
    float z;
    if (kFromLogits) {
      z = logits_in[(size_t)(t0 + t) * E + e];
    } else {
      const T* xr = x + (size_t)(t0 + t) * H;
      float acc = 0.0f;
      for (int k = 0; k < H; ++k) acc = fmaf(Elem<T>::load(xr + k), Elem<T>::load(w + (size_t)k * E + e), acc);
      z = Elem<T>::round(acc);
    }
    sm.tile[t * stride + e] = z;
  }
  __syncthreads();
  router_epilogue<T, 64, 256>(sm, bias, t0, tokens, E, K, route_scale, ids, weights, scores, logits_out,
                              router_scratch(ws, E), score_func);
}

// ---------------------------------------------------------------------------
// bf16 projection on the matrix cores.
//
// ONE summation order for every batch size.  A token's logits must not depend on how many tokens
// share its call (a decode step of 64 tokens and a prefill of 16 384 have to route a row the same
// way), although small batches want the k range shared out over many workgroups and large ones want
// it walked by one.  All the matrix-core kernels below therefore add up a logit in this order:
//   * H is cut into slices of router_slice_rows(H) consecutive k rows (eight slices, or as many
//     128-row chunks as there are, when H is a multiple of 128; one slice otherwise);
//   * inside a slice, v_mfma_f32_16x16x32_bf16 instructions are chained in k order, the first onto a
//     zero accumulator, instruction n of the slice taking k = 32 n + 8 g + j at element j of lane
//     group g (g = lane / 16) of both operands;
//   * the slice sums are added in slice order, starting from the first slice's sum, and the total is
//     rounded to bf16 (the projection's output dtype).
// The large-batch kernel walks the slices one after the other with a second set of accumulators; the
// small-batch kernels compute them in different workgroups and add them up afterwards.
//
// Large batches: one workgroup = 64 tokens = 4 waves of 16 tokens; each wave owns all E columns of
// its tokens (NB = E/16 accumulator tiles).  x is read straight from HBM into MFMA operand registers
// (each lane two 16-byte pieces per 64-wide k chunk, the four lane groups of a token together whole
// 128-byte lines per token row); the router matrix [H,E] is staged chunk by chunk through LDS as it
// is stored and read with the transposing ds_read_b64_tr_b16.
// Requires H % 64 == 0 and E in {16, 32, 64, 128, 256}.
// ---------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
constexpr int kRouterKC = 64;  // k rows of the router matrix per LDS stage
constexpr int kSplitKC = 128;  // k rows per LDS stage of the small-batch kernels; the unit the slices are cut in
constexpr int kPartialMaxSlices = 8;

// k rows per slice of the summation order (see above); a function of H only
__host__ __device__ inline int router_slice_rows(int H) {
  if (H % kSplitKC != 0) return H;
  const int chunks = H / kSplitKC;
  return (chunks + kPartialMaxSlices - 1) / kPartialMaxSlices * kSplitKC;
}

__host__ __device__ inline int router_w_stride(int E) { return E + 32; }  // elements; +64 B between k rows
__host__ __device__ inline size_t router_mfma_smem_bytes(int E, int K, int tokens_per_wg) {
  const size_t w = (size_t)2 * kRouterKC * router_w_stride(E) * 2;
  const size_t ep = router_smem_bytes(E, K, tokens_per_wg);
  return w > ep ? w : ep;
}

template <int NB, int NW>
__global__ __launch_bounds__(64 * NW) void router_mfma_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, const float* __restrict__ bias, int tokens,
    int H, int K, float route_scale, int32_t* __restrict__ ids, bf16_raw* __restrict__ weights,
    float* __restrict__ scores, float* __restrict__ logits_out, void* ws, int score_func) {
  constexpr int kRouterTokens = 16 * NW, kRouterThreads = 64 * NW;
  const int slice_chunks = router_slice_rows(H) / kRouterKC;  // 64-row chunks per slice
  constexpr int E = NB * 16;
  constexpr int WS = E + 32;                      // LDS row stride of the staged matrix (elements)
  constexpr int W_CHUNKS = kRouterKC * E / 8;     // 16-byte chunks per stage
  constexpr int CW = (W_CHUNKS + kRouterThreads - 1) / kRouterThreads;
  constexpr int CPR = E / 8;                      // chunks per k row
  extern __shared__ __align__(16) unsigned char smem_raw[];
  uint16_t* const Ws = reinterpret_cast<uint16_t*>(smem_raw);  // [2][kRouterKC][WS]; reused by the epilogue

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int t0 = blockIdx.x * kRouterTokens;
  const int nrows = min(kRouterTokens, tokens - t0);

  // x: lane (m = lane%16, g = lane/16) holds k = chunk*64 + s*32 + g*8 + [0,8), s = 0, 1, of token t0 + wave*16 + m
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(x + (size_t)t0 * H), 0, nrows * H * 2, kBufferFlags);
  const int x_voff = ((wave * 16 + (lane & 15)) * H + (lane >> 4) * 8) * 2;
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(w), 0, H * E * 2, kBufferFlags);

  // Loads run D chunks ahead of the MFMAs through a ring of registers (chunk c lives in slot
  // c % D), so that the latency of a load is hidden by D - 1 whole iterations instead of by the
  // few MFMAs of one: with a single chunk in flight every iteration waits for memory.
  // The memory pipeline returns loads in order, so what is in flight while a wave waits for the
  // next chunk of the router matrix is everything issued after it: D - 1 chunks of the matrix and of
  // x.  x comes from HBM (the only large stream of this kernel, 2 KB per wave and chunk): with three
  // slots a CU had 16 KB of it in flight and the kernel ran at a quarter of the HBM rate; the ring
  // is as deep as the registers of the matrix chunks allow.
  constexpr int D = CW <= 2 ? 8 : (CW <= 4 ? 6 : (CW <= 8 ? 4 : 2));
  constexpr int UNROLL = D;  // a multiple of D and of the two LDS stages
  static_assert(D % 2 == 0, "the unrolled body alternates between the two LDS stages");
  u32x4_t a_ring[D][2], w_ring[D][CW];
  f32x4_t acc[NB], total[NB];  // the current slice's sum, and the sum of the slices before it
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[nb][i] = total[nb][i] = 0.0f;

#define JT_LOAD_W(slot, k0)                                                                  \
  _Pragma("unroll") for (int i = 0; i < CW; ++i) {                                           \
    const int c = tid + i * kRouterThreads;                                                  \
    if (W_CHUNKS % kRouterThreads == 0 || c < W_CHUNKS)                                      \
      w_ring[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, c * 16, (k0)*E * 2, 0); \
  }
#define JT_STORE_W(slot, stage)                                                              \
  _Pragma("unroll") for (int i = 0; i < CW; ++i) {                                           \
    const int c = tid + i * kRouterThreads;                                                  \
    if (W_CHUNKS % kRouterThreads == 0 || c < W_CHUNKS) {                                    \
      const int kr = c / CPR, nc = c - kr * CPR;                                             \
      *reinterpret_cast<u32x4_t*>(Ws + ((stage)*kRouterKC + kr) * WS + nc * 8) = w_ring[slot][i]; \
    }                                                                                        \
  }
#define JT_LOAD_X(slot, k0)                                                                  \
  {                                                                                          \
    a_ring[slot][0] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, x_voff, (k0)*2, 0);      \
    a_ring[slot][1] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, x_voff + 64, (k0)*2, 0); \
  }

  // transposing read of this lane: 16-lane group g = lane/16 reads rows 32*s + 8*g + 4*h + i/4
  const int w_lane = ((lane >> 4) * 8 + ((lane & 15) >> 2)) * WS + 4 * (lane & 3);
  const int nchunks = H / kRouterKC;
  int in_slice = 0;  // chunks of the current slice done
#pragma unroll
  for (int d = 0; d < D; ++d)
    if (d < nchunks) {
      JT_LOAD_W(d, d * kRouterKC);
      JT_LOAD_X(d, d * kRouterKC);
    }
  JT_STORE_W(0, 0);
  __syncthreads();
  for (int kc0 = 0; kc0 < nchunks; kc0 += UNROLL) {
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
      const int kc = kc0 + j;
      if (kc < nchunks) {  // uniform over the workgroup
        constexpr int kStages = 2;
        const int stage = j % kStages, slot = j % D, next_slot = (j + 1) % D;
        static_assert(D > 1, "a slot is refilled after the MFMAs that read it");
        const uint16_t* wbase = Ws + stage * kRouterKC * WS + w_lane;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const bf16x8_t a = __builtin_bit_cast(bf16x8_t, a_ring[slot][s]);
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            const uint16_t* p = wbase + s * 32 * WS + nb * 16;
            const s16x4_t lo =
                __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p));
            const s16x4_t hi =
                __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p + 4 * WS));
            const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            acc[nb] =
                __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8_t, both), acc[nb], 0, 0, 0);
          }
        }
        if (kc + 1 < nchunks) JT_STORE_W(next_slot, stage ^ 1);
        if (kc + D < nchunks) {
          JT_LOAD_W(slot, (kc + D) * kRouterKC);
          JT_LOAD_X(slot, (kc + D) * kRouterKC);
        }
        // end of a slice (uniform; the last slice may be shorter): its sum joins the total, in slice order
        if (++in_slice == slice_chunks || kc + 1 == nchunks) {
          const bool first = kc < slice_chunks;
          in_slice = 0;
#pragma unroll
          for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              total[nb][i] = first ? acc[nb][i] : total[nb][i] + acc[nb][i];
              acc[nb][i] = 0.0f;
            }
        }
        __syncthreads();
      }
    }
  }
#undef JT_LOAD_W
#undef JT_STORE_W
#undef JT_LOAD_X

  // logits (rounded to bf16, as the projection's output dtype) -> LDS tile; value i of lane l
  // is token row 4*(l/16) + i, expert nb*16 + l%16
  RouterSmem sm = router_smem(smem_raw, E, K, kRouterTokens);
  const int stride = E + 1;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      sm.tile[(wave * 16 + 4 * (lane >> 4) + i) * stride + nb * 16 + (lane & 15)] = round_to_bf16(total[nb][i]);
  __syncthreads();
  router_epilogue<bf16_raw, 16 * NW, 64 * NW>(sm, bias, t0, tokens, E, K, route_scale, ids, weights, scores,
                                              logits_out, router_scratch(ws, E), score_func);
}

// ---------------------------------------------------------------------------
// Small batches: 16 tokens per workgroup, 128 k rows per LDS stage, and the four waves of a workgroup
// share out the EXPERT COLUMNS (wave w owns the 16-column blocks w, w + 4, ...), so that each
// accumulator still sees its k range as one chain in k order -- the summation order above.
// A workgroup then runs H/128 short iterations instead of H/64 longer ones, and 16 tokens already
// make a workgroup, so small batches spread over more CUs.
// ---------------------------------------------------------------------------
constexpr int kSplitMaxTokens = 256;

__host__ __device__ inline size_t router_split_smem_bytes(int E, int K) {
  const size_t w = (size_t)2 * kSplitKC * router_w_stride(E) * 2;
  const size_t ep = router_smem_bytes(E, K, 16);
  return w > ep ? w : ep;
}

// kPartial: the grid's y dimension shares out the slices; a workgroup then only writes the unrounded
// sum of its slice, partial_out[slice][token][expert], and router_finish_kernel adds the slices in
// order and does the rest.  Otherwise the workgroup walks all slices itself.
// (token_block / slice: the workgroup's place in the launch's grid -- blockIdx.x / blockIdx.y in
// router_mfma_split_kernel; the decode launch hands them out among its own workgroups)
template <int NB, bool kPartial>
__device__ __forceinline__ void router_split_body(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, const float* __restrict__ bias, int tokens,
    int H, int K, float route_scale, int32_t* __restrict__ ids, bf16_raw* __restrict__ weights,
    float* __restrict__ scores, float* __restrict__ logits_out, void* ws, float* __restrict__ partial_out,
    int score_func, int token_block, int slice) {
  constexpr int kThreads = 256, kTokens = 16;
  constexpr int E = NB * 16;
  constexpr int WS = E + 32;
  constexpr int W_CHUNKS = kSplitKC * E / 8;
  constexpr int CW = (W_CHUNKS + kThreads - 1) / kThreads;
  constexpr int CPR = E / 8;
  constexpr int NBW = (NB + 3) / 4;  // column blocks per wave
  extern __shared__ __align__(16) unsigned char smem_raw[];
  uint16_t* const Ws = reinterpret_cast<uint16_t*>(smem_raw);  // [2][kSplitKC][WS]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool has_cols = wave < NB;  // with fewer than four column blocks some waves only help to stage the matrix
  const int t0 = token_block * kTokens;
  const int nrows = min(kTokens, tokens - t0);
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(x + (size_t)t0 * H), 0, nrows * H * 2, kBufferFlags);
  // lane (m = lane%16, g = lane/16) holds k = chunk*128 + n*32 + g*8 + [0,8), n = 0..3, of token t0 + m
  const int x_voff = ((lane & 15) * H + (lane >> 4) * 8) * 2;
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(w), 0, H * E * 2, kBufferFlags);

  constexpr int D = CW <= 8 ? 3 : 2;   // chunks in flight (register ring, chunk c in slot c % D)
  constexpr int UNROLL = D == 3 ? 6 : 2;
  u32x4_t a_ring[D][4], w_ring[D][CW];
  f32x4_t acc[NBW], total[NBW];
#pragma unroll
  for (int b = 0; b < NBW; ++b)
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[b][i] = total[b][i] = 0.0f;

#define JT_LOAD(slot, k0)                                                                     \
  {                                                                                           \
    _Pragma("unroll") for (int i = 0; i < CW; ++i) {                                          \
      const int c = tid + i * kThreads;                                                       \
      if (W_CHUNKS % kThreads == 0 || c < W_CHUNKS)                                           \
        w_ring[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, c * 16, (k0)*E * 2, 0); \
    }                                                                                         \
    if (has_cols) {                                                                           \
      _Pragma("unroll") for (int n = 0; n < 4; ++n)                                           \
        a_ring[slot][n] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, x_voff + n * 64, (k0)*2, 0); \
    }                                                                                         \
  }
#define JT_STORE_W(slot, stage)                                                               \
  _Pragma("unroll") for (int i = 0; i < CW; ++i) {                                            \
    const int c = tid + i * kThreads;                                                         \
    if (W_CHUNKS % kThreads == 0 || c < W_CHUNKS) {                                           \
      const int kr = c / CPR, nc = c - kr * CPR;                                              \
      *reinterpret_cast<u32x4_t*>(Ws + ((stage)*kSplitKC + kr) * WS + nc * 8) = w_ring[slot][i]; \
    }                                                                                         \
  }

  // transposing read: the 16-lane group g reads rows n*32 + g*8 + 4*h + i/4, columns 4*(i%4)..
  const int w_lane = ((lane >> 4) * 8 + ((lane & 15) >> 2)) * WS + 4 * (lane & 3);
  // this workgroup's chunks: one slice of them, or all
  const int slice_chunks = router_slice_rows(H) / kSplitKC;
  const int chunk0 = kPartial ? slice * slice_chunks : 0;
  const int nchunks = kPartial ? min(slice_chunks, H / kSplitKC - chunk0) : H / kSplitKC;
  const int kbase = chunk0 * kSplitKC;
  int in_slice = 0;
#pragma unroll
  for (int d = 0; d < D; ++d)
    if (d < nchunks) JT_LOAD(d, kbase + d * kSplitKC);
  JT_STORE_W(0, 0);
  __syncthreads();
  for (int kc0 = 0; kc0 < nchunks; kc0 += UNROLL) {
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
      const int kc = kc0 + j;
      if (kc < nchunks) {  // uniform over the workgroup
        const int stage = j % 2, slot = j % D, next_slot = (j + 1) % D;
        if (has_cols) {
          const uint16_t* wbase = Ws + stage * kSplitKC * WS + w_lane + wave * 16;
#pragma unroll
          for (int n = 0; n < 4; ++n) {
            const bf16x8_t a = __builtin_bit_cast(bf16x8_t, a_ring[slot][n]);
#pragma unroll
            for (int b = 0; b < NBW; ++b) {
              const uint16_t* p = wbase + n * 32 * WS + b * 64;
              const s16x4_t lo =
                  __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p));
              const s16x4_t hi =
                  __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p + 4 * WS));
              const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
              acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8_t, both), acc[b], 0, 0, 0);
            }
          }
        }
        if (kc + 1 < nchunks) JT_STORE_W(next_slot, stage ^ 1);
        if (kc + D < nchunks) JT_LOAD(slot, kbase + (kc + D) * kSplitKC);
        if (!kPartial && (++in_slice == slice_chunks || kc + 1 == nchunks)) {
          // end of a slice: its sum joins the total, in slice order
          const bool first = kc < slice_chunks;
          in_slice = 0;
#pragma unroll
          for (int b = 0; b < NBW; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              total[b][i] = first ? acc[b][i] : total[b][i] + acc[b][i];
              acc[b][i] = 0.0f;
            }
        }
        __syncthreads();
      }
    }
  }
#undef JT_LOAD
#undef JT_STORE_W

  // value i of lane l of block b is token row 4*(l/16) + i, expert (wave + 4 b)*16 + l%16
  if (kPartial) {
    if (has_cols) {
#pragma unroll
      for (int b = 0; b < NBW; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int t = 4 * (lane >> 4) + i;
          if (t < nrows && wave + 4 * b < NB)
            partial_out[((size_t)slice * tokens + t0 + t) * E + (wave + 4 * b) * 16 + (lane & 15)] = acc[b][i];
        }
    }
    return;
  }
  // the total, rounded to bf16 (the projection's output dtype) -> LDS tile (the matrix stages are dead:
  // the loop ends with a barrier)
  RouterSmem sm = router_smem(smem_raw, E, K, kTokens);
  const int stride = E + 1;
  if (has_cols) {
#pragma unroll
    for (int b = 0; b < NBW; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (wave + 4 * b < NB)
          sm.tile[(4 * (lane >> 4) + i) * stride + (wave + 4 * b) * 16 + (lane & 15)] = round_to_bf16(total[b][i]);
  }
  __syncthreads();
  router_epilogue<bf16_raw, kTokens, kThreads>(sm, bias, t0, tokens, E, K, route_scale, ids, weights, scores,
                                               logits_out, router_scratch(ws, E), score_func);
}

template <int NB, bool kPartial>
__global__ __launch_bounds__(256) void router_mfma_split_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, const float* __restrict__ bias, int tokens,
    int H, int K, float route_scale, int32_t* __restrict__ ids, bf16_raw* __restrict__ weights,
    float* __restrict__ scores, float* __restrict__ logits_out, void* ws, float* __restrict__ partial_out,
    int score_func) {
  router_split_body<NB, kPartial>(x, w, bias, tokens, H, K, route_scale, ids, weights, scores, logits_out, ws,
                                  partial_out, score_func, (int)blockIdx.x, (int)blockIdx.y);
}

// Second half of the small-batch router: one workgroup adds the slices of partial sums in slice
// order, rounds to bf16 (the projection's output dtype) and runs the epilogue for every token of
// the call, so the statistics need neither the zeroing nor the finalising launch.
//
// kPlan: the workgroup then goes on to the dispatch plan of these assignments (group sizes, offsets,
// the stable permutation and its inverse) from the ids it holds in LDS; the tables of that step take
// the place of the score tile, which is dead by then.  Requires tokens * K <= kSmallMaxAssignments
// and E <= 4 * kTok.
template <int kTok, bool kPlan>
__device__ __forceinline__ void router_finish_body(
    const float* __restrict__ partial, int slices, const float* __restrict__ bias, int tokens, int E, int K,
    float route_scale, int32_t* __restrict__ ids, bf16_raw* __restrict__ weights, float* __restrict__ scores,
    float* __restrict__ logits_out, float* __restrict__ counts, float* __restrict__ importance,
    int32_t* __restrict__ group_sizes, int32_t* __restrict__ offsets, int32_t* __restrict__ source_order,
    int32_t* __restrict__ inverse, int score_func) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  RouterSmem sm = router_smem(smem_raw, E, K, kTok);
  const int stride = E + 1;
  const size_t plane = (size_t)tokens * E;
#pragma unroll 4
  for (int idx = threadIdx.x; idx < tokens * E; idx += 4 * kTok) {
    const int t = idx / E, e = idx - t * E;
    float part[kPartialMaxSlices];  // all slices requested before the first is needed
#pragma unroll
    for (int sl = 0; sl < kPartialMaxSlices; ++sl) part[sl] = sl < slices ? partial[sl * plane + idx] : 0.0f;
    float v = part[0];
#pragma unroll
    for (int sl = 1; sl < kPartialMaxSlices; ++sl)
      if (sl < slices) v += part[sl];
    sm.tile[t * stride + e] = round_to_bf16(v);
  }
  __syncthreads();
  router_epilogue<bf16_raw, kTok, 4 * kTok>(sm, bias, 0, tokens, E, K, route_scale, ids, weights, scores, logits_out,
                                            RouterScratch{}, score_func, counts, importance);
  if (kPlan) {
    static_assert(kTok >= 1 + 4 * kTok / kWave, "the plan's tables fit into the score tile");
    dispatch_small_body<4 * kTok, false, bf16_raw>(sm.top_id, nullptr, tokens * K, E, group_sizes, offsets,
                                                   source_order, inverse, nullptr, nullptr,
                                                   reinterpret_cast<unsigned char*>(sm.tile));
  }
}

template <int kTok, bool kPlan>
__global__ __launch_bounds__(4 * kTok) void router_finish_kernel(
    const float* __restrict__ partial, int slices, const float* __restrict__ bias, int tokens, int E, int K,
    float route_scale, int32_t* __restrict__ ids, bf16_raw* __restrict__ weights, float* __restrict__ scores,
    float* __restrict__ logits_out, float* __restrict__ counts, float* __restrict__ importance,
    int32_t* __restrict__ group_sizes, int32_t* __restrict__ offsets, int32_t* __restrict__ source_order,
    int32_t* __restrict__ inverse, int score_func) {
  router_finish_body<kTok, kPlan>(partial, slices, bias, tokens, E, K, route_scale, ids, weights, scores, logits_out,
                                  counts, importance, group_sizes, offsets, source_order, inverse, score_func);
}

inline size_t router_arrivals_offset(int64_t E) {
  return router_scratch_bytes(E) + align_up((size_t)kPartialMaxSlices * kSplitMaxTokens * E * sizeof(float), 256);
}

// ---------------------------------------------------------------------------
// The decode launch: ONE launch in which most workgroups stream the gate and up matrices (every token
// through every expert, grouped_gemm_dma_tile in its uniform mode -- nothing of that needs the routing)
// and the first token_blocks * slices workgroups are the small-batch router: each computes the partial
// sums of its (token block, slice), counts itself in, and the last of them to arrive adds the slices up
// in slice order and runs the epilogue and the dispatch plan (router_finish_body) -- the same arithmetic
// in the same order as the two-launch form, so the same bits.  The router's 21 us of dependent steps
// then run beside the 115 us of weight streaming instead of in front of it, with no second stream and
// no dependency between launches other than the stream's own order.
// The arrival counter is a 64-bit word of the caller's workspace: the low byte counts, the rest is a tag
// the host draws per launch.  A word whose tag is not this launch's counts as zero, so the word needs no
// clearing before its first use (the workspace arrives with whatever it held; the first tag of a process
// is random, 56 bits); the workgroup that finishes writes zero, so a captured launch, whose tag is the
// same at every replay, starts from zero as well.  No state outside the workspace: calls are as
// re-entrant as their workspaces are distinct.
// ---------------------------------------------------------------------------
std::atomic<unsigned long long> g_decode_tag{0};

unsigned long long next_decode_tag() {
  unsigned long long t = g_decode_tag.load(std::memory_order_relaxed);
  if (t == 0) {  // first use in this process
    std::random_device rd;
    unsigned long long seed = ((unsigned long long)rd() << 32) ^ rd() ^
                              (unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count();
    unsigned long long expected = 0;
    g_decode_tag.compare_exchange_strong(expected, seed | 1ull, std::memory_order_relaxed);
  }
  t = g_decode_tag.fetch_add(1ull, std::memory_order_relaxed) & 0x00ffffffffffffffull;
  return (t == 0 ? 1ull : t) << 8;
}

template <int NB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3))) void decode_gate_up_router_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ gate, const uint16_t* __restrict__ up,
    uint16_t* __restrict__ act_full, int T, int H, int I, int mtiles, int ntiles_n,
    const uint16_t* __restrict__ w_router, const float* __restrict__ bias, int K, float route_scale, int score_func,
    int32_t* __restrict__ ids, bf16_raw* __restrict__ weights, float* __restrict__ scores,
    float* __restrict__ counts, float* __restrict__ importance, int32_t* __restrict__ group_sizes,
    int32_t* __restrict__ offsets, int32_t* __restrict__ source_order, int32_t* __restrict__ inverse,
    float* __restrict__ partial, int token_blocks, int slices, unsigned long long* __restrict__ arrivals,
    unsigned long long tag) {
  constexpr int E = NB * 16;
  const int router_blocks = token_blocks * slices;
  if ((int)blockIdx.x >= router_blocks) {
    grouped_gemm_dma_tile<GateUpTinyCfg>(x, gate, up, act_full, nullptr, nullptr, E, E * T, H, I, mtiles, ntiles_n,
                                         nullptr, 1, 0, nullptr, nullptr, /*uniform_rows=*/T, 0,
                                         (int)blockIdx.x - router_blocks, (int)gridDim.x - router_blocks);
    return;
  }
  __shared__ int is_last;
  const int token_block = (int)blockIdx.x % token_blocks, slice = (int)blockIdx.x / token_blocks;
  router_split_body<NB, true>(x, w_router, bias, T, H, K, route_scale, ids, weights, scores, nullptr, nullptr, partial,
                              score_func, token_block, slice);
  // Hand-over.  Every thread waits until its own stores have reached the L2 (on this part stores count in
  // vmcnt); after the barrier one thread releases them to the device (the fence writes the L2's dirty
  // lines back, so that the other XCDs can see them) and counts the workgroup in.  The workgroup that
  // finds everyone else counted acquires with one fence (it invalidates this CU's L1 and the stale lines
  // of its L2) before any of its threads reads the others' sums.  One fence per workgroup, not one per
  // thread: each is an operation on whole caches.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    __threadfence();
    unsigned long long seen = atomicAdd(arrivals, 0ull), assumed;
    unsigned count;
    do {  // lock-free: some workgroup's exchange always succeeds
      assumed = seen;
      count = (assumed >> 8) == (tag >> 8) ? (unsigned)(assumed & 0xffull) : 0u;
      seen = atomicCAS(arrivals, assumed, tag | (unsigned long long)(count + 1u));
    } while (seen != assumed);
    is_last = count + 1u == (unsigned)router_blocks;
    if (is_last) __threadfence();
  }
  __syncthreads();
  if (!is_last) return;
  router_finish_body<64, true>(partial, slices, bias, T, E, K, route_scale, ids, weights, scores, nullptr, counts,
                               importance, group_sizes, offsets, source_order, inverse, score_func);
  if (threadIdx.x == 0) *arrivals = 0ull;
}

template <typename KernelT>
int set_max_smem(KernelT kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return JTMOE_OK;
  hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (err != hipSuccess) return fail(JTMOE_ELAUNCH, "hipFuncSetAttribute(router): %s", hipGetErrorString(err));
  return JTMOE_OK;
}

// What a layer call adds to a router call: it may leave the statistics to the dispatch that follows
// (stats_done = false on return), and the small-batch path writes the dispatch plan as well.
struct LayerPlan {
  int32_t* group_sizes;
  int32_t* offsets;
  int32_t* source_order;
  int32_t* inverse;
  bool stats_done;
  bool plan_done;
};

template <typename T, bool kFromLogits>
int launch_router(const void* x, const void* w, const float* logits_in, const float* bias, int64_t tokens,
                  int64_t H, int64_t E, int64_t K, double route_scale, int32_t* ids, void* weights,
                  float* scores, float* counts, float* importance, float* logits_out, void* ws,
                  hipStream_t stream, int score_func, LayerPlan* layer = nullptr) {
  // a stand-alone call always computes the statistics; a layer call only where they cost no launch
  const bool stats = layer == nullptr;
  void* const ws_stats = stats ? ws : nullptr;
  if (layer) layer->stats_done = layer->plan_done = false;
  const bool mfma = Elem<T>::is_bf16 && !kFromLogits && H % kRouterKC == 0 && H * E < ((int64_t)1 << 30) &&
                    (E == 16 || E == 32 || E == 64 || E == 128 || E == 256) && aligned16(x) && aligned16(w);
  if (mfma) {
    // Up to a few hundred tokens the whole call is a handful of workgroups, each waiting on its own
    // chain of chunks: the k-split kernel (16 tokens per workgroup, half as many and shorter
    // iterations) is used; beyond that the 64-token workgroups stage the router matrix four times
    // less often per token and win.
    if (H % kSplitKC == 0 && tokens <= kSplitMaxTokens) {
      const int blocks = (int)((tokens + 15) / 16);
      const size_t smem = router_split_smem_bytes((int)E, (int)K);
      if (smem > 160 * 1024)
        return fail(JTMOE_EUNSUPPORTED, "router: E=%lld K=%lld needs %zu bytes of LDS", (long long)E, (long long)K, smem);
      // Two launches when one workgroup can hold the epilogue of the whole call: partial sums over
      // k slices from many workgroups, then the finishing workgroup.
      const int finish_tok = router_smem_bytes((int)E, (int)K, 256) <= 160 * 1024 ? 256 : 64;
      if (tokens > 0 && tokens <= finish_tok && router_smem_bytes((int)E, (int)K, finish_tok) <= 160 * 1024) {
        const int slice_rows = router_slice_rows((int)H);
        const int slices = (int)((H + slice_rows - 1) / slice_rows);
        float* partial = reinterpret_cast<float*>(static_cast<unsigned char*>(ws) + router_scratch_bytes(E));
#define JT_PARTIAL_CASE(NB)                                                                                   \
  case NB * 16: {                                                                                            \
    auto kernel = router_mfma_split_kernel<NB, true>;                                                        \
    int rc = set_max_smem(kernel, smem);                                                                     \
    if (rc) return rc;                                                                                       \
    kernel<<<dim3(blocks, slices), 256, smem, stream>>>(                                                     \
        static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w), bias, (int)tokens, (int)H, (int)K, \
        (float)route_scale, ids, static_cast<bf16_raw*>(weights), scores, logits_out, ws, partial,           \
        score_func);                                                                                         \
  } break;
        switch ((int)E) {
          JT_PARTIAL_CASE(1)
          JT_PARTIAL_CASE(2)
          JT_PARTIAL_CASE(4)
          JT_PARTIAL_CASE(8)
          JT_PARTIAL_CASE(16)
        }
#undef JT_PARTIAL_CASE
        const size_t fsmem = router_smem_bytes((int)E, (int)K, finish_tok);
        const bool plan = layer != nullptr && tokens * K <= kSmallMaxAssignments && E <= 4 * finish_tok;
#define JT_FINISH(TOK, PLAN)                                                                                       \
  {                                                                                                                \
    auto kernel = router_finish_kernel<TOK, PLAN>;                                                                 \
    int rc = set_max_smem(kernel, fsmem);                                                                          \
    if (rc) return rc;                                                                                             \
    kernel<<<1, 4 * TOK, fsmem, stream>>>(partial, slices, bias, (int)tokens, (int)E, (int)K, (float)route_scale,  \
                                          ids, static_cast<bf16_raw*>(weights), scores, logits_out, counts,        \
                                          importance, PLAN ? layer->group_sizes : nullptr,                         \
                                          PLAN ? layer->offsets : nullptr, PLAN ? layer->source_order : nullptr,   \
                                          PLAN ? layer->inverse : nullptr, score_func);                            \
  }
        if (finish_tok == 256) {
          if (plan) JT_FINISH(256, true) else JT_FINISH(256, false)
        } else {
          if (plan) JT_FINISH(64, true) else JT_FINISH(64, false)
        }
#undef JT_FINISH
        if (layer) {
          layer->stats_done = true;
          layer->plan_done = plan;
        }
        return check_launch("router");
      }
      if (stats) router_zero_kernel<<<1, 256, 0, stream>>>(ws, (int)E);
      if (tokens > 0) {
#define JT_SPLIT_CASE(NB)                                                                                     \
  case NB * 16: {                                                                                            \
    auto kernel = router_mfma_split_kernel<NB, false>;                                                       \
    int rc = set_max_smem(kernel, smem);                                                                     \
    if (rc) return rc;                                                                                       \
    kernel<<<blocks, 256, smem, stream>>>(                                                                   \
        static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w), bias, (int)tokens, (int)H, (int)K, \
        (float)route_scale, ids, static_cast<bf16_raw*>(weights), scores, logits_out, ws_stats, nullptr,     \
        score_func);                                                                                         \
  } break;
        switch ((int)E) {
          JT_SPLIT_CASE(1)
          JT_SPLIT_CASE(2)
          JT_SPLIT_CASE(4)
          JT_SPLIT_CASE(8)
          JT_SPLIT_CASE(16)
        }
#undef JT_SPLIT_CASE
      }
      if (stats) router_finalize_kernel<<<1, 256, 0, stream>>>(ws, (int)E, counts, importance);
      return check_launch("router");
    }
    // four waves (64 tokens) per workgroup: the waves share the work of bringing in the router
    // matrix, which every workgroup reads in full
    constexpr int nw = 4;
    const int tok = 16 * nw;
    const int blocks = (int)((tokens + tok - 1) / tok);
    const size_t smem = router_mfma_smem_bytes((int)E, (int)K, tok);
    if (smem > 160 * 1024) return fail(JTMOE_EUNSUPPORTED, "router: E=%lld K=%lld needs %zu bytes of LDS", (long long)E, (long long)K, smem);
    if (stats) router_zero_kernel<<<1, 256, 0, stream>>>(ws, (int)E);
    if (tokens > 0) {
#define JT_ROUTER_LAUNCH(NB, NW)                                                                             \
  {                                                                                                          \
    auto kernel = router_mfma_kernel<NB, NW>;                                                                \
    int rc = set_max_smem(kernel, smem);                                                                     \
    if (rc) return rc;                                                                                       \
    kernel<<<blocks, 64 * NW, smem, stream>>>(                                                               \
        static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w), bias, (int)tokens, (int)H, (int)K, \
        (float)route_scale, ids, static_cast<bf16_raw*>(weights), scores, logits_out, ws_stats, score_func); \
  }
#define JT_ROUTER_CASE(NB)    \
  case NB * 16:               \
    JT_ROUTER_LAUNCH(NB, nw)  \
    break;
      switch ((int)E) {
        JT_ROUTER_CASE(1)
        JT_ROUTER_CASE(2)
        JT_ROUTER_CASE(4)
        JT_ROUTER_CASE(8)
        JT_ROUTER_CASE(16)
      }
#undef JT_ROUTER_CASE
#undef JT_ROUTER_LAUNCH
    }
  } else {
    const int blocks = (int)((tokens + 63) / 64);
    const size_t smem = router_smem_bytes((int)E, (int)K, 64);
    if (smem > 160 * 1024) return fail(JTMOE_EUNSUPPORTED, "router: E=%lld K=%lld needs %zu bytes of LDS", (long long)E, (long long)K, smem);
    auto kernel = router_kernel<T, kFromLogits>;
    int rc = set_max_smem(kernel, smem);
    if (rc) return rc;
    if (stats) router_zero_kernel<<<1, 256, 0, stream>>>(ws, (int)E);
    if (tokens > 0)
      kernel<<<blocks, 256, smem, stream>>>(
          static_cast<const T*>(x), static_cast<const T*>(w), logits_in, bias, (int)tokens, (int)H, (int)E, (int)K,
          (float)route_scale, ids, static_cast<T*>(weights), scores, logits_out, ws_stats, score_func);
  }
  if (stats) router_finalize_kernel<<<1, 256, 0, stream>>>(ws, (int)E, counts, importance);
  return check_launch("router");
}

int validate_router(int64_t T, int64_t H, int64_t E, int64_t K, double route_scale, int dtype, bool need_h) {
  JT_REQUIRE(dtype_ok(dtype), "router: unknown dtype %d", dtype);
  JT_REQUIRE(T >= 0 && T <= (int64_t)1 << 30, "router: token count %lld out of range", (long long)T);
  JT_REQUIRE(!need_h || (H > 0 && H <= (int64_t)1 << 20), "router: hidden size %lld out of range", (long long)H);
  JT_REQUIRE(E > 0 && K > 0 && K <= E, "router top_k must be positive and <= num_experts (E=%lld K=%lld)",
             (long long)E, (long long)K);
  JT_REQUIRE(route_scale > 0.0, "router route_scale must be positive, got %g", route_scale);
  if (E > JTMOE_MAX_EXPERTS) return fail(JTMOE_EUNSUPPORTED, "router: E=%lld exceeds %d", (long long)E, JTMOE_MAX_EXPERTS);
  if (K > JTMOE_MAX_TOP_K) return fail(JTMOE_EUNSUPPORTED, "router: K=%lld exceeds %d", (long long)K, JTMOE_MAX_TOP_K);
  JT_REQUIRE(T * E < ((int64_t)1 << 31) && T * K < ((int64_t)1 << 31), "router: T*E or T*K exceeds int32");
  return JTMOE_OK;
}

}  // namespace

// ---- the decode path of the layer (declared in common.hpp) ----
bool decode_dense_supported(int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int dtype) {
  // Every token through every expert pays when nearly every expert would be streamed anyway: with
  // T * K >= 2 E assignments thrown at E experts fewer than e^-2 = 14 % of them stay without a row.  One
  // 64-row tile per expert holds every token; the router's workgroups inside the launch need the matrix-core
  // projection (H a multiple of 128) and, so that three workgroups still fit a CU beside each other, a
  // router matrix stage of at most 53 KB (E <= 64); the plan needs E <= 256 and T * K <= kSmallMaxAssignments.
  return dtype == JTMOE_BF16 && T > 0 && T <= 64 && T * K >= 2 * E && T * K <= 32 * E &&
         (E == 16 || E == 32 || E == 64) && K <= JTMOE_MAX_TOP_K && K <= E && H % kSplitKC == 0 && I % 64 == 0 &&
         H * I < ((int64_t)1 << 30) && E * T * (I > H ? I : H) < ((int64_t)1 << 30) &&
         T * K <= kSmallMaxAssignments;
}

int launch_decode_gate_up_router(const void* x, const void* w_router, const float* expert_bias, const void* gate,
                                 const void* up, void* act_full, int64_t T, int64_t H, int64_t E, int64_t K, int64_t I,
                                 double route_scale, int score_func, int32_t* expert_ids, void* weights, float* scores,
                                 float* expert_counts, float* importance, int32_t* group_sizes, int32_t* offsets,
                                 int32_t* source_order, int32_t* inverse, void* router_workspace, hipStream_t stream) {
  if (!(aligned16(x) && aligned16(w_router) && aligned16(gate) && aligned16(up) && aligned16(act_full)))
    return fail(JTMOE_EINVAL, "moe_forward: operands must be 16-byte aligned");
  const int token_blocks = (int)((T + 15) / 16);
  const int slice_rows = router_slice_rows((int)H);
  const int slices = (int)((H + slice_rows - 1) / slice_rows);
  float* partial = reinterpret_cast<float*>(static_cast<unsigned char*>(router_workspace) + router_scratch_bytes(E));
  size_t smem = GateUpTinyCfg::SMEM_BYTES;
  if (router_split_smem_bytes((int)E, (int)K) > smem) smem = router_split_smem_bytes((int)E, (int)K);
  if (router_smem_bytes((int)E, (int)K, 64) > smem) smem = router_smem_bytes((int)E, (int)K, 64);
  if (smem > 53 * 1024) return fail(JTMOE_EUNSUPPORTED, "moe_forward: decode launch needs %zu bytes of LDS", smem);
  const int64_t mtiles = E * ((T + GateUpTinyCfg::BM - 1) / GateUpTinyCfg::BM);
  const int64_t nt = (I + GateUpTinyCfg::BN - 1) / GateUpTinyCfg::BN;
  const int64_t grid = (int64_t)token_blocks * slices + gemm_grid(mtiles, nt);
  if (token_blocks * slices > 255) return fail(JTMOE_EUNSUPPORTED, "moe_forward: decode launch with %d router workgroups", token_blocks * slices);
  unsigned long long* const arrivals = reinterpret_cast<unsigned long long*>(
      static_cast<unsigned char*>(router_workspace) + router_arrivals_offset(E));
  const unsigned long long tag = next_decode_tag();
#define JT_DECODE_CASE(NB)                                                                                       \
  case NB * 16: {                                                                                                \
    auto kernel = decode_gate_up_router_kernel<NB>;                                                              \
    int rc = set_max_smem(kernel, smem);                                                                         \
    if (rc) return rc;                                                                                           \
    kernel<<<(unsigned)grid, 256, smem, stream>>>(                                                               \
        static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(up),   \
        static_cast<uint16_t*>(act_full), (int)T, (int)H, (int)I, (int)mtiles, (int)nt,                          \
        static_cast<const uint16_t*>(w_router), expert_bias, (int)K, (float)route_scale, score_func, expert_ids, \
        static_cast<bf16_raw*>(weights), scores, expert_counts, importance, group_sizes, offsets, source_order,  \
        inverse, partial, token_blocks, slices, arrivals, tag);                                                  \
  } break;
  switch ((int)E) {
    JT_DECODE_CASE(1)
    JT_DECODE_CASE(2)
    JT_DECODE_CASE(4)
    default:
      return fail(JTMOE_EUNSUPPORTED, "moe_forward: decode launch for E=%lld", (long long)E);
  }
#undef JT_DECODE_CASE
  return check_launch("decode gate/up + router");
}

int router_for_layer(const void* x, const void* w_router, const float* expert_bias, int64_t T, int64_t H, int64_t E,
                     int64_t K, double route_scale, int dtype, int32_t* expert_ids, void* weights, float* scores,
                     float* expert_counts, float* importance, int32_t* group_sizes, int32_t* offsets,
                     int32_t* source_order, int32_t* inverse, void* workspace, size_t workspace_bytes,
                     int score_func, bool* stats_done, bool* plan_done, hipStream_t s) {
  int rc = validate_router(T, H, E, K, route_scale, dtype, true);
  if (rc) return rc;
  JT_REQUIRE(score_func_ok(score_func), "router: unknown score function %d", score_func);
  JT_REQUIRE(w_router && expert_counts && importance && workspace, "router: null pointer argument");
  JT_REQUIRE(T == 0 || (x && expert_ids && weights && scores), "router: null pointer argument");
  JT_REQUIRE(group_sizes && offsets && (T == 0 || (source_order && inverse)), "router: null pointer argument");
  if (workspace_bytes < jtmoe_router_workspace_bytes(E))
    return fail(JTMOE_EWORKSPACE, "router: workspace %zu < %zu bytes", workspace_bytes, jtmoe_router_workspace_bytes(E));
  LayerPlan layer{group_sizes, offsets, source_order, inverse, false, false};
  if (dtype == JTMOE_BF16)
    rc = launch_router<bf16_raw, false>(x, w_router, nullptr, expert_bias, T, H, E, K, route_scale, expert_ids, weights,
                                        scores, expert_counts, importance, nullptr, workspace, s, score_func, &layer);
  else
    rc = launch_router<float, false>(x, w_router, nullptr, expert_bias, T, H, E, K, route_scale, expert_ids, weights,
                                     scores, expert_counts, importance, nullptr, workspace, s, score_func, &layer);
  *stats_done = layer.stats_done;
  *plan_done = layer.plan_done;
  return rc;
}

}  // namespace jtmoe

using namespace jtmoe;

extern "C" size_t jtmoe_router_workspace_bytes(int64_t E) {
  if (E <= 0) return 0;
  // the statistics accumulators, the partial sums of the small-batch path, the arrival word of the decode launch
  return router_arrivals_offset(E) + 256;
}

extern "C" int jtmoe_router(const void* x, const void* w_router, const float* expert_bias, int64_t T, int64_t H,
                            int64_t E, int64_t K, double route_scale, int dtype, int32_t* expert_ids,
                            void* weights, float* scores, float* expert_counts, float* importance, float* logits,
                            void* workspace, size_t workspace_bytes, void* stream) {
  return jtmoe_router_sf(x, w_router, expert_bias, T, H, E, K, route_scale, JTMOE_SCORE_SIGMOID, dtype, expert_ids,
                         weights, scores, expert_counts, importance, logits, workspace, workspace_bytes, stream);
}

extern "C" int jtmoe_router_sf(const void* x, const void* w_router, const float* expert_bias, int64_t T, int64_t H,
                               int64_t E, int64_t K, double route_scale, int score_func, int dtype,
                               int32_t* expert_ids, void* weights, float* scores, float* expert_counts,
                               float* importance, float* logits, void* workspace, size_t workspace_bytes,
                               void* stream) {
  clear_error();
  int rc = validate_router(T, H, E, K, route_scale, dtype, true);
  if (rc) return rc;
  JT_REQUIRE(score_func_ok(score_func), "router: unknown score function %d", score_func);
  JT_REQUIRE(w_router && expert_counts && importance && workspace, "router: null pointer argument");
  JT_REQUIRE(T == 0 || (x && expert_ids && weights && scores), "router: null pointer argument");
  if (workspace_bytes < jtmoe_router_workspace_bytes(E))
    return fail(JTMOE_EWORKSPACE, "router: workspace %zu < %zu bytes", workspace_bytes, jtmoe_router_workspace_bytes(E));
  hipStream_t s = as_stream(stream);
  if (dtype == JTMOE_BF16)
    return launch_router<bf16_raw, false>(x, w_router, nullptr, expert_bias, T, H, E, K, route_scale, expert_ids,
                                          weights, scores, expert_counts, importance, logits, workspace, s, score_func);
  return launch_router<float, false>(x, w_router, nullptr, expert_bias, T, H, E, K, route_scale, expert_ids, weights,
                                     scores, expert_counts, importance, logits, workspace, s, score_func);
}

extern "C" int jtmoe_router_from_logits(const float* logits, const float* expert_bias, int64_t T, int64_t E,
                                        int64_t K, double route_scale, int dtype, int32_t* expert_ids,
                                        void* weights, float* scores, float* expert_counts, float* importance,
                                        void* workspace, size_t workspace_bytes, void* stream) {
  return jtmoe_router_from_logits_sf(logits, expert_bias, T, E, K, route_scale, JTMOE_SCORE_SIGMOID, dtype, expert_ids,
                                     weights, scores, expert_counts, importance, workspace, workspace_bytes, stream);
}

extern "C" int jtmoe_router_from_logits_sf(const float* logits, const float* expert_bias, int64_t T, int64_t E,
                                           int64_t K, double route_scale, int score_func, int dtype,
                                           int32_t* expert_ids, void* weights, float* scores, float* expert_counts,
                                           float* importance, void* workspace, size_t workspace_bytes,
                                           void* stream) {
  clear_error();
  int rc = validate_router(T, 1, E, K, route_scale, dtype, false);
  if (rc) return rc;
  JT_REQUIRE(score_func_ok(score_func), "router_from_logits: unknown score function %d", score_func);
  JT_REQUIRE(expert_counts && importance && workspace, "router_from_logits: null pointer argument");
  JT_REQUIRE(T == 0 || (logits && expert_ids && weights && scores), "router_from_logits: null pointer argument");
  if (workspace_bytes < jtmoe_router_workspace_bytes(E))
    return fail(JTMOE_EWORKSPACE, "router_from_logits: workspace %zu < %zu bytes", workspace_bytes,
                jtmoe_router_workspace_bytes(E));
  hipStream_t s = as_stream(stream);
  if (dtype == JTMOE_BF16)
    return launch_router<bf16_raw, true>(nullptr, nullptr, logits, expert_bias, T, 0, E, K, route_scale, expert_ids,
                                         weights, scores, expert_counts, importance, nullptr, workspace, s, score_func);
  return launch_router<float, true>(nullptr, nullptr, logits, expert_bias, T, 0, E, K, route_scale, expert_ids, weights,
                                    scores, expert_counts, importance, nullptr, workspace, s, score_func);
}
