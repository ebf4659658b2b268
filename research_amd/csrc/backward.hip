// Backward pass (vector-Jacobian products) of the MoE layer's four operators.
//
// The reference differentiates SparseMoE with JAX autodiff; what that computes is
// restated here operator by operator (rounding to the compute dtype where the forward
// rounds; straight-through for the roundings themselves):
//
//   combine    y[t] = sum_s Yp[inverse[t,s]] * w[t,s]            (moe.py:663-671)
//     dYp[j] = dy[token(j)] * w[a_j]          dw[a] = <dy[token], Yp[inverse[a]]>
//   experts    G = Xp Wg[e], U = Xp Wu[e], Hh = silu(G) U, Yp = Hh Wd[e]   (moe.py:638-641)
//     Z   = dy[token(j)] Wd[e]^T              (so dHh = w Z and dw[a] = <Z_j, Hh_j>)
//     dG  = dHh * U * silu'(G)                dU = dHh * silu(G)
//     dWd[e] = (w Hh)^T dy[token]             dWg[e] = Xp^T dG      dWu[e] = Xp^T dU
//     dXp = dG Wg[e]^T + dU Wu[e]^T
//   dispatch   Xp[j] = x[token(j)]                                  (moe.py:583-600)
//     dx[t] = sum_s dXp[inverse[t,s]]
//   router     w[t,s] = scale * p_s / (sum_r p_r + 1e-20), p = sigmoid(logits)[ids]  (moe.py:131-147)
//     dp_s = scale * (dw_s / S - sum_r dw_r p_r / S^2)
//     dlogits = (d_scores + scatter(dp)) * p (1 - p);  dW_r = x^T dlogits;  dx += dlogits W_r^T
//   (the expert bias only takes part in the selection and has no gradient: moe.py:139-140)
//
// Every reduction has a fixed order, so repeated calls give identical bits.
#include "common.hpp"
#include "gemm_launch.hpp"

namespace jtmoe {
namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d);
  return v;
}

struct SwigluGrad {
  float dg, du, hw, zh;
};

// one element of the SwiGLU backward; z = (dy Wd^T), w = route weight of the row
template <typename T>
__device__ __forceinline__ SwigluGrad swiglu_grad(float z, float g, float u, float w) {
  const float sig = 1.0f / (1.0f + __expf(-g));
  const float silu = g * sig;
  const float h = Elem<T>::round(silu * u);
  const float dh = Elem<T>::round(w * z);
  SwigluGrad r;
  r.dg = dh * u * (sig * (1.0f + g * (1.0f - sig)));
  r.du = dh * silu;
  r.hw = w * h;
  r.zh = z * h;
  return r;
}

// Packed rows that exist: the groups end at offsets[E-1] + group_sizes[E-1], which is less than the
// number of assignments when the dispatch dropped ids outside [0, E).  Rows past that end hold
// nothing (their entries of the permutation were never written) and are skipped.
__device__ __forceinline__ int packed_rows_end(const int32_t* __restrict__ group_sizes,
                                               const int32_t* __restrict__ offsets, int E, int rows) {
  if (group_sizes == nullptr) return rows;
  return min(rows, offsets[E - 1] + group_sizes[E - 1]);
}

// One wave per packed row.  z_dg holds Z on entry and dG on exit.  row_weight_index[j] (the
// assignment behind packed row j) selects the route weight and the slot of d_weights; with a
// null index (shared experts) the weight is 1 and no weight gradient is produced.
template <typename T>
__global__ __launch_bounds__(256) void swiglu_backward_kernel(T* __restrict__ z_dg, const T* __restrict__ G,
                                                              const T* __restrict__ U,
                                                              const int32_t* __restrict__ row_weight_index,
                                                              const T* __restrict__ weights, int rows, int I,
                                                              T* __restrict__ dU, T* __restrict__ HW,
                                                              T* __restrict__ d_weights,
                                                              const int32_t* __restrict__ group_sizes,
                                                              const int32_t* __restrict__ offsets, int E) {
  const int j = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (j >= packed_rows_end(group_sizes, offsets, E, rows)) return;
  const int lane = threadIdx.x & 63;
  const int a = row_weight_index ? row_weight_index[j] : 0;
  if (a < 0 || a >= rows) return;  // not a permutation entry: nothing to read or write through it
  const float w = row_weight_index ? Elem<T>::load(weights + a) : 1.0f;
  const size_t base = (size_t)j * I;
  float dot = 0.0f;
  for (int i = lane; i < I; i += 64) {
    const SwigluGrad r = swiglu_grad<T>(Elem<T>::load(z_dg + base + i), Elem<T>::load(G + base + i),
                                        Elem<T>::load(U + base + i), w);
    Elem<T>::store(z_dg + base + i, r.dg);
    Elem<T>::store(dU + base + i, r.du);
    Elem<T>::store(HW + base + i, r.hw);
    dot += r.zh;
  }
  dot = wave_sum(dot);
  if (row_weight_index && lane == 0) Elem<T>::store(d_weights + a, dot);
}

// bf16 rows whose length is a multiple of 8, 16-byte aligned: 8 elements per lane and step
__global__ __launch_bounds__(256) void swiglu_backward_bf16_vec_kernel(
    uint4* __restrict__ z_dg, const uint4* __restrict__ G, const uint4* __restrict__ U,
    const int32_t* __restrict__ row_weight_index, const uint16_t* __restrict__ weights, int rows, int row_vecs,
    uint4* __restrict__ dU, uint4* __restrict__ HW, uint16_t* __restrict__ d_weights,
    const int32_t* __restrict__ group_sizes, const int32_t* __restrict__ offsets, int E) {
  const int j = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (j >= packed_rows_end(group_sizes, offsets, E, rows)) return;
  const int lane = threadIdx.x & 63;
  const int a = row_weight_index ? row_weight_index[j] : 0;
  if (a < 0 || a >= rows) return;
  const float w = row_weight_index ? bf16_bits_to_f32(weights[a]) : 1.0f;
  const size_t base = (size_t)j * row_vecs;
  float dot = 0.0f;
  for (int v = lane; v < row_vecs; v += 64) {
    const uint4 zv = load_stream(&z_dg[base + v]), gv = load_stream(&G[base + v]), uv = load_stream(&U[base + v]);
    const uint32_t zw[4] = {zv.x, zv.y, zv.z, zv.w}, gw[4] = {gv.x, gv.y, gv.z, gv.w},
                   uw[4] = {uv.x, uv.y, uv.z, uv.w};
    uint32_t dgw[4], duw[4], hww[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const SwigluGrad lo = swiglu_grad<bf16_raw>(bf16_bits_to_f32(zw[i] & 0xffffu), bf16_bits_to_f32(gw[i] & 0xffffu),
                                                  bf16_bits_to_f32(uw[i] & 0xffffu), w);
      const SwigluGrad hi = swiglu_grad<bf16_raw>(bf16_bits_to_f32(zw[i] >> 16), bf16_bits_to_f32(gw[i] >> 16),
                                                  bf16_bits_to_f32(uw[i] >> 16), w);
      dgw[i] = f32_to_bf16_bits(lo.dg) | (f32_to_bf16_bits(hi.dg) << 16);
      duw[i] = f32_to_bf16_bits(lo.du) | (f32_to_bf16_bits(hi.du) << 16);
      hww[i] = f32_to_bf16_bits(lo.hw) | (f32_to_bf16_bits(hi.hw) << 16);
      dot += lo.zh;
      dot += hi.zh;
    }
    store_stream(&z_dg[base + v], make_uint4(dgw[0], dgw[1], dgw[2], dgw[3]));
    store_stream(&dU[base + v], make_uint4(duw[0], duw[1], duw[2], duw[3]));
    store_stream(&HW[base + v], make_uint4(hww[0], hww[1], hww[2], hww[3]));
  }
  dot = wave_sum(dot);
  if (row_weight_index && lane == 0) d_weights[a] = (uint16_t)f32_to_bf16_bits(dot);
}

// ones[a] = 1 (the unit weights of the combine that sums dXp), and the route-weight gradient of an
// assignment the dispatch dropped (inverse < 0: no packed row, so no one else writes it) is zero
template <typename T>
__global__ __launch_bounds__(256) void fill_one_kernel(T* __restrict__ p, int n, const int32_t* __restrict__ inverse,
                                                       T* __restrict__ d_weights) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  Elem<T>::store(p + i, 1.0f);
  if (inverse[i] < 0) Elem<T>::store(d_weights + i, 0.0f);
}

// out[i] = round(a[i] + b[i])
template <typename T>
__global__ __launch_bounds__(256) void add_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ out,
                                                  size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) Elem<T>::store(out + i, Elem<T>::load(a + i) + Elem<T>::load(b + i));
}

// One wave per token: gradient of the logits from the gradient of the route weights (and,
// optionally, of the scores).  E <= JTMOE_MAX_EXPERTS, K <= JTMOE_MAX_TOP_K.
template <typename T>
__global__ __launch_bounds__(256) void router_backward_kernel(const float* __restrict__ scores,
                                                              const int32_t* __restrict__ ids,
                                                              const T* __restrict__ d_weights,
                                                              const float* __restrict__ d_scores, float route_scale,
                                                              int tokens, int E, int K, T* __restrict__ d_logits,
                                                              int score_func) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= tokens) return;
  const int lane = threadIdx.x & 63;
  const float* sc = scores + (size_t)t * E;
  // S = sum_s p_s + 1e-20 and c = sum_r dw_r p_r / S^2, accumulated in slot order by every lane
  float S = 0.0f, dot = 0.0f;
  for (int s = 0; s < K; ++s) {
    const int e = ids[(size_t)t * K + s];
    const float p = (e >= 0 && e < E) ? sc[e] : 0.0f;
    S += p;
    dot += Elem<T>::load(d_weights + (size_t)t * K + s) * p;
  }
  S += 1e-20f;
  const float c = dot / (S * S);
  // gradient with respect to the score of expert e (lane e, e + 64, ...)
  auto score_grad = [&](int e) {
    float ds = d_scores ? d_scores[(size_t)t * E + e] : 0.0f;
    for (int s = 0; s < K; ++s)
      if (ids[(size_t)t * K + s] == e) ds += route_scale * (Elem<T>::load(d_weights + (size_t)t * K + s) / S - c);
    return ds;
  };
  if (score_func == JTMOE_SCORE_SOFTMAX) {
    // softmax over the experts: d z_e = p_e (g_e - sum_j g_j p_j); the sum by lane, then across the wave
    float inner = 0.0f;
    for (int e = lane; e < E; e += 64) inner += score_grad(e) * sc[e];
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) inner += __shfl_xor(inner, d);
    for (int e = lane; e < E; e += 64) Elem<T>::store(d_logits + (size_t)t * E + e, sc[e] * (score_grad(e) - inner));
    return;
  }
  for (int e = lane; e < E; e += 64) {
    const float ds = score_grad(e);
    const float p = sc[e];
    Elem<T>::store(d_logits + (size_t)t * E + e, ds * p * (1.0f - p));
  }
}

template <typename T>
int run_swiglu_backward(void* z_dg, const void* G, const void* U, const int32_t* row_weight_index, const void* weights,
                        int64_t rows, int64_t I, void* dU, void* HW, void* d_weights, hipStream_t s,
                        const int32_t* group_sizes = nullptr, const int32_t* offsets = nullptr, int64_t E = 0) {
  if (rows == 0) return JTMOE_OK;
  const unsigned grid = (unsigned)((rows + 3) / 4);
  if (Elem<T>::is_bf16 && I % 8 == 0 && aligned16(z_dg) && aligned16(G) && aligned16(U) && aligned16(dU) &&
      aligned16(HW)) {
    swiglu_backward_bf16_vec_kernel<<<grid, 256, 0, s>>>(
        static_cast<uint4*>(z_dg), static_cast<const uint4*>(G), static_cast<const uint4*>(U), row_weight_index,
        static_cast<const uint16_t*>(weights), (int)rows, (int)(I / 8), static_cast<uint4*>(dU),
        static_cast<uint4*>(HW), static_cast<uint16_t*>(d_weights), group_sizes, offsets, (int)E);
  } else {
    swiglu_backward_kernel<T><<<grid, 256, 0, s>>>(static_cast<T*>(z_dg), static_cast<const T*>(G),
                                                   static_cast<const T*>(U), row_weight_index,
                                                   static_cast<const T*>(weights), (int)rows, (int)I,
                                                   static_cast<T*>(dU), static_cast<T*>(HW),
                                                   static_cast<T*>(d_weights), group_sizes, offsets, (int)E);
  }
  return check_launch("swiglu backward");
}

struct Carver {
  unsigned char* base;
  size_t used = 0;
  void* take(size_t bytes) {
    void* p = base ? base + used : nullptr;
    used += align_up(bytes, 256);
    return p;
  }
};

struct ExpertsBwdWs {
  void *dg, *du, *hw, *dxp, *ones, *packed_x, *packed_dy;
  size_t total;
};
ExpertsBwdWs carve_experts(void* base, int64_t A, int64_t H, int64_t I, int dtype) {
  Carver c{static_cast<unsigned char*>(base)};
  const size_t b = dtype_bytes(dtype);
  ExpertsBwdWs w;
  w.dg = c.take((size_t)A * I * b);
  w.du = c.take((size_t)A * I * b);
  w.hw = c.take((size_t)A * I * b);
  w.dxp = c.take((size_t)A * H * b);
  w.ones = c.take((size_t)A * b);
  w.packed_x = c.take((size_t)A * H * b);
  w.packed_dy = c.take((size_t)A * H * b);
  w.total = c.used;
  return w;
}

struct SharedBwdWs {
  void *dg, *du, *hw, *split;
  size_t total;
};
SharedBwdWs carve_shared(void* base, int64_t T, int64_t H, int64_t Is, int dtype) {
  Carver c{static_cast<unsigned char*>(base)};
  const size_t b = dtype_bytes(dtype);
  SharedBwdWs w;
  w.dg = c.take((size_t)T * Is * b);
  w.du = c.take((size_t)T * Is * b);
  w.hw = c.take((size_t)T * Is * b);
  // partial sums of the two weight-gradient reductions (used one after the other)
  const size_t down_split = gemm_tn_split_bytes(dtype, T, Is, H, false);
  const size_t gate_up_split = gemm_tn_split_bytes(dtype, T, H, Is, true);
  const size_t split = down_split > gate_up_split ? down_split : gate_up_split;
  w.split = split ? c.take(split) : nullptr;
  w.total = c.used;
  return w;
}

struct RouterBwdWs {
  void *d_logits, *split;
  size_t total;
};
RouterBwdWs carve_router(void* base, int64_t T, int64_t H, int64_t E, int dtype) {
  Carver c{static_cast<unsigned char*>(base)};
  RouterBwdWs w;
  w.d_logits = c.take((size_t)T * E * dtype_bytes(dtype));
  const size_t split = gemm_tn_split_bytes(dtype, T, H, E, false);
  w.split = split ? c.take(split) : nullptr;
  w.total = c.used;
  return w;
}

// steps of the routed experts up to dXp (in ws.dxp) and d_weights; dx itself is one combine away
int experts_backward_core(const void* x, const void* dy, const int32_t* source_order, const int32_t* inverse,
                          const void* weights, const int32_t* group_sizes, const int32_t* offsets, const void* gate,
                          const void* up, const void* down, const void* gate_pre, const void* up_pre, int64_t T,
                          int64_t K, int64_t H, int64_t I, int64_t E, int dtype, void* d_weights, void* d_gate,
                          void* d_up, void* d_down, const ExpertsBwdWs& ws, hipStream_t s) {
  const int64_t A = T * K;
  int rc;
  // The weight-gradient products walk the rows of a group 64 at a time; fetching those rows through
  // the permutation (64 fresh token rows every step) costs more than writing the permuted copies of
  // x and dy once and streaming them (measured at 131072 rows x 2048: 2.03 vs 1.52 + 0.13 ms for the
  // gate/up product), so the backward pass does materialise them.
  launch_dispatch_rows(x, inverse, T, K, H, dtype, ws.packed_x, s);
  launch_dispatch_rows(dy, inverse, T, K, H, dtype, ws.packed_dy, s);
  rc = check_launch("experts backward (row scatter)");
  if (rc) return rc;
  // Z = dYp @ Wd[e]^T
  rc = launch_gemm_nt(dtype, ws.packed_dy, nullptr, down, nullptr, ws.dg, group_sizes, offsets, A, H, I, E, nullptr, 1,
                      0, 1, s);
  if (rc) return rc;
  rc = dtype == JTMOE_BF16 ? run_swiglu_backward<bf16_raw>(ws.dg, gate_pre, up_pre, source_order, weights, A, I, ws.du,
                                                           ws.hw, d_weights, s, group_sizes, offsets, E)
                           : run_swiglu_backward<float>(ws.dg, gate_pre, up_pre, source_order, weights, A, I, ws.du,
                                                        ws.hw, d_weights, s, group_sizes, offsets, E);
  if (rc) return rc;
  // dWd[e] = (w Hh)^T @ dYp
  rc = launch_gemm_tn(dtype, ws.hw, ws.packed_dy, nullptr, d_down, nullptr, group_sizes, offsets, A, I, H, E, nullptr,
                      1, false, false, 0, s);
  if (rc) return rc;
  // dWg[e], dWu[e] = Xp^T @ (dG, dU)
  rc = launch_gemm_tn(dtype, ws.packed_x, ws.dg, ws.du, d_gate, d_up, group_sizes, offsets, A, H, I, E, nullptr, 1,
                      false, false, 0, s);
  if (rc) return rc;
  // dXp = dG @ Wg[e]^T + dU @ Wu[e]^T
  rc = launch_gemm_nt(dtype, ws.dg, ws.du, gate, up, ws.dxp, group_sizes, offsets, A, I, H, E, nullptr, 1, 0, 2, s);
  if (rc) return rc;
  if (A == 0) return JTMOE_OK;
  const unsigned grid = (unsigned)((A + 255) / 256);
  if (dtype == JTMOE_BF16)
    fill_one_kernel<bf16_raw><<<grid, 256, 0, s>>>(static_cast<bf16_raw*>(ws.ones), (int)A, inverse,
                                                   static_cast<bf16_raw*>(d_weights));
  else
    fill_one_kernel<float><<<grid, 256, 0, s>>>(static_cast<float*>(ws.ones), (int)A, inverse,
                                                static_cast<float*>(d_weights));
  return check_launch("experts backward");
}

int shared_backward_impl(const void* x, const void* dy, const void* gate, const void* up, const void* down,
                         const void* gate_pre, const void* up_pre, int64_t T, int64_t H, int64_t Is, int dtype,
                         void* dx, void* d_gate, void* d_up, void* d_down, const SharedBwdWs& ws, hipStream_t s) {
  int rc = launch_gemm_nt(dtype, dy, nullptr, down, nullptr, ws.dg, nullptr, nullptr, T, H, Is, 1, nullptr, 1, 0, 1, s);
  if (rc) return rc;
  rc = dtype == JTMOE_BF16
           ? run_swiglu_backward<bf16_raw>(ws.dg, gate_pre, up_pre, nullptr, nullptr, T, Is, ws.du, ws.hw, nullptr, s)
           : run_swiglu_backward<float>(ws.dg, gate_pre, up_pre, nullptr, nullptr, T, Is, ws.du, ws.hw, nullptr, s);
  if (rc) return rc;
  rc = launch_gemm_tn(dtype, ws.hw, dy, nullptr, d_down, nullptr, nullptr, nullptr, T, Is, H, 1, nullptr, 1, false,
                      false, 0, s, ws.split);
  if (rc) return rc;
  rc = launch_gemm_tn(dtype, x, ws.dg, ws.du, d_gate, d_up, nullptr, nullptr, T, H, Is, 1, nullptr, 1, false, false, 0,
                      s, ws.split);
  if (rc) return rc;
  rc = launch_gemm_nt(dtype, ws.dg, ws.du, gate, up, dx, nullptr, nullptr, T, Is, H, 1, nullptr, 1, 0, 2, s);
  if (rc) return rc;
  return check_launch("shared backward");
}

int router_backward_impl(const void* x, const void* router_weight, const float* scores, const int32_t* ids,
                         const void* d_weights, const float* d_scores, double route_scale, int64_t T, int64_t H,
                         int64_t E, int64_t K, int dtype, void* dx, void* d_router_weight, const RouterBwdWs& ws,
                         hipStream_t s, int score_func = JTMOE_SCORE_SIGMOID) {
  void* const d_logits = ws.d_logits;
  const unsigned grid = (unsigned)((T + 3) / 4);
  if (T == 0) {
    // no tokens: the weight gradient is all zeros, which the empty reduction below writes
  } else if (dtype == JTMOE_BF16)
    router_backward_kernel<bf16_raw><<<grid, 256, 0, s>>>(scores, ids, static_cast<const bf16_raw*>(d_weights),
                                                          d_scores, (float)route_scale, (int)T, (int)E, (int)K,
                                                          static_cast<bf16_raw*>(d_logits), score_func);
  else
    router_backward_kernel<float><<<grid, 256, 0, s>>>(scores, ids, static_cast<const float*>(d_weights), d_scores,
                                                       (float)route_scale, (int)T, (int)E, (int)K,
                                                       static_cast<float*>(d_logits), score_func);
  int rc = check_launch("router backward");
  if (rc) return rc;
  // dW_r [H, E] = x^T @ dlogits;  dx [T, H] = dlogits @ W_r^T  (W_r is [H, E]: N = H rows of length K = E)
  rc = launch_gemm_tn(dtype, x, d_logits, nullptr, d_router_weight, nullptr, nullptr, nullptr, T, H, E, 1, nullptr, 1,
                      false, false, 0, s, ws.split);
  if (rc) return rc;
  return launch_gemm_nt(dtype, d_logits, nullptr, router_weight, nullptr, dx, nullptr, nullptr, T, E, H, 1, nullptr, 1,
                        0, 1, s);
}

// the same for bf16, eight elements per thread, every byte touched once
__global__ __launch_bounds__(256) void add_bf16_vec_kernel(const uint4* __restrict__ a, const uint4* __restrict__ b,
                                                           uint4* __restrict__ out, size_t nvec) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  const uint4 av = load_stream(&a[i]), bv = load_stream(&b[i]);
  const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
  uint32_t o[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float lo = bf16_bits_to_f32(aw[k] & 0xffffu) + bf16_bits_to_f32(bw[k] & 0xffffu);
    const float hi = bf16_bits_to_f32(aw[k] >> 16) + bf16_bits_to_f32(bw[k] >> 16);
    o[k] = f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
  }
  out[i] = make_uint4(o[0], o[1], o[2], o[3]);  // read again by the combine that follows
}

template <typename T>
void run_add(const void* a, const void* b, void* out, size_t n, hipStream_t s) {
  if (Elem<T>::is_bf16 && n % 8 == 0 && aligned16(a) && aligned16(b) && aligned16(out)) {
    const size_t nvec = n / 8;
    add_bf16_vec_kernel<<<(unsigned)((nvec + 255) / 256), 256, 0, s>>>(
        static_cast<const uint4*>(a), static_cast<const uint4*>(b), static_cast<uint4*>(out), nvec);
    return;
  }
  add_kernel<T><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(static_cast<const T*>(a), static_cast<const T*>(b),
                                                            static_cast<T*>(out), n);
}

int validate_shape(const char* what, int64_t T, int64_t K, int64_t H, int64_t I, int64_t E, int dtype) {
  JT_REQUIRE(dtype_ok(dtype), "%s: unknown dtype %d", what, dtype);
  JT_REQUIRE(T >= 0 && K > 0 && H > 0 && I > 0 && E > 0, "%s: T=%lld K=%lld H=%lld I=%lld E=%lld out of range", what,
             (long long)T, (long long)K, (long long)H, (long long)I, (long long)E);
  JT_REQUIRE(T * K < ((int64_t)1 << 31), "%s: T*K exceeds int32", what);
  JT_REQUIRE(H < ((int64_t)1 << 24) && I < ((int64_t)1 << 24), "%s: H or I too large", what);
  if (E > JTMOE_MAX_EXPERTS) return fail(JTMOE_EUNSUPPORTED, "%s: E=%lld exceeds %d", what, (long long)E, JTMOE_MAX_EXPERTS);
  if (K > JTMOE_MAX_TOP_K) return fail(JTMOE_EUNSUPPORTED, "%s: K=%lld exceeds %d", what, (long long)K, JTMOE_MAX_TOP_K);
  return JTMOE_OK;
}

}  // namespace
}  // namespace jtmoe

using namespace jtmoe;

extern "C" size_t jtmoe_experts_backward_workspace_bytes(int64_t T, int64_t K, int64_t H, int64_t I, int dtype) {
  if (T < 0 || K <= 0 || H <= 0 || I <= 0 || !dtype_ok(dtype)) return 0;
  return carve_experts(nullptr, T * K, H, I, dtype).total;
}

extern "C" int jtmoe_experts_backward(const void* x, const void* dy, const int32_t* source_order,
                                      const int32_t* inverse, const void* weights, const int32_t* group_sizes,
                                      const int32_t* offsets, const void* gate, const void* up, const void* down,
                                      const void* gate_pre, const void* up_pre, int64_t T, int64_t K, int64_t H,
                                      int64_t I, int64_t E, int dtype, const void* dx_extra, void* dx, void* d_weights,
                                      void* d_gate, void* d_up, void* d_down, void* workspace, size_t workspace_bytes,
                                      void* stream) {
  clear_error();
  int rc = validate_shape("experts_backward", T, K, H, I, E, dtype);
  if (rc) return rc;
  JT_REQUIRE(gate && up && down && d_gate && d_up && d_down, "experts_backward: null weight pointer");
  JT_REQUIRE(group_sizes && offsets, "experts_backward: null group pointer");
  if (T > 0)
    JT_REQUIRE(x && dy && source_order && inverse && weights && gate_pre && up_pre && dx && d_weights,
               "experts_backward: null pointer argument");
  const ExpertsBwdWs ws = carve_experts(workspace, T * K, H, I, dtype);
  if (T > 0 && (workspace == nullptr || workspace_bytes < ws.total))
    return fail(JTMOE_EWORKSPACE, "experts_backward: workspace of %zu bytes given, %zu needed", workspace_bytes,
                ws.total);
  hipStream_t s = as_stream(stream);
  // with T == 0 every group is empty and the weight gradients are all zeros
  rc = experts_backward_core(x, dy, source_order, inverse, weights, group_sizes, offsets, gate, up, down, gate_pre,
                             up_pre, T > 0 ? T : 0, K, H, I, E, dtype, d_weights, d_gate, d_up, d_down, ws, s);
  if (rc) return rc;
  if (T == 0) return JTMOE_OK;
  return jtmoe_combine(ws.dxp, inverse, ws.ones, dx_extra, T, H, K, dtype, dx, stream);
}

extern "C" size_t jtmoe_shared_backward_workspace_bytes(int64_t T, int64_t H, int64_t Is, int dtype) {
  if (T < 0 || H <= 0 || Is <= 0 || !dtype_ok(dtype)) return 0;
  return carve_shared(nullptr, T, H, Is, dtype).total;
}

extern "C" int jtmoe_shared_backward(const void* x, const void* dy, const void* gate, const void* up, const void* down,
                                     const void* gate_pre, const void* up_pre, int64_t T, int64_t H, int64_t Is,
                                     int dtype, void* dx, void* d_gate, void* d_up, void* d_down, void* workspace,
                                     size_t workspace_bytes, void* stream) {
  clear_error();
  int rc = validate_shape("shared_backward", T, 1, H, Is, 1, dtype);
  if (rc) return rc;
  JT_REQUIRE(gate && up && down && d_gate && d_up && d_down, "shared_backward: null weight pointer");
  if (T > 0) JT_REQUIRE(x && dy && gate_pre && up_pre && dx, "shared_backward: null pointer argument");
  const SharedBwdWs ws = carve_shared(workspace, T, H, Is, dtype);
  if (T > 0 && (workspace == nullptr || workspace_bytes < ws.total))
    return fail(JTMOE_EWORKSPACE, "shared_backward: workspace of %zu bytes given, %zu needed", workspace_bytes,
                ws.total);
  return shared_backward_impl(x, dy, gate, up, down, gate_pre, up_pre, T, H, Is, dtype, dx, d_gate, d_up, d_down, ws,
                              as_stream(stream));
}

extern "C" size_t jtmoe_router_backward_workspace_bytes(int64_t T, int64_t H, int64_t E, int dtype) {
  if (T < 0 || H <= 0 || E <= 0 || !dtype_ok(dtype)) return 0;
  return carve_router(nullptr, T, H, E, dtype).total;
}

extern "C" int jtmoe_router_backward(const void* x, const void* router_weight, const float* scores,
                                     const int32_t* expert_ids, const void* d_weights, const float* d_scores,
                                     double route_scale, int64_t T, int64_t H, int64_t E, int64_t K, int dtype,
                                     void* dx, void* d_router_weight, void* workspace, size_t workspace_bytes,
                                     void* stream) {
  return jtmoe_router_backward_sf(x, router_weight, scores, expert_ids, d_weights, d_scores, route_scale,
                                  JTMOE_SCORE_SIGMOID, T, H, E, K, dtype, dx, d_router_weight, workspace,
                                  workspace_bytes, stream);
}

extern "C" int jtmoe_router_backward_sf(const void* x, const void* router_weight, const float* scores,
                                        const int32_t* expert_ids, const void* d_weights, const float* d_scores,
                                        double route_scale, int score_func, int64_t T, int64_t H, int64_t E,
                                        int64_t K, int dtype, void* dx, void* d_router_weight, void* workspace,
                                        size_t workspace_bytes, void* stream) {
  clear_error();
  int rc = validate_shape("router_backward", T, K, H, 1, E, dtype);
  if (rc) return rc;
  JT_REQUIRE(score_func_ok(score_func), "router_backward: unknown score function %d", score_func);
  JT_REQUIRE(router_weight && d_router_weight, "router_backward: null weight pointer");
  if (T > 0) JT_REQUIRE(x && scores && expert_ids && d_weights && dx, "router_backward: null pointer argument");
  const RouterBwdWs ws = carve_router(workspace, T, H, E, dtype);
  if (T > 0 && (workspace == nullptr || workspace_bytes < ws.total))
    return fail(JTMOE_EWORKSPACE, "router_backward: workspace of %zu bytes given, %zu needed", workspace_bytes,
                ws.total);
  return router_backward_impl(x, router_weight, scores, expert_ids, d_weights, d_scores, route_scale, T, H, E, K,
                              dtype, dx, d_router_weight, ws, as_stream(stream), score_func);
}

extern "C" size_t jtmoe_moe_backward_workspace_bytes(int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                                                     int dtype) {
  if (T < 0 || K <= 0 || H <= 0 || I <= 0 || E <= 0 || Is < 0 || !dtype_ok(dtype)) return 0;
  size_t total = carve_experts(nullptr, T * K, H, I, dtype).total;
  if (Is > 0) total += carve_shared(nullptr, T, H, Is, dtype).total;
  total += carve_router(nullptr, T, H, E, dtype).total;
  total += 3 * align_up((size_t)T * H * dtype_bytes(dtype), 256);  // dx of the shared experts, of the router, their sum
  total += align_up((size_t)T * K * dtype_bytes(dtype), 256);      // gradient of the route weights
  return total;
}

extern "C" int jtmoe_moe_backward(const void* x, const void* dy, const float* d_scores, const void* router_weight,
                                  const void* gate, const void* up, const void* down, const void* shared_gate,
                                  const void* shared_up, const void* shared_down, const float* scores,
                                  const int32_t* expert_ids, const void* weights, const int32_t* source_order,
                                  const int32_t* inverse, const int32_t* group_sizes, const int32_t* offsets,
                                  const void* gate_pre, const void* up_pre, const void* shared_gate_pre,
                                  const void* shared_up_pre, double route_scale, int64_t T, int64_t H, int64_t E,
                                  int64_t K, int64_t I, int64_t Is, int dtype, void* dx, void* d_router_weight,
                                  void* d_gate, void* d_up, void* d_down, void* d_shared_gate, void* d_shared_up,
                                  void* d_shared_down, void* workspace, size_t workspace_bytes, void* stream) {
  return jtmoe_moe_backward_sf(x, dy, d_scores, router_weight, gate, up, down, shared_gate, shared_up, shared_down,
                               scores, expert_ids, weights, source_order, inverse, group_sizes, offsets, gate_pre,
                               up_pre, shared_gate_pre, shared_up_pre, route_scale, JTMOE_SCORE_SIGMOID, T, H, E, K, I,
                               Is, dtype, dx, d_router_weight, d_gate, d_up, d_down, d_shared_gate, d_shared_up,
                               d_shared_down, workspace, workspace_bytes, stream);
}

extern "C" int jtmoe_moe_backward_sf(const void* x, const void* dy, const float* d_scores, const void* router_weight,
                                     const void* gate, const void* up, const void* down, const void* shared_gate,
                                     const void* shared_up, const void* shared_down, const float* scores,
                                     const int32_t* expert_ids, const void* weights, const int32_t* source_order,
                                     const int32_t* inverse, const int32_t* group_sizes, const int32_t* offsets,
                                     const void* gate_pre, const void* up_pre, const void* shared_gate_pre,
                                     const void* shared_up_pre, double route_scale, int score_func, int64_t T,
                                     int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is, int dtype, void* dx,
                                     void* d_router_weight, void* d_gate, void* d_up, void* d_down,
                                     void* d_shared_gate, void* d_shared_up, void* d_shared_down, void* workspace,
                                     size_t workspace_bytes, void* stream) {
  clear_error();
  int rc = validate_shape("moe_backward", T, K, H, I, E, dtype);
  if (rc) return rc;
  JT_REQUIRE(score_func_ok(score_func), "moe_backward: unknown score function %d", score_func);
  JT_REQUIRE(Is >= 0, "moe_backward: Is=%lld out of range", (long long)Is);
  JT_REQUIRE(router_weight && gate && up && down && d_router_weight && d_gate && d_up && d_down,
             "moe_backward: null weight pointer");
  JT_REQUIRE(group_sizes && offsets, "moe_backward: null group pointer");
  if (Is > 0)
    JT_REQUIRE(shared_gate && shared_up && shared_down && d_shared_gate && d_shared_up && d_shared_down,
               "moe_backward: null shared-expert weight pointer");
  if (T > 0) {
    JT_REQUIRE(x && dy && scores && expert_ids && weights && source_order && inverse && gate_pre && up_pre && dx,
               "moe_backward: null pointer argument");
    if (Is > 0) JT_REQUIRE(shared_gate_pre && shared_up_pre, "moe_backward: null shared-expert residual");
  }
  const size_t need = jtmoe_moe_backward_workspace_bytes(T, H, E, K, I, Is, dtype);
  if (T > 0 && (workspace == nullptr || workspace_bytes < need))
    return fail(JTMOE_EWORKSPACE, "moe_backward: workspace of %zu bytes given, %zu needed", workspace_bytes, need);
  hipStream_t s = as_stream(stream);
  Carver c{static_cast<unsigned char*>(workspace)};
  const ExpertsBwdWs ews = carve_experts(c.take(carve_experts(nullptr, T * K, H, I, dtype).total), T * K, H, I, dtype);
  SharedBwdWs sws{};
  if (Is > 0) sws = carve_shared(c.take(carve_shared(nullptr, T, H, Is, dtype).total), T, H, Is, dtype);
  const RouterBwdWs rws = carve_router(c.take(carve_router(nullptr, T, H, E, dtype).total), T, H, E, dtype);
  const size_t th = (size_t)T * H * dtype_bytes(dtype);
  void* dx_shared = c.take(th);
  void* dx_router = c.take(th);
  void* dx_sum = c.take(th);
  void* d_weights = c.take((size_t)T * K * dtype_bytes(dtype));

  rc = experts_backward_core(x, dy, source_order, inverse, weights, group_sizes, offsets, gate, up, down, gate_pre,
                             up_pre, T, K, H, I, E, dtype, d_weights, d_gate, d_up, d_down, ews, s);
  if (rc) return rc;
  if (Is > 0) {
    rc = shared_backward_impl(x, dy, shared_gate, shared_up, shared_down, shared_gate_pre, shared_up_pre, T, H, Is,
                              dtype, dx_shared, d_shared_gate, d_shared_up, d_shared_down, sws, s);
    if (rc) return rc;
  }
  rc = router_backward_impl(x, router_weight, scores, expert_ids, d_weights, d_scores, route_scale, T, H, E, K, dtype,
                            dx_router, d_router_weight, rws, s, score_func);
  if (rc) return rc;
  if (T == 0) return JTMOE_OK;
  const void* extra = dx_router;
  if (Is > 0) {
    if (dtype == JTMOE_BF16)
      run_add<bf16_raw>(dx_shared, dx_router, dx_sum, (size_t)T * H, s);
    else
      run_add<float>(dx_shared, dx_router, dx_sum, (size_t)T * H, s);
    rc = check_launch("moe backward");
    if (rc) return rc;
    extra = dx_sum;
  }
  return jtmoe_combine(ews.dxp, inverse, ews.ones, extra, T, H, K, dtype, dx, stream);
}
