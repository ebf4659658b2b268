// Library-level pieces of libjtmoe: error state, the sequence balance loss and
// the whole-layer launcher that chains the stage launchers on one stream.
#include "common.hpp"

#include <cstdarg>
#include <cstdio>

namespace jtmoe {

namespace {
thread_local char g_error[512] = "";
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_error[0] = '\0'; }

thread_local StageTimer* g_stage_timer = nullptr;

int check_launch(const char* what) {
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return fail(JTMOE_ELAUNCH, "%s: %s", what, hipGetErrorString(err));
  return JTMOE_OK;
}

namespace {

// ---- sequence balance loss (reference moe.py:828-840) --------------------------
constexpr int kBalThreads = 256;
constexpr int kBalWaves = kBalThreads / kWave;
constexpr int kBalPerLane = JTMOE_MAX_EXPERTS / kWave;

__global__ __launch_bounds__(kBalThreads) void balance_partial_kernel(const int32_t* __restrict__ ids,
                                                                      const float* __restrict__ scores, int S, int E,
                                                                      int K, float* __restrict__ partial) {
  extern __shared__ float smem[];
  float* psum = smem;                                        // [kBalWaves][E]
  int* cnt = reinterpret_cast<int*>(smem + kBalWaves * E);   // [E]
  __shared__ float red[kBalWaves];
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int e = tid; e < E; e += kBalThreads) cnt[e] = 0;
  __syncthreads();
  const int32_t* ids_b = ids + (size_t)b * S * K;
  for (int i = tid; i < S * K; i += kBalThreads) {
    const int id = ids_b[i];
    if (id >= 0 && id < E) atomicAdd(&cnt[id], 1);
  }
  float acc[kBalPerLane];
#pragma unroll
  for (int j = 0; j < kBalPerLane; ++j) acc[j] = 0.0f;
  for (int s = wave; s < S; s += kBalWaves) {
    const float* row = scores + ((size_t)b * S + s) * E;
    float v[kBalPerLane];
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < kBalPerLane; ++j) {
      const int e = lane + j * kWave;
      v[j] = e < E ? row[e] : 0.0f;
      sum += v[j];
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) sum += __shfl_xor(sum, m);
    const float d = fmaxf(sum, 1e-20f);
#pragma unroll
    for (int j = 0; j < kBalPerLane; ++j) acc[j] += v[j] / d;
  }
#pragma unroll
  for (int j = 0; j < kBalPerLane; ++j) {
    const int e = lane + j * kWave;
    if (e < E) psum[wave * E + e] = acc[j];
  }
  __syncthreads();
  const float fscale = (float)E / ((float)K * (float)S);
  float local = 0.0f;
  for (int e = tid; e < E; e += kBalThreads) {
    float p = 0.0f;
    for (int w = 0; w < kBalWaves; ++w) p += psum[w * E + e];
    p = p / (float)S;
    local += fscale * (float)cnt[e] * p;
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) local += __shfl_xor(local, m);
  if (lane == 0) red[wave] = local;
  __syncthreads();
  if (tid == 0) {
    float t = 0.0f;
    for (int w = 0; w < kBalWaves; ++w) t += red[w];
    partial[b] = t;
  }
}

// Gradient of the loss with respect to the scores (the counts are piecewise constant and carry none):
//   d loss / d scores[b,s,e] = g / (B S) * ( f[b,e] / D - (sum_i f[b,i] scores[b,s,i]) / D^2 ),  D = sum_e scores[b,s,e]
// (for D <= 1e-20, where the forward divides by the constant 1e-20 instead: g / (B S) * f[b,e] / 1e-20).
// One workgroup per sequence, a wave per token at a time; g is *d_loss, or 1 when d_loss is null.
__global__ __launch_bounds__(kBalThreads) void balance_backward_kernel(const int32_t* __restrict__ ids,
                                                                       const float* __restrict__ scores,
                                                                       const float* __restrict__ d_loss, int B, int S,
                                                                       int E, int K, float* __restrict__ d_scores) {
  extern __shared__ float smem[];
  int* cnt = reinterpret_cast<int*>(smem);  // [E]
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int e = tid; e < E; e += kBalThreads) cnt[e] = 0;
  __syncthreads();
  const int32_t* ids_b = ids + (size_t)b * S * K;
  for (int i = tid; i < S * K; i += kBalThreads) {
    const int id = ids_b[i];
    if (id >= 0 && id < E) atomicAdd(&cnt[id], 1);
  }
  __syncthreads();
  const float fscale = (float)E / ((float)K * (float)S);
  const float g = (d_loss ? d_loss[0] : 1.0f) / ((float)B * (float)S);
  float f[kBalPerLane];
#pragma unroll
  for (int j = 0; j < kBalPerLane; ++j) {
    const int e = lane + j * kWave;
    f[j] = e < E ? fscale * (float)cnt[e] : 0.0f;
  }
  for (int s = wave; s < S; s += kBalWaves) {
    const size_t row = ((size_t)b * S + s) * E;
    float v[kBalPerLane];
    float sum = 0.0f, dot = 0.0f;
#pragma unroll
    for (int j = 0; j < kBalPerLane; ++j) {
      const int e = lane + j * kWave;
      v[j] = e < E ? scores[row + e] : 0.0f;
      sum += v[j];
      dot += f[j] * v[j];
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
      sum += __shfl_xor(sum, m);
      dot += __shfl_xor(dot, m);
    }
    const bool clamped = sum <= 1e-20f;
    const float d = clamped ? 1e-20f : sum;
    const float second = clamped ? 0.0f : dot / (d * d);
#pragma unroll
    for (int j = 0; j < kBalPerLane; ++j) {
      const int e = lane + j * kWave;
      if (e < E) d_scores[row + e] = g * (f[j] / d - second);
    }
  }
}

__global__ void balance_final_kernel(const float* __restrict__ partial, int B, float* __restrict__ loss) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    float t = 0.0f;
    for (int b = 0; b < B; ++b) t += partial[b];
    loss[0] = t / (float)B;
  }
}

// ---- scalar router statistics (reference moe.py:806-813) -----------------------
// out = {total, load_min, load_max, load_mean, max_vio, load_entropy}
__global__ __launch_bounds__(256) void router_stats_kernel(const float* __restrict__ counts, int E,
                                                           float* __restrict__ out) {
  __shared__ float s_sum[256], s_min[256], s_max[256];
  const int tid = threadIdx.x;
  float sum = 0.0f, mn = 3.402823466e38f, mx = -3.402823466e38f;
  for (int e = tid; e < E; e += 256) {
    const float c = counts[e];
    sum += c;
    mn = fminf(mn, c);
    mx = fmaxf(mx, c);
  }
  s_sum[tid] = sum;
  s_min[tid] = mn;
  s_max[tid] = mx;
  __syncthreads();
  for (int d = 128; d >= 1; d >>= 1) {
    if (tid < d) {
      s_sum[tid] += s_sum[tid + d];
      s_min[tid] = fminf(s_min[tid], s_min[tid + d]);
      s_max[tid] = fmaxf(s_max[tid], s_max[tid + d]);
    }
    __syncthreads();
  }
  const float total = s_sum[0];
  const float lmin = s_min[0], lmax = s_max[0];
  __syncthreads();
  float ent = 0.0f;
  const float denom = fmaxf(total, 1e-6f);
  for (int e = tid; e < E; e += 256) {
    const float p = counts[e] / denom;
    if (p > 0.0f) ent += p * logf(p);
  }
  s_sum[tid] = ent;
  __syncthreads();
  for (int d = 128; d >= 1; d >>= 1) {
    if (tid < d) s_sum[tid] += s_sum[tid + d];
    __syncthreads();
  }
  if (tid == 0) {
    const float mean = total / (float)E;
    out[0] = total;
    out[1] = lmin;
    out[2] = lmax;
    out[3] = mean;
    out[4] = (lmax - mean) / fmaxf(mean, 1e-6f);
    out[5] = -s_sum[0];
  }
}

// ---- SMEBU balancing update (reference steps/moe_balance.py:123-161, 174-184) ----------------
// One workgroup of 16 waves; a wave owns a layer at a time and reduces over its experts with
// shuffles (no barriers inside a layer).  Per layer: mean = sum(counts) / E;
// violation = (mean - counts) / max(mean, 1e-6); delta = load_lr * tanh(clamp * violation), centred on
// its mean; momentum' = f * momentum + (1 - f) * delta; bias' = bias + momentum'.
// metrics = {max over layers of max_vio, min of load_min, max of load_max, mean of the load entropy,
//            sqrt(sum bias'^2), sqrt(sum momentum'^2)}.  Every sum has a fixed order: a lane adds its
// experts in ascending order, the wave combines lanes in a butterfly, thread 0 adds layers in order.
constexpr int kSmebuWaves = 16;

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d);
  return v;
}

__global__ __launch_bounds__(kSmebuWaves * 64) void smebu_update_kernel(
    const float* __restrict__ counts, float* __restrict__ momentum, float* __restrict__ bias, int L, int E,
    float load_lr, float factor, float clamp, float* __restrict__ metrics) {
  __shared__ float s_vio[kSmebuWaves], s_min[kSmebuWaves], s_max[kSmebuWaves], s_ent[kSmebuWaves],
      s_bsq[kSmebuWaves], s_msq[kSmebuWaves];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float all_vio = -3.402823466e38f, all_min = 3.402823466e38f, all_max = -3.402823466e38f;
  float entropy_sum = 0.0f, bias_sq = 0.0f, momentum_sq = 0.0f;  // kept by thread 0
  for (int l0 = 0; l0 < L; l0 += kSmebuWaves) {
    const int l = l0 + wave;
    if (l < L) {
      const float* c = counts + (size_t)l * E;
      float* m = momentum + (size_t)l * E;
      float* b = bias + (size_t)l * E;
      float sum = 0.0f, mn = 3.402823466e38f, mx = -3.402823466e38f;
      for (int e = lane; e < E; e += 64) {
        const float v = c[e];
        sum += v;
        mn = fminf(mn, v);
        mx = fmaxf(mx, v);
      }
      const float total = wave_sum_f32(sum);
#pragma unroll
      for (int d = 32; d > 0; d >>= 1) {
        mn = fminf(mn, __shfl_xor(mn, d));
        mx = fmaxf(mx, __shfl_xor(mx, d));
      }
      const float mean = total / (float)E;
      const float denom = fmaxf(mean, 1e-6f);
      float dsum = 0.0f;
      for (int e = lane; e < E; e += 64) dsum += load_lr * tanhf(clamp * ((mean - c[e]) / denom));
      const float dmean = wave_sum_f32(dsum) / (float)E;
      float ent = 0.0f, bsq = 0.0f, msq = 0.0f;
      const float pden = fmaxf(total, 1e-6f);
      for (int e = lane; e < E; e += 64) {
        const float delta = load_lr * tanhf(clamp * ((mean - c[e]) / denom)) - dmean;
        const float next_m = factor * m[e] + (1.0f - factor) * delta;
        const float next_b = b[e] + next_m;
        m[e] = next_m;
        b[e] = next_b;
        msq += next_m * next_m;
        bsq += next_b * next_b;
        const float p = c[e] / pden;
        if (p > 0.0f) ent += p * logf(p);
      }
      ent = wave_sum_f32(ent);
      bsq = wave_sum_f32(bsq);
      msq = wave_sum_f32(msq);
      if (lane == 0) {
        s_vio[wave] = (mx - mean) / denom;
        s_min[wave] = mn;
        s_max[wave] = mx;
        s_ent[wave] = -ent;
        s_bsq[wave] = bsq;
        s_msq[wave] = msq;
      }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      const int n = min(kSmebuWaves, L - l0);
      for (int w = 0; w < n; ++w) {
        all_vio = fmaxf(all_vio, s_vio[w]);
        all_min = fminf(all_min, s_min[w]);
        all_max = fmaxf(all_max, s_max[w]);
        entropy_sum += s_ent[w];
        bias_sq += s_bsq[w];
        momentum_sq += s_msq[w];
      }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    metrics[0] = all_vio;
    metrics[1] = all_min;
    metrics[2] = all_max;
    metrics[3] = entropy_sum / (float)L;
    metrics[4] = sqrtf(bias_sq);
    metrics[5] = sqrtf(momentum_sq);
  }
}

struct Carve {
  unsigned char* base;
  size_t used;
  void* take(size_t bytes) {
    void* p = base ? base + used : nullptr;
    used += align_up(bytes, 256);
    return p;
  }
};

struct LayerWorkspace {
  void* router;
  size_t router_bytes;
  void* dispatch;
  size_t dispatch_bytes;
  void* packed_x;
  void* act;
  void* packed_y;
  void* shared_act;
  void* shared_y;
  size_t total;
};

LayerWorkspace carve_layer(void* base, int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is, int dtype) {
  const size_t b = dtype_bytes(dtype);
  const size_t A = (size_t)T * (size_t)K;
  Carve c{static_cast<unsigned char*>(base), 0};
  LayerWorkspace w;
  w.router_bytes = jtmoe_router_workspace_bytes(E);
  w.router = c.take(w.router_bytes);
  w.dispatch_bytes = dispatch_layer_workspace_bytes((int64_t)A, E);
  w.dispatch = c.take(w.dispatch_bytes);
  // the permuted copy of x exists only where the grouped GEMM cannot fetch its rows through the
  // permutation itself (a third of the workspace at 64 experts x top-8 x 2048)
  w.packed_x = jtmoe_grouped_swiglu_gather_supported(T, H, I, dtype) ? nullptr : c.take(A * (size_t)H * b);
  // (the decode path keeps the activations of all tokens through every expert)
  const size_t act_rows = decode_dense_supported(T, H, E, K, I, dtype) ? (size_t)E * (size_t)T : A;
  w.act = c.take((act_rows > A ? act_rows : A) * (size_t)I * b);
  w.packed_y = c.take(A * (size_t)H * b);
  w.shared_act = Is > 0 ? c.take((size_t)T * (size_t)Is * b) : nullptr;
  w.shared_y = Is > 0 ? c.take((size_t)T * (size_t)H * b) : nullptr;
  w.total = c.used;
  return w;
}

}  // namespace
}  // namespace jtmoe

using namespace jtmoe;

extern "C" int jtmoe_version(void) { return JTMOE_VERSION; }

extern "C" const char* jtmoe_last_error(void) { return g_error; }

extern "C" size_t jtmoe_balance_workspace_bytes(int64_t B, int64_t E) {
  (void)E;
  if (B <= 0) return 0;
  return align_up((size_t)B * sizeof(float), 256);
}

extern "C" int jtmoe_sequence_balance_loss(const int32_t* expert_ids, const float* scores, int64_t B, int64_t S,
                                           int64_t E, int64_t K, float* loss, void* workspace,
                                           size_t workspace_bytes, void* stream) {
  clear_error();
  JT_REQUIRE(B > 0 && S > 0 && E > 0 && K > 0, "sequence_balance_loss: B=%lld S=%lld E=%lld K=%lld out of range",
             (long long)B, (long long)S, (long long)E, (long long)K);
  if (E > JTMOE_MAX_EXPERTS) return fail(JTMOE_EUNSUPPORTED, "sequence_balance_loss: E=%lld exceeds %d", (long long)E, JTMOE_MAX_EXPERTS);
  JT_REQUIRE(B * S * E < ((int64_t)1 << 40) && S * K < ((int64_t)1 << 31) && B < ((int64_t)1 << 24),
             "sequence_balance_loss: sizes out of range");
  JT_REQUIRE(expert_ids && scores && loss && workspace, "sequence_balance_loss: null pointer argument");
  if (workspace_bytes < jtmoe_balance_workspace_bytes(B, E))
    return fail(JTMOE_EWORKSPACE, "sequence_balance_loss: workspace %zu < %zu bytes", workspace_bytes,
                jtmoe_balance_workspace_bytes(B, E));
  hipStream_t s = as_stream(stream);
  float* partial = static_cast<float*>(workspace);
  const size_t smem = (size_t)(kBalWaves + 1) * E * sizeof(float);
  balance_partial_kernel<<<(unsigned)B, kBalThreads, smem, s>>>(expert_ids, scores, (int)S, (int)E, (int)K, partial);
  balance_final_kernel<<<1, 64, 0, s>>>(partial, (int)B, loss);
  return check_launch("sequence_balance_loss");
}

extern "C" int jtmoe_sequence_balance_loss_backward(const int32_t* expert_ids, const float* scores,
                                                    const float* d_loss, int64_t B, int64_t S, int64_t E, int64_t K,
                                                    float* d_scores, void* stream) {
  clear_error();
  JT_REQUIRE(B > 0 && S > 0 && E > 0 && K > 0,
             "sequence_balance_loss_backward: B=%lld S=%lld E=%lld K=%lld out of range", (long long)B, (long long)S,
             (long long)E, (long long)K);
  if (E > JTMOE_MAX_EXPERTS)
    return fail(JTMOE_EUNSUPPORTED, "sequence_balance_loss_backward: E=%lld exceeds %d", (long long)E, JTMOE_MAX_EXPERTS);
  JT_REQUIRE(B * S * E < ((int64_t)1 << 40) && S * K < ((int64_t)1 << 31) && B < ((int64_t)1 << 24),
             "sequence_balance_loss_backward: sizes out of range");
  JT_REQUIRE(expert_ids && scores && d_scores, "sequence_balance_loss_backward: null pointer argument");
  balance_backward_kernel<<<(unsigned)B, kBalThreads, (size_t)E * sizeof(int), as_stream(stream)>>>(
      expert_ids, scores, d_loss, (int)B, (int)S, (int)E, (int)K, d_scores);
  return check_launch("sequence_balance_loss_backward");
}

extern "C" int jtmoe_router_stats(const float* expert_counts, int64_t E, float* stats6, void* stream) {
  clear_error();
  JT_REQUIRE(E > 0 && E < ((int64_t)1 << 24), "router_stats: E=%lld out of range", (long long)E);
  JT_REQUIRE(expert_counts && stats6, "router_stats: null pointer argument");
  router_stats_kernel<<<1, 256, 0, as_stream(stream)>>>(expert_counts, (int)E, stats6);
  return check_launch("router_stats");
}

extern "C" int jtmoe_smebu_update(const float* router_counts, float* momentum, float* expert_bias, int64_t L,
                                  int64_t E, float load_lr, float momentum_factor, float clamp, float* metrics6,
                                  void* stream) {
  clear_error();
  JT_REQUIRE(L > 0 && L < ((int64_t)1 << 20) && E > 0 && E < ((int64_t)1 << 24), "smebu_update: L=%lld E=%lld out of range",
             (long long)L, (long long)E);
  JT_REQUIRE(load_lr > 0.0f && momentum_factor > 0.0f && clamp > 0.0f,
             "smebu_update: load_lr, momentum and clamp must be positive");
  JT_REQUIRE(router_counts && momentum && expert_bias && metrics6, "smebu_update: null pointer argument");
  smebu_update_kernel<<<1, kSmebuWaves * 64, 0, as_stream(stream)>>>(router_counts, momentum, expert_bias, (int)L, (int)E, load_lr,
                                                       momentum_factor, clamp, metrics6);
  return check_launch("smebu_update");
}

extern "C" int jtmoe_moe_forward_takes_decode_path(int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int dtype) {
  if (T < 0 || H <= 0 || E <= 0 || K <= 0 || I <= 0 || !dtype_ok(dtype)) return 0;
  return decode_dense_supported(T, H, E, K, I, dtype) ? 1 : 0;
}

extern "C" size_t jtmoe_workspace_bytes(int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                                        int dtype) {
  if (T < 0 || H <= 0 || E <= 0 || K <= 0 || I <= 0 || Is < 0 || !dtype_ok(dtype)) return 0;
  return carve_layer(nullptr, T, H, E, K, I, Is, dtype).total;
}

// gate_pre .. shared_up_pre: where the training forward keeps the four rounded products that the
// backward pass reads; all null for the plain forward
static int moe_forward_impl(const void* x, const void* w_router, const float* expert_bias, const void* gate,
                            const void* up, const void* down, const void* shared_gate, const void* shared_up,
                            const void* shared_down, int64_t T, int64_t H, int64_t E, int64_t K, int64_t I,
                            int64_t Is, double route_scale, int dtype, void* y, int32_t* expert_ids, void* weights,
                            float* scores, float* expert_counts, float* importance, int32_t* group_sizes,
                            int32_t* offsets, int32_t* source_order, int32_t* inverse, void* workspace,
                            size_t workspace_bytes, void* stream, void* gate_pre, void* up_pre,
                            void* shared_gate_pre, void* shared_up_pre, const void* residual = nullptr,
                            const float* post_scale = nullptr, double eps = 0.0,
                            int score_func = JTMOE_SCORE_SIGMOID) {
  clear_error();
  const bool train = gate_pre != nullptr;
  JT_REQUIRE(dtype_ok(dtype), "moe_forward: unknown dtype %d", dtype);
  JT_REQUIRE(T >= 0 && H > 0 && E > 0 && K > 0 && I > 0 && Is >= 0, "moe_forward: shape out of range");
  JT_REQUIRE((Is == 0) == (shared_gate == nullptr) && (Is == 0) == (shared_up == nullptr) &&
                 (Is == 0) == (shared_down == nullptr),
             "moe_forward: shared expert matrices and Is=%lld disagree", (long long)Is);
  JT_REQUIRE(workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
             "moe_forward: workspace must be non-null and 256-byte aligned");
  const LayerWorkspace w = carve_layer(workspace, T, H, E, K, I, Is, dtype);
  if (workspace_bytes < w.total)
    return fail(JTMOE_EWORKSPACE, "moe_forward: workspace %zu < %zu bytes", workspace_bytes, w.total);
  // where the GEMM can apply the permutation while it fetches its A tiles, the permuted copy of
  // x is never written: dispatch then only computes the histogram, offsets and permutation
  const bool gather = train || (T > 0 && jtmoe_grouped_swiglu_gather_supported(T, H, I, dtype));
  // the workspace of such a shape holds no permuted copy of x to fall back on
  if (gather && !train &&
      ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up) |
        reinterpret_cast<uintptr_t>(down)) & 15u) != 0)
    return fail(JTMOE_EINVAL, "moe_forward: x and the expert matrices must be 16-byte aligned");
  // The router of a layer call leaves out what the dispatch behind it can do in passing: at large
  // batches the statistics (no zeroing and no finalising launch, no global atomics), at small ones
  // its finishing workgroup writes the dispatch plan as well.
  // Decode path (a handful of tokens): one launch runs every token through every expert's gate and up
  // matrices, which needs nothing of the routing, and a few of its workgroups are the router and write
  // the dispatch plan; the down launch then picks the routed rows.
  hipStream_t main_stream = as_stream(stream);
  const bool decode = !train && decode_dense_supported(T, H, E, K, I, dtype);
  bool stats_done = false, plan_done = false;
  int rc;
  if (decode) {
    rc = launch_decode_gate_up_router(x, w_router, expert_bias, gate, up, w.act, T, H, E, K, I, route_scale,
                                      score_func, expert_ids, weights, scores, expert_counts, importance, group_sizes,
                                      offsets, source_order, inverse, w.router, main_stream);
    if (rc) return rc;
    stage_mark(kStageGateUp, main_stream);
    rc = launch_down_from_all_tokens(w.act, down, group_sizes, offsets, source_order, T, K, H, I, E, w.packed_y,
                                     main_stream);
    if (rc) return rc;
    stage_mark(kStageDown, main_stream);
    rc = check_launch("grouped gemm");
  } else {
    rc = router_for_layer(x, w_router, expert_bias, T, H, E, K, route_scale, dtype, expert_ids, weights, scores,
                          expert_counts, importance, group_sizes, offsets, source_order, inverse, w.router,
                          w.router_bytes, score_func, &stats_done, &plan_done, main_stream);
    if (rc) return rc;
    stage_mark(kStageRouter, main_stream);
    rc = dispatch_for_layer(expert_ids, weights, (T > 0 && !gather) ? x : nullptr, T, H, E, K, dtype, group_sizes,
                            offsets, source_order, inverse, w.packed_x, expert_counts, importance, w.dispatch,
                            !stats_done, plan_done, main_stream);
  }
  if (rc) return rc;
  if (!decode) {  // (the decode path has enqueued both of its GEMM launches above)
    if (train)
      rc = jtmoe_grouped_swiglu_train(x, source_order, gate, up, down, group_sizes, offsets, T, K, H, I, E, dtype,
                                      gate_pre, up_pre, w.act, w.packed_y, stream);
    else if (gather)
      rc = jtmoe_grouped_swiglu_gather(x, source_order, gate, up, down, group_sizes, offsets, T, K, H, I, E, dtype,
                                       w.act, w.packed_y, stream);
    else
      rc = jtmoe_grouped_swiglu(w.packed_x, gate, up, down, group_sizes, offsets, T * K, H, I, E, dtype, w.act,
                                w.packed_y, stream);
    if (rc) return rc;
  }
  if (Is > 0) {
    if (train)
      rc = jtmoe_shared_swiglu_train(x, shared_gate, shared_up, shared_down, T, H, Is, dtype, shared_gate_pre,
                                     shared_up_pre, w.shared_act, w.shared_y, stream);
    else
      rc = jtmoe_shared_swiglu(x, shared_gate, shared_up, shared_down, T, H, Is, dtype, w.shared_act, w.shared_y,
                               stream);
    if (rc) return rc;
  }
  if (residual)  // the decoder block's tail fused into the combine: y = residual + rmsnorm(layer output)
    rc = jtmoe_combine_norm_residual(w.packed_y, inverse, weights, Is > 0 ? w.shared_y : nullptr, residual, post_scale,
                                     eps, T, H, K, dtype, y, stream);
  else
    rc = jtmoe_combine(w.packed_y, inverse, weights, Is > 0 ? w.shared_y : nullptr, T, H, K, dtype, y, stream);
  stage_mark(kStageCombine, as_stream(stream));
  return rc;
}

extern "C" int jtmoe_moe_forward(const void* x, const void* w_router, const float* expert_bias, const void* gate,
                                 const void* up, const void* down, const void* shared_gate, const void* shared_up,
                                 const void* shared_down, int64_t T, int64_t H, int64_t E, int64_t K, int64_t I,
                                 int64_t Is, double route_scale, int dtype, void* y, int32_t* expert_ids,
                                 void* weights, float* scores, float* expert_counts, float* importance,
                                 int32_t* group_sizes, int32_t* offsets, int32_t* source_order, int32_t* inverse,
                                 void* workspace, size_t workspace_bytes, void* stream) {
  return moe_forward_impl(x, w_router, expert_bias, gate, up, down, shared_gate, shared_up, shared_down, T, H, E, K, I,
                          Is, route_scale, dtype, y, expert_ids, weights, scores, expert_counts, importance,
                          group_sizes, offsets, source_order, inverse, workspace, workspace_bytes, stream, nullptr,
                          nullptr, nullptr, nullptr);
}

extern "C" int jtmoe_moe_forward_sf(const void* x, const void* w_router, const float* expert_bias, const void* gate,
                                    const void* up, const void* down, const void* shared_gate, const void* shared_up,
                                    const void* shared_down, int64_t T, int64_t H, int64_t E, int64_t K, int64_t I,
                                    int64_t Is, double route_scale, int score_func, int dtype, void* y,
                                    int32_t* expert_ids, void* weights, float* scores, float* expert_counts,
                                    float* importance, int32_t* group_sizes, int32_t* offsets, int32_t* source_order,
                                    int32_t* inverse, void* workspace, size_t workspace_bytes, void* stream) {
  return moe_forward_impl(x, w_router, expert_bias, gate, up, down, shared_gate, shared_up, shared_down, T, H, E, K, I,
                          Is, route_scale, dtype, y, expert_ids, weights, scores, expert_counts, importance,
                          group_sizes, offsets, source_order, inverse, workspace, workspace_bytes, stream, nullptr,
                          nullptr, nullptr, nullptr, nullptr, nullptr, 0.0, score_func);
}

extern "C" int jtmoe_moe_forward_train(const void* x, const void* w_router, const float* expert_bias,
                                       const void* gate, const void* up, const void* down, const void* shared_gate,
                                       const void* shared_up, const void* shared_down, int64_t T, int64_t H,
                                       int64_t E, int64_t K, int64_t I, int64_t Is, double route_scale, int dtype,
                                       void* y, int32_t* expert_ids, void* weights, float* scores,
                                       float* expert_counts, float* importance, int32_t* group_sizes,
                                       int32_t* offsets, int32_t* source_order, int32_t* inverse, void* gate_pre,
                                       void* up_pre, void* shared_gate_pre, void* shared_up_pre, void* workspace,
                                       size_t workspace_bytes, void* stream) {
  return jtmoe_moe_forward_train_sf(x, w_router, expert_bias, gate, up, down, shared_gate, shared_up, shared_down, T, H,
                                    E, K, I, Is, route_scale, JTMOE_SCORE_SIGMOID, dtype, y, expert_ids, weights, scores,
                                    expert_counts, importance, group_sizes, offsets, source_order, inverse, gate_pre,
                                    up_pre, shared_gate_pre, shared_up_pre, workspace, workspace_bytes, stream);
}

extern "C" int jtmoe_moe_forward_train_sf(const void* x, const void* w_router, const float* expert_bias,
                                          const void* gate, const void* up, const void* down,
                                          const void* shared_gate, const void* shared_up, const void* shared_down,
                                          int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                                          double route_scale, int score_func, int dtype, void* y, int32_t* expert_ids,
                                          void* weights, float* scores, float* expert_counts, float* importance,
                                          int32_t* group_sizes, int32_t* offsets, int32_t* source_order,
                                          int32_t* inverse, void* gate_pre, void* up_pre, void* shared_gate_pre,
                                          void* shared_up_pre, void* workspace, size_t workspace_bytes, void* stream) {
  if (T > 0 && (gate_pre == nullptr || up_pre == nullptr || (Is > 0 && (!shared_gate_pre || !shared_up_pre)))) {
    clear_error();
    return fail(JTMOE_EINVAL, "moe_forward_train: null residual buffer");
  }
  // without tokens there is nothing to keep and the plain path (which launches nothing) serves
  return moe_forward_impl(x, w_router, expert_bias, gate, up, down, shared_gate, shared_up, shared_down, T, H, E, K, I,
                          Is, route_scale, dtype, y, expert_ids, weights, scores, expert_counts, importance,
                          group_sizes, offsets, source_order, inverse, workspace, workspace_bytes, stream,
                          gate_pre, up_pre, shared_gate_pre, shared_up_pre, nullptr, nullptr, 0.0, score_func);
}

extern "C" size_t jtmoe_ffn_block_workspace_bytes(int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                                                  int dtype) {
  const size_t layer = jtmoe_workspace_bytes(T, H, E, K, I, Is, dtype);
  if (layer == 0) return 0;
  return layer + align_up((size_t)T * (size_t)H * dtype_bytes(dtype), 256);
}

extern "C" int jtmoe_ffn_block_forward(const void* x, const float* pre_scale, const float* post_scale, double eps,
                                       const void* w_router, const float* expert_bias, const void* gate,
                                       const void* up, const void* down, const void* shared_gate,
                                       const void* shared_up, const void* shared_down, int64_t T, int64_t H,
                                       int64_t E, int64_t K, int64_t I, int64_t Is, double route_scale, int dtype,
                                       void* out, int32_t* expert_ids, void* weights, float* scores,
                                       float* expert_counts, float* importance, int32_t* group_sizes,
                                       int32_t* offsets, int32_t* source_order, int32_t* inverse, void* workspace,
                                       size_t workspace_bytes, void* stream) {
  clear_error();
  JT_REQUIRE(dtype_ok(dtype), "ffn_block_forward: unknown dtype %d", dtype);
  JT_REQUIRE(T >= 0 && H > 0 && E > 0 && K > 0 && I > 0 && Is >= 0, "ffn_block_forward: shape out of range");
  JT_REQUIRE(pre_scale && post_scale, "ffn_block_forward: null norm scale");
  JT_REQUIRE(workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
             "ffn_block_forward: workspace must be non-null and 256-byte aligned");
  const size_t layer_bytes = jtmoe_workspace_bytes(T, H, E, K, I, Is, dtype);
  const size_t need = jtmoe_ffn_block_workspace_bytes(T, H, E, K, I, Is, dtype);
  if (workspace_bytes < need)
    return fail(JTMOE_EWORKSPACE, "ffn_block_forward: workspace %zu < %zu bytes", workspace_bytes, need);
  void* normed = static_cast<unsigned char*>(workspace) + layer_bytes;
  int rc = jtmoe_rmsnorm(x, pre_scale, T, H, eps, dtype, normed, stream);
  if (rc) return rc;
  return moe_forward_impl(normed, w_router, expert_bias, gate, up, down, shared_gate, shared_up, shared_down, T, H, E,
                          K, I, Is, route_scale, dtype, out, expert_ids, weights, scores, expert_counts, importance,
                          group_sizes, offsets, source_order, inverse, workspace, layer_bytes, stream, nullptr,
                          nullptr, nullptr, nullptr, T > 0 ? x : nullptr, post_scale, eps);
}

extern "C" int jtmoe_moe_forward_timed(const void* x, const void* w_router, const float* expert_bias,
                                       const void* gate, const void* up, const void* down, const void* shared_gate,
                                       const void* shared_up, const void* shared_down, int64_t T, int64_t H,
                                       int64_t E, int64_t K, int64_t I, int64_t Is, double route_scale, int dtype,
                                       void* y, int32_t* expert_ids, void* weights, float* scores,
                                       float* expert_counts, float* importance, int32_t* group_sizes,
                                       int32_t* offsets, int32_t* source_order, int32_t* inverse, void* workspace,
                                       size_t workspace_bytes, void* stream, float* stage_ms) {
  clear_error();
  JT_REQUIRE(stage_ms != nullptr, "moe_forward_timed: stage_ms is null");
  StageTimer timer;
  int created = 0;
  for (; created < kStageCount; ++created)
    if (hipEventCreate(&timer.ev[created]) != hipSuccess) break;
  int rc = JTMOE_OK;
  if (created != kStageCount) {
    rc = fail(JTMOE_ELAUNCH, "moe_forward_timed: hipEventCreate failed");
  } else {
    hipStream_t s = as_stream(stream);
    // every event is recorded once up front so that a skipped stage reads as zero
    for (int i = kStageCount - 1; i >= 0; --i) (void)hipEventRecord(timer.ev[i], s);
    g_stage_timer = &timer;
    rc = jtmoe_moe_forward(x, w_router, expert_bias, gate, up, down, shared_gate, shared_up, shared_down, T, H, E, K,
                           I, Is, route_scale, dtype, y, expert_ids, weights, scores, expert_counts, importance,
                           group_sizes, offsets, source_order, inverse, workspace, workspace_bytes, stream);
    g_stage_timer = nullptr;
    if (hipStreamSynchronize(s) != hipSuccess && rc == JTMOE_OK)
      rc = fail(JTMOE_ELAUNCH, "moe_forward_timed: stream synchronisation failed");
    if (rc == JTMOE_OK) {
      int last = kStageBegin;
      for (int i = 1; i < kStageCount; ++i) {
        float ms = 0.0f;
        // a stage that did not run keeps its up-front record, which precedes kStageBegin
        if (hipEventElapsedTime(&ms, timer.ev[last], timer.ev[i]) != hipSuccess || ms < 0.0f) {
          stage_ms[i - 1] = 0.0f;
          continue;
        }
        stage_ms[i - 1] = ms;
        last = i;
      }
    }
  }
  for (int i = 0; i < created; ++i) (void)hipEventDestroy(timer.ev[i]);
  return rc;
}
