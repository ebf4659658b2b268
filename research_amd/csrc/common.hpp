// Shared host/device helpers of libjtmoe (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "jtmoe.h"

namespace jtmoe {

// ---- host side: status + thread-local message -----------------------------
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();
// hipGetLastError() after a launch -> JTMOE_OK or JTMOE_ELAUNCH (message set).
int check_launch(const char* what);

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline size_t dtype_bytes(int dtype) { return dtype == JTMOE_F32 ? 4 : 2; }
inline bool dtype_ok(int dtype) { return dtype == JTMOE_BF16 || dtype == JTMOE_F32; }
inline bool score_func_ok(int f) { return f == JTMOE_SCORE_SIGMOID || f == JTMOE_SCORE_SOFTMAX; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- optional per-stage timing (only jtmoe_moe_forward_timed installs a timer) ----
enum Stage {
  kStageBegin = 0,
  kStageRouter,
  kStageDispatchMeta,
  kStageDispatchRows,
  kStageGateUp,
  kStageDown,
  kStageSharedGateUp,
  kStageSharedDown,
  kStageCombine,
  kStageCount
};
struct StageTimer {
  hipEvent_t ev[kStageCount];
};
extern thread_local StageTimer* g_stage_timer;
// records the event that closes `stage` on `s`; a no-op unless a timer is installed
inline void stage_mark(int stage, hipStream_t s) {
  if (g_stage_timer) (void)hipEventRecord(g_stage_timer->ev[stage], s);
}

#define JT_REQUIRE(cond, ...)                          \
  do {                                                 \
    if (!(cond)) return ::jtmoe::fail(JTMOE_EINVAL, __VA_ARGS__); \
  } while (0)

// ---- device side: element types --------------------------------------------
// bf16 values travel as raw 16-bit patterns; fp32 as float.
struct bf16_raw {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits) { return __uint_as_float(bits << 16); }

// round-to-nearest-even fp32 -> bf16 bit pattern (NaN stays a quiet NaN)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x0040u;
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ float round_to_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

template <typename T>
struct Elem;

template <>
struct Elem<float> {
  static constexpr bool is_bf16 = false;
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};

template <>
struct Elem<bf16_raw> {
  static constexpr bool is_bf16 = true;
  static __device__ __forceinline__ float load(const bf16_raw* p) { return bf16_bits_to_f32(p->bits); }
  static __device__ __forceinline__ void store(bf16_raw* p, float v) { p->bits = (uint16_t)f32_to_bf16_bits(v); }
  static __device__ __forceinline__ float round(float v) { return round_to_bf16(v); }
};

constexpr int kWave = 64;

// 16-byte loads and stores of data that is touched once (rows streamed through an HBM-bound kernel):
// the non-temporal forms keep them from displacing each other in the L2.  On the 537 MB gather of
// the combine they are worth 4.9 -> 6.2 TB/s.
typedef unsigned int stream_u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_stream(const uint4* p) {
  const stream_u32x4_t r = __builtin_nontemporal_load(reinterpret_cast<const stream_u32x4_t*>(p));
  return make_uint4(r[0], r[1], r[2], r[3]);
}
__device__ __forceinline__ void store_stream(uint4* p, const uint4& v) {
  const stream_u32x4_t r = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(r, reinterpret_cast<stream_u32x4_t*>(p));
}
// scalar element types go through the same names
template <typename V>
__device__ __forceinline__ V load_stream(const V* p) {
  return __builtin_nontemporal_load(p);
}
template <typename V>
__device__ __forceinline__ void store_stream(V* p, const V& v) {
  __builtin_nontemporal_store(v, p);
}

// dispatch.hip: packed[inverse[t*K + s]] = x[t] (the row scatter of jtmoe_dispatch on its own)
void launch_dispatch_rows(const void* x, const int32_t* inverse, int64_t T, int64_t K, int64_t H, int dtype,
                          void* packed_x, hipStream_t stream);

// dispatch.hip: the dispatch as the layer runs it.  want_stats (weights of element type = dtype): the
// histogram pass also sums the route weights per expert, and expert_counts / importance get the
// statistics that the router left out (router_for_layer).  The workspace holds
// dispatch_layer_workspace_bytes(T*K, E) bytes.  plan_done: only the row scatter is left to do.
size_t dispatch_layer_workspace_bytes(int64_t A, int64_t E);
int dispatch_for_layer(const int32_t* expert_ids, const void* weights, const void* x, int64_t T, int64_t H, int64_t E,
                       int64_t K, int dtype, int32_t* group_sizes, int32_t* offsets, int32_t* source_order,
                       int32_t* inverse, void* packed_x, float* expert_counts, float* importance, void* workspace,
                       bool want_stats, bool plan_done, hipStream_t stream);

// router.hip: the router as the layer runs it, with the dispatch plan behind it where that is free.
// On return *stats_done says whether expert_counts / importance have been written (the small-batch
// path gets them from its one finishing workgroup); if not, the caller's dispatch computes them from
// the ids and weights.  *plan_done says whether group_sizes / offsets / source_order / inverse have
// been written as well (the finishing workgroup of the small-batch router goes on to the plan while
// it still holds the ids in LDS).
int router_for_layer(const void* x, const void* w_router, const float* expert_bias, int64_t T, int64_t H, int64_t E,
                     int64_t K, double route_scale, int dtype, int32_t* expert_ids, void* weights, float* scores,
                     float* expert_counts, float* importance, int32_t* group_sizes, int32_t* offsets,
                     int32_t* source_order, int32_t* inverse, void* workspace, size_t workspace_bytes,
                     int score_func, bool* stats_done, bool* plan_done, hipStream_t stream);


// The decode path of the layer (a handful of tokens, nearly every expert chosen by some token).  A tile is
// 64 rows tall whether it holds an expert's few routed rows or all T <= 64 tokens, so ONE launch runs every
// token through every expert's gate and up matrices -- act_full [E][T][I], which needs nothing of the
// routing -- while a few of its workgroups are the router and write the dispatch plan (router.hip); the
// down launch (grouped_gemm.hip) then takes packed row j from act_full[expert of j][source_order[j] / K].
// The launches stream the same expert matrices in the same time as the gathering ones, the router's
// dependent steps no longer stand in front of them, and the rows that were routed come out bit for bit as
// from the gathering launch.
bool decode_dense_supported(int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int dtype);
int launch_decode_gate_up_router(const void* x, const void* w_router, const float* expert_bias, const void* gate,
                                 const void* up, void* act_full, int64_t T, int64_t H, int64_t E, int64_t K, int64_t I,
                                 double route_scale, int score_func, int32_t* expert_ids, void* weights, float* scores,
                                 float* expert_counts, float* importance, int32_t* group_sizes, int32_t* offsets,
                                 int32_t* source_order, int32_t* inverse, void* router_workspace, hipStream_t stream);
int launch_down_from_all_tokens(const void* act_full, const void* down, const int32_t* group_sizes,
                                const int32_t* offsets, const int32_t* source_order, int64_t T, int64_t K, int64_t H,
                                int64_t I, int64_t E, void* packed_y, hipStream_t stream);

}  // namespace jtmoe
