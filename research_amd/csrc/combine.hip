// Combine: gate-weighted gather-reduce of the expert outputs back to token order,
// plus the unweighted shared-expert add.
//
// Follows moe.py:663-671 and :415/:429 of the reference:
//   y[t] = round( sum_s round(packed_y[inverse[t*K+s]] * w[t,s]) )     (fp32 sum, slot order)
//   y[t] = round( y[t] + shared_y[t] )                                  (if shared experts exist)
// Compiled with floating-point contraction OFF so that the product is rounded
// before it is accumulated, exactly as stated.
//
// The fused variant also applies what the decoder block does next (blocks.py:224-230):
//   out[t] = round( residual[t] + rmsnorm(y[t]; post_scale, eps) )
// with the RMSNorm of norm.hip (fp32 statistics of the rounded y, mul = 1/sqrt(var + eps) * scale).
// A wave holds the whole row of its token, so the row never leaves registers in between.
#include "common.hpp"

namespace jtmoe {
namespace {

// 8 bf16 values per 16-byte vector
__device__ __forceinline__ void unpack8(const uint4& v, float* f) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;

// fp32 -> bf16 -> fp32 with the hardware conversion (round to nearest even, same result as the
// integer formula of f32_to_bf16_bits for every finite value)
__device__ __forceinline__ float round_bf16_hw(float f) { return (float)(__bf16)f; }

__device__ __forceinline__ uint4 pack8_hw(const float* f) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f32x2_t v = {f[2 * i], f[2 * i + 1]};
    w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// bf16, rows a multiple of 8 elements, 16-byte aligned.  One wave per token; a lane owns NV
// 16-byte vectors of the row and requests them from all K source rows before it starts adding,
// so K*NV independent loads are in flight per lane.  KT = K when K is one of the unrolled
// values, 0 for a run-time loop.
__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d);
  return v;
}

template <int NV, int KT, bool kNorm>
__global__ __launch_bounds__(256) void combine_bf16_vec_kernel(const uint4* __restrict__ packed_y,
                                                               const int32_t* __restrict__ inverse,
                                                               const uint16_t* __restrict__ weights,
                                                               const uint4* __restrict__ shared_y, int tokens, int K,
                                                               int A, int row_vecs, uint4* __restrict__ y,
                                                               const uint4* __restrict__ residual,
                                                               const float* __restrict__ post_scale, float eps) {
#pragma clang fp contract(off)
  const int t = blockIdx.x * blockDim.y + threadIdx.y;
  if (t >= tokens) return;
  const int lane = threadIdx.x;
  float acc[NV][8];
#pragma unroll
  for (int j = 0; j < NV; ++j)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[j][i] = 0.0f;

  auto add_row = [&](const uint4* r, float w) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      float f[8];
      unpack8(r[j], f);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float p = round_bf16_hw(f[i] * w);
        acc[j][i] = acc[j][i] + p;
      }
    }
  };

  if (KT > 0) {
    int pos[KT > 0 ? KT : 1];
    float w[KT > 0 ? KT : 1];
#pragma unroll
    for (int s = 0; s < KT; ++s) {
      pos[s] = inverse[(size_t)t * KT + s];
      w[s] = bf16_bits_to_f32(weights[(size_t)t * KT + s]);
    }
    uint4 rows[KT > 0 ? KT : 1][NV];
#pragma unroll
    for (int s = 0; s < KT; ++s) {
      const bool ok = pos[s] >= 0 && pos[s] < A;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int v = lane + j * 64;
        rows[s][j] = (ok && v < row_vecs) ? load_stream(&packed_y[(size_t)pos[s] * row_vecs + v]) : make_uint4(0, 0, 0, 0);
      }
    }
#pragma unroll
    for (int s = 0; s < KT; ++s) add_row(rows[s], w[s]);  // a dropped assignment contributes +0
  } else {
    for (int s = 0; s < K; ++s) {
      const int pos = inverse[(size_t)t * K + s];
      if (pos < 0 || pos >= A) continue;
      const float w = bf16_bits_to_f32(weights[(size_t)t * K + s]);
      uint4 r[NV];
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int v = lane + j * 64;
        r[j] = v < row_vecs ? load_stream(&packed_y[(size_t)pos * row_vecs + v]) : make_uint4(0, 0, 0, 0);
      }
      add_row(r, w);
    }
  }
  float ss = 0.0f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int v = lane + j * 64;
    if (v >= row_vecs) continue;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[j][i] = round_bf16_hw(acc[j][i]);
    if (shared_y) {
      float f[8];
      unpack8(load_stream(&shared_y[(size_t)t * row_vecs + v]), f);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[j][i] = acc[j][i] + f[i];  // rounded by the packing
    }
    if (!kNorm) {
      store_stream(&y[(size_t)t * row_vecs + v], pack8_hw(acc[j]));
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        acc[j][i] = round_bf16_hw(acc[j][i]);
        ss += acc[j][i] * acc[j][i];
      }
    }
  }
  if (kNorm) {
    ss = wave_sum_f32(ss);
    const float inv = 1.0f / sqrtf(ss / (float)(row_vecs * 8) + eps);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int v = lane + j * 64;
      if (v >= row_vecs) continue;
      float r[8];
      unpack8(load_stream(&residual[(size_t)t * row_vecs + v]), r);
      const float4 s0 = reinterpret_cast<const float4*>(post_scale)[v * 2];
      const float4 s1 = reinterpret_cast<const float4*>(post_scale)[v * 2 + 1];
      const float sc[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float n = round_bf16_hw(acc[j][i] * (inv * sc[i]));
        acc[j][i] = r[i] + n;  // rounded by the packing
      }
      store_stream(&y[(size_t)t * row_vecs + v], pack8_hw(acc[j]));
    }
  }
}

// any dtype / row length, one element per lane
template <typename T>
__global__ __launch_bounds__(256) void combine_generic_kernel(const T* __restrict__ packed_y,
                                                              const int32_t* __restrict__ inverse,
                                                              const T* __restrict__ weights,
                                                              const T* __restrict__ shared_y, int tokens, int K, int A,
                                                              int H, T* __restrict__ y, const T* __restrict__ residual,
                                                              const float* __restrict__ post_scale, float eps) {
#pragma clang fp contract(off)
  const int t = blockIdx.x * blockDim.y + threadIdx.y;
  if (t >= tokens) return;
  float ss = 0.0f;
  for (int h = threadIdx.x; h < H; h += blockDim.x) {
    float acc = 0.0f;
    for (int s = 0; s < K; ++s) {
      const int pos = inverse[(size_t)t * K + s];
      if (pos < 0 || pos >= A) continue;
      const float w = Elem<T>::load(weights + (size_t)t * K + s);
      const float p = Elem<T>::round(Elem<T>::load(packed_y + (size_t)pos * H + h) * w);
      acc = acc + p;
    }
    acc = Elem<T>::round(acc);
    if (shared_y) acc = Elem<T>::round(acc + Elem<T>::load(shared_y + (size_t)t * H + h));
    Elem<T>::store(y + (size_t)t * H + h, acc);
    ss += acc * acc;
  }
  if (residual == nullptr) return;
  // fused post-norm and residual: the lane re-reads the elements it has just written
  ss = wave_sum_f32(ss);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  for (int h = threadIdx.x; h < H; h += blockDim.x) {
    const float n = Elem<T>::round(Elem<T>::load(y + (size_t)t * H + h) * (inv * post_scale[h]));
    Elem<T>::store(y + (size_t)t * H + h, Elem<T>::load(residual + (size_t)t * H + h) + n);
  }
}

}  // namespace
}  // namespace jtmoe

using namespace jtmoe;

namespace jtmoe {
namespace {

// residual == nullptr: plain combine; otherwise the fused post-norm + residual variant
int combine_launch(const char* what, const void* packed_y, const int32_t* inverse, const void* weights,
                   const void* shared_y, const void* residual, const float* post_scale, double eps, int64_t T,
                   int64_t H, int64_t K, int dtype, void* y, void* stream) {
  JT_REQUIRE(dtype_ok(dtype), "%s: unknown dtype %d", what, dtype);
  JT_REQUIRE(T >= 0 && H > 0 && K > 0, "%s: T=%lld H=%lld K=%lld out of range", what, (long long)T, (long long)H,
             (long long)K);
  if (K > JTMOE_MAX_TOP_K) return fail(JTMOE_EUNSUPPORTED, "%s: K=%lld exceeds %d", what, (long long)K, JTMOE_MAX_TOP_K);
  JT_REQUIRE(T * K < ((int64_t)1 << 31), "%s: T*K exceeds int32", what);
  JT_REQUIRE(H * (int64_t)dtype_bytes(dtype) < ((int64_t)1 << 31), "%s: row too long", what);
  if (T == 0) return JTMOE_OK;
  JT_REQUIRE(packed_y && inverse && weights && y, "%s: null pointer argument", what);
  const bool norm = residual != nullptr;
  hipStream_t s = as_stream(stream);
  const int A = (int)(T * K);
  const float epsf = (float)eps;
  const bool vec = dtype == JTMOE_BF16 && H % 8 == 0 && H <= 4096 && aligned16(packed_y) && aligned16(y) &&
                   (shared_y == nullptr || aligned16(shared_y)) &&
                   (!norm || (aligned16(residual) && aligned16(post_scale)));
  if (vec) {
    const int row_vecs = (int)(H / 8);
    dim3 block(64, 4);
    const int grid = (int)((T + block.y - 1) / block.y);
    const int nv = (row_vecs + 63) / 64;
#define JT_COMBINE_N(NV, KT, NORM)                                                                          \
  combine_bf16_vec_kernel<NV, KT, NORM><<<grid, block, 0, s>>>(                                             \
      static_cast<const uint4*>(packed_y), inverse, static_cast<const uint16_t*>(weights),                   \
      static_cast<const uint4*>(shared_y), (int)T, (int)K, A, row_vecs, static_cast<uint4*>(y),              \
      static_cast<const uint4*>(residual), post_scale, epsf)
#define JT_COMBINE(NV, KT)       \
  if (norm)                      \
    JT_COMBINE_N(NV, KT, true);  \
  else                           \
    JT_COMBINE_N(NV, KT, false)
#define JT_COMBINE_K(NV)      \
  if (K == 8) {               \
    JT_COMBINE(NV, 8);        \
  } else if (K == 2) {        \
    JT_COMBINE(NV, 2);        \
  } else {                    \
    JT_COMBINE(NV, 0);        \
  }
    if (nv <= 1) {
      JT_COMBINE_K(1);
    } else if (nv <= 2) {
      JT_COMBINE_K(2);
    } else if (nv <= 4) {
      JT_COMBINE_K(4);
    } else {
      JT_COMBINE(8, 0);
    }
#undef JT_COMBINE_K
#undef JT_COMBINE
#undef JT_COMBINE_N
  } else {
    dim3 block(64, 4);
    const int grid = (int)((T + block.y - 1) / block.y);
    if (dtype == JTMOE_BF16)
      combine_generic_kernel<bf16_raw><<<grid, block, 0, s>>>(
          static_cast<const bf16_raw*>(packed_y), inverse, static_cast<const bf16_raw*>(weights),
          static_cast<const bf16_raw*>(shared_y), (int)T, (int)K, A, (int)H, static_cast<bf16_raw*>(y),
          static_cast<const bf16_raw*>(residual), post_scale, epsf);
    else
      combine_generic_kernel<float><<<grid, block, 0, s>>>(
          static_cast<const float*>(packed_y), inverse, static_cast<const float*>(weights),
          static_cast<const float*>(shared_y), (int)T, (int)K, A, (int)H, static_cast<float*>(y),
          static_cast<const float*>(residual), post_scale, epsf);
  }
  return check_launch(what);
}

}  // namespace
}  // namespace jtmoe

extern "C" int jtmoe_combine(const void* packed_y, const int32_t* inverse, const void* weights, const void* shared_y,
                             int64_t T, int64_t H, int64_t K, int dtype, void* y, void* stream) {
  clear_error();
  return combine_launch("combine", packed_y, inverse, weights, shared_y, nullptr, nullptr, 0.0, T, H, K, dtype, y,
                        stream);
}

extern "C" int jtmoe_combine_norm_residual(const void* packed_y, const int32_t* inverse, const void* weights,
                                           const void* shared_y, const void* residual, const float* post_scale,
                                           double eps, int64_t T, int64_t H, int64_t K, int dtype, void* out,
                                           void* stream) {
  clear_error();
  JT_REQUIRE(eps >= 0.0, "combine_norm_residual: eps must not be negative");
  if (T > 0) JT_REQUIRE(residual && post_scale, "combine_norm_residual: null pointer argument");
  return combine_launch("combine_norm_residual", packed_y, inverse, weights, shared_y, T > 0 ? residual : nullptr,
                        post_scale, eps, T, H, K, dtype, out, stream);
}
