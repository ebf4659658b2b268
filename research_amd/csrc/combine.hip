// Combine: gate-weighted gather-reduce of the expert outputs back to token order,
// plus the unweighted shared-expert add.
//
// Follows moe.py:663-671 and :415/:429 of the reference:
//   y[t] = round( sum_s round(packed_y[inverse[t*K+s]] * w[t,s]) )     (fp32 sum, slot order)
//   y[t] = round( y[t] + shared_y[t] )                                  (if shared experts exist)
// Compiled with floating-point contraction OFF so that the product is rounded
// before it is accumulated, exactly as stated.
#include "common.hpp"

namespace jtmoe {
namespace {

constexpr int kMaxK = JTMOE_MAX_TOP_K;

// 8 bf16 values per 16-byte vector
__device__ __forceinline__ void unpack8(const uint4& v, float* f) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

__device__ __forceinline__ uint4 pack8(const float* f) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = f32_to_bf16_bits(f[2 * i]) | (f32_to_bf16_bits(f[2 * i + 1]) << 16);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// bf16, rows a multiple of 8 elements, 16-byte aligned: one wave streams rows
__global__ __launch_bounds__(256) void combine_bf16_vec_kernel(const uint4* __restrict__ packed_y,
                                                               const int32_t* __restrict__ inverse,
                                                               const uint16_t* __restrict__ weights,
                                                               const uint4* __restrict__ shared_y, int tokens, int K,
                                                               int A, int row_vecs, uint4* __restrict__ y) {
#pragma clang fp contract(off)
  const int t = blockIdx.x * blockDim.y + threadIdx.y;
  if (t >= tokens) return;
  int pos[kMaxK];
  float w[kMaxK];
#pragma unroll
  for (int s = 0; s < kMaxK; ++s) {
    if (s < K) {
      pos[s] = inverse[(size_t)t * K + s];
      w[s] = bf16_bits_to_f32(weights[(size_t)t * K + s]);
    }
  }
  for (int v = threadIdx.x; v < row_vecs; v += blockDim.x) {
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int s = 0; s < kMaxK; ++s) {
      if (s < K && pos[s] >= 0 && pos[s] < A) {
        float f[8];
        unpack8(packed_y[(size_t)pos[s] * row_vecs + v], f);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float p = round_to_bf16(f[i] * w[s]);
          acc[i] = acc[i] + p;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = round_to_bf16(acc[i]);
    if (shared_y) {
      float f[8];
      unpack8(shared_y[(size_t)t * row_vecs + v], f);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = acc[i] + f[i];  // rounded by pack8
    }
    y[(size_t)t * row_vecs + v] = pack8(acc);
  }
}

// any dtype / row length, one element per lane
template <typename T>
__global__ __launch_bounds__(256) void combine_generic_kernel(const T* __restrict__ packed_y,
                                                              const int32_t* __restrict__ inverse,
                                                              const T* __restrict__ weights,
                                                              const T* __restrict__ shared_y, int tokens, int K, int A,
                                                              int H, T* __restrict__ y) {
#pragma clang fp contract(off)
  const int t = blockIdx.x * blockDim.y + threadIdx.y;
  if (t >= tokens) return;
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
    if (shared_y) acc = acc + Elem<T>::load(shared_y + (size_t)t * H + h);
    Elem<T>::store(y + (size_t)t * H + h, acc);
  }
}

}  // namespace
}  // namespace jtmoe

using namespace jtmoe;

extern "C" int jtmoe_combine(const void* packed_y, const int32_t* inverse, const void* weights, const void* shared_y,
                             int64_t T, int64_t H, int64_t K, int dtype, void* y, void* stream) {
  clear_error();
  JT_REQUIRE(dtype_ok(dtype), "combine: unknown dtype %d", dtype);
  JT_REQUIRE(T >= 0 && H > 0 && K > 0, "combine: T=%lld H=%lld K=%lld out of range", (long long)T, (long long)H,
             (long long)K);
  if (K > JTMOE_MAX_TOP_K) return fail(JTMOE_EUNSUPPORTED, "combine: K=%lld exceeds %d", (long long)K, JTMOE_MAX_TOP_K);
  JT_REQUIRE(T * K < ((int64_t)1 << 31), "combine: T*K exceeds int32");
  JT_REQUIRE(H * (int64_t)dtype_bytes(dtype) < ((int64_t)1 << 31), "combine: row too long");
  if (T == 0) return JTMOE_OK;
  JT_REQUIRE(packed_y && inverse && weights && y, "combine: null pointer argument");
  hipStream_t s = as_stream(stream);
  const int A = (int)(T * K);
  const bool vec = dtype == JTMOE_BF16 && H % 8 == 0 && aligned16(packed_y) && aligned16(y) &&
                   (shared_y == nullptr || aligned16(shared_y));
  if (vec) {
    const int row_vecs = (int)(H / 8);
    int bx = 64;
    while (bx < 256 && bx * 2 <= row_vecs) bx *= 2;
    dim3 block(bx, 256 / bx);
    const int grid = (int)((T + block.y - 1) / block.y);
    combine_bf16_vec_kernel<<<grid, block, 0, s>>>(static_cast<const uint4*>(packed_y), inverse,
                                                   static_cast<const uint16_t*>(weights),
                                                   static_cast<const uint4*>(shared_y), (int)T, (int)K, A, row_vecs,
                                                   static_cast<uint4*>(y));
  } else {
    dim3 block(64, 4);
    const int grid = (int)((T + block.y - 1) / block.y);
    if (dtype == JTMOE_BF16)
      combine_generic_kernel<bf16_raw><<<grid, block, 0, s>>>(
          static_cast<const bf16_raw*>(packed_y), inverse, static_cast<const bf16_raw*>(weights),
          static_cast<const bf16_raw*>(shared_y), (int)T, (int)K, A, (int)H, static_cast<bf16_raw*>(y));
    else
      combine_generic_kernel<float><<<grid, block, 0, s>>>(static_cast<const float*>(packed_y), inverse,
                                                           static_cast<const float*>(weights),
                                                           static_cast<const float*>(shared_y), (int)T, (int)K, A,
                                                           (int)H, static_cast<float*>(y));
  }
  return check_launch("combine");
}
