// RMSNorm over the last axis, the normalisation the decoder block puts in front of the MoE
// layer (ffn_pre_norm) and behind it (ffn_post_norm): blocks.py:224-230 of the reference,
// modules built by build_rms_norm (models/components/norm.py:12-31) = flax nnx.RMSNorm with
// a float32 scale, and the reference's own forward-only kernel boundary
// (kernels/rmsnorm.py:14-21, kernels/cuda/rmsnorm/rmsnorm_ffi.cu).
//
//   var = mean(f32(x)^2)        (fp32)
//   mul = rsqrt(var + eps) * scale                      (fp32, one factor per column)
//   y   = round_dtype(f32(x) * mul)
//
// 1/sqrt is computed as a correctly rounded square root followed by a correctly rounded
// division, so that a NumPy float32 restatement agrees bit for bit given the same sum.
#include "common.hpp"

namespace jtmoe {
namespace {

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d);
  return v;
}

// One wave per row; any row length.  bf16 rows of a multiple of 8 elements with 16-byte
// alignment take the vector path (kVec).
template <typename T, bool kVec>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const T* __restrict__ x, const float* __restrict__ scale,
                                                      int rows, int H, float eps, T* __restrict__ y) {
#pragma clang fp contract(off)
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int lane = threadIdx.x & 63;
  const T* xr = x + (size_t)r * H;
  T* yr = y + (size_t)r * H;
  float ss = 0.0f;
  if (kVec) {
    const uint4* xv = reinterpret_cast<const uint4*>(xr);
    for (int v = lane; v < H / 8; v += 64) {
      const uint4 q = xv[v];
      const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float lo = bf16_bits_to_f32(w[i] & 0xffffu), hi = bf16_bits_to_f32(w[i] >> 16);
        ss += lo * lo;
        ss += hi * hi;
      }
    }
  } else {
    for (int i = lane; i < H; i += 64) {
      const float v = Elem<T>::load(xr + i);
      ss += v * v;
    }
  }
  ss = wave_sum_f32(ss);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  if (kVec) {
    const uint4* xv = reinterpret_cast<const uint4*>(xr);
    uint4* yv = reinterpret_cast<uint4*>(yr);
    for (int v = lane; v < H / 8; v += 64) {
      const uint4 q = xv[v];
      const uint32_t w[4] = {q.x, q.y, q.z, q.w};
      uint32_t o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float lo = bf16_bits_to_f32(w[i] & 0xffffu) * (inv * scale[v * 8 + 2 * i]);
        const float hi = bf16_bits_to_f32(w[i] >> 16) * (inv * scale[v * 8 + 2 * i + 1]);
        o[i] = f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
      }
      yv[v] = make_uint4(o[0], o[1], o[2], o[3]);
    }
  } else {
    for (int i = lane; i < H; i += 64) Elem<T>::store(yr + i, Elem<T>::load(xr + i) * (inv * scale[i]));
  }
}

}  // namespace
}  // namespace jtmoe

using namespace jtmoe;

extern "C" int jtmoe_rmsnorm(const void* x, const float* scale, int64_t T, int64_t H, double eps, int dtype, void* y,
                             void* stream) {
  clear_error();
  JT_REQUIRE(dtype_ok(dtype), "rmsnorm: unknown dtype %d", dtype);
  JT_REQUIRE(T >= 0 && H > 0 && H < ((int64_t)1 << 24) && T < ((int64_t)1 << 31), "rmsnorm: T=%lld H=%lld out of range",
             (long long)T, (long long)H);
  JT_REQUIRE(eps >= 0.0, "rmsnorm: eps must not be negative");
  if (T == 0) return JTMOE_OK;
  JT_REQUIRE(x && scale && y, "rmsnorm: null pointer argument");
  hipStream_t s = as_stream(stream);
  const unsigned grid = (unsigned)((T + 3) / 4);
  if (dtype == JTMOE_BF16) {
    if (H % 8 == 0 && aligned16(x) && aligned16(y))
      rmsnorm_kernel<bf16_raw, true><<<grid, 256, 0, s>>>(static_cast<const bf16_raw*>(x), scale, (int)T, (int)H,
                                                          (float)eps, static_cast<bf16_raw*>(y));
    else
      rmsnorm_kernel<bf16_raw, false><<<grid, 256, 0, s>>>(static_cast<const bf16_raw*>(x), scale, (int)T, (int)H,
                                                           (float)eps, static_cast<bf16_raw*>(y));
  } else {
    rmsnorm_kernel<float, false><<<grid, 256, 0, s>>>(static_cast<const float*>(x), scale, (int)T, (int)H, (float)eps,
                                                      static_cast<float*>(y));
  }
  return check_launch("rmsnorm");
}
