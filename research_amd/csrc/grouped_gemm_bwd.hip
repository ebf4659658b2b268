// Grouped GEMMs of the backward pass: data gradients (A @ B^T per group) and weight
// gradients (P^T @ D reduced over the rows of each group).  The reference obtains both from
// jax.lax.ragged_dot by automatic differentiation (moe.py:638-641); here they are two kernels
// of their own, see grouped_gemm_bwd.hpp.
#include "gemm_launch.hpp"
#include "grouped_gemm_bwd.hpp"

#include <algorithm>
#include <mutex>

namespace jtmoe {
namespace {

constexpr int QB = 64, QK = 16;  // tile edge and reduction step of the staged kernels

// ---------------------------------------------------------------------------
// Staged kernels: any dtype, shape and alignment.  64 x 64 output tile, 256 threads, each
// accumulating a 4 x 4 block in fp32 from operands staged through LDS as floats.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gemm_nt_staged_kernel(
    const T* __restrict__ A0, const T* __restrict__ A1, const T* __restrict__ B0, const T* __restrict__ B1,
    T* __restrict__ C, const int32_t* __restrict__ group_sizes, const int32_t* __restrict__ offsets, int E,
    int dense_rows, int Kdim, int N, int ntiles_n, const int32_t* __restrict__ row_map, int row_div, int segs) {
  __shared__ float As[QK][QB + 1];
  __shared__ float Bs[QK][QB + 1];
  __shared__ int a_row_of[QB];
  const int mt = blockIdx.x / ntiles_n;
  const int nt = blockIdx.x - mt * ntiles_n;
  const TileRows tr = find_tile_wave(mt, QB, group_sizes, offsets, E, dense_rows);
  if (tr.rows <= 0) return;
  const int n0 = nt * QB;
  const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
  if (tid < tr.rows) a_row_of[tid] = row_map ? row_map[tr.row0 + tid] / row_div : tr.row0 + tid;
  __syncthreads();
  float acc[4][4] = {};
  for (int s = 0; s < segs; ++s) {
    const T* A = s ? A1 : A0;
    const T* B = (s ? B1 : B0) + (size_t)tr.expert * N * Kdim;
    for (int k0 = 0; k0 < Kdim; k0 += QK) {
      for (int idx = tid; idx < QB * QK; idx += 256) {
        const int r = idx / QK, k = idx - r * QK;
        const int gk = k0 + k;
        As[k][r] = (r < tr.rows && gk < Kdim) ? Elem<T>::load(A + (size_t)a_row_of[r] * Kdim + gk) : 0.0f;
        Bs[k][r] = (n0 + r < N && gk < Kdim) ? Elem<T>::load(B + (size_t)(n0 + r) * Kdim + gk) : 0.0f;
      }
      __syncthreads();
#pragma unroll
      for (int k = 0; k < QK; ++k) {
        float a[4], b[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          a[i] = As[k][ty * 4 + i];
          b[i] = Bs[k][tx * 4 + i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
      }
      __syncthreads();
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (r >= tr.rows) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (col < N) Elem<T>::store(C + (size_t)(tr.row0 + r) * N + col, acc[i][j]);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gemm_tn_staged_kernel(
    const T* __restrict__ P, const T* __restrict__ D, T* __restrict__ C, const int32_t* __restrict__ group_sizes,
    const int32_t* __restrict__ offsets, int dense_rows, int KA, int N, int mtiles_o, int ntiles_o,
    const int32_t* __restrict__ row_map, int row_div, int p_gather, int d_gather) {
  __shared__ float Ps[QK][QB + 1];
  __shared__ float Ds[QK][QB + 1];
  __shared__ int p_row_of[QK], d_row_of[QK];
  const int per_group = mtiles_o * ntiles_o;
  const int e = blockIdx.x / per_group;
  const int in_e = blockIdx.x - e * per_group;
  const int mt = in_e / ntiles_o, nt = in_e - mt * ntiles_o;
  const int m0 = mt * QB, n0 = nt * QB;
  const int row0 = group_sizes ? offsets[e] : 0;
  const int rows = group_sizes ? group_sizes[e] : dense_rows;
  const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
  float acc[4][4] = {};
  for (int r0 = 0; r0 < rows; r0 += QK) {
    if (tid < QK && r0 + tid < rows) {
      const int mapped = (p_gather || d_gather) ? row_map[row0 + r0 + tid] / row_div : 0;
      p_row_of[tid] = p_gather ? mapped : row0 + r0 + tid;
      d_row_of[tid] = d_gather ? mapped : row0 + r0 + tid;
    }
    __syncthreads();
    for (int idx = tid; idx < QK * QB; idx += 256) {
      const int k = idx / QB, c = idx - k * QB;
      const bool live = r0 + k < rows;
      Ps[k][c] = (live && m0 + c < KA) ? Elem<T>::load(P + (size_t)p_row_of[k] * KA + m0 + c) : 0.0f;
      Ds[k][c] = (live && n0 + c < N) ? Elem<T>::load(D + (size_t)d_row_of[k] * N + n0 + c) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < QK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[i] = Ps[k][ty * 4 + i];
        b[i] = Ds[k][tx * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
    }
    __syncthreads();
  }
  T* const Ce = C + (size_t)e * KA * N;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = m0 + ty * 4 + i;
    if (r >= KA) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (col < N) Elem<T>::store(Ce + (size_t)r * N + col, acc[i][j]);
    }
  }
}

inline int64_t max_m_tiles(int64_t rows, int64_t groups, int BM) {
  return (rows + BM - 1) / BM + (groups < rows ? groups : rows);
}

template <typename Kernel>
hipError_t allow_lds(Kernel kernel, size_t bytes) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                             (int)bytes);
}

constexpr int64_t kOperandLimit = (int64_t)1 << 30;  // elements: byte offsets stay below 2^31

}  // namespace

int launch_gemm_nt(int dtype, const void* a0, const void* a1, const void* b0, const void* b1, void* c,
                   const int32_t* group_sizes, const int32_t* offsets, int64_t rows, int64_t Kdim, int64_t N,
                   int64_t E, const int32_t* row_map, int row_div, int64_t a_rows, int segs, hipStream_t stream) {
  if (rows == 0) return JTMOE_OK;
  const bool dense = group_sizes == nullptr;
  const bool fast = dtype == JTMOE_BF16 && Kdim % 64 == 0 && N % 8 == 0 && N * Kdim < kOperandLimit &&
                    (row_map ? a_rows : rows) * Kdim < kOperandLimit && aligned16(a0) && aligned16(b0) &&
                    (segs == 1 || (aligned16(a1) && aligned16(b1))) && aligned16(c);
  if (fast) {
    using Cfg = DgradCfg;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    auto kernel = grouped_gemm_nt_kernel<Cfg>;
    std::call_once(once, [&] { attr_err = allow_lds(kernel, Cfg::SMEM_BYTES); });
    if (attr_err != hipSuccess)
      return fail(JTMOE_ELAUNCH, "grouped gemm (nt): hipFuncSetAttribute: %s", hipGetErrorString(attr_err));
    const int64_t mtiles = dense ? (rows + Cfg::BM - 1) / Cfg::BM : max_m_tiles(rows, E, Cfg::BM);
    const int64_t nt = (N + Cfg::BN - 1) / Cfg::BN;
    const int64_t tiles_grid = gemm_grid(mtiles, nt);
    if (tiles_grid >= ((int64_t)1 << 31)) return fail(JTMOE_EUNSUPPORTED, "grouped gemm (nt): grid too large");
    // persistent workgroups: one per CU, each walking its share of the tiles
    const int64_t grid = tiles_grid > persistent_grid_size() ? persistent_grid_size() : tiles_grid;
    kernel<<<(unsigned)grid, Cfg::NT, Cfg::SMEM_BYTES, stream>>>(
        static_cast<const uint16_t*>(a0), static_cast<const uint16_t*>(a1), static_cast<const uint16_t*>(b0),
        static_cast<const uint16_t*>(b1), static_cast<uint16_t*>(c), group_sizes, offsets, (int)E, (int)rows,
        (int)Kdim, (int)N, (int)mtiles, (int)nt, row_map, row_div, (int)a_rows, segs);
    return JTMOE_OK;
  }
  const int64_t mtiles = dense ? (rows + QB - 1) / QB : max_m_tiles(rows, E, QB);
  const int64_t nt = (N + QB - 1) / QB;
  if (mtiles * nt >= ((int64_t)1 << 31)) return fail(JTMOE_EUNSUPPORTED, "grouped gemm (nt): grid too large");
  if (dtype == JTMOE_BF16)
    gemm_nt_staged_kernel<bf16_raw><<<(unsigned)(mtiles * nt), 256, 0, stream>>>(
        static_cast<const bf16_raw*>(a0), static_cast<const bf16_raw*>(a1), static_cast<const bf16_raw*>(b0),
        static_cast<const bf16_raw*>(b1), static_cast<bf16_raw*>(c), group_sizes, offsets, (int)E, (int)rows,
        (int)Kdim, (int)N, (int)nt, row_map, row_div, segs);
  else
    gemm_nt_staged_kernel<float><<<(unsigned)(mtiles * nt), 256, 0, stream>>>(
        static_cast<const float*>(a0), static_cast<const float*>(a1), static_cast<const float*>(b0),
        static_cast<const float*>(b1), static_cast<float*>(c), group_sizes, offsets, (int)E, (int)rows, (int)Kdim,
        (int)N, (int)nt, row_map, row_div, segs);
  return JTMOE_OK;
}

namespace {

// out[i] = round(sum over s of partial[s][i]), s ascending
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float* __restrict__ partial, int splits,
                                                              size_t n, uint16_t* __restrict__ out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float acc = 0.0f;
  for (int s = 0; s < splits; ++s) acc += partial[(size_t)s * n + i];
  out[i] = (uint16_t)f32_to_bf16_bits(acc);
}

// four elements per thread; the partial sums are read once
typedef float stream_f32x4_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void reduce_partials_vec_kernel(const stream_f32x4_t* __restrict__ partial,
                                                                  int splits, size_t nvec, uint2* __restrict__ out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  stream_f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int s = 0; s < splits; ++s) {
    const stream_f32x4_t v = __builtin_nontemporal_load(&partial[(size_t)s * nvec + i]);
    acc += v;
  }
  out[i] = make_uint2(f32_to_bf16_bits(acc[0]) | (f32_to_bf16_bits(acc[1]) << 16),
                      f32_to_bf16_bits(acc[2]) | (f32_to_bf16_bits(acc[3]) << 16));
}

void launch_reduce_partials(const float* partial, int splits, size_t n, uint16_t* out, hipStream_t stream) {
  if (n % 4 == 0 && aligned16(partial) && (reinterpret_cast<uintptr_t>(out) & 7) == 0) {
    const size_t nvec = n / 4;
    reduce_partials_vec_kernel<<<(unsigned)((nvec + 255) / 256), 256, 0, stream>>>(
        reinterpret_cast<const stream_f32x4_t*>(partial), splits, nvec, reinterpret_cast<uint2*>(out));
  } else {
    reduce_partials_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(partial, splits, n, out);
  }
}

struct SplitPlan {
  int splits;  // 0: do not split
  int chunk;   // rows per run, a multiple of the k step
};

// A one-group reduction whose output tiles cannot occupy the chip is split into runs of rows.
// The number of runs minimises an estimate of the launch in k steps: rounds of (tile, run) pairs over
// the CUs times the steps of a run (plus a fixed cost per pair), plus the reduction of the float32
// partial sums (written and read once per run: about 0.8 steps per million result elements).  A
// split is taken only when it is estimated to save a tenth of the time.
template <typename Cfg>
SplitPlan split_plan(int64_t rows, int64_t KA, int64_t N) {
  const int64_t tiles = ((KA + Cfg::BMO - 1) / Cfg::BMO) * ((N + Cfg::BNO - 1) / Cfg::BNO);
  SplitPlan p{0, 0};
  const int64_t cus = persistent_grid_size();
  if (tiles > cus || rows < 2048) return p;
  constexpr int64_t kStep = 64;  // the estimate counts in steps of 64 rows, whatever the kernel's k step
  static_assert(kStep % Cfg::BK == 0, "a run is a whole number of k steps");
  const double reduce_steps = 0.84e-6 * (double)KA * (double)N * (Cfg::kDual ? 2.0 : 1.0);
  auto cost = [&](int64_t runs) {
    const int64_t chunk = ((rows + runs - 1) / runs + kStep - 1) / kStep * kStep;
    const int64_t real_runs = (rows + chunk - 1) / chunk;
    const int64_t rounds = (tiles * real_runs + cus - 1) / cus;
    return (double)rounds * (double)(chunk / kStep + 3) + (real_runs > 1 ? reduce_steps * (double)real_runs : 0.0);
  };
  const int64_t max_runs = std::min<int64_t>(64, rows / 256);
  int64_t best = 1;
  double best_cost = cost(1);
  for (int64_t runs = 2; runs <= max_runs; ++runs) {
    const double c = cost(runs);
    if (c < best_cost) {
      best_cost = c;
      best = runs;
    }
  }
  if (best < 2 || best_cost > 0.9 * cost(1)) return p;
  const int64_t chunk = ((rows + best - 1) / best + kStep - 1) / kStep * kStep;
  p.splits = (int)((rows + chunk - 1) / chunk);
  p.chunk = (int)chunk;
  return p;
}

template <typename Cfg>
int launch_tn_fast(const void* p, const void* d0, const void* d1, void* c0, void* c1, const int32_t* group_sizes,
                   const int32_t* offsets, int64_t rows, int64_t KA, int64_t N, int64_t E, const int32_t* row_map,
                   int row_div, bool p_gather, bool d_gather, int64_t gathered_rows, hipStream_t stream,
                   void* split_ws) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto kernel = grouped_gemm_tn_kernel<Cfg>;
  std::call_once(once, [&] { attr_err = allow_lds(kernel, Cfg::SMEM_BYTES); });
  if (attr_err != hipSuccess)
    return fail(JTMOE_ELAUNCH, "grouped gemm (tn): hipFuncSetAttribute: %s", hipGetErrorString(attr_err));
  const int64_t mt = (KA + Cfg::BMO - 1) / Cfg::BMO, nt = (N + Cfg::BNO - 1) / Cfg::BNO;
  SplitPlan plan{0, 0};
  if (split_ws != nullptr && group_sizes == nullptr && !p_gather && !d_gather) plan = split_plan<Cfg>(rows, KA, N);
  if (plan.splits > 0) {
    const size_t n = (size_t)KA * N;
    float* part0 = static_cast<float*>(split_ws);
    float* part1 = part0 + (size_t)plan.splits * n;
    const int64_t tiles_grid = gemm_grid(plan.splits * mt, nt);
    const int64_t grid = tiles_grid > persistent_grid_size() ? persistent_grid_size() : tiles_grid;
    kernel<<<(unsigned)grid, Cfg::NT, Cfg::SMEM_BYTES, stream>>>(
        static_cast<const uint16_t*>(p), static_cast<const uint16_t*>(d0), static_cast<const uint16_t*>(d1),
        reinterpret_cast<uint16_t*>(part0), reinterpret_cast<uint16_t*>(part1), nullptr, nullptr, plan.splits,
        (int)rows, (int)KA, (int)N, (int)mt, (int)nt, nullptr, 1, 0, 0, 0, plan.chunk);
    launch_reduce_partials(part0, plan.splits, n, static_cast<uint16_t*>(c0), stream);
    if (Cfg::kDual) launch_reduce_partials(part1, plan.splits, n, static_cast<uint16_t*>(c1), stream);
    return JTMOE_OK;
  }
  const int64_t tiles_grid = gemm_grid(E * mt, nt);
  if (tiles_grid >= ((int64_t)1 << 31)) return fail(JTMOE_EUNSUPPORTED, "grouped gemm (tn): grid too large");
  // persistent workgroups: one per CU, each walking its share of the (group, tile) pairs
  const int64_t grid = tiles_grid > persistent_grid_size() ? persistent_grid_size() : tiles_grid;
  kernel<<<(unsigned)grid, Cfg::NT, Cfg::SMEM_BYTES, stream>>>(
      static_cast<const uint16_t*>(p), static_cast<const uint16_t*>(d0), static_cast<const uint16_t*>(d1),
      static_cast<uint16_t*>(c0), static_cast<uint16_t*>(c1), group_sizes, offsets, (int)E, (int)rows, (int)KA,
      (int)N, (int)mt, (int)nt, row_map, row_div, p_gather ? 1 : 0, d_gather ? 1 : 0, (int)gathered_rows, 0);
  return JTMOE_OK;
}
}  // namespace

int launch_gemm_tn(int dtype, const void* p, const void* d0, const void* d1, void* c0, void* c1,
                   const int32_t* group_sizes, const int32_t* offsets, int64_t rows, int64_t KA, int64_t N, int64_t E,
                   const int32_t* row_map, int row_div, bool p_gather, bool d_gather, int64_t gathered_rows,
                   hipStream_t stream, void* split_ws) {
  const bool dual = d1 != nullptr;
  const int64_t p_rows = p_gather ? gathered_rows : rows, d_rows = d_gather ? gathered_rows : rows;
  const bool fast = dtype == JTMOE_BF16 && KA % 8 == 0 && N % 8 == 0 && p_rows * KA < kOperandLimit &&
                    d_rows * N < kOperandLimit && aligned16(p) && aligned16(d0) && aligned16(c0) &&
                    (!dual || (aligned16(d1) && aligned16(c1)));
  if (fast && (p_gather || d_gather)) {
    if (dual)
      return launch_tn_fast<WgradDualGatherCfg>(p, d0, d1, c0, c1, group_sizes, offsets, rows, KA, N, E, row_map,
                                                row_div, p_gather, d_gather, gathered_rows, stream, split_ws);
    return launch_tn_fast<WgradGatherCfg>(p, d0, nullptr, c0, nullptr, group_sizes, offsets, rows, KA, N, E, row_map,
                                          row_div, p_gather, d_gather, gathered_rows, stream, split_ws);
  }
  if (fast) {
    if (dual)
      return launch_tn_fast<WgradDualCfg>(p, d0, d1, c0, c1, group_sizes, offsets, rows, KA, N, E, nullptr, 1, false,
                                          false, 0, stream, split_ws);
    return launch_tn_fast<WgradCfg>(p, d0, nullptr, c0, nullptr, group_sizes, offsets, rows, KA, N, E, nullptr, 1,
                                    false, false, 0, stream, split_ws);
  }
  const int64_t mt = (KA + QB - 1) / QB, nt = (N + QB - 1) / QB;
  if (E * mt * nt >= ((int64_t)1 << 31)) return fail(JTMOE_EUNSUPPORTED, "grouped gemm (tn): grid too large");
  for (int i = 0; i < (dual ? 2 : 1); ++i) {
    const void* d = i ? d1 : d0;
    void* c = i ? c1 : c0;
    if (dtype == JTMOE_BF16)
      gemm_tn_staged_kernel<bf16_raw><<<(unsigned)(E * mt * nt), 256, 0, stream>>>(
          static_cast<const bf16_raw*>(p), static_cast<const bf16_raw*>(d), static_cast<bf16_raw*>(c), group_sizes,
          offsets, (int)rows, (int)KA, (int)N, (int)mt, (int)nt, row_map, row_div, p_gather ? 1 : 0, d_gather ? 1 : 0);
    else
      gemm_tn_staged_kernel<float><<<(unsigned)(E * mt * nt), 256, 0, stream>>>(
          static_cast<const float*>(p), static_cast<const float*>(d), static_cast<float*>(c), group_sizes, offsets,
          (int)rows, (int)KA, (int)N, (int)mt, (int)nt, row_map, row_div, p_gather ? 1 : 0, d_gather ? 1 : 0);
  }
  return JTMOE_OK;
}

size_t gemm_tn_split_bytes(int dtype, int64_t rows, int64_t KA, int64_t N, bool dual) {
  if (dtype != JTMOE_BF16 || KA % 8 != 0 || N % 8 != 0) return 0;
  const SplitPlan plan = dual ? split_plan<WgradDualCfg>(rows, KA, N) : split_plan<WgradCfg>(rows, KA, N);
  if (plan.splits == 0) return 0;
  return align_up((size_t)plan.splits * KA * N * sizeof(float) * (dual ? 2 : 1), 256);
}

}  // namespace jtmoe
