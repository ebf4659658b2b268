// Grouped SwiGLU expert FFN: two grouped GEMM launches over variable-size,
// expert-contiguous row groups.
//
// Follows the three jax.lax.ragged_dot calls of the reference and the SwiGLU
// between them (moe.py:638-641), and SharedSwiGLU.__call__ (moe.py:361-364) as
// the one-group dense case:
//   launch 1 (dual):  act = round(silu(round(X Wg[e])) * round(X Wu[e]))   [rows, I]
//   launch 2:         Y   = round(act Wd[e])                                [rows, H]
// `round` is the rounding to the compute dtype (identity for fp32); products
// are accumulated in fp32 on the matrix cores (v_mfma_f32_32x32x16_bf16 for
// bf16, v_mfma_f32_32x32x2_f32 for fp32).
#include "common.hpp"
#include "grouped_gemm_dma.hpp"
#include "grouped_gemm_stream.hpp"

#include <mutex>

namespace jtmoe {
namespace {

// ---------------------------------------------------------------------------
// Generic kernel: any shape, any alignment, both dtypes.  64x64x32 tiles, four
// waves (2x2), each owning one 32x32 accumulator tile (two when kDual).
// Operands are staged element by element through LDS with bounds checks; B is
// transposed on the way in so that both MFMA operands are k-contiguous.
// ---------------------------------------------------------------------------
constexpr int GBM = 64, GBN = 64, GBK = 32;
constexpr int GPAD = 8;  // elements; keeps 16-byte alignment of bf16 rows

template <typename T>
__device__ __forceinline__ void mfma_tile(const T* __restrict__ a_row, const T* __restrict__ b_row, int khalf,
                                          f32x16_t& acc);

// a_row / b_row point at the k = 0 element of this lane's A row / B column in LDS
template <>
__device__ __forceinline__ void mfma_tile<bf16_raw>(const bf16_raw* __restrict__ a_row,
                                                    const bf16_raw* __restrict__ b_row, int khalf, f32x16_t& acc) {
#pragma unroll
  for (int kk = 0; kk < GBK / 16; ++kk) {
    const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(a_row + kk * 16 + khalf * 8);
    const bf16x8_t b = *reinterpret_cast<const bf16x8_t*>(b_row + kk * 16 + khalf * 8);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
  }
}

template <>
__device__ __forceinline__ void mfma_tile<float>(const float* __restrict__ a_row, const float* __restrict__ b_row,
                                                 int khalf, f32x16_t& acc) {
#pragma unroll
  for (int kk = 0; kk < GBK / 2; ++kk) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_row[kk * 2 + khalf], b_row[kk * 2 + khalf], acc, 0, 0, 0);
  }
}

template <typename T, bool kDual>
__global__ __launch_bounds__(256) void grouped_gemm_generic_kernel(
    const T* __restrict__ A, const T* __restrict__ B0, const T* __restrict__ B1, T* __restrict__ C,
    const int32_t* __restrict__ group_sizes, const int32_t* __restrict__ offsets, int E, int dense_rows, int Kdim,
    int N, int ntiles_n, const int32_t* __restrict__ row_map, int row_div, T* __restrict__ save0,
    T* __restrict__ save1) {
  __shared__ __align__(16) T As[GBM][GBK + GPAD];
  __shared__ int a_row_of[GBM];  // row of A behind tile row r (through the row map, if there is one)
  __shared__ __align__(16) T Bs0[GBN][GBK + GPAD];
  __shared__ __align__(16) T Bs1[kDual ? GBN : 1][GBK + GPAD];

  const int mt = blockIdx.x / ntiles_n;
  const int nt = blockIdx.x - mt * ntiles_n;
  const TileRows tr = find_tile_wave(mt, GBM, group_sizes, offsets, E, dense_rows);
  if (tr.rows <= 0) return;
  const int n0 = nt * GBN;
  const size_t wofs = (size_t)tr.expert * Kdim * N;
  const T* Bg0 = B0 + wofs;
  const T* Bg1 = kDual ? B1 + wofs : nullptr;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int frag_row = lane & 31, khalf = lane >> 5;

  f32x16_t acc0, acc1;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    acc0[i] = 0.0f;
    acc1[i] = 0.0f;
  }

  T zero;
  __builtin_memset(&zero, 0, sizeof(T));
  if (tid < GBM && tid < tr.rows) a_row_of[tid] = row_map ? row_map[tr.row0 + tid] / row_div : tr.row0 + tid;
  __syncthreads();

  for (int k0 = 0; k0 < Kdim; k0 += GBK) {
    for (int idx = tid; idx < GBM * GBK; idx += 256) {
      const int r = idx / GBK, c = idx - r * GBK;
      const int gk = k0 + c;
      T v = zero;
      if (r < tr.rows && gk < Kdim) v = A[(size_t)a_row_of[r] * Kdim + gk];
      As[r][c] = v;
    }
    for (int idx = tid; idx < GBK * GBN; idx += 256) {
      const int k = idx / GBN, n = idx - k * GBN;
      const int gk = k0 + k, gn = n0 + n;
      const bool ok = gk < Kdim && gn < N;
      Bs0[n][k] = ok ? Bg0[(size_t)gk * N + gn] : zero;
      if (kDual) Bs1[n][k] = ok ? Bg1[(size_t)gk * N + gn] : zero;
    }
    __syncthreads();
    const T* a_row = &As[wm * 32 + frag_row][0];
    mfma_tile<T>(a_row, &Bs0[wn * 32 + frag_row][0], khalf, acc0);
    if (kDual) mfma_tile<T>(a_row, &Bs1[wn * 32 + frag_row][0], khalf, acc1);
    __syncthreads();
  }

  // 32x32 accumulator layout: value i of lane l is row 8*(i/4) + 4*(l/32) + i%4, column l%32
  const int col = n0 + wn * 32 + (lane & 31);
  if (col < N) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int r = wm * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
      if (r < tr.rows) {
        float v;
        if (kDual) {
          const float g = Elem<T>::round(acc0[i]);
          const float u = Elem<T>::round(acc1[i]);
          v = silu_fast(g) * u;
          if (save0) {
            Elem<T>::store(save0 + (size_t)(tr.row0 + r) * N + col, g);
            Elem<T>::store(save1 + (size_t)(tr.row0 + r) * N + col, u);
          }
        } else {
          v = acc0[i];
        }
        Elem<T>::store(C + (size_t)(tr.row0 + r) * N + col, v);
      }
    }
  }
}

// upper bound on the number of m-tiles when the group sizes live on the device
inline int64_t max_m_tiles(int64_t rows, int64_t groups, int BM) {
  return (rows + BM - 1) / BM + (groups < rows ? groups : rows);
}

template <typename T, bool kDual>
int launch_generic(const void* a, const void* b0, const void* b1, void* c, const int32_t* group_sizes,
                   const int32_t* offsets, int64_t rows, int64_t Kdim, int64_t N, int64_t E, hipStream_t stream,
                   const int32_t* row_map = nullptr, int row_div = 1, void* save0 = nullptr, void* save1 = nullptr) {
  const bool dense = group_sizes == nullptr;
  const int64_t mtiles = dense ? (rows + GBM - 1) / GBM : max_m_tiles(rows, E, GBM);
  const int64_t nt = (N + GBN - 1) / GBN;
  if (mtiles * nt >= ((int64_t)1 << 31)) return fail(JTMOE_EUNSUPPORTED, "grouped gemm: grid too large");
  grouped_gemm_generic_kernel<T, kDual><<<(unsigned)(mtiles * nt), 256, 0, stream>>>(
      static_cast<const T*>(a), static_cast<const T*>(b0), static_cast<const T*>(b1), static_cast<T*>(c), group_sizes,
      offsets, (int)E, (int)rows, (int)Kdim, (int)N, (int)nt, row_map, row_div, static_cast<T*>(save0),
      static_cast<T*>(save1));
  return JTMOE_OK;
}

template <typename Cfg>
int launch_fast(const void* a, const void* b0, const void* b1, void* c, const int32_t* group_sizes,
                const int32_t* offsets, int64_t rows, int64_t Kdim, int64_t N, int64_t E, hipStream_t stream,
                const int32_t* row_map = nullptr, int row_div = 1, int64_t a_rows = 0, void* save0 = nullptr,
                void* save1 = nullptr, int64_t uniform_rows = 0, int64_t a_group_rows = 0) {
  // the 256-row configurations run as persistent workgroups (see persistent_schedule), the others one
  // tile per workgroup
  constexpr bool kPersistent = Cfg::BM == 256 && Cfg::NSTAGE == 2 && Cfg::BK == 64;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto kernel = [] {
    if constexpr (kPersistent)
      return &grouped_gemm_dma_persistent_kernel<Cfg>;
    else
      return &grouped_gemm_dma_kernel<Cfg>;
  }();
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)Cfg::SMEM_BYTES);
  });
  if (attr_err != hipSuccess)
    return fail(JTMOE_ELAUNCH, "grouped gemm: kernel set-up: %s", hipGetErrorString(attr_err));
  const bool dense = group_sizes == nullptr;
  const int64_t mtiles = uniform_rows > 0 ? E * ((uniform_rows + Cfg::BM - 1) / Cfg::BM)
                         : dense          ? (rows + Cfg::BM - 1) / Cfg::BM
                                          : max_m_tiles(rows, E, Cfg::BM);
  const int64_t nt = (N + Cfg::BN - 1) / Cfg::BN;
  const int64_t tiles_grid = gemm_grid(mtiles, nt);
  if (tiles_grid >= ((int64_t)1 << 31)) return fail(JTMOE_EUNSUPPORTED, "grouped gemm: grid too large");
  if constexpr (kPersistent) {
    if (uniform_rows > 0 || a_group_rows > 0)
      return fail(JTMOE_EUNSUPPORTED, "grouped gemm: the decode forms run one tile per workgroup");
    const PersistentSchedule ps = persistent_schedule(tiles_grid, persistent_grid_size(), kTilesPerWorkgroup<Cfg>);
    kernel<<<(unsigned)ps.grid, Cfg::NT, Cfg::SMEM_BYTES, stream>>>(
        static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(b0), static_cast<const uint16_t*>(b1),
        static_cast<uint16_t*>(c), group_sizes, offsets, (int)E, (int)rows, (int)Kdim, (int)N, (int)mtiles, (int)nt,
        row_map, row_div, (int)a_rows, static_cast<uint16_t*>(save0), static_cast<uint16_t*>(save1), ps.window,
        ps.chunk);
  } else {
    kernel<<<(unsigned)tiles_grid, Cfg::NT, Cfg::SMEM_BYTES, stream>>>(
        static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(b0), static_cast<const uint16_t*>(b1),
        static_cast<uint16_t*>(c), group_sizes, offsets, (int)E, (int)rows, (int)Kdim, (int)N, (int)mtiles, (int)nt,
        row_map, row_div, (int)a_rows, static_cast<uint16_t*>(save0), static_cast<uint16_t*>(save1), (int)uniform_rows,
        (int)a_group_rows);
  }
  return JTMOE_OK;
}


// The stream kernel (grouped_gemm_stream.hpp) for the gate/up launch of the 256-row configurations: the
// same tiles as one software pipeline through all tiles of a workgroup, results written straight from
// the accumulators.  Its envelope is narrower than launch_fast's (see stream_ok).
template <typename Cfg>
int launch_stream(const void* a, const void* b0, const void* b1, void* c, const int32_t* group_sizes,
                  const int32_t* offsets, int64_t rows, int64_t Kdim, int64_t N, int64_t E, hipStream_t stream,
                  const int32_t* row_map, int row_div, int64_t a_rows, void* save0, void* save1) {
  using L = StreamLayout<Cfg>;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto kernel = &grouped_gemm_stream_kernel<Cfg>;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)L::kSmemBytes);
  });
  if (attr_err != hipSuccess)
    return fail(JTMOE_ELAUNCH, "grouped gemm: kernel set-up: %s", hipGetErrorString(attr_err));
  const bool dense = group_sizes == nullptr;
  const int64_t mtiles = dense ? (rows + Cfg::BM - 1) / Cfg::BM : max_m_tiles(rows, E, Cfg::BM);
  const int64_t nt = (N + Cfg::BN - 1) / Cfg::BN;
  const int64_t tiles_grid = gemm_grid(mtiles, nt);
  if (tiles_grid >= ((int64_t)1 << 31)) return fail(JTMOE_EUNSUPPORTED, "grouped gemm: grid too large");
  const PersistentSchedule ps = persistent_schedule(tiles_grid, persistent_grid_size(), kTilesPerWorkgroup<Cfg>);
  kernel<<<(unsigned)ps.grid, Cfg::NT, L::kSmemBytes, stream>>>(
      static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(b0), static_cast<const uint16_t*>(b1),
      static_cast<uint16_t*>(c), group_sizes, offsets, (int)E, (int)rows, (int)Kdim, (int)N, (int)mtiles, (int)nt,
      row_map, row_div, (int)a_rows, static_cast<uint16_t*>(save0), static_cast<uint16_t*>(save1), ps.window, ps.chunk);
  return JTMOE_OK;
}

// what the stream kernel needs beyond fast_ok: enough k steps to fill its pipeline, a result of at most
// 0x7ffe0000 bytes (32-bit store offsets; the kernel drops a store by giving it the offset 0x7fff0000,
// which must lie past the end of every admitted result) and, with a row map, fewer than 2^27 rows and a
// divisor of at most 32
template <typename Cfg>
inline bool stream_ok(int64_t rows, int64_t Kdim, int64_t N, const int32_t* row_map, int row_div) {
  return Kdim % Cfg::BK == 0 && Kdim / Cfg::BK >= 2 * Cfg::NSTAGE && rows * N * 2 <= (int64_t)0x7ffe0000 &&
         (row_map == nullptr || (rows < ((int64_t)1 << 27) && row_div >= 1 && row_div <= 32));
}

// Mean rows per group below which the 64-row tiles are used.
constexpr int64_t kSmallGroupRows = 128;
inline bool small_groups(int64_t rows, int64_t E) { return rows < kSmallGroupRows * E; }
// Mean rows per group up to which nearly every group is a single tile tall, so that no workgroup
// reads an expert matrix after another has: its loads are then marked non-temporal.
constexpr int64_t kTinyGroupRows = 32;
inline bool tiny_groups(int64_t rows, int64_t E) { return rows <= kTinyGroupRows * E; }

inline bool fast_ok(const void* a, const void* b0, const void* b1, const void* c, int64_t Kdim, int64_t N) {
  return Kdim % 64 == 0 && N % 8 == 0 && Kdim * N < ((int64_t)1 << 30) && aligned16(a) && aligned16(b0) && (b1 == nullptr || aligned16(b1)) &&
         aligned16(c);
}

template <typename T>
int launch_pair(const void* x, const void* gate, const void* up, const void* down, const int32_t* group_sizes,
                const int32_t* offsets, int64_t rows, int64_t H, int64_t I, int64_t E, void* act, void* y,
                hipStream_t stream, int first_stage, const int32_t* row_map = nullptr, int row_div = 1,
                int64_t x_rows = 0, void* save_gate = nullptr, void* save_up = nullptr) {
  if (rows == 0) return JTMOE_OK;
  int rc;
  const bool small = small_groups(rows, E), tiny = tiny_groups(rows, E);
  const bool gather_ok = row_map == nullptr || x_rows * H < ((int64_t)1 << 30);
  const bool saves_ok = save_gate == nullptr || (aligned16(save_gate) && aligned16(save_up));
  if (Elem<T>::is_bf16 && fast_ok(x, gate, up, act, H, I) && gather_ok && saves_ok)
    rc = tiny    ? launch_fast<GateUpTinyCfg>(x, gate, up, act, group_sizes, offsets, rows, H, I, E, stream, row_map,
                                              row_div, x_rows, save_gate, save_up)
         : small ? launch_fast<GateUpSmallCfg>(x, gate, up, act, group_sizes, offsets, rows, H, I, E, stream, row_map,
                                               row_div, x_rows, save_gate, save_up)
         : stream_ok<GateUpStreamCfg>(rows, H, I, row_map, row_div)
             ? launch_stream<GateUpStreamCfg>(x, gate, up, act, group_sizes, offsets, rows, H, I, E, stream, row_map,
                                              row_div, x_rows, save_gate, save_up)
             : launch_fast<GateUpCfg>(x, gate, up, act, group_sizes, offsets, rows, H, I, E, stream, row_map,
                                      row_div, x_rows, save_gate, save_up);
  else
    rc = launch_generic<T, true>(x, gate, up, act, group_sizes, offsets, rows, H, I, E, stream, row_map, row_div,
                                 save_gate, save_up);
  if (rc) return rc;
  stage_mark(first_stage, stream);
  if (Elem<T>::is_bf16 && fast_ok(act, down, nullptr, y, I, H))
    rc = tiny    ? launch_fast<DownTinyCfg>(act, down, nullptr, y, group_sizes, offsets, rows, I, H, E, stream)
         : small ? launch_fast<DownSmallCfg>(act, down, nullptr, y, group_sizes, offsets, rows, I, H, E, stream)
                 : launch_fast<DownCfg>(act, down, nullptr, y, group_sizes, offsets, rows, I, H, E, stream);
  else
    rc = launch_generic<T, false>(act, down, nullptr, y, group_sizes, offsets, rows, I, H, E, stream);
  if (rc) return rc;
  stage_mark(first_stage + 1, stream);
  return check_launch("grouped gemm");
}

int validate_gemm(const char* what, int64_t rows, int64_t H, int64_t I, int64_t E, int dtype) {
  JT_REQUIRE(dtype_ok(dtype), "%s: unknown dtype %d", what, dtype);
  JT_REQUIRE(rows >= 0 && rows < ((int64_t)1 << 31), "%s: row count %lld out of range", what, (long long)rows);
  JT_REQUIRE(H > 0 && I > 0 && E > 0, "%s: H=%lld I=%lld E=%lld out of range", what, (long long)H, (long long)I,
             (long long)E);
  JT_REQUIRE(H < ((int64_t)1 << 24) && I < ((int64_t)1 << 24), "%s: H or I too large", what);
  return JTMOE_OK;
}

}  // namespace

// ---- the down launch of the layer's decode path (declared in common.hpp) ----
int launch_down_from_all_tokens(const void* act_full, const void* down, const int32_t* group_sizes,
                                const int32_t* offsets, const int32_t* source_order, int64_t T, int64_t K, int64_t H,
                                int64_t I, int64_t E, void* packed_y, hipStream_t stream) {
  if (!fast_ok(act_full, down, nullptr, packed_y, I, H))
    return fail(JTMOE_EINVAL, "moe_forward: operands must be 16-byte aligned");
  return launch_fast<DownTinyCfg>(act_full, down, nullptr, packed_y, group_sizes, offsets, T * K, I, H, E, stream,
                                  source_order, (int)K, T, nullptr, nullptr, 0, /*a_group_rows=*/T);
}

}  // namespace jtmoe

using namespace jtmoe;

extern "C" int jtmoe_grouped_swiglu(const void* packed_x, const void* gate, const void* up, const void* down,
                                    const int32_t* group_sizes, const int32_t* offsets, int64_t A, int64_t H,
                                    int64_t I, int64_t E, int dtype, void* act, void* packed_y, void* stream) {
  clear_error();
  int rc = validate_gemm("grouped_swiglu", A, H, I, E, dtype);
  if (rc) return rc;
  if (E > JTMOE_MAX_EXPERTS) return fail(JTMOE_EUNSUPPORTED, "grouped_swiglu: E=%lld exceeds %d", (long long)E, JTMOE_MAX_EXPERTS);
  if (A == 0) return JTMOE_OK;
  JT_REQUIRE(packed_x && gate && up && down && group_sizes && offsets && act && packed_y,
             "grouped_swiglu: null pointer argument");
  hipStream_t s = as_stream(stream);
  if (dtype == JTMOE_BF16)
    return launch_pair<bf16_raw>(packed_x, gate, up, down, group_sizes, offsets, A, H, I, E, act, packed_y, s, kStageGateUp);
  return launch_pair<float>(packed_x, gate, up, down, group_sizes, offsets, A, H, I, E, act, packed_y, s, kStageGateUp);
}

extern "C" int jtmoe_shared_swiglu(const void* x, const void* gate, const void* up, const void* down, int64_t T,
                                   int64_t H, int64_t Is, int dtype, void* act, void* shared_y, void* stream) {
  clear_error();
  int rc = validate_gemm("shared_swiglu", T, H, Is, 1, dtype);
  if (rc) return rc;
  if (T == 0) return JTMOE_OK;
  JT_REQUIRE(x && gate && up && down && act && shared_y, "shared_swiglu: null pointer argument");
  hipStream_t s = as_stream(stream);
  if (dtype == JTMOE_BF16)
    return launch_pair<bf16_raw>(x, gate, up, down, nullptr, nullptr, T, H, Is, 1, act, shared_y, s, kStageSharedGateUp);
  return launch_pair<float>(x, gate, up, down, nullptr, nullptr, T, H, Is, 1, act, shared_y, s, kStageSharedGateUp);
}

extern "C" int jtmoe_grouped_swiglu_gather_supported(int64_t T, int64_t H, int64_t I, int dtype) {
  return dtype == JTMOE_BF16 && H % 64 == 0 && I % 64 == 0 && H * I < ((int64_t)1 << 30) &&
         T * H < ((int64_t)1 << 29);
}

extern "C" int jtmoe_grouped_swiglu_gather(const void* x, const int32_t* source_order, const void* gate,
                                           const void* up, const void* down, const int32_t* group_sizes,
                                           const int32_t* offsets, int64_t T, int64_t K, int64_t H, int64_t I,
                                           int64_t E, int dtype, void* act, void* packed_y, void* stream) {
  clear_error();
  JT_REQUIRE(T >= 0 && K > 0 && T * K < ((int64_t)1 << 31), "grouped_swiglu_gather: T=%lld K=%lld out of range",
             (long long)T, (long long)K);
  const int64_t A = T * K;
  int rc = validate_gemm("grouped_swiglu_gather", A, H, I, E, dtype);
  if (rc) return rc;
  if (E > JTMOE_MAX_EXPERTS)
    return fail(JTMOE_EUNSUPPORTED, "grouped_swiglu_gather: E=%lld exceeds %d", (long long)E, JTMOE_MAX_EXPERTS);
  if (A == 0) return JTMOE_OK;
  JT_REQUIRE(x && source_order && gate && up && down && group_sizes && offsets && act && packed_y,
             "grouped_swiglu_gather: null pointer argument");
  if (!jtmoe_grouped_swiglu_gather_supported(T, H, I, dtype) || !aligned16(x))
    return fail(JTMOE_EUNSUPPORTED,
                "grouped_swiglu_gather: needs bf16, H and I multiples of 64 and 16-byte aligned rows "
                "(use jtmoe_dispatch + jtmoe_grouped_swiglu otherwise)");
  return launch_pair<bf16_raw>(x, gate, up, down, group_sizes, offsets, A, H, I, E, act, packed_y, as_stream(stream),
                               kStageGateUp, source_order, (int)K, T);
}

// Forward pass that keeps what the backward pass needs: the two rounded products
// gate_pre = round(X Wg[e]) and up_pre = round(X Wu[e]) are stored next to act and packed_y.
// With source_order the rows of x are fetched through the permutation (packed row j is token
// source_order[j] / K); without it x is already packed and has T rows.
extern "C" int jtmoe_grouped_swiglu_train(const void* x, const int32_t* source_order, const void* gate, const void* up,
                                          const void* down, const int32_t* group_sizes, const int32_t* offsets,
                                          int64_t T, int64_t K, int64_t H, int64_t I, int64_t E, int dtype,
                                          void* gate_pre, void* up_pre, void* act, void* packed_y, void* stream) {
  clear_error();
  JT_REQUIRE(T >= 0 && K > 0 && T * K < ((int64_t)1 << 31), "grouped_swiglu_train: T=%lld K=%lld out of range",
             (long long)T, (long long)K);
  const int64_t A = source_order ? T * K : T;
  int rc = validate_gemm("grouped_swiglu_train", A, H, I, E, dtype);
  if (rc) return rc;
  if (E > JTMOE_MAX_EXPERTS)
    return fail(JTMOE_EUNSUPPORTED, "grouped_swiglu_train: E=%lld exceeds %d", (long long)E, JTMOE_MAX_EXPERTS);
  if (A == 0) return JTMOE_OK;
  JT_REQUIRE(x && gate && up && down && group_sizes && offsets && gate_pre && up_pre && act && packed_y,
             "grouped_swiglu_train: null pointer argument");
  hipStream_t s = as_stream(stream);
  if (dtype == JTMOE_BF16)
    return launch_pair<bf16_raw>(x, gate, up, down, group_sizes, offsets, A, H, I, E, act, packed_y, s, kStageGateUp,
                                 source_order, (int)K, T, gate_pre, up_pre);
  return launch_pair<float>(x, gate, up, down, group_sizes, offsets, A, H, I, E, act, packed_y, s, kStageGateUp,
                            source_order, (int)K, T, gate_pre, up_pre);
}

extern "C" int jtmoe_shared_swiglu_train(const void* x, const void* gate, const void* up, const void* down, int64_t T,
                                         int64_t H, int64_t Is, int dtype, void* gate_pre, void* up_pre, void* act,
                                         void* shared_y, void* stream) {
  clear_error();
  int rc = validate_gemm("shared_swiglu_train", T, H, Is, 1, dtype);
  if (rc) return rc;
  if (T == 0) return JTMOE_OK;
  JT_REQUIRE(x && gate && up && down && gate_pre && up_pre && act && shared_y,
             "shared_swiglu_train: null pointer argument");
  hipStream_t s = as_stream(stream);
  if (dtype == JTMOE_BF16)
    return launch_pair<bf16_raw>(x, gate, up, down, nullptr, nullptr, T, H, Is, 1, act, shared_y, s,
                                 kStageSharedGateUp, nullptr, 1, 0, gate_pre, up_pre);
  return launch_pair<float>(x, gate, up, down, nullptr, nullptr, T, H, Is, 1, act, shared_y, s, kStageSharedGateUp,
                            nullptr, 1, 0, gate_pre, up_pre);
}
