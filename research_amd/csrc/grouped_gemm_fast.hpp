// LDS-tiled, double-buffered bf16 grouped GEMM for gfx950 matrix cores.
//
//   C[rows of group e, :] = A[rows of group e, :] @ B[e]          (kDual = false)
//   C = silu(round(A @ B0[e])) * round(A @ B1[e])                  (kDual = true)
//
// A is [rows, K] row-major (k contiguous), B[e] is [K, N] row-major (n
// contiguous), exactly as the expert matrices are stored ([E,H,I] / [E,I,H]).
// A tiles sit in LDS as [m][k]; B tiles sit in LDS as [k][n], untouched, and
// are turned into k-contiguous MFMA operands by the transposing LDS read
// ds_read_b64_tr_b16: inside a group of 16 lanes, lane i supplies the address
// of 4 consecutive n at row k0 + i/4, columns 4*(i%4).., and lane j receives
// column j of that 4x16 block, i.e. 4 consecutive k for its own n.
//
// Requirements of this path: K % BK == 0, N % 8 == 0, 16-byte aligned pointers,
// every expert matrix and every group of rows smaller than 2 GiB.
#pragma once

#include "common.hpp"

namespace jtmoe {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;

// word 3 of a raw buffer descriptor on gfx9: 32-bit data format, untyped
constexpr int kBufferFlags = 0x00020000;

struct TileRows {
  int expert;
  int row0;  // first row of the tile
  int rows;  // valid rows in the tile (0 = no such tile)
};

// m-tile `mt` counted expert by expert (ceil(group_size / BM) tiles each).  Every
// lane of the calling wave gets the same answer.  E <= 256.
__device__ __forceinline__ TileRows find_tile_wave(int mt, int BM, const int32_t* __restrict__ group_sizes,
                                                   const int32_t* __restrict__ offsets, int E, int dense_rows) {
  TileRows r;
  r.expert = 0;
  r.row0 = 0;
  r.rows = 0;
  if (group_sizes == nullptr) {
    const int row0 = mt * BM;
    if (row0 < dense_rows) {
      r.row0 = row0;
      r.rows = min(BM, dense_rows - row0);
    }
    return r;
  }
  const int lane = threadIdx.x & 63;
  constexpr int kPer = JTMOE_MAX_EXPERTS / 64;  // experts per lane, contiguous
  int n[kPer], tiles[kPer];
  int local = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int e = lane * kPer + j;
    n[j] = e < E ? group_sizes[e] : 0;
    tiles[j] = (n[j] + BM - 1) / BM;
    local += tiles[j];
  }
  int incl = local;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int v = __shfl_up(incl, d);
    if (lane >= d) incl += v;
  }
  int first = incl - local;  // tiles before this lane's experts
  const bool mine = mt >= first && mt < incl;
  const unsigned long long owners = __ballot(mine);
  if (owners == 0ull) return r;
  const int owner = __ffsll((long long)owners) - 1;
  int expert = 0, local_tile = 0, rows_e = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    if (mine && mt >= first && mt < first + tiles[j]) {
      expert = lane * kPer + j;
      local_tile = mt - first;
      rows_e = n[j];
    }
    first += tiles[j];
  }
  expert = __shfl(expert, owner);
  local_tile = __shfl(local_tile, owner);
  rows_e = __shfl(rows_e, owner);
  r.expert = expert;
  r.row0 = offsets[expert] + local_tile * BM;
  r.rows = min(BM, rows_e - local_tile * BM);
  return r;
}

__device__ __forceinline__ float silu_fast(float g) { return g / (1.0f + __expf(-g)); }

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, bool kDual_>
struct FastGemmCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr bool kDual = kDual_;
  static constexpr int BNE = kDual ? 2 * BN : BN;  // columns of the B tile in LDS
  static constexpr int NT = WAVES_M * WAVES_N * 64;
  static constexpr int WM = BM / WAVES_M, WN = BNE / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int A_STRIDE = BK + 8;    // elements; +16 B keeps ds_read_b128 conflict-free
  static constexpr int B_STRIDE = BNE + 32;  // elements; +64 B spreads the 4 rows of a transposing read
  static constexpr int A_STAGE = BM * A_STRIDE;
  static constexpr int B_STAGE = BK * B_STRIDE;
  static constexpr size_t SMEM_BYTES = (size_t)2 * (A_STAGE + B_STAGE) * 2;
  static constexpr int A_CHUNKS = BM * BK / 8;  // 16-byte chunks per A tile
  static constexpr int B_CHUNKS = BK * BN / 8;  // per B matrix
  static constexpr int CA = A_CHUNKS / NT, CB = B_CHUNKS / NT;
  static constexpr int NB = kDual ? 2 : 1;
  static constexpr int GROUP_M = 4;  // m-tiles walked together so that they share B panels in L2
  static_assert(A_CHUNKS % NT == 0 && B_CHUNKS % NT == 0, "tile must divide evenly over the threads");
  static_assert(WM % 32 == 0 && WN % 32 == 0 && BK % 16 == 0, "wave tile must be made of 32x32x16 MFMAs");
  static_assert(!kDual || TN % 2 == 0, "dual tiles need gate and up halves in every wave");
};

template <typename Cfg>
__global__ __launch_bounds__(Cfg::NT) void grouped_gemm_fast_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B0, const uint16_t* __restrict__ B1,
    uint16_t* __restrict__ C, const int32_t* __restrict__ group_sizes, const int32_t* __restrict__ offsets, int E,
    int dense_rows, int Kdim, int N, int mtiles, int ntiles_n) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, WM = Cfg::WM, WN = Cfg::WN;
  constexpr int AS = Cfg::A_STRIDE, BS = Cfg::B_STRIDE;
  constexpr bool kDual = Cfg::kDual;
  extern __shared__ __align__(16) uint16_t smem[];
  uint16_t* const As = smem;                     // [2][BM][AS]
  uint16_t* const Bs = smem + 2 * Cfg::A_STAGE;  // [2][BK][BS]

  // ---- block -> (m-tile, n-tile): consecutive workgroup ids go round-robin to the 8
  // XCDs, so give each XCD a contiguous range of the logical order, and walk that order
  // in groups of GROUP_M m-tiles x all n-tiles so that neighbours share panels in L2.
  const int total = mtiles * ntiles_n;
  const int per_xcd = (int)gridDim.x >> 3;
  const int logical = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
  if (logical >= total) return;
  const int group_span = Cfg::GROUP_M * ntiles_n;
  const int group = logical / group_span;
  const int in_group = logical - group * group_span;
  const int gm = min(Cfg::GROUP_M, mtiles - group * Cfg::GROUP_M);
  const int nt = in_group / gm;
  const int mt = group * Cfg::GROUP_M + (in_group - nt * gm);

  const TileRows tr = find_tile_wave(mt, BM, group_sizes, offsets, E, dense_rows);
  if (tr.rows <= 0) return;
  const int n0 = nt * BN;
  const size_t wofs = (size_t)tr.expert * Kdim * N;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / Cfg::WAVES_N, wn = wave - wm * Cfg::WAVES_N;

  // ---- per-thread global -> LDS copy plan (16-byte chunks) ----
  // chunk i of this thread is chunk tid + i*NT of the tile; consecutive i differ by a
  // fixed number of rows, so one base offset per operand is enough.
  constexpr int A_CPR = BK / 8;          // chunks per A row
  constexpr int A_ROWS_STEP = NT / A_CPR;  // rows between consecutive chunks of a thread
  constexpr int B_CPR = BN / 8;          // chunks per B row (per matrix)
  constexpr int B_ROWS_STEP = NT / B_CPR;
  static_assert(NT % A_CPR == 0 && NT % B_CPR == 0, "thread count must cover whole tile rows");
  // Operands are fetched with raw buffer loads: a read past the end of the tile's rows
  // (A) or of the expert's matrix (B) returns zeros instead of faulting, so the tile
  // tails need no branches.  Offsets are in bytes.
  const int a_row = tid / A_CPR, a_kc = (tid - a_row * A_CPR) * 8;
  const int a_voff = (a_row * Kdim + a_kc) * 2;
  const int a_dst = a_row * AS + a_kc;
  const int b_krow = tid / B_CPR, b_nc = (tid - b_krow * B_CPR) * 8;
  const int b_voff = (b_krow * N + n0 + b_nc) * 2;
  const int b_dst = b_krow * BS + b_nc;
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(A + (size_t)tr.row0 * Kdim), 0, tr.rows * Kdim * 2, kBufferFlags);
  __amdgpu_buffer_rsrc_t b_rsrc[Cfg::NB];
#pragma unroll
  for (int m = 0; m < Cfg::NB; ++m)
    b_rsrc[m] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>((m == 0 ? B0 : B1) + wofs), 0,
                                                  Kdim * N * 2, kBufferFlags);

  u32x4_t a_reg[Cfg::CA];
  u32x4_t b_reg[Cfg::NB][Cfg::CB];

#define JT_LOAD_GLOBAL(k0)                                                                                   \
  {                                                                                                          \
    _Pragma("unroll") for (int i = 0; i < Cfg::CA; ++i) a_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(    \
        a_rsrc, a_voff + i * A_ROWS_STEP * Kdim * 2, (k0)*2, 0);                                             \
    _Pragma("unroll") for (int m = 0; m < Cfg::NB; ++m) _Pragma("unroll") for (int i = 0; i < Cfg::CB; ++i)  \
        b_reg[m][i] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc[m], b_voff + i * B_ROWS_STEP * N * 2,     \
                                                            (k0)*N * 2, 0);                                  \
  }
#define JT_STORE_LDS(stage)                                                                                  \
  {                                                                                                          \
    uint16_t* as_w = As + (stage)*Cfg::A_STAGE + a_dst;                                                      \
    uint16_t* bs_w = Bs + (stage)*Cfg::B_STAGE + b_dst;                                                      \
    _Pragma("unroll") for (int i = 0; i < Cfg::CA; ++i)                                                      \
        *reinterpret_cast<u32x4_t*>(as_w + i * A_ROWS_STEP * AS) = a_reg[i];                                 \
    _Pragma("unroll") for (int m = 0; m < Cfg::NB; ++m) _Pragma("unroll") for (int i = 0; i < Cfg::CB; ++i)  \
        *reinterpret_cast<u32x4_t*>(bs_w + i * B_ROWS_STEP * BS + m * BN) = b_reg[m][i];                     \
  }

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int mi = 0; mi < TM; ++mi)
#pragma unroll
    for (int jj = 0; jj < TN; ++jj)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mi][jj][i] = 0.0f;

  // LDS read offsets of this lane (elements)
  const int a_lane = (wm * WM + (lane & 31)) * AS + (lane >> 5) * 8;
  // transposing read: 16-lane group g = lane/16 covers n block 16*(g&1), k block 8*(g>>1)
  const int b_lane = (8 * (lane >> 5) + ((lane & 15) >> 2)) * BS + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  int b_col[TN];
#pragma unroll
  for (int jj = 0; jj < TN; ++jj) {
    if (kDual)
      b_col[jj] = (jj < TN / 2 ? 0 : BN) + wn * (WN / 2) + (jj % (TN / 2)) * 32;
    else
      b_col[jj] = wn * WN + jj * 32;
  }

  const int nk = Kdim / BK;
  JT_LOAD_GLOBAL(0);
  JT_STORE_LDS(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int stage = kt & 1;
    if (kt + 1 < nk) JT_LOAD_GLOBAL((kt + 1) * BK);
    const uint16_t* as = As + stage * Cfg::A_STAGE + a_lane;
    const uint16_t* bs = Bs + stage * Cfg::B_STAGE + b_lane;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8_t af[TM], bf[TN];
#pragma unroll
      for (int mi = 0; mi < TM; ++mi)
        af[mi] = *reinterpret_cast<const bf16x8_t*>(as + mi * 32 * AS + kk * 16);
#pragma unroll
      for (int jj = 0; jj < TN; ++jj) {
        const uint16_t* p = bs + kk * 16 * BS + b_col[jj];
        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4_t*)(p));
        const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4_t*)(p + 4 * BS));
        const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        bf[jj] = __builtin_bit_cast(bf16x8_t, both);
      }
#pragma unroll
      for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int jj = 0; jj < TN; ++jj)
          acc[mi][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mi], bf[jj], acc[mi][jj], 0, 0, 0);
    }
    if (kt + 1 < nk) JT_STORE_LDS(stage ^ 1);
    __syncthreads();
  }
#undef JT_LOAD_GLOBAL
#undef JT_STORE_LDS

  // ---- epilogue: value i of lane l is row 8*(i/4) + 4*(l/32) + i%4, column l%32 ----
  constexpr int TNO = kDual ? TN / 2 : TN;  // output column blocks per wave
  const int col_base = n0 + (kDual ? wn * (WN / 2) : wn * WN) + (lane & 31);
#pragma unroll
  for (int mi = 0; mi < TM; ++mi) {
#pragma unroll
    for (int jj = 0; jj < TNO; ++jj) {
      const int col = col_base + jj * 32;
      if (col >= N) continue;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int r = wm * WM + mi * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
        if (r >= tr.rows) continue;
        float v;
        if (kDual) {
          const float g = round_to_bf16(acc[mi][jj][i]);
          const float u = round_to_bf16(acc[mi][jj + TN / 2][i]);
          v = silu_fast(g) * u;
        } else {
          v = acc[mi][jj][i];
        }
        C[(size_t)(tr.row0 + r) * N + col] = (uint16_t)f32_to_bf16_bits(v);
      }
    }
  }
}

// number of workgroups for `mtiles x ntiles_n` tiles: a multiple of 8 (one slice per XCD)
inline int64_t fast_gemm_grid(int64_t mtiles, int64_t ntiles_n) { return (mtiles * ntiles_n + 7) / 8 * 8; }

}  // namespace jtmoe
