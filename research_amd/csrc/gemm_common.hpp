// Pieces shared by the grouped GEMM kernels: vector types, the m-tile -> expert
// lookup and the workgroup -> tile order.
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

// number of workgroups for `mtiles x ntiles_n` tiles: a multiple of 8 (one slice per XCD)
inline int64_t gemm_grid(int64_t mtiles, int64_t ntiles_n) { return (mtiles * ntiles_n + 7) / 8 * 8; }

}  // namespace jtmoe
