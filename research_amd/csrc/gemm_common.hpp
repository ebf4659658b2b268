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

// Tiles are counted expert by expert, ceil(group_size / BM) m-tiles each.  group_scan computes, in
// every lane of the calling wave, the tile counts of the lane's own experts, their exclusive
// prefix and the total; locate_tile then finds the expert and row range of m-tile `mt`.
// E <= JTMOE_MAX_EXPERTS.
struct GroupScan {
  static constexpr int kPer = JTMOE_MAX_EXPERTS / 64;  // experts per lane, contiguous
  int n[kPer], tiles[kPer];
  int first;  // tiles before this lane's experts
  int total;  // tiles of all experts
};

__device__ __forceinline__ GroupScan group_scan(int BM, const int32_t* __restrict__ group_sizes, int E) {
  GroupScan g;
  const int lane = threadIdx.x & 63;
  int local = 0;
#pragma unroll
  for (int j = 0; j < GroupScan::kPer; ++j) {
    const int e = lane * GroupScan::kPer + j;
    g.n[j] = e < E ? group_sizes[e] : 0;
    g.tiles[j] = (g.n[j] + BM - 1) / BM;
    local += g.tiles[j];
  }
  int incl = local;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int v = __shfl_up(incl, d);
    if (lane >= d) incl += v;
  }
  g.first = incl - local;
  g.total = __shfl(incl, 63);
  return g;
}

__device__ __forceinline__ TileRows locate_tile(const GroupScan& g, int mt, int BM,
                                                const int32_t* __restrict__ offsets) {
  TileRows r;
  r.expert = 0;
  r.row0 = 0;
  r.rows = 0;
  const int lane = threadIdx.x & 63;
  int first = g.first;
  int last = first;
#pragma unroll
  for (int j = 0; j < GroupScan::kPer; ++j) last += g.tiles[j];
  const bool mine = mt >= first && mt < last;
  const unsigned long long owners = __ballot(mine);
  if (owners == 0ull) return r;
  const int owner = __ffsll((long long)owners) - 1;
  int expert = 0, local_tile = 0, rows_e = 0;
#pragma unroll
  for (int j = 0; j < GroupScan::kPer; ++j) {
    if (mine && mt >= first && mt < first + g.tiles[j]) {
      expert = lane * GroupScan::kPer + j;
      local_tile = mt - first;
      rows_e = g.n[j];
    }
    first += g.tiles[j];
  }
  expert = __shfl(expert, owner);
  local_tile = __shfl(local_tile, owner);
  rows_e = __shfl(rows_e, owner);
  r.expert = expert;
  r.row0 = offsets[expert] + local_tile * BM;
  r.rows = min(BM, rows_e - local_tile * BM);
  return r;
}

// m-tile `mt` of a grouped (or, with group_sizes == nullptr, dense) row range.  Every lane of the
// calling wave gets the same answer.
__device__ __forceinline__ TileRows find_tile_wave(int mt, int BM, const int32_t* __restrict__ group_sizes,
                                                   const int32_t* __restrict__ offsets, int E, int dense_rows) {
  if (group_sizes == nullptr) {
    TileRows r;
    r.expert = 0;
    r.row0 = 0;
    r.rows = 0;
    const int row0 = mt * BM;
    if (row0 < dense_rows) {
      r.row0 = row0;
      r.rows = min(BM, dense_rows - row0);
    }
    return r;
  }
  return locate_tile(group_scan(BM, group_sizes, E), mt, BM, offsets);
}

__device__ __forceinline__ float silu_fast(float g) { return g / (1.0f + __expf(-g)); }

struct TileCoord {
  int mt, nt;  // mt < 0: this workgroup has no tile
};

// Workgroup id -> (m-tile, n-tile).  Consecutive workgroup ids go round-robin to the 8 XCDs, so
// each XCD gets a contiguous range of the logical order, and that order is walked in groups of
// group_m m-tiles x all n-tiles so that neighbours share operand panels in their L2.
// (block / blocks: this workgroup's index among the workgroups that share out the tiles, and their number --
// the launch's own unless other workgroups of the launch do something else)
__device__ __forceinline__ TileCoord xcd_tile_order(int mtiles, int ntiles_n, int group_m, int block, int blocks) {
  TileCoord t;
  const int total = mtiles * ntiles_n;
  const int per_xcd = blocks >> 3;
  const int logical = (block & 7) * per_xcd + (block >> 3);
  if (logical >= total) {
    t.mt = -1;
    t.nt = 0;
    return t;
  }
  const int group_span = group_m * ntiles_n;
  const int group = logical / group_span;
  const int in_group = logical - group * group_span;
  const int gm = min(group_m, mtiles - group * group_m);
  t.nt = in_group / gm;
  t.mt = group * group_m + (in_group - t.nt * gm);
  return t;
}

// The tile of this workgroup when the launch was sized for an upper bound of `mtiles_bound` m-tiles
// and only `mtiles` of them exist (group sizes live on the device): the XCD ranges are cut from the
// real count, so that the surplus workgroups are spread over all XCDs instead of idling one of them.
// Requires gridDim.x / 8 >= ceil(mtiles * ntiles_n / 8), which the bound guarantees.
__device__ __forceinline__ TileCoord xcd_tile_order_balanced(int mtiles, int ntiles_n, int group_m, int block) {
  TileCoord t;
  t.mt = -1;
  t.nt = 0;
  const int total = mtiles * ntiles_n;
  const int per_xcd = (total + 7) >> 3;
  const int idx = block >> 3;
  const int logical = (block & 7) * per_xcd + idx;
  if (idx >= per_xcd || logical >= total) return t;
  const int group_span = group_m * ntiles_n;
  const int group = logical / group_span;
  const int in_group = logical - group * group_span;
  const int gm = min(group_m, mtiles - group * group_m);
  t.nt = in_group / gm;
  t.mt = group * group_m + (in_group - t.nt * gm);
  return t;
}

__device__ __forceinline__ TileCoord xcd_tile_order(int mtiles, int ntiles_n, int group_m) {
  return xcd_tile_order(mtiles, ntiles_n, group_m, (int)blockIdx.x, (int)gridDim.x);
}
__device__ __forceinline__ TileCoord xcd_tile_order_balanced(int mtiles, int ntiles_n, int group_m) {
  return xcd_tile_order_balanced(mtiles, ntiles_n, group_m, (int)blockIdx.x);
}

// Second half of every epilogue: a wave has parked its WM x WNO block of bf16 results in its own
// LDS slice `cw` (row stride CS elements) and streams it out row by row with 16-byte stores.
// Row r of the block is output row out_row0 + r; rows at or past rows_end and columns at or past
// N are dropped.
template <int WM, int WNO, int CS, bool kStream = false>
__device__ __forceinline__ void store_wave_block(const uint16_t* __restrict__ cw, int lane, uint16_t* __restrict__ out,
                                                 int N, size_t out_row0, int rows_end, int col0) {
  constexpr int CPR_OUT = WNO / 8;
  constexpr int OUT_CHUNKS = WM * CPR_OUT;
#pragma unroll
  for (int j = 0; j < OUT_CHUNKS / 64; ++j) {
    const int c = lane + j * 64;
    const int r = c / CPR_OUT, ch = c - r * CPR_OUT;
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(cw + r * CS + ch * 8);
    const int col = col0 + ch * 8;
    if (r < rows_end && col < N) {
      u32x4_t* const dst = reinterpret_cast<u32x4_t*>(out + (out_row0 + r) * N + col);
      if (kStream)
        __builtin_nontemporal_store(v, dst);  // the result is not read again by this kernel
      else
        *dst = v;
    }
  }
}

// number of workgroups for `mtiles x ntiles_n` tiles: a multiple of 8 (one slice per XCD)
inline int64_t gemm_grid(int64_t mtiles, int64_t ntiles_n) { return (mtiles * ntiles_n + 7) / 8 * 8; }

// number of workgroups of a persistent launch: one per CU of the current device, a whole number per
// XCD (the 256-row configurations fit one workgroup per CU); looked up once per process
inline int persistent_grid_size() {
  static const int size = [] {
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus < 8)
      return 8;
    return cus / 8 * 8;
  }();
  return size;
}

}  // namespace jtmoe
