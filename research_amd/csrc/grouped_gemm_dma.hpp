// Multi-stage bf16 grouped GEMM for gfx950 whose operand tiles are written into
// LDS by the memory system itself (buffer_load_dwordx4 ... lds), not through
// vector registers.
//
//   C[rows of group e, :] = A[rows of group e, :] @ B[e]          (kDual = false)
//   C = silu(round(A @ B0[e])) * round(A @ B1[e])                  (kDual = true)
//
// A is [rows, K] row-major, B[e] is [K, N] row-major, as the expert matrices are
// stored.  One wave-wide LDS load fills 1 KiB of LDS, lane i supplying bytes
// [16 i, 16 i + 16); which 16 global bytes a lane fetches is free, so the tiles
// are stored without padding and bank conflicts are avoided by permuting the
// 16-byte chunks inside each row (an XOR swizzle applied to the *source* chunk):
//   A tile [BM][BK]:        chunk c of row r sits in slot c ^ ((r / (16/CPR)) % CPR)
//   B tile [BK][128] x NSUB: stored as blocks of 4 k rows x 16 columns (128 bytes, one
//                            16-lane transposing read touches one block) or, in the large
//                            configurations, 4 k rows x 64 columns (512 bytes: eight lanes
//                            fetch a whole 128-byte line; rows 2 and 3 keep their 64-byte
//                            halves swapped so a transposing read meets no bank twice)
// A fragments are read with ds_read_b128, B fragments with the transposing
// ds_read_b64_tr_b16 (lane i of a 16-lane group addresses row i/4, columns
// 4*(i%4)..; lane j receives the four k values of its column j).
//
// NSTAGE tiles are in flight: iteration kt waits (s_waitcnt vmcnt) only for its own
// tile, passes one barrier, re-arms the buffer that iteration kt-1 just released
// and computes.  The loads are issued from inline assembly because the compiler
// would otherwise drain every outstanding load before each LDS read.
//
// Requirements: K % BK == 0, N % 8 == 0, 16-byte aligned pointers, K*N*2 < 2^31.
#pragma once

#include "gemm_common.hpp"

#include <type_traits>

namespace jtmoe {

typedef __attribute__((ext_vector_type(4))) int i32x4_t;

__device__ __forceinline__ unsigned lds_byte_addr(const void* p) {
  return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}

// 16 bytes per lane from a raw buffer straight into LDS at lds_base + lane*16.
// Reads past the end of the buffer store zeros.  The LDS base travels in M0; the hardware wants one
// wait state between a scalar write of M0 and an LDS-DMA load that reads it, and the compiler's
// hazard handling does not look inside inline assembly, so the s_nop is written out here.
__device__ __forceinline__ void buffer_load_lds16(i32x4_t rsrc, unsigned lds_base, int voffset, int soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset)
               : "memory", "m0");
}

// The same with the LDS address given as a scalar base plus a compile-time offset: a kernel that
// issues many loads per stage then keeps one scalar per stage instead of one per load.
template <int kOffset>
__device__ __forceinline__ void buffer_load_lds16_at(i32x4_t rsrc, unsigned lds_base, int voffset, int soffset) {
  asm volatile("s_add_u32 m0, %0, %4\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset), "n"(kOffset)
               : "memory", "scc", "m0");
}

// The same with the non-temporal hint, for operands no other workgroup reads again (the expert
// matrices when every group is a single tile tall).
__device__ __forceinline__ void buffer_load_lds16_nt(i32x4_t rsrc, unsigned lds_base, int voffset, int soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen nt lds"
               :
               : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset)
               : "memory", "m0");
}

// s_waitcnt lgkmcnt(0) vmcnt(N), then the workgroup barrier.  The "memory" clobber keeps the
// compiler from moving LDS accesses across it.
template <int N>
__device__ __forceinline__ void wait_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// fp32 -> bf16 by the hardware conversion (round to nearest even)
__device__ __forceinline__ uint16_t bf16_bits_fast(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
__device__ __forceinline__ float bf16_round_fast(float f) { return (float)(__bf16)f; }
// silu with the hardware exp2 and reciprocal (about 1 ulp each); results are rounded to bf16 anyway
__device__ __forceinline__ float silu_rcp(float g) {
  return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g));
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ i32x4_t make_rsrc(const void* base, int bytes) {
  const unsigned long long p = (unsigned long long)base;
  i32x4_t r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(unsigned)p);
  r[1] = __builtin_amdgcn_readfirstlane((int)(unsigned)(p >> 32));
  r[2] = __builtin_amdgcn_readfirstlane(bytes);
  r[3] = kBufferFlags;
  return r;
}

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, bool kDual_, int NSTAGE_, int OPT_ = 16>
struct DmaGemmCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, NSTAGE = NSTAGE_;
  // scheduling options: 16 = request the fragments of MFMA step kk+1 before issuing step kk,
  // 32 = raise the wave priority around the MFMA burst, 64 = ask the scheduler to interleave
  // one MFMA with up to three LDS reads, 128 = B tiles in 4 x 64 blocks, 2048 = (persistent kernel) results written
  // straight from transposed accumulators instead of through LDS, 4096 = non-temporal loads of B, 8192 / 16384 = 8 / 2 m-tiles per group of the tile order instead of 4, 32768 = non-temporal stores of the result
  static constexpr int OPT = OPT_;
  static constexpr bool kDual = kDual_;
  static constexpr int BNE = kDual ? 2 * BN : BN;  // columns of the B tile in LDS
  static constexpr int NSUB = BNE / 128;           // 128-column sub-tiles of B
  static constexpr int NT = WAVES_M * WAVES_N * 64;
  static constexpr int WM = BM / WAVES_M, WN = BNE / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int TNO = kDual ? TN / 2 : TN;
  static constexpr int WNO = TNO * 32;
  static constexpr int CPRA = BK / 8;  // 16-byte chunks per A row
  static constexpr int A_BYTES = BM * BK * 2;
  static constexpr int BSUB_BYTES = BK * 256;
  static constexpr int STAGE_BYTES = A_BYTES + NSUB * BSUB_BYTES;
  static constexpr int A_LOADS = BM * CPRA / NT;   // per thread per stage
  static constexpr int BSUB_LOADS = BK * 16 / NT;  // per thread per sub-tile per stage
  static constexpr int LPS = A_LOADS + NSUB * BSUB_LOADS;
  static constexpr int CS = WNO + 8;  // epilogue staging row stride (elements)
  static constexpr size_t EPI_BYTES = (size_t)WAVES_M * WAVES_N * WM * CS * 2;
  static constexpr size_t PIPE_BYTES = (size_t)NSTAGE * STAGE_BYTES;
  static constexpr size_t SMEM_BYTES = PIPE_BYTES > EPI_BYTES ? PIPE_BYTES : EPI_BYTES;
  // m-tiles per group of the tile order (a group = GROUP_M m-tiles x all n-tiles, walked n-tile by n-tile);
  // option bits 8192 / 16384 select 8 / 2 for the stand-alone check's comparison of schedules
  static constexpr int GROUP_M = (OPT_ & 8192) ? 8 : ((OPT_ & 16384) ? 2 : 4);
  // A four-wave workgroup whose waves hold 128 accumulators each is meant to share its CU with a second
  // one (two waves per SIMD): the register allocation is held to half of the file.
  static constexpr int MIN_WAVES_PER_EU = (NT == 256 && TM * TN * 16 >= 128) ? 2 : 1;
  static_assert(BNE % 128 == 0, "B tile is made of 128-column sub-tiles");
  static_assert(BK == 32 || BK == 64, "BK must be 32 or 64");
  static_assert((BM * CPRA) % NT == 0 && (BK * 16) % NT == 0, "tile must divide evenly over the threads");
  static_assert((NT / CPRA) % 16 == 0 && NT % 64 == 0, "swizzle must not depend on the load index");
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be made of 32x32x16 MFMAs");
  static_assert(!kDual || (TN % 2 == 0 && BN == 128), "dual tiles: one sub-tile per matrix");
  static_assert(NSTAGE >= 2 && (NSTAGE - 2) * LPS < 64, "vmcnt is a 6-bit counter");
  static_assert(SMEM_BYTES <= 160 * 1024, "LDS budget");
};

// two fp32 values -> their bf16 roundings packed in one dword (lo in the low half): one hardware conversion
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
__device__ __forceinline__ unsigned pack_bf16x2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2_t));
}

// Epilogue of the kernels that issue their MFMAs with the WEIGHT fragment as the first operand: a
// 32 x 32 accumulator then holds the TRANSPOSED block -- value i of lane l is row l % 32, column
// 8 * (i / 4) + 4 * (l / 32) + i % 4 of the block, i.e. a lane owns runs of four neighbouring columns
// of one row.  Two such runs are packed to bf16 pairs, the half-waves swap one of them
// (v_permlane32_swap), and every lane stores 16 contiguous bytes: no LDS staging, no barrier.
// Stores go through a buffer descriptor of the whole result (out_rows_total rows of N columns, at most
// 0x7ffe0000 bytes): one 32-bit offset per row, the column of each store as an immediate, and rows
// past the end of the group (or columns past N) get the offset 0x7fff0000, which lies outside every
// admitted result, so the hardware drops the store.
// With save0 / save1 (dual tiles only) the two rounded products are written as well.
template <typename Cfg>
__device__ __forceinline__ void store_transposed_accumulators(const f32x16_t (&acc)[Cfg::TM][Cfg::TN], int wm, int wn,
                                                              int row0, int rows, int n0, int N, int out_rows_total,
                                                              uint16_t* __restrict__ C, uint16_t* __restrict__ save0,
                                                              uint16_t* __restrict__ save1) {
  constexpr int TM = Cfg::TM, TN = Cfg::TN, WM = Cfg::WM, TNO = Cfg::TNO, WNO = Cfg::WNO;
  constexpr bool kDual = Cfg::kDual;
  // (the lane id is taken afresh so that nothing of the epilogue's addressing is kept in registers
  // through the k loops, where every register is spoken for)
  int lane_e;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_e));
  const int col0 = n0 + wn * WNO;
  const int half = lane_e >> 5;
  const int cols_left = N - (col0 + 8 * half);
  auto write_pass = [&](auto pass_tag) {
    constexpr int pass = decltype(pass_tag)::value;  // 0: the result, 1 and 2: the two rounded products
    uint16_t* const out = pass == 0 ? C : (pass == 1 ? save0 : save1);
    const __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(out, 0, out_rows_total * N * 2, kBufferFlags);
#pragma unroll
    for (int mi = 0; mi < TM; ++mi) {
      const int r = wm * WM + mi * 32 + (lane_e & 31);
      const int row_off = r < rows ? ((row0 + r) * N + col0 + 8 * half) * 2 : 0x7fff0000;
#pragma unroll
      for (int jj = 0; jj < TNO; ++jj) {
#pragma unroll
        for (int qq = 0; qq < 4; qq += 2) {
          unsigned pk[2][2];
#pragma unroll
          for (int dq = 0; dq < 2; ++dq) {
#pragma unroll
            for (int tp = 0; tp < 2; ++tp) {  // two neighbouring columns at a time
              const int i = (qq + dq) * 4 + tp * 2;
              if (kDual) {
                // both products rounded to bf16 (one packed conversion each), then silu(g) * u on them
                const unsigned gb = pack_bf16x2(acc[mi][jj][i], acc[mi][jj][i + 1]);
                const unsigned ub = pack_bf16x2(acc[mi][jj + TN / 2][i], acc[mi][jj + TN / 2][i + 1]);
                if (pass == 0) {
                  const float g0 = __uint_as_float(gb << 16), g1 = __uint_as_float(gb & 0xffff0000u);
                  const float u0 = __uint_as_float(ub << 16), u1 = __uint_as_float(ub & 0xffff0000u);
                  pk[dq][tp] = pack_bf16x2(silu_rcp(g0) * u0, silu_rcp(g1) * u1);
                } else {
                  pk[dq][tp] = pass == 1 ? gb : ub;
                }
              } else {
                pk[dq][tp] = pack_bf16x2(acc[mi][jj][i], acc[mi][jj][i + 1]);
              }
            }
          }
          // before: this lane has columns 8 qq + 4 half + 0..3 (pk[0]) and 8 (qq + 1) + 4 half + 0..3
          // (pk[1]); after: columns 8 (qq + half) + 0..7
          const auto lo = __builtin_amdgcn_permlane32_swap(pk[0][0], pk[1][0], false, false);
          const auto hi = __builtin_amdgcn_permlane32_swap(pk[0][1], pk[1][1], false, false);
          const u32x4_t val = {lo[0], hi[0], lo[1], hi[1]};
          const int col = jj * 32 + 8 * qq;  // + 8 * half, already in row_off
          const int off = col < cols_left ? row_off : 0x7fff0000;
          // plain stores: a 128-byte line of the result is put together from four of these stores in the
          // L2 (as non-temporal stores the 32-byte pieces cost 17 % of the down projection)
          __builtin_amdgcn_raw_buffer_store_b128(val, out_rsrc, off + col * 2, 0, 0);
          // keeps the compiler from computing many column runs at once (register pressure)
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };
  write_pass(std::integral_constant<int, 0>{});
  if (kDual && save0 != nullptr) {
    write_pass(std::integral_constant<int, 1>{});
    write_pass(std::integral_constant<int, 2>{});
  }
}

// One tile per workgroup.  block / blocks: this workgroup's index among the workgroups that share out the
// tiles and their number (the launch's own in grouped_gemm_dma_kernel below; a launch may also give some of
// its workgroups other work, see the decode launch of the router).
template <typename Cfg>
__device__ __forceinline__ void grouped_gemm_dma_tile(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B0, const uint16_t* __restrict__ B1,
    uint16_t* __restrict__ C, const int32_t* __restrict__ group_sizes, const int32_t* __restrict__ offsets, int E,
    int dense_rows, int Kdim, int N, int mtiles, int ntiles_n, const int32_t* __restrict__ row_map, int row_div,
    int a_rows, uint16_t* __restrict__ save0, uint16_t* __restrict__ save1, int uniform_rows, int a_group_rows,
    int block, int blocks) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT, NSTAGE = Cfg::NSTAGE;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, WM = Cfg::WM, WN = Cfg::WN;
  constexpr int CPRA = Cfg::CPRA;
  constexpr bool kDual = Cfg::kDual;
  extern __shared__ __align__(16) unsigned char smem_raw[];

  // the grid covers an upper bound of the m-tiles; the tile order is cut from their real number
  TileCoord tc;
  TileRows tr;
  int a_row0;  // first row of the tile inside A (without a row map)
  if (uniform_rows > 0) {
    // Every group takes the SAME uniform_rows rows of A (all tokens through every expert: the decode
    // path, which does not wait for the routing): group e writes rows [e, e + 1) * uniform_rows of C.
    const int per_group = (uniform_rows + BM - 1) / BM;
    tc = xcd_tile_order(E * per_group, ntiles_n, Cfg::GROUP_M, block, blocks);
    if (tc.mt < 0) return;
    tr.expert = tc.mt / per_group;
    const int local_row0 = (tc.mt - tr.expert * per_group) * BM;
    tr.row0 = tr.expert * uniform_rows + local_row0;
    tr.rows = min(BM, uniform_rows - local_row0);
    a_row0 = local_row0;
  } else if (group_sizes) {
    const GroupScan scan = group_scan(BM, group_sizes, E);
    tc = xcd_tile_order_balanced(scan.total, ntiles_n, Cfg::GROUP_M, block);
    if (tc.mt < 0) return;
    tr = locate_tile(scan, tc.mt, BM, offsets);
  } else {
    tc = xcd_tile_order(mtiles, ntiles_n, Cfg::GROUP_M, block, blocks);
    if (tc.mt < 0) return;
    tr = find_tile_wave(tc.mt, BM, nullptr, nullptr, E, dense_rows);
  }
  if (uniform_rows <= 0) a_row0 = tr.row0;
  a_row0 = __builtin_amdgcn_readfirstlane(a_row0);
  const int nt = tc.nt;
  tr.expert = __builtin_amdgcn_readfirstlane(tr.expert);
  tr.row0 = __builtin_amdgcn_readfirstlane(tr.row0);
  tr.rows = __builtin_amdgcn_readfirstlane(tr.rows);
  if (tr.rows <= 0) return;
  const int n0 = nt * BN;
  const size_t wofs = (size_t)tr.expert * Kdim * N;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WAVES_N, wn = wave - wm * Cfg::WAVES_N;

  // ---- load plan ----
  i32x4_t b_rsrc[Cfg::NSUB];
#pragma unroll
  for (int u = 0; u < Cfg::NSUB; ++u)
    b_rsrc[u] = make_rsrc((kDual && u == 1 ? B1 : B0) + wofs, Kdim * N * 2);
  // Without a row map, tile row r is row tr.row0 + r of A.  With one (gather on load), it is row
  // row_map[tr.row0 + r] / row_div of A: the expert-major permutation is applied while the tile is
  // fetched, so the permuted copy of the activations never exists in memory.
  // (a_group_rows > 0: A holds a block of a_group_rows rows per group, and the map's rows are rows of the
  // tile's group's block -- the activations of the decode path above, [E][tokens][K])
  const bool gather = row_map != nullptr;
  const i32x4_t a_rsrc = gather ? make_rsrc(A + (size_t)tr.expert * a_group_rows * Kdim, a_rows * Kdim * 2)
                                : make_rsrc(A + (size_t)a_row0 * Kdim, tr.rows * Kdim * 2);
  // A: slot s = j*NT + tid -> row s / CPRA, slot-in-row s % CPRA holds source chunk c
  const int a_r = tid / CPRA, a_slot = tid - a_r * CPRA;
  const int a_c = a_slot ^ ((a_r / (16 / CPRA)) % CPRA);
  int a_voff[Cfg::A_LOADS];
#pragma unroll
  for (int j = 0; j < Cfg::A_LOADS; ++j) {
    const int r = a_r + j * (NT / CPRA);
    if (gather) {
      // rows past the end of the group get an offset beyond the buffer: they read as zeros
      a_voff[j] = r < tr.rows ? ((row_map[tr.row0 + r] / row_div) * Kdim + a_c * 8) * 2 : 0x70000000;
    } else {
      a_voff[j] = (r * Kdim + a_c * 8) * 2;
    }
  }
  // B sub-tile [BK][128]: stored as 128-byte blocks of 4 k rows x 16 columns, block (k/4, n/16) at
  // index (k/4)*8 + n/16; slot s (16 bytes) -> block s/8, row (s/2)%4 of the block, half s%2.
  // OPT & 128: 512-byte blocks of 4 k rows x 64 columns instead (block (k/4, n/64) at index
  // (k/4)*2 + n/64, slot s -> block s/32, row (s/8)%4, chunk s%8), so that eight lanes fetch one
  // whole 128-byte line of the matrix; rows 2 and 3 of a block hold their two 64-byte halves
  // swapped, which keeps the four 32-byte pieces of a transposing read in different banks.
  constexpr bool kWide = (Cfg::OPT & 128) != 0;
  const int b_blk_id = kWide ? tid >> 5 : tid >> 3;
  const int b_k = kWide ? (b_blk_id >> 1) * 4 + ((tid >> 3) & 3) : (b_blk_id >> 3) * 4 + ((tid >> 1) & 3);
  const int b_c = kWide ? (b_blk_id & 1) * 8 + ((tid & 7) ^ (((tid >> 4) & 1) << 2)) : (b_blk_id & 7) * 2 + (tid & 1);
  int b_voff[Cfg::NSUB];
#pragma unroll
  for (int u = 0; u < Cfg::NSUB; ++u) b_voff[u] = (b_k * N + n0 + (kDual ? 0 : u * 128) + b_c * 8) * 2;
  const unsigned lds0 = lds_byte_addr(smem_raw);
  const unsigned wave_lds = lds0 + wave * 1024;  // this wave's 1 KiB inside every NT*16-byte load round

  auto issue = [&](int kt) {
    const unsigned base = wave_lds + (kt % NSTAGE) * Cfg::STAGE_BYTES;
    const int k0 = kt * BK;
#pragma unroll
    for (int j = 0; j < Cfg::A_LOADS; ++j)
      buffer_load_lds16(a_rsrc, base + j * NT * 16, a_voff[j], k0 * 2);
#pragma unroll
    for (int u = 0; u < Cfg::NSUB; ++u)
#pragma unroll
      for (int j = 0; j < Cfg::BSUB_LOADS; ++j) {
        if (Cfg::OPT & 4096)
          buffer_load_lds16_nt(b_rsrc[u], base + Cfg::A_BYTES + u * Cfg::BSUB_BYTES + j * NT * 16,
                               b_voff[u] + j * (NT / 16) * N * 2, k0 * N * 2);
        else
          buffer_load_lds16(b_rsrc[u], base + Cfg::A_BYTES + u * Cfg::BSUB_BYTES + j * NT * 16,
                            b_voff[u] + j * (NT / 16) * N * 2, k0 * N * 2);
      }
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int mi = 0; mi < TM; ++mi)
#pragma unroll
    for (int jj = 0; jj < TN; ++jj)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mi][jj][i] = 0.0f;

  // ---- fragment addresses of this lane (bytes inside a stage) ----
  const int a_row = wm * WM + (lane & 31);
  const int a_sw = (a_row / (16 / CPRA)) % CPRA;
  const int a_rowoff = a_row * (BK * 2);
  // transposing read: the 16 lanes of a group read one whole 128-byte block, lane i its bytes
  // [8 i, 8 i + 8) = row i/4, columns 4*(i%4)..; groups: column half (lane/16)%2, k half lane/32
  const int b_laneoff = kWide ? ((lane & 15) >> 2) * 128 + (lane & 3) * 8 + ((lane >> 4) & 1) * 32 + (lane >> 5) * 2048
                              : (lane & 15) * 8 + ((lane >> 4) & 1) * 128 + (lane >> 5) * (2 * 8 * 128);
  const int half_swap = kWide ? ((lane >> 3) & 1) * 64 : 0;  // the swapped halves, seen from the reading lane
  int b_blk[TN];  // byte offset of column block jj: sub-tile base + its first 16-column block
#pragma unroll
  for (int jj = 0; jj < TN; ++jj) {
    int col;  // first column of the block inside the BNE-wide tile
    if (kDual)
      col = (jj < TN / 2 ? 0 : BN) + wn * (WN / 2) + (jj % (TN / 2)) * 32;
    else
      col = wn * WN + jj * 32;
    const int u = col >> 7;
    if (kWide)
      b_blk[jj] = Cfg::A_BYTES + u * Cfg::BSUB_BYTES + ((col & 127) >> 6) * 512 + (col & 63) * 2 +
                  ((col & 32) ? -half_swap : half_swap);
    else
      b_blk[jj] = Cfg::A_BYTES + u * Cfg::BSUB_BYTES + ((col & 127) >> 4) * 128;
  }

  auto load_frags = [&](const unsigned char* st, int kk, bf16x8_t* af, bf16x8_t* bf) {
#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
      af[mi] = *reinterpret_cast<const bf16x8_t*>(st + a_rowoff + mi * 32 * BK * 2 +
                                                  (((kk * 2 + (lane >> 5)) ^ a_sw) << 4));
#pragma unroll
    for (int jj = 0; jj < TN; ++jj) {
      const unsigned char* p = st + b_blk[jj] + b_laneoff + kk * (4 * 8 * 128);
      const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p));
      const s16x4_t hi =
          __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p + 8 * 128));
      const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      bf[jj] = __builtin_bit_cast(bf16x8_t, both);
    }
  };

  const int nk = Kdim / BK;
  // The last tile of a group is usually partly empty.  A wave whose WM rows all lie past the end of
  // the group (or whose columns all lie past N) still takes part in the loads and the barriers but
  // skips its fragment reads and MFMAs.
  const bool wave_has_rows = wm * WM < tr.rows && n0 + wn * Cfg::WNO < N;
#pragma unroll
  for (int s = 0; s < NSTAGE - 1; ++s)
    if (s < nk) issue(s);

  for (int kt = 0; kt < nk; ++kt) {
    if (kt + NSTAGE - 2 < nk)
      wait_vmcnt<(NSTAGE - 2) * Cfg::LPS>();
    else
      wait_vmcnt<0>();
    __syncthreads();
    if (kt + NSTAGE - 1 < nk) issue(kt + NSTAGE - 1);
    const unsigned char* st = smem_raw + (kt % NSTAGE) * Cfg::STAGE_BYTES;
    if (!wave_has_rows) continue;  // a tile at the end of a group: this wave's rows lie past it
    if (Cfg::OPT & 16) {
      // fragments of step kk+1 are requested before the MFMAs of step kk are issued
      bf16x8_t af[2][TM], bf[2][TN];
      load_frags(st, 0, af[0], bf[0]);
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
        if (kk + 1 < BK / 16) load_frags(st, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
        if (Cfg::OPT & 32) __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
          for (int jj = 0; jj < TN; ++jj)
            acc[mi][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk & 1][mi], bf[kk & 1][jj], acc[mi][jj], 0, 0, 0);
        if (Cfg::OPT & 32) __builtin_amdgcn_s_setprio(0);
        if (Cfg::OPT & 64) {
          // interleave: one MFMA, then up to three LDS reads, repeated
#pragma unroll
          for (int g = 0; g < TM * TN; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
          }
        }
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
        bf16x8_t af[TM], bf[TN];
        load_frags(st, kk, af, bf);
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
          for (int jj = 0; jj < TN; ++jj)
            acc[mi][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mi], bf[jj], acc[mi][jj], 0, 0, 0);
      }
    }
  }
  wait_vmcnt<0>();
  __syncthreads();  // every wave is done reading the tiles: LDS becomes the output staging area

  // ---- epilogue ----
  // Value i of lane l in a 32x32 accumulator is row 8*(i/4) + 4*(l/32) + i%4, column l%32: a
  // lane holds single elements of many rows.  Each wave parks its WM x WNO block of results
  // in its own slice of the idle LDS and streams it out row by row with 16-byte stores.
  // With save0 / save1 (dual tiles only) the two rounded products themselves, which the backward
  // pass needs, are written as well: pass 0 stores the result, passes 1 and 2 the two products.
  constexpr int TNO = Cfg::TNO, WNO = Cfg::WNO, CS = Cfg::CS;
  uint16_t* const cw = reinterpret_cast<uint16_t*>(smem_raw) + wave * (WM * CS);
  const int col0 = n0 + wn * WNO;
  const int row_base = wm * WM;
  const int passes = (kDual && save0 != nullptr) ? 3 : 1;
  for (int pass = 0; pass < passes; ++pass) {
#pragma unroll
    for (int mi = 0; mi < TM; ++mi) {
#pragma unroll
      for (int jj = 0; jj < TNO; ++jj) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int r = mi * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
          float v;
          if (kDual) {
            const float g = bf16_round_fast(acc[mi][jj][i]);
            const float u = bf16_round_fast(acc[mi][jj + TN / 2][i]);
            v = pass == 0 ? silu_rcp(g) * u : (pass == 1 ? g : u);
          } else {
            v = acc[mi][jj][i];
          }
          cw[r * CS + jj * 32 + (lane & 31)] = bf16_bits_fast(v);
        }
      }
    }
    uint16_t* const out = pass == 0 ? C : (pass == 1 ? save0 : save1);
    // the kept products are read again only by the backward pass: always streamed out
    if (pass == 0)
      store_wave_block<WM, WNO, CS, (Cfg::OPT & 32768) != 0>(cw, lane, out, N, (size_t)tr.row0 + row_base,
                                                            tr.rows - row_base, col0);
    else
      store_wave_block<WM, WNO, CS, true>(cw, lane, out, N, (size_t)tr.row0 + row_base, tr.rows - row_base, col0);
  }
}

template <typename Cfg>
__global__ __launch_bounds__(Cfg::NT) __attribute__((amdgpu_waves_per_eu(Cfg::MIN_WAVES_PER_EU))) void grouped_gemm_dma_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B0, const uint16_t* __restrict__ B1,
    uint16_t* __restrict__ C, const int32_t* __restrict__ group_sizes, const int32_t* __restrict__ offsets, int E,
    int dense_rows, int Kdim, int N, int mtiles, int ntiles_n, const int32_t* __restrict__ row_map, int row_div,
    int a_rows, uint16_t* __restrict__ save0 = nullptr, uint16_t* __restrict__ save1 = nullptr, int uniform_rows = 0,
    int a_group_rows = 0) {
  grouped_gemm_dma_tile<Cfg>(A, B0, B1, C, group_sizes, offsets, E, dense_rows, Kdim, N, mtiles, ntiles_n, row_map,
                             row_div, a_rows, save0, save1, uniform_rows, a_group_rows, (int)blockIdx.x,
                             (int)gridDim.x);
}

// ---------------------------------------------------------------------------------------------
// The same tile computation for launches with many tiles per CU: a workgroup walks a sequence of
// tiles of its XCD's contiguous range of the logical order.  The tile after the current one is
// looked up when the current one starts, and its first operand tiles are requested right after the
// current k loop, before the epilogue: the latency of those loads, the tile look-up and the start
// of a new workgroup no longer stand between two tiles.  At the C3 shape the down projection (22 k
// steps, 128 KB of results per tile) goes from 0.78 to 0.735 ms, gate/up from 1.465 to 1.44 ms.
// The epilogue stages results above the first stage buffer (which the next tile's loads are
// filling), in two halves where a wave's block does not fit its share of that area.
// Two schedules (launch with a multiple of 8 workgroups):
//   chunk == 0: one workgroup per CU for the whole launch; workgroup i of an XCD takes tiles
//     i, i + n, i + 2n, ... of the range (n workgroups per XCD).
//   chunk > 0: many workgroups of `chunk` tiles each, which the hardware starts in order as CUs
//     become free.  With `window` workgroups resident per XCD, workgroup j takes tiles
//     (j / window) * window * chunk + j % window + p * window, p < chunk: the resident workgroups
//     stay within window * chunk consecutive tiles of each other, where fully persistent ones drift
//     apart and share fewer operand panels in the L2 (gate/up at C3: 5.9 GB leave the L2 per launch
//     with chunk 0, 4.4 GB with chunk 4, 4.1 GB with one tile per workgroup; the run time is the
//     same for chunk 0, 2, 4 and 8).
// ---------------------------------------------------------------------------------------------
template <typename Cfg>
__global__ __launch_bounds__(Cfg::NT) void grouped_gemm_dma_persistent_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B0, const uint16_t* __restrict__ B1,
    uint16_t* __restrict__ C, const int32_t* __restrict__ group_sizes, const int32_t* __restrict__ offsets, int E,
    int dense_rows, int Kdim, int N, int mtiles, int ntiles_n, const int32_t* __restrict__ row_map, int row_div,
    int a_rows, uint16_t* __restrict__ save0, uint16_t* __restrict__ save1, int window, int chunk) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, WM = Cfg::WM, WN = Cfg::WN;
  constexpr int CPRA = Cfg::CPRA;
  constexpr bool kDual = Cfg::kDual;
  static_assert(Cfg::NSTAGE == 2, "two stages");
  // results straight from (transposed) accumulators: the weight fragment is the MFMA's first operand
  constexpr bool kDirect = (Cfg::OPT & 2048) != 0;
  extern __shared__ __align__(16) unsigned char smem_raw[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WAVES_N, wn = wave - wm * Cfg::WAVES_N;
  const bool gather = row_map != nullptr;

  // ---- schedule: the XCD's contiguous range of the logical tile order, walked with the stride of
  // the workgroups this XCD has ----
  GroupScan scan;
  int real_mtiles = mtiles;
  if (group_sizes) {
    scan = group_scan(BM, group_sizes, E);
    real_mtiles = __builtin_amdgcn_readfirstlane(scan.total);
  }
  const int total = real_mtiles * ntiles_n;
  const int per_xcd = (total + 7) >> 3;
  const int xcd = (int)blockIdx.x & 7;  // the launch uses a multiple of 8 workgroups
  int idx = (int)blockIdx.x >> 3, stride = max(1, (int)gridDim.x >> 3), left = 0x7fffffff;
  if (chunk > 0) {
    idx = (idx / window) * (window * chunk) + idx % window;
    stride = window;
    left = chunk;
  }

  struct Tile {
    int expert, row0, rows, n0;
  };
  auto locate = [&](int i) -> Tile {
    Tile t;
    t.expert = 0; t.row0 = 0; t.rows = 0; t.n0 = 0;
    const int logical = xcd * per_xcd + i;
    if (i >= per_xcd || logical >= total) return t;
    const int group_span = Cfg::GROUP_M * ntiles_n;
    const int group = logical / group_span;
    const int in_group = logical - group * group_span;
    const int gm = min(Cfg::GROUP_M, real_mtiles - group * Cfg::GROUP_M);
    const int nt = in_group / gm;
    const int mt = group * Cfg::GROUP_M + (in_group - nt * gm);
    TileRows tr;
    if (group_sizes) {
      tr = locate_tile(scan, mt, BM, offsets);
    } else {
      tr.expert = 0;
      tr.row0 = mt * BM;
      tr.rows = min(BM, dense_rows - mt * BM);
    }
    t.expert = __builtin_amdgcn_readfirstlane(tr.expert);
    t.row0 = __builtin_amdgcn_readfirstlane(tr.row0);
    t.rows = __builtin_amdgcn_readfirstlane(tr.rows);
    t.n0 = nt * BN;
    return t;
  };

  // ---- load plan (rewritten for every tile) ----
  i32x4_t b_rsrc[Cfg::NSUB];
  i32x4_t a_rsrc;
  int a_voff[Cfg::A_LOADS];
  int b_voff[Cfg::NSUB];
  const int a_r = tid / CPRA, a_slot = tid - a_r * CPRA;
  const int a_c = a_slot ^ ((a_r / (16 / CPRA)) % CPRA);
  constexpr bool kWide = (Cfg::OPT & 128) != 0;
  const int b_blk_id = kWide ? tid >> 5 : tid >> 3;
  const int b_k = kWide ? (b_blk_id >> 1) * 4 + ((tid >> 3) & 3) : (b_blk_id >> 3) * 4 + ((tid >> 1) & 3);
  const int b_c = kWide ? (b_blk_id & 1) * 8 + ((tid & 7) ^ (((tid >> 4) & 1) << 2)) : (b_blk_id & 7) * 2 + (tid & 1);
  // the A offsets of a tile's rows (with a row map they are fetched through it)
  auto row_offsets = [&](const Tile& t, int* voff) {
#pragma unroll
    for (int j = 0; j < Cfg::A_LOADS; ++j) {
      const int r = a_r + j * (NT / CPRA);
      if (gather)
        voff[j] = r < t.rows ? ((row_map[t.row0 + r] / row_div) * Kdim + a_c * 8) * 2 : 0x70000000;
      else
        voff[j] = (r * Kdim + a_c * 8) * 2;
    }
  };
  auto plan = [&](const Tile& t, const int* voff) {
    const size_t wofs = (size_t)t.expert * Kdim * N;
#pragma unroll
    for (int u = 0; u < Cfg::NSUB; ++u) b_rsrc[u] = make_rsrc((kDual && u == 1 ? B1 : B0) + wofs, Kdim * N * 2);
    a_rsrc = gather ? make_rsrc(A, a_rows * Kdim * 2) : make_rsrc(A + (size_t)t.row0 * Kdim, t.rows * Kdim * 2);
#pragma unroll
    for (int j = 0; j < Cfg::A_LOADS; ++j) a_voff[j] = voff[j];
#pragma unroll
    for (int u = 0; u < Cfg::NSUB; ++u) b_voff[u] = (b_k * N + t.n0 + (kDual ? 0 : u * 128) + b_c * 8) * 2;
  };
  const unsigned lds0 = lds_byte_addr(smem_raw);
  const unsigned wave_lds = lds0 + wave * 1024;
  auto issue = [&](int kt) {
    const unsigned base = wave_lds + (kt & 1) * Cfg::STAGE_BYTES;
    const int k0 = kt * BK;
#pragma unroll
    for (int j = 0; j < Cfg::A_LOADS; ++j) buffer_load_lds16(a_rsrc, base + j * NT * 16, a_voff[j], k0 * 2);
#pragma unroll
    for (int u = 0; u < Cfg::NSUB; ++u)
#pragma unroll
      for (int j = 0; j < Cfg::BSUB_LOADS; ++j)
        buffer_load_lds16(b_rsrc[u], base + Cfg::A_BYTES + u * Cfg::BSUB_BYTES + j * NT * 16,
                          b_voff[u] + j * (NT / 16) * N * 2, k0 * N * 2);
  };

  // ---- fragment addresses of this lane (the same for every tile) ----
  const int a_row = wm * WM + (lane & 31);
  const int a_sw = (a_row / (16 / CPRA)) % CPRA;
  const int a_rowoff = a_row * (BK * 2);
  const int b_laneoff = kWide ? ((lane & 15) >> 2) * 128 + (lane & 3) * 8 + ((lane >> 4) & 1) * 32 + (lane >> 5) * 2048
                              : (lane & 15) * 8 + ((lane >> 4) & 1) * 128 + (lane >> 5) * (2 * 8 * 128);
  const int half_swap = kWide ? ((lane >> 3) & 1) * 64 : 0;
  int b_blk[TN];
#pragma unroll
  for (int jj = 0; jj < TN; ++jj) {
    int col;
    if (kDual)
      col = (jj < TN / 2 ? 0 : BN) + wn * (WN / 2) + (jj % (TN / 2)) * 32;
    else
      col = wn * WN + jj * 32;
    const int u = col >> 7;
    if (kWide)
      b_blk[jj] = Cfg::A_BYTES + u * Cfg::BSUB_BYTES + ((col & 127) >> 6) * 512 + (col & 63) * 2 +
                  ((col & 32) ? -half_swap : half_swap);
    else
      b_blk[jj] = Cfg::A_BYTES + u * Cfg::BSUB_BYTES + ((col & 127) >> 4) * 128;
  }
  auto load_frags = [&](const unsigned char* st, int kk, bf16x8_t* af, bf16x8_t* bf) {
#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
      af[mi] = *reinterpret_cast<const bf16x8_t*>(st + a_rowoff + mi * 32 * BK * 2 +
                                                  (((kk * 2 + (lane >> 5)) ^ a_sw) << 4));
#pragma unroll
    for (int jj = 0; jj < TN; ++jj) {
      const unsigned char* p = st + b_blk[jj] + b_laneoff + kk * (4 * 8 * 128);
      const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p));
      const s16x4_t hi =
          __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p + 8 * 128));
      const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      bf[jj] = __builtin_bit_cast(bf16x8_t, both);
    }
  };

  const int nk = Kdim / BK;
  constexpr int TNO = Cfg::TNO, WNO = Cfg::WNO, CS = Cfg::CS;
  // Epilogue staging lives above the first stage buffer, which the next tile's first loads fill
  // while the epilogue runs.  If a wave's block does not fit its share, it goes out in two halves.
  constexpr int kStageArea = (int)Cfg::SMEM_BYTES - Cfg::STAGE_BYTES;
  constexpr int kHalves = (NT / 64) * WM * CS * 2 <= kStageArea ? 1 : 2;
  constexpr int TMH = TM / kHalves, WMH = WM / kHalves;
  static_assert((NT / 64) * WMH * CS * 2 <= kStageArea && TM % kHalves == 0, "epilogue staging must fit above stage 0");
  uint16_t* const cw = reinterpret_cast<uint16_t*>(smem_raw + Cfg::STAGE_BYTES) + wave * (WMH * CS);

  Tile cur = locate(idx);
  if (cur.rows <= 0) return;
  {
    int voff[Cfg::A_LOADS];
    row_offsets(cur, voff);
    plan(cur, voff);
  }
  issue(0);

  while (true) {
    f32x16_t acc[TM][TN];
#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
#pragma unroll
      for (int jj = 0; jj < TN; ++jj)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mi][jj][i] = 0.0f;
    const bool wave_has_rows = wm * WM < cur.rows && cur.n0 + wn * Cfg::WNO < N;
    // the tile after this one is looked up now, and its row offsets requested, so that nothing but the
    // issue of its first loads stands between the end of this tile's k loop and its epilogue
    idx += stride;
    --left;
    const Tile nxt = locate(left > 0 ? idx : 0x3fffffff);
    int nxt_voff[Cfg::A_LOADS];
    if (nxt.rows > 0) row_offsets(nxt, nxt_voff);

    for (int kt = 0; kt < nk; ++kt) {
      wait_vmcnt<0>();
      __syncthreads();
      if (kt + 1 < nk) issue(kt + 1);
      const unsigned char* st = smem_raw + (kt & 1) * Cfg::STAGE_BYTES;
      if (!wave_has_rows) continue;
      bf16x8_t af[2][TM], bf[2][TN];
      load_frags(st, 0, af[0], bf[0]);
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
        if (kk + 1 < BK / 16) load_frags(st, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
          for (int jj = 0; jj < TN; ++jj)
            acc[mi][jj] = kDirect ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf[kk & 1][jj], af[kk & 1][mi], acc[mi][jj], 0, 0, 0)
                                  : __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk & 1][mi], bf[kk & 1][jj], acc[mi][jj], 0, 0, 0);
        if (Cfg::OPT & 64) {
#pragma unroll
          for (int g = 0; g < TM * TN; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
          }
        }
      }
    }
    __syncthreads();  // every wave is done reading the stage buffers

    // the next tile: its first operand tiles are on their way while this one's results go out
    const int out_row0 = cur.row0, out_rows = cur.rows, out_n0 = cur.n0;
    if (nxt.rows > 0) {
      plan(nxt, nxt_voff);
      issue(0);
    }

    if constexpr (kDirect) {
      store_transposed_accumulators<Cfg>(acc, wm, wn, out_row0, out_rows, out_n0, N, dense_rows, C, save0, save1);
      if (nxt.rows <= 0) break;
      cur = nxt;
      continue;
    }
    const int col0 = out_n0 + wn * WNO;
    const int passes = (kDual && save0 != nullptr) ? 3 : 1;
    for (int pass = 0; pass < passes; ++pass) {
#pragma unroll
      for (int h = 0; h < kHalves; ++h) {
        const int row_base = wm * WM + h * WMH;
#pragma unroll
        for (int mh = 0; mh < TMH; ++mh) {
          const int mi = h * TMH + mh;
#pragma unroll
          for (int jj = 0; jj < TNO; ++jj) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int r = mh * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
              float v;
              if (kDual) {
                const float g = bf16_round_fast(acc[mi][jj][i]);
                const float u = bf16_round_fast(acc[mi][jj + TN / 2][i]);
                v = pass == 0 ? silu_rcp(g) * u : (pass == 1 ? g : u);
              } else {
                v = acc[mi][jj][i];
              }
              cw[r * CS + jj * 32 + (lane & 31)] = bf16_bits_fast(v);
            }
          }
        }
        uint16_t* const out = pass == 0 ? C : (pass == 1 ? save0 : save1);
        if (pass == 0)
          store_wave_block<WMH, WNO, CS, (Cfg::OPT & 32768) != 0>(cw, lane, out, N, (size_t)out_row0 + row_base,
                                                                 out_rows - row_base, col0);
        else
          store_wave_block<WMH, WNO, CS, true>(cw, lane, out, N, (size_t)out_row0 + row_base, out_rows - row_base, col0);
      }
    }
    if (nxt.rows <= 0) break;
    cur = nxt;
  }
}


// Grid and schedule of a persistent launch over `tiles_grid` (a multiple of 8) tiles on a device with
// `cus` CUs (a multiple of 8): see the two schedules above.
struct PersistentSchedule {
  int64_t grid;
  int window, chunk;
};
inline PersistentSchedule persistent_schedule(int64_t tiles_grid, int cus, int tiles_per_workgroup) {
  if (tiles_grid <= cus) return {tiles_grid, 0, 0};  // a tile per workgroup, no second tile to look up
  if (tiles_per_workgroup <= 0) return {cus, 0, 0};
  const int window = cus / 8;
  const int64_t per_xcd = tiles_grid / 8, span = (int64_t)window * tiles_per_workgroup;
  return {8 * ((per_xcd + span - 1) / span) * window, window, tiles_per_workgroup};
}

// The two configurations the library launches: 256 x 256 output tiles (gate and up share the A
// tile: 128 + 128 columns), 64-deep k steps, two LDS stages, 8 waves, B tiles in 4 x 64 blocks
// (whole 128-byte lines per eight lanes; about 1 % faster than 4 x 16 blocks at 131072 rows).
using GateUpCfg = DmaGemmCfg<256, 128, 64, 4, 2, true, 2, 16 + 128>;
// tiles per workgroup of a persistent launch (0: one workgroup per CU walks them all).  The down
// projection measures 0.8 % faster fully persistent (and sheds 7 % of its L2 misses with 4); gate/up
// runs as fast either way and sheds a quarter of them.
template <typename Cfg>
constexpr int kTilesPerWorkgroup = Cfg::kDual ? 4 : 0;
using DownCfg = DmaGemmCfg<256, 256, 64, 2, 4, false, 2, 16 + 64 + 128 + 32768>;  // 537 MB of results at C3: streamed out
// Few rows per group (decode-sized batches): the layer streams every expert matrix once and
// is bound by HBM, so the tiles are only 64 rows tall to keep the padded-row MFMA work below
// the time the weights take to arrive, and the k steps 32 deep so that four workgroups of four
// waves fit a CU: at 64 experts x 11 column tiles every workgroup of the launch is then resident
// at once and all of them stream together (with 64-deep steps and two workgroups per CU the
// last third of the workgroups ran alone on a mostly idle memory system: 0.140 vs 0.126 ms).
using GateUpSmallCfg = DmaGemmCfg<64, 128, 32, 1, 4, true, 2, 16 + 128>;
using DownSmallCfg = DmaGemmCfg<64, 256, 32, 1, 4, false, 2, 16>;
// The same tiles when nearly every group fits one tile (a decode step): each expert matrix is then
// read by exactly one row of workgroups, and non-temporal loads stream it past the L2
// (64 tokens, 64 experts: gate/up 0.126 -> 0.110 ms = 6.7 TB/s, down 0.061 -> 0.054 ms = 6.8 TB/s).
using GateUpTinyCfg = DmaGemmCfg<64, 128, 32, 1, 4, true, 2, 16 + 128 + 4096>;
using DownTinyCfg = DmaGemmCfg<64, 256, 32, 1, 4, false, 2, 16 + 4096>;

}  // namespace jtmoe
