// The grouped bf16 GEMM of grouped_gemm_dma.hpp (same tiles, same LDS layouts, same LDS-DMA operand
// loads) as ONE software pipeline that runs through all the tiles of a workgroup:
//
//   * NSTAGE operand stages are in flight.  The loads of k step c + NSTAGE are issued during step c,
//     as soon as the stage they overwrite has been read for the last time, so a load has NSTAGE - 1
//     steps to arrive instead of one, and the wait in front of the barrier (s_waitcnt vmcnt(n),
//     n > 0) leaves the younger stages in flight.
//   * The barrier of a step stands before its LAST 16-deep sub-step, and guarantees the NEXT step's
//     stage: the first fragments of step c + 1 are read from LDS while the matrix cores work on the
//     last sub-step of step c, so no wave starts a step by waiting for LDS.
//   * The stream of k steps does not stop at the end of a tile: the loads of the next tile's first
//     steps are issued during the last steps of the current one, and its first fragments are in
//     registers before the epilogue.  The epilogue writes the accumulators straight to memory (they
//     hold transposed blocks, so a lane owns runs of neighbouring columns): no LDS, no barrier.
//   * Nothing in the steady state returns data to vector registers through the memory pipe (the
//     row map of the next tile arrives by LDS-DMA as well, group sizes and offsets are read from a copy
//     in LDS), so the compiler never inserts a wait that drains the operand loads.
//
// Requirements: those of grouped_gemm_dma.hpp, and K / BK >= 2 * NSTAGE, a result of at most 0x7ffe0000
// bytes, with a row map fewer than 2^27 rows and row_div <= 32; launch with a multiple of 8 workgroups
// (persistent schedule).
#pragma once

#include "grouped_gemm_dma.hpp"

#include <type_traits>

namespace jtmoe {

// 4 bytes per lane from a raw buffer into LDS at lds_base + lane * 4 (zeros past the end)
__device__ __forceinline__ void buffer_load_lds4(i32x4_t rsrc, unsigned lds_base, int voffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds"
               :
               : "s"(lds_base), "v"(voffset), "s"(rsrc)
               : "memory", "m0");
}

template <typename Cfg>
struct StreamLayout {
  static constexpr int kRowBufBytes = Cfg::NT * 4;
  static constexpr int kPipeBytes = Cfg::NSTAGE * Cfg::STAGE_BYTES;
  static constexpr int kRowBufBase = kPipeBytes;
  static constexpr int kGroupBase = kRowBufBase + kRowBufBytes;  // group sizes, then first rows: 2 x JTMOE_MAX_EXPERTS ints
  static constexpr int kSmemBytes = kGroupBase + 2 * JTMOE_MAX_EXPERTS * 4;
  static_assert(kSmemBytes <= 160 * 1024, "LDS budget");
  static_assert(Cfg::BM <= Cfg::NT, "one row-map entry per thread");
};

// kNT = false: C = A @ B[e] with B[e] stored [K, N] (the forward products; kDual: two of them sharing the A tile).
// kNT = true:  C = sum over segs segments of A_s @ B_s[e]^T with B_s[e] stored [N, K] (the data gradients of
//              the backward pass, grouped_gemm_bwd.hpp): the B tile is then k-contiguous like the A tile,
//              lives in LDS in the same swizzled row layout and is read with ds_read_b128; the k loop
//              runs through the segments one after the other.
template <typename Cfg, bool kNT>
__device__ __forceinline__ void stream_gemm_body(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ A1, const uint16_t* __restrict__ B0,
    const uint16_t* __restrict__ B1, uint16_t* __restrict__ C, const int32_t* __restrict__ group_sizes,
    const int32_t* __restrict__ offsets, int E, int dense_rows, int Kdim, int N, int mtiles, int ntiles_n,
    const int32_t* __restrict__ row_map, int row_div, int a_rows, uint16_t* __restrict__ save0,
    uint16_t* __restrict__ save1, int segs, int window, int chunk) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT, NS = Cfg::NSTAGE;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, WM = Cfg::WM, WN = Cfg::WN;
  constexpr int CPRA = Cfg::CPRA, KK = BK / 16, LPS = Cfg::LPS;
  constexpr bool kDual = Cfg::kDual;
  using L = StreamLayout<Cfg>;
  static_assert(KK % 2 == 0, "fragment double buffer wants an even number of sub-steps");
  static_assert(kNT || (Cfg::OPT & 128) != 0, "weight tiles in 4 x 64 blocks");
  static_assert(!kNT || !kDual, "the transposed-B form has one output per tile");
  static_assert(!kNT || (BN * CPRA) % NT == 0, "the B tile must divide evenly over the threads");
  // Timing experiments of the stand-alone check's time_ablation mode, which bounds what any schedule of
  // this loop can reach (wrong results by construction, never launched by the library): OPT & 256 leaves out the operand loads of the steady part of the k loop, OPT & 512 its
  // fragment reads (the MFMAs then run on the fragments read once before the loop).
  // OPT & 1024 makes every load of the steady part fetch the tile's first k step again (operands that
  // are in the nearest cache: the cost of issuing the loads without the memory system behind them).
  constexpr bool kNoLoads = (Cfg::OPT & 256) != 0, kNoFragReads = (Cfg::OPT & 512) != 0;
  constexpr bool kSameTile = (Cfg::OPT & 1024) != 0;
  extern __shared__ __align__(16) unsigned char smem_raw[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WAVES_N, wn = wave - wm * Cfg::WAVES_N;
  const bool gather = row_map != nullptr;
  const int nk1 = Kdim / BK;               // k steps of one segment
  const int nk = kNT ? nk1 * segs : nk1;   // k steps of a tile

  // ---- schedule (as in grouped_gemm_dma_persistent_kernel) ----
  // Group sizes and first rows are copied into LDS once; every tile look-up scans them from there, so
  // that no look-up touches global memory while operand loads are in flight.
  int* const gs_l = reinterpret_cast<int*>(smem_raw + L::kGroupBase);
  int* const row0_l = gs_l + JTMOE_MAX_EXPERTS;
  int real_mtiles = mtiles;
  if (group_sizes) {
    for (int e = tid; e < JTMOE_MAX_EXPERTS; e += NT) {
      gs_l[e] = e < E ? group_sizes[e] : 0;
      row0_l[e] = e < E ? offsets[e] : 0;
    }
    __syncthreads();
    real_mtiles = __builtin_amdgcn_readfirstlane(group_scan(BM, gs_l, JTMOE_MAX_EXPERTS).total);
  }
  const int total = real_mtiles * ntiles_n;
  const int per_xcd = (total + 7) >> 3;
  const int xcd = (int)blockIdx.x & 7;
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
    if (group_sizes) {
      const TileRows tr = locate_tile(group_scan(BM, gs_l, JTMOE_MAX_EXPERTS), mt, BM, row0_l);
      t.expert = __builtin_amdgcn_readfirstlane(tr.expert);
      t.row0 = __builtin_amdgcn_readfirstlane(tr.row0);
      t.rows = __builtin_amdgcn_readfirstlane(tr.rows);
    } else {
      t.row0 = mt * BM;
      t.rows = min(BM, dense_rows - mt * BM);
    }
    t.n0 = nt * BN;
    return t;
  };

  // ---- the load plan: descriptors and offsets of the tile whose operands are being requested.  The
  // last NS steps of a tile request the next tile's first steps, so the plan switches over to the next
  // tile NS steps before the current tile ends; nothing else of the current tile depends on it. ----
  constexpr int NSEG = kNT ? 2 : 1;                        // A descriptors (one per segment)
  constexpr int NBD = kNT ? 2 : Cfg::NSUB;                 // B descriptors (per segment / per 128-column sub-tile)
  constexpr int B_LOADS = kNT ? BN * CPRA / NT : Cfg::NSUB;  // entries of b_voff
  static_assert(!kNT || B_LOADS == Cfg::NSUB * Cfg::BSUB_LOADS, "a stage has LPS loads in either form");
  struct Plan {
    i32x4_t a_rsrc[NSEG];
    i32x4_t b_rsrc[NBD];
    int a_voff[Cfg::A_LOADS];
    int b_voff[B_LOADS];
  };
  const int a_r = tid / CPRA, a_slot = tid - a_r * CPRA;
  const int a_c = a_slot ^ ((a_r / (16 / CPRA)) % CPRA);
  const int b_blk_id = tid >> 5;
  const int b_k = (b_blk_id >> 1) * 4 + ((tid >> 3) & 3);
  const int b_c = (b_blk_id & 1) * 8 + ((tid & 7) ^ (((tid >> 4) & 1) << 2));
  const unsigned lds0 = lds_byte_addr(smem_raw);
  const unsigned wave_lds = lds0 + wave * 1024;
  int* const rowbuf = reinterpret_cast<int*>(smem_raw + L::kRowBufBase);

  // everything of a plan but the A row offsets
  auto plan_tile = [&](Plan& p, const Tile& t) {
    const size_t wofs = (size_t)t.expert * Kdim * N;
    if constexpr (kNT) {
#pragma unroll
      for (int sg = 0; sg < 2; ++sg) {
        const uint16_t* a = (sg == 1 && segs > 1) ? A1 : A;
        const uint16_t* b = (sg == 1 && segs > 1) ? B1 : B0;
        p.a_rsrc[sg] = gather ? make_rsrc(a, a_rows * Kdim * 2) : make_rsrc(a + (size_t)t.row0 * Kdim, t.rows * Kdim * 2);
        p.b_rsrc[sg] = make_rsrc(b + wofs, N * Kdim * 2);  // rows of B past N lie outside it and read as zeros
      }
      // the B tile's rows are output columns: row n0 + r of B[e], the same slots and swizzle as the A tile
#pragma unroll
      for (int j = 0; j < B_LOADS; ++j) p.b_voff[j] = ((t.n0 + a_r + j * (NT / CPRA)) * Kdim + a_c * 8) * 2;
    } else {
#pragma unroll
      for (int u = 0; u < Cfg::NSUB; ++u) p.b_rsrc[u] = make_rsrc((kDual && u == 1 ? B1 : B0) + wofs, Kdim * N * 2);
      p.a_rsrc[0] = gather ? make_rsrc(A, a_rows * Kdim * 2) : make_rsrc(A + (size_t)t.row0 * Kdim, t.rows * Kdim * 2);
#pragma unroll
      for (int u = 0; u < Cfg::NSUB; ++u) p.b_voff[u] = (b_k * N + t.n0 + (kDual ? 0 : u * 128) + b_c * 8) * 2;
    }
#pragma unroll
    for (int j = 0; j < Cfg::A_LOADS; ++j) p.a_voff[j] = ((a_r + j * (NT / CPRA)) * Kdim + a_c * 8) * 2;
  };
  // gathered rows: the offsets come from row ids (rows past the end of the group read as zeros)
  // row_map entries are divided by row_div (the top-k of the routing) with a multiply: for
  // 0 <= n < 2^27 and 1 <= d <= 32, floor(n / d) == (n * ceil(2^32 / d)) >> 32  (the product stays
  // below 2^60, and n * (d * ceil(2^32 / d) - 2^32) < 2^27 * 32 = 2^32)
  const unsigned long long div_magic = ((1ull << 32) + (unsigned)row_div - 1) / (unsigned)row_div;
  auto plan_rows = [&](Plan& p, const Tile& t, auto row_id) {
#pragma unroll
    for (int j = 0; j < Cfg::A_LOADS; ++j) {
      const int r = a_r + j * (NT / CPRA);
      const int src = (int)(((unsigned long long)(unsigned)row_id(r) * div_magic) >> 32);
      p.a_voff[j] = r < t.rows ? (src * Kdim + a_c * 8) * 2 : 0x70000000;
    }
  };
  // load i of the LPS loads of a stage (A loads first, then B) of k step kt of the planned tile
  auto issue_one = [&](const Plan& p, int kt, int stage, int i) {
    const unsigned base = wave_lds + stage * Cfg::STAGE_BYTES;
    if constexpr (kNT) {
      const bool second = kt >= nk1;  // uniform: the step belongs to the second segment
      const int k0 = (second ? kt - nk1 : kt) * BK;
      if (i < Cfg::A_LOADS)
        buffer_load_lds16(second ? p.a_rsrc[1] : p.a_rsrc[0], base + i * NT * 16, p.a_voff[i], k0 * 2);
      else
        buffer_load_lds16(second ? p.b_rsrc[1] : p.b_rsrc[0], base + Cfg::A_BYTES + (i - Cfg::A_LOADS) * NT * 16,
                          p.b_voff[i - Cfg::A_LOADS], k0 * 2);
    } else {
      const int k0 = kt * BK;
      if (i < Cfg::A_LOADS) {
        buffer_load_lds16(p.a_rsrc[0], base + i * NT * 16, p.a_voff[i], k0 * 2);
      } else {
        const int u = (i - Cfg::A_LOADS) / Cfg::BSUB_LOADS, jb = (i - Cfg::A_LOADS) % Cfg::BSUB_LOADS;
        buffer_load_lds16(p.b_rsrc[u], base + Cfg::A_BYTES + u * Cfg::BSUB_BYTES + jb * NT * 16,
                          p.b_voff[u] + jb * (NT / 16) * N * 2, k0 * N * 2);
      }
    }
  };
  auto issue = [&](const Plan& p, int kt, int stage) {
#pragma unroll
    for (int i = 0; i < LPS; ++i) issue_one(p, kt, stage, i);
  };

  // ---- fragment addresses of this lane (bytes inside a stage) ----
  const int a_row = wm * WM + (lane & 31);
  const int a_sw = (a_row / (16 / CPRA)) % CPRA;
  const int a_rowoff = a_row * (BK * 2);
  const int b_laneoff = ((lane & 15) >> 2) * 128 + (lane & 3) * 8 + ((lane >> 4) & 1) * 32 + (lane >> 5) * 2048;
  const int half_swap = ((lane >> 3) & 1) * 64;
  int b_blk[TN];
  // kNT: the B tile in the A tile's layout, this lane's row = its output column
  const int bt_row = wn * WN + (lane & 31);
  const int bt_sw = (bt_row / (16 / CPRA)) % CPRA;
  const int bt_rowoff = Cfg::A_BYTES + bt_row * (BK * 2);
#pragma unroll
  for (int jj = 0; jj < TN; ++jj) {
    int col;
    if (kDual)
      col = (jj < TN / 2 ? 0 : BN) + wn * (WN / 2) + (jj % (TN / 2)) * 32;
    else
      col = wn * WN + jj * 32;
    const int u = col >> 7;
    b_blk[jj] = Cfg::A_BYTES + u * Cfg::BSUB_BYTES + ((col & 127) >> 6) * 512 + (col & 63) * 2 +
                ((col & 32) ? -half_swap : half_swap);
  }
  auto load_frag_a = [&](int stage, int kk, int mi) -> bf16x8_t {
    const unsigned char* st = smem_raw + stage * Cfg::STAGE_BYTES;
    return *reinterpret_cast<const bf16x8_t*>(st + a_rowoff + mi * 32 * BK * 2 + (((kk * 2 + (lane >> 5)) ^ a_sw) << 4));
  };
  auto load_frag_b = [&](int stage, int kk, int jj) -> bf16x8_t {
    if constexpr (kNT) {
      const unsigned char* st = smem_raw + stage * Cfg::STAGE_BYTES;
      return *reinterpret_cast<const bf16x8_t*>(st + bt_rowoff + jj * 32 * BK * 2 + (((kk * 2 + (lane >> 5)) ^ bt_sw) << 4));
    }
    const unsigned char* p = smem_raw + stage * Cfg::STAGE_BYTES + b_blk[jj] + b_laneoff + kk * (4 * 8 * 128);
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p));
    const s16x4_t hi =
        __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p + 8 * 128));
    const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8_t, both);
  };
  auto load_frags = [&](int stage, int kk, bf16x8_t* af, bf16x8_t* bf) {
#pragma unroll
    for (int mi = 0; mi < TM; ++mi) af[mi] = load_frag_a(stage, kk, mi);
#pragma unroll
    for (int jj = 0; jj < TN; ++jj) bf[jj] = load_frag_b(stage, kk, jj);
  };

  // ---- first tile: plan, all NS stages requested, first fragments read ----
  Tile cur = locate(idx);
  if (cur.rows <= 0) return;
  Plan pl;
  plan_tile(pl, cur);
  // (a partial tile's rows past the group end are not read: the map may end with the group)
  if (gather) plan_rows(pl, cur, [&](int r) { return r < cur.rows ? row_map[cur.row0 + r] : 0; });
#pragma unroll
  for (int s = 0; s < NS; ++s) issue(pl, s, s);
  f32x16_t acc[TM][TN];
  bf16x8_t af[2][TM], bf[2][TN];
  wait_and_barrier<(NS - 1) * LPS>();
  load_frags(0, 0, af[0], bf[0]);
  if (kNoFragReads) load_frags(0, 1, af[1], bf[1]);
  int cs = 0;  // stage of the current k step

  while (true) {
    const bool wave_has_rows = wm * WM < cur.rows && cur.n0 + wn * Cfg::WNO < N;
    idx += stride;
    --left;
    const Tile nxt = locate(left > 0 ? idx : 0x3fffffff);
    const bool have_next = nxt.rows > 0;

    // row ids of the next tile: one LDS-DMA dword per thread, requested now and read NS steps before
    // this tile ends (it is older than every operand load issued from here on, so the waits below
    // cover it)
    if (gather && have_next) {
      const i32x4_t map_rsrc = make_rsrc(row_map + nxt.row0, nxt.rows * 4);
      buffer_load_lds4(map_rsrc, lds0 + L::kRowBufBase + wave * 256, lane * 4 + wave * 256);
    }

    // MFMAs of one 16-deep sub-step on fragment set `cur_set`, interleaved by the scheduler with the
    // LDS reads (two per MFMA) that were written before them
    // (`first`: the tile's first sub-step, which accumulates onto zero instead of clearing 128 registers)
    auto mfma_substep = [&](int cur_set, bool first = false) {
      if (Cfg::OPT & 32) __builtin_amdgcn_s_setprio(1);
      f32x16_t zero;
#pragma unroll
      for (int i = 0; i < 16; ++i) zero[i] = 0.0f;
#pragma unroll
      for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int jj = 0; jj < TN; ++jj)
          acc[mi][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf[cur_set][jj], af[cur_set][mi],
                                                                first ? zero : acc[mi][jj], 0, 0, 0);
#pragma unroll
      for (int g = 0; g < TM * TN; ++g) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      if (Cfg::OPT & 32) __builtin_amdgcn_s_setprio(0);
    };
    // sub-steps 0 .. KK-2 of a step: fragments of the following sub-step are requested, then this one's MFMAs
    auto leading_substeps = [&](auto first_tag) {
#pragma unroll
      for (int kk = 0; kk < KK - 1; ++kk) {
        if (!kNoFragReads) load_frags(cs, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
        mfma_substep(kk & 1, decltype(first_tag)::value && kk == 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    };

    // ---- steady part: every step has NS successors inside this tile ----
    int j = 0;
    if (wave_has_rows) {
      auto steady_step = [&](auto first_tag) {
        leading_substeps(first_tag);
        // the next step's stage has arrived (own loads: the wait; everyone's: the barrier), and every
        // wave holds its last fragments of the current stage, which is therefore free
        wait_and_barrier<(NS - 2) * LPS>();
        __builtin_amdgcn_sched_barrier(0);
        // last sub-step, in a fixed order: after each of its MFMAs one operand load of step j + NS
        // (into the stage just released) and one fragment read of step j + 1 are issued
        const int ns = (cs + 1) & (NS - 1);
        constexpr int cur_set = (KK - 1) & 1;
        if (Cfg::OPT & 32) __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int g = 0; g < TM * TN; ++g) {
          acc[g / TN][g % TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf[cur_set][g % TN], af[cur_set][g / TN],
                                                                        acc[g / TN][g % TN], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          constexpr int kLoadsPer = (LPS + TM * TN - 1) / (TM * TN);
#pragma unroll
          for (int q = 0; q < kLoadsPer; ++q)
            if (!kNoLoads && g * kLoadsPer + q < LPS) issue_one(pl, kSameTile ? 0 : j + NS, cs, g * kLoadsPer + q);
          if (kNoFragReads) {
          } else if (g < TM)
            af[0][g] = load_frag_a(ns, 0, g);
          else if (g < TM + TN)
            bf[0][g - TM] = load_frag_b(ns, 0, g - TM);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (Cfg::OPT & 32) __builtin_amdgcn_s_setprio(0);
        cs = ns;
      };
      steady_step(std::true_type{});  // nk >= 2 NS: the steady part has at least NS steps
      for (j = 1; j < nk - NS; ++j) steady_step(std::false_type{});
    } else {
      // a tile at the end of a group: this wave's rows lie past it; it only keeps the loads going
#pragma unroll
      for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int jj = 0; jj < TN; ++jj)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[mi][jj][i] = 0.0f;
      for (; j < nk - NS; ++j) {
        wait_and_barrier<(NS - 2) * LPS>();
        issue(pl, j + NS, cs);
        cs = (cs + 1) & (NS - 1);
      }
    }

    // ---- last NS steps: requests go to the next tile, if there is one ----
    for (; j < nk; ++j) {
      if (wave_has_rows) leading_substeps(std::false_type{});
      // k steps of this workgroup's stream after this one (only the next tile counts: a load is
      // never issued more than NS <= nk steps ahead)
      const int rem = (nk - 1 - j) + (have_next ? nk : 0);
      if (rem > 0) {
        if (rem >= NS - 1)
          wait_and_barrier<(NS - 2) * LPS>();
        else if (NS > 3 && rem == NS - 2)
          wait_and_barrier<(NS > 3 ? NS - 3 : 0) * LPS>();
        else
          wait_and_barrier<0>();
        if (rem >= NS) {
          const int kt = j + NS - nk;  // a step of the next tile
          if (kt == 0) {               // from here on the plan is the next tile's
            plan_tile(pl, nxt);
            if (gather) plan_rows(pl, nxt, [&](int r) { return rowbuf[r]; });
          }
          issue(pl, kt, cs);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      cs = (cs + 1) & (NS - 1);
      if (rem > 0) load_frags(cs, 0, af[0], bf[0]);
      if (wave_has_rows) mfma_substep((KK - 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- epilogue: straight from the accumulators to memory (no LDS, no barrier) ----
    store_transposed_accumulators<Cfg>(acc, wm, wn, cur.row0, cur.rows, cur.n0, N, dense_rows, C, save0, save1);
    if (!have_next) break;
    cur = nxt;
  }
}

template <typename Cfg>
__global__ __launch_bounds__(Cfg::NT) void grouped_gemm_stream_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B0, const uint16_t* __restrict__ B1,
    uint16_t* __restrict__ C, const int32_t* __restrict__ group_sizes, const int32_t* __restrict__ offsets, int E,
    int dense_rows, int Kdim, int N, int mtiles, int ntiles_n, const int32_t* __restrict__ row_map, int row_div,
    int a_rows, uint16_t* __restrict__ save0, uint16_t* __restrict__ save1, int window, int chunk) {
  stream_gemm_body<Cfg, false>(A, nullptr, B0, B1, C, group_sizes, offsets, E, dense_rows, Kdim, N, mtiles, ntiles_n,
                               row_map, row_div, a_rows, save0, save1, 1, window, chunk);
}

// The transposed-B form: the arguments of grouped_gemm_nt_kernel (grouped_gemm_bwd.hpp) plus the schedule.
// Requirements: (Kdim / BK) * segs >= 2 * NSTAGE, and those of the kernel above.
template <typename Cfg>
__global__ __launch_bounds__(Cfg::NT) void grouped_gemm_stream_nt_kernel(
    const uint16_t* __restrict__ A0, const uint16_t* __restrict__ A1, const uint16_t* __restrict__ B0,
    const uint16_t* __restrict__ B1, uint16_t* __restrict__ C, const int32_t* __restrict__ group_sizes,
    const int32_t* __restrict__ offsets, int E, int dense_rows, int Kdim, int N, int mtiles, int ntiles_n,
    const int32_t* __restrict__ row_map, int row_div, int a_rows, int segs, int window, int chunk) {
  stream_gemm_body<Cfg, true>(A0, A1, B0, B1, C, group_sizes, offsets, E, dense_rows, Kdim, N, mtiles, ntiles_n,
                              row_map, row_div, a_rows, nullptr, nullptr, segs, window, chunk);
}

// The configuration the library launches for gate/up (routed and shared experts): the tile of GateUpCfg
// with 32-deep steps and four stages.  Measured on 64 groups of 2048 gathered rows x 2048 x 1408
// (alternating in one process): 1.306 ms against 1.400-1.409 ms for grouped_gemm_dma_persistent_kernel
// and 1.315-1.320 ms for 64-deep steps with two stages.
using GateUpStreamCfg = DmaGemmCfg<256, 128, 32, 4, 2, true, 4, 16 + 128>;
// Variants kept for the stand-alone check and its timings (time_stream, time_down): 64-deep steps with
// two stages, and the down projection's tile (within 2 % of grouped_gemm_dma_persistent_kernel, which
// the library keeps for that launch, at 12, 22 and 44 k steps per tile).
using GateUpStream2Cfg = DmaGemmCfg<256, 128, 64, 4, 2, true, 2, 16 + 128>;
using DownStreamCfg = DmaGemmCfg<256, 256, 32, 2, 4, false, 4, 16 + 128 + 32768>;
using DownStream2Cfg = DmaGemmCfg<256, 256, 64, 2, 4, false, 2, 16 + 128 + 32768>;
// The data-gradient products of the backward pass (transposed-B form): 256 x 256 tiles, 2 x 4 waves.
// Checked and timed by the stand-alone check (time_stream_nt) against grouped_gemm_nt_kernel, which
// the library launches: the transposed-B form measures equal or slower there.
using DgradStreamCfg = DmaGemmCfg<256, 256, 32, 2, 4, false, 4, 16 + 128>;

}  // namespace jtmoe
