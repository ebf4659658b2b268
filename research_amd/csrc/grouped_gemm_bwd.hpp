// The two grouped GEMM forms the backward pass of the expert FFN needs, built from
// the same parts as grouped_gemm_dma.hpp (tiles written into LDS by
// buffer_load ... lds, two stages, v_mfma_f32_32x32x16_bf16):
//
//   "NT"  C[rows of group e, :] = sum over segments s of  A_s[rows of e, :] @ B_s[e]^T
//         B_s[e] is [N, K] row-major, i.e. an expert matrix exactly as the forward
//         pass stores it, used transposed (the data gradient of y = x W is dy W^T).
//         Both operands are k-contiguous, so both tiles use the row layout with the
//         XOR swizzle and are read with ds_read_b128.
//
//   "TN"  C_i[e] = P[rows of group e, :]^T @ D_i[rows of group e, :]        (i = 0, 1)
//         one [KA, N] matrix per group, reduced over the rows of the group (the weight
//         gradient of y = x W is x^T dy).  Both operands are row-major with the
//         reduction index as the row, so both tiles use the 4 x 16 block layout and are
//         read with the transposing ds_read_b64_tr_b16.  An empty group yields zeros.
//
// Either kernel can fetch operand rows through a row map (packed row j reads row
// row_map[j] / row_div), the way the forward gate/up launch does, so neither the
// permuted activations nor the permuted output gradient are ever written to memory.
//
// Requirements: bf16, K % 64 == 0 (NT), row lengths multiples of 8, 16-byte aligned
// pointers, every operand smaller than 2 GiB.
#pragma once

#include "grouped_gemm_dma.hpp"

namespace jtmoe {

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int OPT_ = 16>
struct NtGemmCfg {
  static constexpr int BM = BM_, BN = BN_, BK = 64, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, OPT = OPT_;
  static constexpr int NT = WAVES_M * WAVES_N * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int A_LOADS = BM * 8 / NT, B_LOADS = BN * 8 / NT;
  static constexpr int CS = WN + 8;
  static constexpr size_t EPI_BYTES = (size_t)WAVES_M * WAVES_N * WM * CS * 2;
  static constexpr size_t PIPE_BYTES = 2 * (size_t)STAGE_BYTES;
  static constexpr size_t SMEM_BYTES = PIPE_BYTES > EPI_BYTES ? PIPE_BYTES : EPI_BYTES;
  static constexpr int GROUP_M = 4;
  static_assert((BM * 8) % NT == 0 && (BN * 8) % NT == 0, "tiles must divide evenly over the threads");
  static_assert((NT / 8) % 16 == 0, "swizzle must not depend on the load index");
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be made of 32x32x16 MFMAs");
  static_assert(SMEM_BYTES <= 160 * 1024, "LDS budget");
};

// A0/A1: [rows, Kdim] (or [a_rows, Kdim] fetched through row_map); B0/B1: [E, N, Kdim];
// C: [rows, N].  segs = 1 uses A0/B0 only; segs = 2 adds A1 @ B1^T into the same output.
template <typename Cfg>
__global__ __launch_bounds__(Cfg::NT) void grouped_gemm_nt_kernel(
    const uint16_t* __restrict__ A0, const uint16_t* __restrict__ A1, const uint16_t* __restrict__ B0,
    const uint16_t* __restrict__ B1, uint16_t* __restrict__ C, const int32_t* __restrict__ group_sizes,
    const int32_t* __restrict__ offsets, int E, int dense_rows, int Kdim, int N, int mtiles, int ntiles_n,
    const int32_t* __restrict__ row_map, int row_div, int a_rows, int segs) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, WM = Cfg::WM, WN = Cfg::WN;
  extern __shared__ __align__(16) unsigned char smem_raw[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WAVES_N, wn = wave - wm * Cfg::WAVES_N;
  const bool gather = row_map != nullptr;

  // Persistent workgroups, as in grouped_gemm_dma_persistent_kernel: this one walks the tiles
  // idx, idx + stride, ... of its XCD's contiguous range of the logical order.
  GroupScan scan;
  int real_mtiles = mtiles;
  if (group_sizes) {
    scan = group_scan(BM, group_sizes, E);
    real_mtiles = __builtin_amdgcn_readfirstlane(scan.total);
  }
  const int total = real_mtiles * ntiles_n;
  const int per_xcd = (total + 7) >> 3;
  const int xcd = (int)blockIdx.x & 7, stride = max(1, (int)gridDim.x >> 3);
  int idx = (int)blockIdx.x >> 3;
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
  i32x4_t a_rsrc[2], b_rsrc[2];
  // both tiles: slot s = j*NT + tid -> row s/8, slot-in-row s%8 holds source chunk (s%8) ^ ((row/2)%8)
  const int l_r = tid >> 3, l_slot = tid & 7;
  const int l_c = l_slot ^ ((l_r >> 1) & 7);
  int a_voff[Cfg::A_LOADS];
  int b_voff = 0;
  auto row_offsets = [&](const Tile& t, int* voff) {
#pragma unroll
    for (int j = 0; j < Cfg::A_LOADS; ++j) {
      const int r = l_r + j * (NT / 8);
      if (gather)
        voff[j] = r < t.rows ? ((row_map[t.row0 + r] / row_div) * Kdim + l_c * 8) * 2 : 0x70000000;
      else
        voff[j] = (r * Kdim + l_c * 8) * 2;
    }
  };
  auto plan = [&](const Tile& t, const int* voff) {
    const size_t wofs = (size_t)t.expert * Kdim * N;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const uint16_t* a = s ? A1 : A0;
      const uint16_t* b = s ? B1 : B0;
      if (s >= segs) {
        a = A0;
        b = B0;
      }
      a_rsrc[s] = gather ? make_rsrc(a, a_rows * Kdim * 2) : make_rsrc(a + (size_t)t.row0 * Kdim, t.rows * Kdim * 2);
      // rows of B past N lie outside the descriptor and read as zeros
      b_rsrc[s] = make_rsrc(b + wofs, N * Kdim * 2);
    }
#pragma unroll
    for (int j = 0; j < Cfg::A_LOADS; ++j) a_voff[j] = voff[j];
    b_voff = ((t.n0 + l_r) * Kdim + l_c * 8) * 2;
  };
  const unsigned lds0 = lds_byte_addr(smem_raw);
  const unsigned wave_lds = lds0 + wave * 1024;
  const int nk1 = Kdim / BK;
  const int nk = nk1 * segs;

  auto issue = [&](int kt) {
    const unsigned base = wave_lds + (kt & 1) * Cfg::STAGE_BYTES;
    const bool second = kt >= nk1;
    const int k0 = (second ? kt - nk1 : kt) * BK;
    const i32x4_t ar = second ? a_rsrc[1] : a_rsrc[0];
    const i32x4_t br = second ? b_rsrc[1] : b_rsrc[0];
#pragma unroll
    for (int j = 0; j < Cfg::A_LOADS; ++j) buffer_load_lds16(ar, base + j * NT * 16, a_voff[j], k0 * 2);
#pragma unroll
    for (int j = 0; j < Cfg::B_LOADS; ++j)
      buffer_load_lds16(br, base + Cfg::A_BYTES + j * NT * 16, b_voff + j * (NT / 8) * Kdim * 2, k0 * 2);
  };

  const int sw = ((lane & 31) >> 1) & 7;
  const int a_rowoff = (wm * WM + (lane & 31)) * (BK * 2);
  const int b_rowoff = Cfg::A_BYTES + (wn * WN + (lane & 31)) * (BK * 2);

  auto load_frags = [&](const unsigned char* st, int kk, bf16x8_t* af, bf16x8_t* bf) {
    const int chunk = ((kk * 2 + (lane >> 5)) ^ sw) << 4;
#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
      af[mi] = *reinterpret_cast<const bf16x8_t*>(st + a_rowoff + mi * 32 * BK * 2 + chunk);
#pragma unroll
    for (int jj = 0; jj < TN; ++jj)
      bf[jj] = *reinterpret_cast<const bf16x8_t*>(st + b_rowoff + jj * 32 * BK * 2 + chunk);
  };

  // Epilogue staging lives above the first stage buffer, which the next tile's first loads fill
  // while the epilogue runs; a wave's block goes out in halves where it does not fit its share.
  constexpr int CS = Cfg::CS;
  constexpr int kStageArea = (int)Cfg::SMEM_BYTES - Cfg::STAGE_BYTES;
  constexpr int kHalves = (NT / 64) * WM * CS * 2 <= kStageArea ? 1 : 2;
  constexpr int TMH = TM / kHalves, WMH = WM / kHalves;
  static_assert((NT / 64) * WMH * CS * 2 <= kStageArea && TM % kHalves == 0, "epilogue staging must fit above stage 0");
  uint16_t* const cw = reinterpret_cast<uint16_t*>(smem_raw + Cfg::STAGE_BYTES) + wave * (WMH * CS);

  Tile cur = locate(idx);
  if (cur.rows <= 0 || nk <= 0) return;
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
    // a wave whose rows all lie past the end of the group skips its fragment reads and MFMAs
    // a wave whose rows lie past the end of the group, or whose columns lie past N, has nothing to add
    const bool wave_has_rows = wm * WM < cur.rows && cur.n0 + wn * WN < N;
    // the tile after this one is looked up now, and its row offsets requested
    idx += stride;
    const Tile nxt = locate(idx);
    int nxt_voff[Cfg::A_LOADS];
    if (nxt.rows > 0) row_offsets(nxt, nxt_voff);

    for (int kt = 0; kt < nk; ++kt) {
      wait_vmcnt<0>();
      __syncthreads();
      if (kt + 1 < nk) issue(kt + 1);
      if (!wave_has_rows) continue;
      const unsigned char* st = smem_raw + (kt & 1) * Cfg::STAGE_BYTES;
      bf16x8_t af[2][TM], bf[2][TN];
      load_frags(st, 0, af[0], bf[0]);
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
        if (kk + 1 < BK / 16) load_frags(st, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
          for (int jj = 0; jj < TN; ++jj)
            acc[mi][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk & 1][mi], bf[kk & 1][jj], acc[mi][jj], 0, 0, 0);
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

    // the first operand tiles of the next tile are on their way while this one's results go out
    const int out_row0 = cur.row0, out_rows = cur.rows, out_n0 = cur.n0;
    if (nxt.rows > 0) {
      plan(nxt, nxt_voff);
      issue(0);
    }
#pragma unroll
    for (int h = 0; h < kHalves; ++h) {
      const int row_base = wm * WM + h * WMH;
#pragma unroll
      for (int mh = 0; mh < TMH; ++mh)
#pragma unroll
        for (int jj = 0; jj < TN; ++jj)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int r = mh * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
            cw[r * CS + jj * 32 + (lane & 31)] = bf16_bits_fast(acc[h * TMH + mh][jj][i]);
          }
      store_wave_block<WMH, WN, CS, (Cfg::OPT & 32768) != 0>(cw, lane, C, N, (size_t)out_row0 + row_base,
                                                            out_rows - row_base, out_n0 + wn * WN);
    }
    if (nxt.rows <= 0) break;
    cur = nxt;
  }
}

// ---------------------------------------------------------------------------------------------

// BK_ rows of the reduction per k step, NSTAGE_ operand stages in LDS: a step's loads are issued
// NSTAGE_ - 1 steps before they are read.  More than two stages only for streamed operands (no row map).
template <int BMO_, int BNO_, int WAVES_M_, int WAVES_N_, bool kDual_, int OPT_ = 16, int BK_ = 64, int NSTAGE_ = 2>
struct TnGemmCfg {
  static constexpr int BMO = BMO_, BNO = BNO_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, OPT = OPT_;
  static constexpr int NSTAGE = NSTAGE_;
  static constexpr bool kDual = kDual_;
  static constexpr int BNE = kDual ? 2 * BNO : BNO;
  static constexpr int PSUB = BMO / 128, DSUB = BNE / 128;  // 128-column sub-tiles of the two operands
  static constexpr int NT = WAVES_M * WAVES_N * 64;
  static constexpr int WM = BMO / WAVES_M, WN = BNE / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int TNO = kDual ? TN / 2 : TN;
  static constexpr int WNO = TNO * 32;
  static constexpr int SUB_BYTES = BK * 256;
  static constexpr int P_BYTES = PSUB * SUB_BYTES;
  static constexpr int STAGE_BYTES = (PSUB + DSUB) * SUB_BYTES;
  static constexpr int SUB_LOADS = BK * 16 / NT;
  static constexpr int CS = WNO + 8;
  static constexpr size_t EPI_BYTES = (size_t)WAVES_M * WAVES_N * WM * CS * 2;
  static constexpr int LOADS_PER_STAGE = (PSUB + DSUB) * SUB_LOADS;
  static constexpr size_t PIPE_BYTES = NSTAGE * (size_t)STAGE_BYTES;
  static constexpr size_t SMEM_BYTES = PIPE_BYTES > EPI_BYTES ? PIPE_BYTES : EPI_BYTES;
  static_assert(NSTAGE >= 2 && NSTAGE <= 4 && (BK == 32 || BK == 64), "two to four stages of 32 or 64 rows");
  static_assert(BMO % 128 == 0 && BNE % 128 == 0, "operand tiles are made of 128-column sub-tiles");
  static_assert((BK * 16) % NT == 0, "sub-tile must divide evenly over the threads");
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be made of 32x32x16 MFMAs");
  static_assert(!kDual || (TN % 2 == 0 && BNO == 128), "dual tiles: one sub-tile per matrix");
  static_assert(SMEM_BYTES <= 160 * 1024, "LDS budget");
};

// P: [rows, KA] (or [p_rows, KA] through row_map when p_gather); D0/D1: [rows, N] (or [d_rows, N]
// through row_map when d_gather); C0/C1: [E, KA, N].
template <typename Cfg>
__global__ __launch_bounds__(Cfg::NT) void grouped_gemm_tn_kernel(
    const uint16_t* __restrict__ P, const uint16_t* __restrict__ D0, const uint16_t* __restrict__ D1,
    uint16_t* __restrict__ C0, uint16_t* __restrict__ C1, const int32_t* __restrict__ group_sizes,
    const int32_t* __restrict__ offsets, int E, int dense_rows, int KA, int N, int mtiles_o, int ntiles_o,
    const int32_t* __restrict__ row_map, int row_div, int p_gather, int d_gather, int gathered_rows,
    int split_chunk) {
  constexpr int BMO = Cfg::BMO, BNO = Cfg::BNO, BK = Cfg::BK, NT = Cfg::NT;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, WM = Cfg::WM, WN = Cfg::WN;
  constexpr bool kDual = Cfg::kDual;
  extern __shared__ __align__(16) unsigned char smem_raw[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WAVES_N, wn = wave - wm * Cfg::WAVES_N;

  // Persistent workgroups: consecutive workgroup ids go round-robin to the 8 XCDs, each XCD owns a
  // contiguous range of (group, tile) pairs (so that all tiles of one group read its rows through
  // the same L2).  A pair's k loop is as long as its group.  With groups of about the same size
  // the ranges hold the same number of pairs and this workgroup walks the pairs idx, idx + stride,
  // ... of its XCD's range.  With unequal groups the ranges are cut by work (k steps plus a fixed
  // cost per pair), and the pairs of a range are dealt longest group first, each to the workgroup
  // with the least work so far: every workgroup of the XCD runs the same deterministic deal and
  // keeps its own list.
  const int per_group = mtiles_o * ntiles_o;
  const int total = E * per_group;
  const int xcd = (int)blockIdx.x & 7, stride = max(1, (int)gridDim.x >> 3);
  int idx = (int)blockIdx.x >> 3;
  int pair_lo = min(total, xcd * ((total + 7) >> 3)), pair_hi = min(total, (xcd + 1) * ((total + 7) >> 3));
  constexpr int kMaxList = 2048;  // pairs a range may hold for the deal (else: round-robin)
  __shared__ int s_work[JTMOE_MAX_EXPERTS], s_count[JTMOE_MAX_EXPERTS], s_first[JTMOE_MAX_EXPERTS];
  __shared__ int s_order[JTMOE_MAX_EXPERTS];
  __shared__ int s_list[kMaxList];
  __shared__ int s_len;
  int listed = -1;  // >= 0: this workgroup's pairs are s_list[0 .. listed)
  if (group_sizes) {
    constexpr int kPer = JTMOE_MAX_EXPERTS / 64;  // groups per lane, contiguous
    constexpr int kFixedSteps = 3 * 64 / BK;      // look-up and epilogue of a pair, in k steps
    int w[kPer], local = 0, wmin = 0x7fffffff, wmax = 0;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int e = lane * kPer + j;
      w[j] = e < E ? (group_sizes[e] + BK - 1) / BK + kFixedSteps : 0;
      local += w[j];
      if (e < E) {
        wmin = min(wmin, w[j]);
        wmax = max(wmax, w[j]);
      }
    }
    int incl = local;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int v = __shfl_up(incl, d);
      if (lane >= d) incl += v;
    }
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      wmin = min(wmin, __shfl_xor(wmin, d));
      wmax = max(wmax, __shfl_xor(wmax, d));
    }
    const long long first = (long long)(incl - local) * per_group;  // work before this lane's groups
    const long long all = (long long)__shfl(incl, 63) * per_group;
    // the first pair that starts at or after `target` units of work
    auto first_pair_at = [&](long long target) -> int {
      const bool mine = target >= first && target < first + (long long)local * per_group;
      const unsigned long long owners = __ballot(mine);
      if (owners == 0ull) return total;  // target == all
      const int owner = __ffsll((long long)owners) - 1;
      int pair = 0;
      long long s = first;
      bool found = false;
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const long long span = (long long)w[j] * per_group;
        if (mine && !found && target < s + span) {
          pair = (lane * kPer + j) * per_group + ((int)(target - s) + w[j] - 1) / w[j];
          found = true;
        }
        s += span;
      }
      return __builtin_amdgcn_readfirstlane(__shfl(pair, owner));
    };
    wmin = __builtin_amdgcn_readfirstlane(wmin);
    wmax = __builtin_amdgcn_readfirstlane(wmax);
    const bool unequal = (long long)wmax * 4 > (long long)wmin * 5;  // longest group > 1.25 x shortest
    const bool keys_fit = __builtin_amdgcn_readfirstlane((int)(all < ((long long)1 << 26))) != 0;
    if (unequal) {
      pair_lo = first_pair_at(all * xcd / 8);
      pair_hi = first_pair_at(all * (xcd + 1) / 8);
    }
    // the deal (work of one XCD must fit the 26 bits the arg-min key leaves for it)
    if (unequal && pair_hi - pair_lo <= kMaxList && stride <= 32 && keys_fit) {
      if (wave == 0) {
        // groups with pairs inside the range: work, number of pairs inside, first pair inside
        int inside = 0;
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
          const int e = lane * kPer + j;
          const int lo = max(pair_lo, e * per_group), hi = min(pair_hi, (e + 1) * per_group);
          s_work[e] = w[j];
          s_count[e] = e < E ? max(0, hi - lo) : 0;
          s_first[e] = lo;
          inside += e < E && hi > lo;
        }
        // (same wave: LDS writes above are visible to the reads below after the wait the compiler places)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        // order: longer groups first, equal ones by index
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
          const int e = lane * kPer + j;
          if (e < E && s_count[e] > 0) {
            int rank = 0;
            for (int o = 0; o < E; ++o)
              rank += s_count[o] > 0 && (s_work[o] > w[j] || (s_work[o] == w[j] && o < e));
            s_order[rank] = e;
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        int n_inside = inside;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) n_inside += __shfl_xor(n_inside, d);
        n_inside = __builtin_amdgcn_readfirstlane(n_inside);
        // lanes 0 .. stride-1 stand for the workgroups of this XCD
        int load = lane < stride ? 0 : (1 << 26) - 1;
        int len = 0;
        for (int r = 0; r < n_inside; ++r) {
          const int e = __builtin_amdgcn_readfirstlane(s_order[r]);
          const int we = __builtin_amdgcn_readfirstlane(s_work[e]);
          const int cnt = __builtin_amdgcn_readfirstlane(s_count[e]);
          const int fst = __builtin_amdgcn_readfirstlane(s_first[e]);
          for (int c = 0; c < cnt; ++c) {
            int key = (load << 5) | (lane & 31);
            key = min(key, __builtin_amdgcn_mov_dpp(key, 0xB1, 0xF, 0xF, false));   // lanes ^ 1
            key = min(key, __builtin_amdgcn_mov_dpp(key, 0x4E, 0xF, 0xF, false));   // lanes ^ 2
            key = min(key, __builtin_amdgcn_mov_dpp(key, 0x141, 0xF, 0xF, false));  // mirror within 8
            key = min(key, __builtin_amdgcn_mov_dpp(key, 0x140, 0xF, 0xF, false));  // mirror within 16
            const int least = min(__builtin_amdgcn_readlane(key, 0), __builtin_amdgcn_readlane(key, 16)) & 31;
            if (lane == least) load += we;
            if (least == idx) {
              if (lane == 0) s_list[len] = fst + c;
              ++len;
            }
          }
        }
        if (lane == 0) s_len = len;
      }
      __syncthreads();
      listed = __builtin_amdgcn_readfirstlane(s_len);
    }
  }
  int step = 0;  // number of pairs this workgroup has taken

  // split_chunk > 0 (one dense group only): "group" e is the e-th run of split_chunk rows, and the
  // outputs are float32 partial sums [E, KA, N] that the caller adds up in a fixed order.  This
  // gives a reduction over many rows into a small matrix enough workgroups to fill the chip.
  struct Tile {
    int e, m0, n0, row0, rows;
    bool valid;
  };
  auto locate = [&](int i) -> Tile {
    Tile t;
    t.e = 0; t.m0 = 0; t.n0 = 0; t.row0 = 0; t.rows = 0;
    int logical;
    if (listed >= 0) {
      t.valid = i < listed;
      logical = t.valid ? __builtin_amdgcn_readfirstlane(s_list[i]) : 0;
    } else {
      logical = pair_lo + idx + i * stride;
      t.valid = logical < pair_hi;
    }
    if (!t.valid) return t;
    t.e = logical / per_group;
    const int in_e = logical - t.e * per_group;
    const int nt = in_e / mtiles_o;
    t.m0 = (in_e - nt * mtiles_o) * BMO;
    t.n0 = nt * BNO;
    if (group_sizes) {
      t.row0 = __builtin_amdgcn_readfirstlane(offsets[t.e]);
      t.rows = __builtin_amdgcn_readfirstlane(group_sizes[t.e]);
    } else if (split_chunk > 0) {
      t.row0 = t.e * split_chunk;
      t.rows = max(0, min(split_chunk, dense_rows - t.row0));
    } else {
      t.row0 = 0;
      t.rows = dense_rows;
    }
    return t;
  };

  // ---- load plan (rewritten for every tile) ----
  i32x4_t p_rsrc;
  i32x4_t d_rsrc[Cfg::DSUB];
  // sub-tile [BK rows][128 columns] as 128-byte blocks of 4 rows x 16 columns, block (r/4, c/16) at
  // index (r/4)*8 + c/16; slot s (16 bytes) -> block s/8, row (s/2)%4 of the block, half s%2
  // (OPT & 128: 512-byte blocks of 4 rows x 64 columns instead, block (r/4, c/64) at index
  // (r/4)*2 + c/64, so that eight lanes fetch one whole 128-byte line)
  constexpr bool kWide = (Cfg::OPT & 128) != 0;
  const int b_blk_id = kWide ? tid >> 5 : tid >> 3;
  // row inside the k step (first load) and 16-byte chunk inside the 128 columns
  const int l_r = kWide ? (b_blk_id >> 1) * 4 + ((tid >> 3) & 3) : (b_blk_id >> 3) * 4 + ((tid >> 1) & 3);
  // (wide blocks: rows 2 and 3 of a block hold their eight chunks with the two halves swapped, which
  // puts the four 32-byte pieces of a transposing read into four different groups of banks)
  const int l_c = kWide ? (b_blk_id & 1) * 8 + ((tid & 7) ^ (((tid >> 4) & 1) << 2)) : (b_blk_id & 7) * 2 + (tid & 1);
  constexpr int ROWS_PER_LOAD = NT / 16;
  int p_col = 0, d_col = 0;  // byte offset inside a row
  int row0 = 0, rows = 0, nk = 0;
  auto plan = [&](const Tile& t) {
    row0 = t.row0;
    rows = t.rows;
    nk = (rows + BK - 1) / BK;
    p_rsrc = p_gather ? make_rsrc(P, gathered_rows * KA * 2) : make_rsrc(P + (size_t)row0 * KA, rows * KA * 2);
#pragma unroll
    for (int u = 0; u < Cfg::DSUB; ++u) {
      const uint16_t* d = (kDual && u == 1) ? D1 : D0;
      d_rsrc[u] = d_gather ? make_rsrc(d, gathered_rows * N * 2) : make_rsrc(d + (size_t)row0 * N, rows * N * 2);
    }
    p_col = (t.m0 + l_c * 8) * 2;
    d_col = (t.n0 + l_c * 8) * 2;
  };
  const unsigned lds0 = lds_byte_addr(smem_raw);
  const unsigned wave_lds = lds0 + wave * 1024;

  // row ids of a k step (only used by gathered operands); -1 = past the end of the group
  int ids[Cfg::SUB_LOADS];
  auto fetch_ids = [&](int kt) {
#pragma unroll
    for (int j = 0; j < Cfg::SUB_LOADS; ++j) {
      const int r = kt * BK + l_r + j * ROWS_PER_LOAD;
      ids[j] = r < rows ? row_map[row0 + r] / row_div : -1;
    }
  };
  // (row ids are fetched one step ahead of their loads: with more than two stages the row map is not used)
  if (Cfg::NSTAGE > 2) {
    p_gather = 0;
    d_gather = 0;
  }
  const bool any_gather = p_gather || d_gather;

  // Rows past the end of the group must contribute zeros: their offsets lie outside the
  // descriptor (which ends with the group, or is pushed there explicitly for gathered rows).
  auto issue = [&](int kt) {
    const unsigned base = wave_lds + (kt % Cfg::NSTAGE) * Cfg::STAGE_BYTES;
    int pv[Cfg::SUB_LOADS], dv[Cfg::SUB_LOADS];
#pragma unroll
    for (int j = 0; j < Cfg::SUB_LOADS; ++j) {
      const int r = kt * BK + l_r + j * ROWS_PER_LOAD;
      pv[j] = p_gather ? (ids[j] >= 0 ? ids[j] * KA * 2 + p_col : 0x70000000) : r * KA * 2 + p_col;
      dv[j] = d_gather ? (ids[j] >= 0 ? ids[j] * N * 2 + d_col : 0x70000000) : r * N * 2 + d_col;
    }
    // LDS address = one scalar per stage + a compile-time offset per load (this kernel is short of
    // scalar registers)
    static_assert(Cfg::PSUB <= 2 && Cfg::DSUB <= 2 && Cfg::SUB_LOADS <= 2, "load list written out below");
    constexpr int L = Cfg::SUB_LOADS - 1;  // index of a sub-tile's second load (its first if there is one only)
    buffer_load_lds16_at<0>(p_rsrc, base, pv[0], 0);
    if (Cfg::SUB_LOADS == 2) buffer_load_lds16_at<NT * 16>(p_rsrc, base, pv[L], 0);
    if (Cfg::PSUB == 2) {
      buffer_load_lds16_at<Cfg::SUB_BYTES>(p_rsrc, base, pv[0] + 256, 0);
      if (Cfg::SUB_LOADS == 2) buffer_load_lds16_at<Cfg::SUB_BYTES + NT * 16>(p_rsrc, base, pv[L] + 256, 0);
    }
    buffer_load_lds16_at<Cfg::P_BYTES>(d_rsrc[0], base, dv[0], 0);
    if (Cfg::SUB_LOADS == 2) buffer_load_lds16_at<Cfg::P_BYTES + NT * 16>(d_rsrc[0], base, dv[L], 0);
    if (Cfg::DSUB == 2) {
      buffer_load_lds16_at<Cfg::P_BYTES + Cfg::SUB_BYTES>(d_rsrc[Cfg::DSUB - 1], base, dv[0] + (kDual ? 0 : 256), 0);
      if (Cfg::SUB_LOADS == 2)
        buffer_load_lds16_at<Cfg::P_BYTES + Cfg::SUB_BYTES + NT * 16>(d_rsrc[Cfg::DSUB - 1], base,
                                                                    dv[L] + (kDual ? 0 : 256), 0);
    }
  };
  // first loads of a tile (and, for gathered operands, the row ids they need)
  auto start_tile = [&]() {
    if (nk > 0) {
      if (any_gather) fetch_ids(0);
      issue(0);
      if (any_gather && nk > 1) fetch_ids(1);
    }
  };

  // transposing read: the 16 lanes of a group read one whole 128-byte block, lane i its bytes
  // [8 i, 8 i + 8) = row i/4, columns 4*(i%4)..; groups: column half (lane/16)%2, row half lane/32
  const int laneoff = kWide ? ((lane & 15) >> 2) * 128 + (lane & 3) * 8 + ((lane >> 4) & 1) * 32 + (lane >> 5) * 2048
                            : (lane & 15) * 8 + ((lane >> 4) & 1) * 128 + (lane >> 5) * (2 * 8 * 128);
  auto block_of = [&](int col) {
    return kWide ? (col >> 7) * Cfg::SUB_BYTES + ((col & 127) >> 6) * 512 + (col & 63) * 2
                 : (col >> 7) * Cfg::SUB_BYTES + ((col & 127) >> 4) * 128;
  };
  // the swap of the two 64-byte halves in rows 2 and 3 of a wide block, seen from the reading lane
  const int half_swap = kWide ? ((lane >> 3) & 1) * 64 : 0;
  auto swapped = [&](int col) { return (col & 32) ? -half_swap : half_swap; };
  int p_blk[TM], d_blk[TN];
#pragma unroll
  for (int mi = 0; mi < TM; ++mi) p_blk[mi] = block_of(wm * WM + mi * 32) + swapped(mi * 32);
#pragma unroll
  for (int jj = 0; jj < TN; ++jj) {
    int col;
    if (kDual)
      col = (jj < TN / 2 ? 0 : BNO) + wn * (WN / 2) + (jj % (TN / 2)) * 32;
    else
      col = wn * WN + jj * 32;
    d_blk[jj] = Cfg::P_BYTES + block_of(col) + swapped(col);
  }
  auto read_tr = [&](const unsigned char* p) {
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p));
    const s16x4_t hi =
        __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p + 8 * 128));
    const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8_t, both);
  };
  auto load_frags = [&](const unsigned char* st, int kk, bf16x8_t* af, bf16x8_t* bf) {
#pragma unroll
    for (int mi = 0; mi < TM; ++mi) af[mi] = read_tr(st + p_blk[mi] + laneoff + kk * (4 * 8 * 128));
#pragma unroll
    for (int jj = 0; jj < TN; ++jj) bf[jj] = read_tr(st + d_blk[jj] + laneoff + kk * (4 * 8 * 128));
  };

  // Epilogue staging lives above the first stage buffer, which the next tile's first loads fill
  // while the epilogue runs; a wave's block goes out in halves where it does not fit its share.
  constexpr int TNO = Cfg::TNO, WNO = Cfg::WNO, CS = Cfg::CS;
  constexpr int kStageArea = (int)Cfg::SMEM_BYTES - Cfg::STAGE_BYTES;
  constexpr int kHalves = (NT / 64) * WM * CS * 2 <= kStageArea ? 1 : 2;
  constexpr int TMH = TM / kHalves, WMH = WM / kHalves;
  static_assert((NT / 64) * WMH * CS * 2 <= kStageArea && TM % kHalves == 0, "epilogue staging must fit above stage 0");
  uint16_t* const cw = reinterpret_cast<uint16_t*>(smem_raw + Cfg::STAGE_BYTES) + wave * (WMH * CS);

  Tile cur = locate(step);
  if (!cur.valid) return;
  plan(cur);
  start_tile();

  while (true) {
    f32x16_t acc[TM][TN];
#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
#pragma unroll
      for (int jj = 0; jj < TN; ++jj)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mi][jj][i] = 0.0f;

    // a wave whose block of the result lies wholly outside [KA, N] has nothing to add
    const bool wave_has_output = cur.m0 + wm * WM < KA && cur.n0 + wn * (kDual ? WN / 2 : WN) < N;
    auto mfma_substep = [&](const bf16x8_t* af, const bf16x8_t* bf) {
#pragma unroll
      for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int jj = 0; jj < TN; ++jj)
          acc[mi][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mi], bf[jj], acc[mi][jj], 0, 0, 0);
    };
    // Stage 0 of the tile is on its way (start_tile); the stages above it share their LDS with the
    // epilogue's staging area, so their loads start behind the first barrier of the tile, by which
    // every wave has stored its results: steps 1 .. NSTAGE - 1 all at once there, then one step per
    // step, each NSTAGE - 1 steps ahead of its use.
    int issued = 1;
    {
      for (int kt = 0; kt < nk; ++kt) {
        // the stages younger than this step's stay in flight when the pipeline is full
        if (Cfg::NSTAGE > 2 && issued - kt == Cfg::NSTAGE - 1)
          wait_vmcnt<(Cfg::NSTAGE - 2) * Cfg::LOADS_PER_STAGE>();
        else
          wait_vmcnt<0>();
        __syncthreads();
        while (issued < nk && issued < kt + Cfg::NSTAGE) {
          issue(issued);
          ++issued;
          if (any_gather && issued < nk) fetch_ids(issued);
        }
        if (!wave_has_output) continue;
        const unsigned char* st = smem_raw + (kt % Cfg::NSTAGE) * Cfg::STAGE_BYTES;
        bf16x8_t af[2][TM], bf[2][TN];
        load_frags(st, 0, af[0], bf[0]);
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
          if (kk + 1 < BK / 16) load_frags(st, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
          mfma_substep(af[kk & 1], bf[kk & 1]);
        }
      }
    }
    __syncthreads();  // every wave is done reading the stage buffers (and, for an empty group, with
                      // the previous tile's staging area)

    // the first operand tiles of the next pair are on their way while this one's results go out
    // (the pair is looked up only now: this kernel has no scalar registers to spare during the k loop)
    const int out_e = cur.e, out_m0 = cur.m0, out_n0 = cur.n0;
    ++step;
    const Tile nxt = locate(step);
    if (nxt.valid) {
      plan(nxt);
      start_tile();
    }

    if (split_chunk > 0) {
      // float32 partial sums straight from the accumulators: for a fixed i the 32 lanes of a half
      // wave write 128 contiguous bytes of one row
#pragma unroll
      for (int which = 0; which < (kDual ? 2 : 1); ++which) {
        float* const Cm = reinterpret_cast<float*>(which ? C1 : C0) + (size_t)out_e * KA * N;
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
          for (int jj = 0; jj < TNO; ++jj) {
            const int col = out_n0 + wn * WNO + jj * 32 + (lane & 31);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int r = out_m0 + wm * WM + mi * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
              if (r < KA && col < N) Cm[(size_t)r * N + col] = acc[mi][jj + which * (TN / 2)][i];
            }
          }
      }
    } else {
      // per matrix, each wave parks its block in LDS (in halves) and streams it out in rows
      const int col0 = out_n0 + wn * WNO;
#pragma unroll
      for (int which = 0; which < (kDual ? 2 : 1); ++which) {
        uint16_t* const Cm = (which ? C1 : C0) + (size_t)out_e * KA * N;
#pragma unroll
        for (int h = 0; h < kHalves; ++h) {
          const int row_base = out_m0 + wm * WM + h * WMH;
#pragma unroll
          for (int mh = 0; mh < TMH; ++mh)
#pragma unroll
            for (int jj = 0; jj < TNO; ++jj)
#pragma unroll
              for (int i = 0; i < 16; ++i) {
                const int r = mh * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
                cw[r * CS + jj * 32 + (lane & 31)] = bf16_bits_fast(acc[h * TMH + mh][jj + which * (TN / 2)][i]);
              }
          // the staging area is private to the wave: program order within the wave suffices between
          // one block's row stores and the next block's LDS writes
          store_wave_block<WMH, WNO, CS, (Cfg::OPT & 32768) != 0>(cw, lane, Cm, N, (size_t)row_base, KA - row_base,
                                                                 col0);
        }
      }
    }
    if (!nxt.valid) break;
    cur = nxt;
  }
}

// Configurations the library launches.
using DgradCfg = NtGemmCfg<256, 256, 2, 4, 16 + 64 + 32768>;   // data gradients: 256 x 256 tiles
// narrow LDS blocks: the fastest layout when the operands are streamed (1.52 vs 1.60 ms for the
// gate/up product of the C3 shape); the wide blocks pay off only when rows are gathered.
// Four stages of 32 rows against two of 64 (the same LDS): 1.39-1.43 against 1.47-1.49 ms for the gate/up
// gradients of that shape, 0.73-0.75 against 0.76-0.77 ms for the down gradient; three stages measure
// the same as four; moving a step's barrier in front of its last sub-step, which pays in the forward
// kernel, costs 3-9 % here, and asking the scheduler to put two transposing reads behind every MFMA 2-4 %.
using WgradDualCfg = TnGemmCfg<256, 128, 4, 2, true, 16 + 32768, 32, 4>;  // gate and up weight gradients share the x tile
using WgradCfg = TnGemmCfg<256, 256, 2, 4, false, 16 + 32768, 32, 4>;     // down weight gradient
// the same products with an operand fetched through a row map (row ids run one step ahead of their loads)
using WgradDualGatherCfg = TnGemmCfg<256, 128, 4, 2, true, 16 + 32768>;
using WgradGatherCfg = TnGemmCfg<256, 256, 2, 4, false, 16 + 32768>;

}  // namespace jtmoe
