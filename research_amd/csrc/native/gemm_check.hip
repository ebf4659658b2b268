// Stand-alone check of the grouped GEMM kernels (no Python, no torch), in the manner of the
// reference's rmsnorm_test.cu (src/jaxtitan/kernels/cuda/rmsnorm/rmsnorm_test.cu:126-149):
// deterministic inputs, an independent reference (one thread per output element, fp32
// accumulation in k order), a tolerance, and PASS / FAIL on stdout.
//
//   gemm_check            correctness on ragged groups, gather-on-load and the dense case
//   gemm_check time_backward   + timing of the four backward launches at the C3 shape
//   gemm_check time       + timing of the library's two configurations at the C3 shape,
//                           once on N(0,1)-like data and once on all-zero data
//   gemm_check time_stream / time_ablation / counters_stream   the stream kernel against the older one,
//                           with parts of its loop left out, and a fixed launch sequence for counter runs
//   gemm_check time_stream_nt   the transposed-B form of the stream kernel against grouped_gemm_nt_kernel
//   gemm_check time_ragged      the C3 launches on random against equal group sizes
//   gemm_check time_decode      the decode-shape launches (64 groups of about 8 rows), also with the head of
//                               every expert matrix read into the memory-side cache beforehand
//   gemm_check time_tn_stages   the weight-gradient kernel with two, three and four operand stages
//   gemm_check time_c2_down     the down projection with 256 x 256 against 256 x 128 tiles, caches warm and cold
//   gemm_check time_chunks / counters_chunks   the stream kernel's gate/up launch with its tiles cut into workgroups
//                               of 1, 2, 4, 8 tiles or one per CU, and tile-order groups of 2, 4, 8 m-tiles
//   gemm_check time_down        the down projection's kernels at the three large configurations' shapes, caches cold
//   gemm_check time_prio        the stream kernel with and without raised wave priority around its MFMAs
//   (a second argument "nocheck" skips the correctness cases)
#include "grouped_gemm_bwd.hpp"
#include "grouped_gemm_stream.hpp"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

using namespace jtmoe;
namespace jtmoe {
thread_local StageTimer* g_stage_timer = nullptr;
}

#define CK(x)                                                                              \
  do {                                                                                     \
    hipError_t e_ = (x);                                                                   \
    if (e_ != hipSuccess) {                                                                \
      printf("HIP error %s at %s:%d\nFAIL\n", hipGetErrorString(e_), __FILE__, __LINE__);   \
      exit(1);                                                                             \
    }                                                                                      \
  } while (0)

static uint16_t f2bf(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
static float bf2f(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

__global__ void reference_kernel(const uint16_t* A, const uint16_t* B0, const uint16_t* B1, float* C,
                                 const int* row_expert, const int* a_row_of, int rows, int K, int N, int dual) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
  if (n >= N || r >= rows) return;
  const int e = row_expert[r];
  const uint16_t* a = A + (size_t)a_row_of[r] * K;
  float g = 0, u = 0;
  for (int k = 0; k < K; ++k) {
    const float av = bf16_bits_to_f32(a[k]);
    g += av * bf16_bits_to_f32(B0[((size_t)e * K + k) * N + n]);
    if (dual) u += av * bf16_bits_to_f32(B1[((size_t)e * K + k) * N + n]);
  }
  if (dual) {
    g = round_to_bf16(g);
    u = round_to_bf16(u);
    C[(size_t)r * N + n] = g / (1.0f + expf(-g)) * u;
  } else {
    C[(size_t)r * N + n] = g;
  }
}

struct Problem {
  int E, rows, K, N, a_rows, top_k;
  std::vector<int> gs, off, row_expert, a_row_of, row_map;
  uint16_t *A, *B0, *B1, *C;
  int *dgs, *doff, *drow, *darow, *dmap;
};

// rows are spread over E groups (skewed, some empty); with top_k > 0 the A matrix has
// rows/top_k rows and packed row j reads A row row_map[j] / top_k (gather on load)
static bool g_equal_groups = false;  // every group rows / E rows (no ragged last tiles) instead of random sizes
static Problem make(int E, int rows, int K, int N, unsigned seed, bool skew, int top_k, float scale) {
  Problem p;
  p.E = E; p.rows = rows; p.K = K; p.N = N; p.top_k = top_k;
  std::mt19937 rng(seed);
  p.gs.assign(E, 0);
  for (int r = 0; r < rows; ++r) {
    int e = skew ? (int)(std::pow((double)(rng() % 10000) / 10000.0, 3.0) * E) : (int)(rng() % E);
    if (skew && e % 5 == 3) e = 0;
    if (g_equal_groups) e = r % E;
    p.gs[e]++;
  }
  p.off.assign(E, 0);
  for (int e = 1; e < E; ++e) p.off[e] = p.off[e - 1] + p.gs[e - 1];
  p.row_expert.resize(rows);
  for (int e = 0; e < E; ++e)
    for (int i = 0; i < p.gs[e]; ++i) p.row_expert[p.off[e] + i] = e;
  p.a_rows = top_k > 0 ? rows / top_k : rows;
  p.row_map.resize(rows);
  p.a_row_of.resize(rows);
  for (int r = 0; r < rows; ++r) p.row_map[r] = r;
  if (top_k > 0) std::shuffle(p.row_map.begin(), p.row_map.end(), rng);
  for (int r = 0; r < rows; ++r) p.a_row_of[r] = top_k > 0 ? p.row_map[r] / top_k : r;
  std::vector<uint16_t> hA((size_t)p.a_rows * K), hB((size_t)E * K * N);
  std::normal_distribution<float> nd(0.f, 1.f);
  for (auto& v : hA) v = f2bf(nd(rng) * scale);
  CK(hipMalloc(&p.A, hA.size() * 2));
  CK(hipMemcpy(p.A, hA.data(), hA.size() * 2, hipMemcpyHostToDevice));
  for (auto& v : hB) v = f2bf(nd(rng) * 0.05f * scale);
  CK(hipMalloc(&p.B0, hB.size() * 2));
  CK(hipMemcpy(p.B0, hB.data(), hB.size() * 2, hipMemcpyHostToDevice));
  for (auto& v : hB) v = f2bf(nd(rng) * 0.05f * scale);
  CK(hipMalloc(&p.B1, hB.size() * 2));
  CK(hipMemcpy(p.B1, hB.data(), hB.size() * 2, hipMemcpyHostToDevice));
  CK(hipMalloc(&p.C, (size_t)rows * N * 2));
  CK(hipMalloc(&p.dgs, E * 4)); CK(hipMalloc(&p.doff, E * 4)); CK(hipMalloc(&p.drow, rows * 4));
  CK(hipMalloc(&p.darow, rows * 4)); CK(hipMalloc(&p.dmap, rows * 4));
  CK(hipMemcpy(p.dgs, p.gs.data(), E * 4, hipMemcpyHostToDevice));
  CK(hipMemcpy(p.doff, p.off.data(), E * 4, hipMemcpyHostToDevice));
  CK(hipMemcpy(p.drow, p.row_expert.data(), rows * 4, hipMemcpyHostToDevice));
  CK(hipMemcpy(p.darow, p.a_row_of.data(), rows * 4, hipMemcpyHostToDevice));
  CK(hipMemcpy(p.dmap, p.row_map.data(), rows * 4, hipMemcpyHostToDevice));
  return p;
}
static void release(Problem& p) {
  hipFree(p.A); hipFree(p.B0); hipFree(p.B1); hipFree(p.C);
  hipFree(p.dgs); hipFree(p.doff); hipFree(p.drow); hipFree(p.darow); hipFree(p.dmap);
}

// The 256-row configurations run as the library runs them: persistent workgroups, one per CU (256
// here), unless g_one_tile_per_workgroup asks for the plain kernel.
static bool g_one_tile_per_workgroup = false;
static int g_chunk = -1;  // tiles per workgroup of a persistent launch; -1: as the library chooses
// the stream kernel (grouped_gemm_stream.hpp): one software pipeline through all tiles of a workgroup
template <typename Cfg>
static void launch_stream(Problem& p, bool dense) {
  using L = StreamLayout<Cfg>;
  if (p.K / Cfg::BK < 2 * Cfg::NSTAGE) { printf("stream kernel: K too short\n"); exit(1); }
  const long mt = dense ? (p.rows + Cfg::BM - 1) / Cfg::BM
                        : (p.rows + Cfg::BM - 1) / Cfg::BM + (p.E < p.rows ? p.E : p.rows);
  const long nt = (p.N + Cfg::BN - 1) / Cfg::BN;
  const long tiles_grid = gemm_grid(mt, nt);
  auto kernel = grouped_gemm_stream_kernel<Cfg>;
  CK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                         (int)L::kSmemBytes));
  PersistentSchedule ps = persistent_schedule(tiles_grid, 256, g_chunk < 0 ? kTilesPerWorkgroup<Cfg> : g_chunk);
  if (tiles_grid <= 256) ps = {tiles_grid, 0, 0};
  kernel<<<(unsigned)ps.grid, Cfg::NT, L::kSmemBytes>>>(
      p.A, p.B0, Cfg::kDual ? p.B1 : nullptr, p.C, dense ? nullptr : p.dgs, dense ? nullptr : p.doff, p.E, p.rows, p.K,
      p.N, (int)mt, (int)nt, p.top_k > 0 ? p.dmap : nullptr, p.top_k > 0 ? p.top_k : 1, p.a_rows, nullptr, nullptr,
      ps.window, ps.chunk);
}

static bool g_stream = false;
template <typename Cfg>
static void launch(Problem& p, bool dense) {
  if constexpr (Cfg::BM == 256 && (Cfg::OPT & 128) != 0) {
    if (g_stream) return launch_stream<Cfg>(p, dense);
  }
  constexpr bool kCanPersist = Cfg::BM == 256 && Cfg::NSTAGE == 2 && Cfg::BK == 64;
  const bool persist = kCanPersist && !g_one_tile_per_workgroup;
  const long mt = dense ? (p.rows + Cfg::BM - 1) / Cfg::BM
                        : (p.rows + Cfg::BM - 1) / Cfg::BM + (p.E < p.rows ? p.E : p.rows);
  const long nt = (p.N + Cfg::BN - 1) / Cfg::BN;
  const long tiles_grid = gemm_grid(mt, nt);
  if constexpr (kCanPersist) {
    if (persist) {
      auto kernel = grouped_gemm_dma_persistent_kernel<Cfg>;
      CK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                             (int)Cfg::SMEM_BYTES));
      const PersistentSchedule ps = persistent_schedule(tiles_grid, 256, g_chunk < 0 ? kTilesPerWorkgroup<Cfg> : g_chunk);
      kernel<<<(unsigned)ps.grid, Cfg::NT, Cfg::SMEM_BYTES>>>(
          p.A, p.B0, Cfg::kDual ? p.B1 : nullptr, p.C, dense ? nullptr : p.dgs, dense ? nullptr : p.doff, p.E, p.rows,
          p.K, p.N, (int)mt, (int)nt, p.top_k > 0 ? p.dmap : nullptr, p.top_k > 0 ? p.top_k : 1, p.a_rows, nullptr,
          nullptr, ps.window, ps.chunk);
      return;
    }
  }
  auto kernel = grouped_gemm_dma_kernel<Cfg>;
  CK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                         (int)Cfg::SMEM_BYTES));
  kernel<<<(unsigned)tiles_grid, Cfg::NT, Cfg::SMEM_BYTES>>>(
      p.A, p.B0, Cfg::kDual ? p.B1 : nullptr, p.C, dense ? nullptr : p.dgs, dense ? nullptr : p.doff, p.E, p.rows,
      p.K, p.N, (int)mt, (int)nt, p.top_k > 0 ? p.dmap : nullptr, p.top_k > 0 ? p.top_k : 1, p.a_rows, nullptr, nullptr, 0,
      0);
}

template <typename Cfg>
static bool check(const char* name, Problem& p, bool dense = false) {
  float* ref;
  CK(hipMalloc(&ref, (size_t)p.rows * p.N * 4));
  reference_kernel<<<dim3((p.N + 255) / 256, p.rows), 256>>>(p.A, p.B0, p.B1, ref, p.drow, p.darow, p.rows, p.K, p.N,
                                                            Cfg::kDual);
  CK(hipMemset(p.C, 0xff, (size_t)p.rows * p.N * 2));
  launch<Cfg>(p, dense);
  CK(hipDeviceSynchronize());
  std::vector<float> hr((size_t)p.rows * p.N);
  std::vector<uint16_t> hc(hr.size());
  CK(hipMemcpy(hr.data(), ref, hr.size() * 4, hipMemcpyDeviceToHost));
  CK(hipMemcpy(hc.data(), p.C, hc.size() * 2, hipMemcpyDeviceToHost));
  double maxref = 0, maxerr = 0;
  size_t bad = 0;
  for (float v : hr) maxref = std::max(maxref, (double)std::fabs(v));
  for (size_t i = 0; i < hr.size(); ++i) {
    const double e = std::fabs((double)bf2f(hc[i]) - hr[i]);
    if (!(e <= 0.02 * maxref)) ++bad;  // also catches NaN and untouched 0xffff outputs
    maxerr = std::max(maxerr, e);
  }
  printf("case %-34s E=%d rows=%d K=%d N=%d max_err/max_ref=%.3e tolerance=2e-2 bad=%zu\n", name, p.E, p.rows, p.K,
         p.N, maxerr / maxref, bad);
  fflush(stdout);
  hipFree(ref);
  return bad == 0;
}

template <typename Cfg>
static void timeit(const char* name, Problem& p, int iters) {
  hipEvent_t a, b;
  CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  // a long warm-up: the first tens of milliseconds after a pause on the host side (here, filling
  // the operands) run several per cent slower, whichever kernel is timed
  for (int i = 0; i < 60; ++i) launch<Cfg>(p, false);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(a));
  for (int i = 0; i < iters; ++i) launch<Cfg>(p, false);
  CK(hipEventRecord(b)); CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  ms /= iters;
  const double flops = 2.0 * p.rows * (double)p.K * p.N * (Cfg::kDual ? 2 : 1);
  printf("time %-36s rows=%d K=%d N=%d: %.3f ms  %.1f TFLOP/s  (%.1f%% of 2500)\n", name, p.rows, p.K, p.N, ms,
         flops / ms / 1e9, flops / ms / 1e9 / 25.0);
  fflush(stdout);
}

// The same with the caches cold: between two timed launches a fill of 1 GiB goes through the L2s and
// the memory-side cache, so that the operands come from HBM as they do inside a layer, where the
// launch before has streamed other matrices.  Each launch is timed by its own pair of events.
__global__ __launch_bounds__(256) void flush_fill_kernel(u32x4_t* out, size_t n) {
  const u32x4_t v = {1u, 2u, 3u, 4u};
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) out[i] = v;
}
template <typename Cfg>
static void timeit_cold(const char* name, Problem& p, int iters) {
  static u32x4_t* junk = nullptr;
  const size_t junk_vecs = (size_t)1 << 26;
  if (junk == nullptr) CK(hipMalloc(&junk, junk_vecs * 16));
  hipEvent_t a, b;
  CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  for (int i = 0; i < 20; ++i) launch<Cfg>(p, false);
  double total = 0;
  for (int i = 0; i < iters; ++i) {
    flush_fill_kernel<<<4096, 256>>>(junk, junk_vecs);
    CK(hipEventRecord(a));
    launch<Cfg>(p, false);
    CK(hipEventRecord(b)); CK(hipEventSynchronize(b));
    float ms;
    CK(hipEventElapsedTime(&ms, a, b));
    total += ms;
  }
  const double ms = total / iters;
  const double flops = 2.0 * p.rows * (double)p.K * p.N * (Cfg::kDual ? 2 : 1);
  printf("time %-36s rows=%d K=%d N=%d: %.3f ms  %.1f TFLOP/s  (%.1f%% of 2500), caches cold\n", name, p.rows, p.K,
         p.N, ms, flops / ms / 1e9, flops / ms / 1e9 / 25.0);
  fflush(stdout);
}

// ---- the two backward forms -------------------------------------------------------------------

// C[r, n] = sum_s sum_k A_s[arow(r), k] * B_s[e(r), n, k]
__global__ void reference_nt_kernel(const uint16_t* A0, const uint16_t* A1, const uint16_t* B0, const uint16_t* B1,
                                    float* C, const int* row_expert, const int* a_row_of, int rows, int K, int N,
                                    int segs) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
  if (n >= N || r >= rows) return;
  const int e = row_expert[r];
  float acc = 0;
  for (int s = 0; s < segs; ++s) {
    const uint16_t* a = (s ? A1 : A0) + (size_t)a_row_of[r] * K;
    const uint16_t* b = (s ? B1 : B0) + ((size_t)e * N + n) * K;
    for (int k = 0; k < K; ++k) acc += bf16_bits_to_f32(a[k]) * bf16_bits_to_f32(b[k]);
  }
  C[(size_t)r * N + n] = acc;
}

// C[e, ka, n] = sum over rows r of group e of P[prow(r), ka] * D[drow(r), n]
__global__ void reference_tn_kernel(const uint16_t* P, const uint16_t* D, float* C, const int* gs, const int* off,
                                    const int* p_row_of, const int* d_row_of, int KA, int N) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x, ka = blockIdx.y, e = blockIdx.z;
  if (n >= N) return;
  float acc = 0;
  for (int r = off[e]; r < off[e] + gs[e]; ++r)
    acc += bf16_bits_to_f32(P[(size_t)p_row_of[r] * KA + ka]) * bf16_bits_to_f32(D[(size_t)d_row_of[r] * N + n]);
  C[((size_t)e * KA + ka) * N + n] = acc;
}

static uint16_t* random_bf16(size_t n, unsigned seed, float scale) {
  std::vector<uint16_t> h(n);
  std::mt19937 rng(seed);
  std::normal_distribution<float> nd(0.f, 1.f);
  for (auto& v : h) v = f2bf(nd(rng) * scale);
  uint16_t* d;
  CK(hipMalloc(&d, n * 2));
  CK(hipMemcpy(d, h.data(), n * 2, hipMemcpyHostToDevice));
  return d;
}

static bool compare(const char* name, const float* dref, const uint16_t* dgot, size_t n, const char* shape) {
  std::vector<float> hr(n);
  std::vector<uint16_t> hc(n);
  CK(hipMemcpy(hr.data(), dref, n * 4, hipMemcpyDeviceToHost));
  CK(hipMemcpy(hc.data(), dgot, n * 2, hipMemcpyDeviceToHost));
  double maxref = 0, maxerr = 0;
  size_t bad = 0;
  for (float v : hr) maxref = std::max(maxref, (double)std::fabs(v));
  for (size_t i = 0; i < n; ++i) {
    const double e = std::fabs((double)bf2f(hc[i]) - hr[i]);
    if (!(e <= 0.02 * maxref)) ++bad;
    maxerr = std::max(maxerr, e);
  }
  printf("case %-34s %s max_err/max_ref=%.3e tolerance=2e-2 bad=%zu\n", name, shape, maxerr / maxref, bad);
  fflush(stdout);
  return bad == 0;
}

// the transposed-B form of the stream kernel (what the library launches for the data gradients where it fits)
static int g_stream_nt = 0;  // 0: the older kernel; 1: DgradStreamCfg; 2 and 3: its variants below
using DgradStream42Cfg = DmaGemmCfg<256, 256, 32, 4, 2, false, 4, 16 + 128>;  // 4 x 2 waves of 64 x 128
using DgradStream2Cfg = DmaGemmCfg<256, 256, 64, 2, 4, false, 2, 16 + 128>;   // 64-deep steps, two stages
template <typename Cfg>
static void launch_stream_nt_cfg(Problem& p, const uint16_t* A1, int segs, bool dense) {
  using L = StreamLayout<Cfg>;
  if ((p.K / Cfg::BK) * segs < 2 * Cfg::NSTAGE || p.K % Cfg::BK != 0) {
    printf("stream nt: K=%d segs=%d is outside the kernel's envelope\n", p.K, segs);
    exit(1);
  }
  auto kernel = grouped_gemm_stream_nt_kernel<Cfg>;
  CK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                         (int)L::kSmemBytes));
  const long mt = dense ? (p.rows + Cfg::BM - 1) / Cfg::BM
                        : (p.rows + Cfg::BM - 1) / Cfg::BM + (p.E < p.rows ? p.E : p.rows);
  const long nt = (p.N + Cfg::BN - 1) / Cfg::BN;
  const long tiles_grid = gemm_grid(mt, nt);
  PersistentSchedule ps = persistent_schedule(tiles_grid, 256, g_chunk < 0 ? kTilesPerWorkgroup<Cfg> : g_chunk);
  if (tiles_grid <= 256) ps = {tiles_grid, 0, 0};
  kernel<<<(unsigned)ps.grid, Cfg::NT, L::kSmemBytes>>>(
      p.A, A1, p.B0, p.B1, p.C, dense ? nullptr : p.dgs, dense ? nullptr : p.doff, p.E, p.rows, p.K, p.N, (int)mt,
      (int)nt, p.top_k > 0 ? p.dmap : nullptr, p.top_k > 0 ? p.top_k : 1, p.a_rows, segs, ps.window, ps.chunk);
}
static void launch_stream_nt(Problem& p, const uint16_t* A1, int segs, bool dense) {
  if (g_stream_nt == 2) return launch_stream_nt_cfg<DgradStream42Cfg>(p, A1, segs, dense);
  if (g_stream_nt == 3) return launch_stream_nt_cfg<DgradStream2Cfg>(p, A1, segs, dense);
  launch_stream_nt_cfg<DgradStreamCfg>(p, A1, segs, dense);
}

template <typename Cfg>
static void launch_nt(Problem& p, const uint16_t* A1, int segs, bool dense) {
  if (g_stream_nt) return launch_stream_nt(p, A1, segs, dense);
  auto kernel = grouped_gemm_nt_kernel<Cfg>;
  CK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                         (int)Cfg::SMEM_BYTES));
  const long mt = dense ? (p.rows + Cfg::BM - 1) / Cfg::BM
                        : (p.rows + Cfg::BM - 1) / Cfg::BM + (p.E < p.rows ? p.E : p.rows);
  const long nt = (p.N + Cfg::BN - 1) / Cfg::BN;
  // persistent workgroups, as the library launches it; g_one_tile_per_workgroup gives every tile its own
  const long tiles_grid = gemm_grid(mt, nt);
  kernel<<<(unsigned)(!g_one_tile_per_workgroup && tiles_grid > 256 ? 256 : tiles_grid), Cfg::NT, Cfg::SMEM_BYTES>>>(
      p.A, A1, p.B0, p.B1, p.C, dense ? nullptr : p.dgs, dense ? nullptr : p.doff, p.E, p.rows, p.K, p.N, (int)mt,
      (int)nt, p.top_k > 0 ? p.dmap : nullptr, p.top_k > 0 ? p.top_k : 1, p.a_rows, segs);
}

// B0 / B1 of the problem are read as [E, N, K] here
template <typename Cfg>
static bool check_nt(const char* name, Problem& p, int segs, bool dense = false) {
  uint16_t* A1 = segs == 2 ? random_bf16((size_t)p.a_rows * p.K, 77, 1.0f) : nullptr;
  float* ref;
  CK(hipMalloc(&ref, (size_t)p.rows * p.N * 4));
  reference_nt_kernel<<<dim3((p.N + 255) / 256, p.rows), 256>>>(p.A, A1, p.B0, p.B1, ref, p.drow, p.darow, p.rows,
                                                               p.K, p.N, segs);
  CK(hipMemset(p.C, 0xff, (size_t)p.rows * p.N * 2));
  launch_nt<Cfg>(p, A1, segs, dense);
  CK(hipDeviceSynchronize());
  char shape[128];
  snprintf(shape, sizeof shape, "E=%d rows=%d K=%d N=%d segs=%d", p.E, p.rows, p.K, p.N, segs);
  const bool ok = compare(name, ref, p.C, (size_t)p.rows * p.N, shape);
  hipFree(ref);
  if (A1) hipFree(A1);
  return ok;
}

template <typename Cfg>
static void launch_tn(Problem& p, const uint16_t* D0, const uint16_t* D1, uint16_t* C0, uint16_t* C1, bool p_gather,
                      bool d_gather, bool dense) {
  auto kernel = grouped_gemm_tn_kernel<Cfg>;
  CK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                         (int)Cfg::SMEM_BYTES));
  const long mt = (p.K + Cfg::BMO - 1) / Cfg::BMO, nt = (p.N + Cfg::BNO - 1) / Cfg::BNO;
  const int groups = dense ? 1 : p.E;
  const long tiles_grid = gemm_grid(groups * mt, nt);
  kernel<<<(unsigned)(!g_one_tile_per_workgroup && tiles_grid > 256 ? 256 : tiles_grid), Cfg::NT, Cfg::SMEM_BYTES>>>(
      p.A, D0, D1, C0, C1, dense ? nullptr : p.dgs, dense ? nullptr : p.doff, groups, p.rows, p.K, p.N, (int)mt,
      (int)nt, p.dmap, p.top_k > 0 ? p.top_k : 1, p_gather, d_gather, p.a_rows, 0);
}

// which operand goes through the row map: 0 none, 1 the transposed one (P), 2 the other (D)
template <typename Cfg>
static bool check_tn(const char* name, Problem& p, int gather_which, bool dense = false) {
  const bool pg = gather_which == 1, dg = gather_which == 2;
  // P is p.A ([a_rows, K] if gathered, else its first rows are used as [rows, K]: make sure it is big enough)
  uint16_t* P = pg ? p.A : random_bf16((size_t)p.rows * p.K, 91, 1.0f);
  const size_t d_rows = dg ? p.a_rows : p.rows;
  uint16_t* D0 = random_bf16(d_rows * p.N, 92, 1.0f);
  uint16_t* D1 = random_bf16(d_rows * p.N, 93, 1.0f);
  const size_t out = (size_t)(dense ? 1 : p.E) * p.K * p.N;
  uint16_t *C0, *C1;
  CK(hipMalloc(&C0, out * 2)); CK(hipMalloc(&C1, out * 2));
  CK(hipMemset(C0, 0xff, out * 2)); CK(hipMemset(C1, 0xff, out * 2));
  // identity row lookup for operands that are not gathered
  std::vector<int> ident(p.rows);
  for (int r = 0; r < p.rows; ++r) ident[r] = r;
  int* dident;
  CK(hipMalloc(&dident, p.rows * 4));
  CK(hipMemcpy(dident, ident.data(), p.rows * 4, hipMemcpyHostToDevice));
  std::vector<int> one_gs{p.rows}, one_off{0};
  int *dgs1, *doff1;
  CK(hipMalloc(&dgs1, 4)); CK(hipMalloc(&doff1, 4));
  CK(hipMemcpy(dgs1, one_gs.data(), 4, hipMemcpyHostToDevice));
  CK(hipMemcpy(doff1, one_off.data(), 4, hipMemcpyHostToDevice));
  float *ref0, *ref1;
  CK(hipMalloc(&ref0, out * 4)); CK(hipMalloc(&ref1, out * 4));
  const dim3 grid((p.N + 255) / 256, p.K, dense ? 1 : p.E);
  reference_tn_kernel<<<grid, 256>>>(P, D0, ref0, dense ? dgs1 : p.dgs, dense ? doff1 : p.doff, pg ? p.darow : dident,
                                     dg ? p.darow : dident, p.K, p.N);
  reference_tn_kernel<<<grid, 256>>>(P, D1, ref1, dense ? dgs1 : p.dgs, dense ? doff1 : p.doff, pg ? p.darow : dident,
                                     dg ? p.darow : dident, p.K, p.N);
  Problem q = p;
  q.A = P;
  launch_tn<Cfg>(q, D0, D1, C0, C1, pg, dg, dense);
  CK(hipDeviceSynchronize());
  char shape[128];
  snprintf(shape, sizeof shape, "E=%d rows=%d KA=%d N=%d gather=%d", p.E, p.rows, p.K, p.N, gather_which);
  bool ok = compare(name, ref0, C0, out, shape);
  if (Cfg::kDual) ok &= compare(name, ref1, C1, out, shape);
  hipFree(ref0); hipFree(ref1); hipFree(C0); hipFree(C1); hipFree(D0); hipFree(D1); hipFree(dident);
  hipFree(dgs1); hipFree(doff1);
  if (!pg) hipFree(P);
  return ok;
}

template <typename F>
static void time_launches(const char* name, double flops, int iters, F launch_once) {
  hipEvent_t a, b;
  CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  for (int i = 0; i < 40; ++i) launch_once();  // long warm-up, as in timeit
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(a));
  for (int i = 0; i < iters; ++i) launch_once();
  CK(hipEventRecord(b)); CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  ms /= iters;
  printf("time %-52s %.3f ms  %.1f TFLOP/s  (%.1f%% of 2500)\n", name, ms, flops / ms / 1e9, flops / ms / 1e9 / 25.0);
  fflush(stdout);
}

// the four backward launches of the routed experts at the layer shape: 64 groups, 131072 packed
// rows that are 16384 token rows fetched through a permutation, hidden 2048, intermediate 1408
static void time_backward() {
  const int E = 64, T = 16384, topk = 8, H = 2048, I = 1408, rows = T * topk;
  {  // forward gate/up launch that also stores the two products for the backward pass
    Problem p = make(E, rows, H, I, 20, false, topk, 1.0f);
    uint16_t *s0, *s1;
    CK(hipMalloc(&s0, (size_t)rows * I * 2)); CK(hipMalloc(&s1, (size_t)rows * I * 2));
    auto kernel = grouped_gemm_dma_kernel<GateUpCfg>;
    CK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                           (int)GateUpCfg::SMEM_BYTES));
    const long mt = (rows + GateUpCfg::BM - 1) / GateUpCfg::BM + E, nt = (I + GateUpCfg::BN - 1) / GateUpCfg::BN;
    for (int save = 0; save < 2; ++save)
      time_launches(save ? "forward gate/up, products kept" : "forward gate/up", 4.0 * rows * H * I, 10, [&] {
        kernel<<<(unsigned)gemm_grid(mt, nt), GateUpCfg::NT, GateUpCfg::SMEM_BYTES>>>(
            p.A, p.B0, p.B1, p.C, p.dgs, p.doff, E, rows, H, I, (int)mt, (int)nt, p.dmap, topk, p.a_rows,
            save ? s0 : nullptr, save ? s1 : nullptr, 0, 0);
      });
    hipFree(s0); hipFree(s1);
    release(p);
  }
  {  // d act = dy[token of row] @ Wd^T : A gathered [T, H], B [E, I, H]
    Problem p = make(E, rows, H, I, 21, false, topk, 1.0f);
    time_launches("dgrad down (gathered dy @ Wd^T)", 2.0 * rows * H * I, 10, [&] { launch_nt<DgradCfg>(p, nullptr, 1, false); });
    // dWg, dWu = x[token of row]^T @ (dG, dU)
    uint16_t* D0 = random_bf16((size_t)rows * I, 31, 1.0f);
    uint16_t* D1 = random_bf16((size_t)rows * I, 32, 1.0f);
    uint16_t *C0, *C1;
    CK(hipMalloc(&C0, (size_t)E * H * I * 2)); CK(hipMalloc(&C1, (size_t)E * H * I * 2));
    time_launches("wgrad gate/up (gathered x^T @ dG, dU)", 4.0 * rows * H * I, 10,
                  [&] { launch_tn<WgradDualGatherCfg>(p, D0, D1, C0, C1, true, false, false); });
    {  // the same product on a permuted copy of x: what the library runs
      uint16_t* Xp = random_bf16((size_t)rows * H, 36, 1.0f);
      Problem q = p;
      q.A = Xp;
      time_launches("wgrad gate/up (packed x^T @ dG, dU)", 4.0 * rows * H * I, 10,
                    [&] { launch_tn<WgradDualCfg>(q, D0, D1, C0, C1, false, false, false); });
      hipFree(Xp);
    }
    hipFree(D0); hipFree(D1); hipFree(C0); hipFree(C1);
    release(p);
  }
  {  // dXp = dG @ Wg^T + dU @ Wu^T : A [rows, I] twice, B [E, H, I] twice
    Problem p = make(E, rows, I, H, 22, false, 0, 1.0f);
    uint16_t* A1 = random_bf16((size_t)rows * I, 33, 1.0f);
    time_launches("dgrad gate/up (dG @ Wg^T + dU @ Wu^T)", 4.0 * rows * H * I, 10, [&] { launch_nt<DgradCfg>(p, A1, 2, false); });
    hipFree(A1);
    release(p);
  }
  {  // dWd = (w * act)^T @ dy[token of row] : P [rows, I], D gathered [T, H]
    Problem p = make(E, rows, I, H, 23, false, topk, 1.0f);  // p.A is [T, I] here and unused as P
    uint16_t* P = random_bf16((size_t)rows * I, 34, 1.0f);
    uint16_t* D = random_bf16((size_t)T * H, 35, 1.0f);
    uint16_t* C0;
    CK(hipMalloc(&C0, (size_t)E * H * I * 2));
    Problem q = p;
    q.A = P;
    time_launches("wgrad down (act^T @ gathered dy)", 2.0 * rows * H * I, 10,
                  [&] { launch_tn<WgradGatherCfg>(q, D, nullptr, C0, nullptr, false, true, false); });
    {
      uint16_t* dYp = random_bf16((size_t)rows * H, 37, 1.0f);
      time_launches("wgrad down (act^T @ packed dy)", 2.0 * rows * H * I, 10,
                    [&] { launch_tn<WgradCfg>(q, dYp, nullptr, C0, nullptr, false, false, false); });
      hipFree(dYp);
    }
    hipFree(P); hipFree(D); hipFree(C0);
    release(p);
  }
}

// decode-sized batch: 8 rows per group, bound by streaming the expert matrices
// Reads the first `rows` rows of every expert's [K, N] matrix (both matrices of a dual launch) and
// throws the data away: what is left behind is the data in the memory-side cache.
__global__ __launch_bounds__(1024) void touch_rows_kernel(const u32x4_t* b0, const u32x4_t* b1, int E, size_t matrix_vecs,
                                                          size_t head_vecs, unsigned* sink) {
  const size_t total = (size_t)E * 2 * head_vecs;
  u32x4_t acc = {0u, 0u, 0u, 0u};
  for (size_t i = (size_t)blockIdx.x * 1024 + threadIdx.x; i < total; i += (size_t)gridDim.x * 1024) {
    const size_t region = i / head_vecs, within = i - region * head_vecs;
    const u32x4_t* base = (region & 1) ? b1 : b0;
    const u32x4_t v = base[(region >> 1) * matrix_vecs + within];
    acc[0] ^= v[0]; acc[1] ^= v[1]; acc[2] ^= v[2]; acc[3] ^= v[3];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) *sink = 1;  // keeps the loads alive
}

// The decode-shape gate/up launch with the caches cold (a 1 GiB fill before every launch), and with the
// first `head_rows` rows of every expert matrix read once between the fill and the launch.
static void time_decode_prefetch(Problem& g, int head_rows, int iters) {
  static u32x4_t* junk = nullptr;
  static unsigned* sink = nullptr;
  const size_t junk_vecs = (size_t)1 << 26;
  if (junk == nullptr) { CK(hipMalloc(&junk, junk_vecs * 16)); CK(hipMalloc(&sink, 4)); }
  hipEvent_t a, b, c;
  CK(hipEventCreate(&a)); CK(hipEventCreate(&b)); CK(hipEventCreate(&c));
  const size_t matrix_vecs = (size_t)g.K * g.N * 2 / 16, head_vecs = (size_t)head_rows * g.N * 2 / 16;
  double touch_ms = 0, gemm_ms = 0;
  for (int i = 0; i < iters + 3; ++i) {
    flush_fill_kernel<<<4096, 256>>>(junk, junk_vecs);
    CK(hipEventRecord(a));
    if (head_rows > 0)
      touch_rows_kernel<<<255, 1024>>>(reinterpret_cast<const u32x4_t*>(g.B0), reinterpret_cast<const u32x4_t*>(g.B1),
                                       g.E, matrix_vecs, head_vecs, sink);
    CK(hipEventRecord(b));
    launch<GateUpTinyCfg>(g, false);
    CK(hipEventRecord(c)); CK(hipEventSynchronize(c));
    float t0, t1;
    CK(hipEventElapsedTime(&t0, a, b)); CK(hipEventElapsedTime(&t1, b, c));
    if (i >= 3) { touch_ms += t0; gemm_ms += t1; }
  }
  printf("time decode gate/up, caches cold, first %4d rows of each matrix touched before (%.1f MB): touch %.1f us, launch %.1f us\n",
         head_rows, (double)g.E * 2 * head_vecs * 16 / 1e6, touch_ms / iters * 1e3, gemm_ms / iters * 1e3);
  fflush(stdout);
}

static void time_decode() {
  Problem g = make(64, 512, 2048, 1408, 8, false, 0, 1.0f);
  Problem d = make(64, 512, 1408, 2048, 9, false, 0, 1.0f);
  for (int rep = 0; rep < 2; ++rep)
    for (int head : {0, 128, 256, 384, 512, 2048}) time_decode_prefetch(g, head, 20);
  timeit<GateUpCfg>("gate/up 64 groups, 256-row tiles", g, 20);
  timeit<DownCfg>("down 64 groups, 256-row tiles", d, 20);
  for (int rep = 0; rep < 3; ++rep) {
    timeit<GateUpSmallCfg>("gate/up 64 groups, 64-row tiles", g, 50);
    timeit<GateUpTinyCfg>("gate/up 64 groups, 64-row tiles, weights non-temporal", g, 50);
    timeit<DownSmallCfg>("down 64 groups, 64-row tiles", d, 50);
    timeit<DownTinyCfg>("down 64 groups, 64-row tiles, weights non-temporal", d, 50);
  }
  release(g);
  release(d);
}

int main(int argc, char** argv) {
  bool ok = true;
  // "<mode> nocheck": only the timing mode (for counter collection); otherwise every check runs first
  const bool nocheck = argc > 2 && !strcmp(argv[2], "nocheck");
  if (!nocheck) {
  {
    Problem p = make(7, 3001, 576, 392, 1, true, 0, 1.0f);  // ragged groups, N not a multiple of the tile
    ok &= check<GateUpCfg>("gate/up ragged", p);
    ok &= check<DownCfg>("down ragged", p);
    release(p);
  }
  {
    Problem p = make(5, 2400, 512, 384, 2, true, 3, 1.0f);  // rows fetched through a permutation
    ok &= check<GateUpCfg>("gate/up gather on load", p);
    release(p);
  }
  {
    Problem p = make(1, 777, 512, 520, 3, false, 0, 1.0f);  // one group covering every row
    ok &= check<GateUpCfg>("gate/up dense", p, true);
    ok &= check<DownCfg>("down dense", p, true);
    release(p);
  }
  {
    Problem p = make(16, 150, 512, 392, 6, true, 0, 1.0f);  // a handful of rows per group: the 64-row tiles
    ok &= check<GateUpSmallCfg>("gate/up few rows per group", p);
    ok &= check<DownSmallCfg>("down few rows per group", p);
    release(p);
  }
  {
    Problem p = make(5, 300, 512, 384, 7, true, 3, 1.0f);
    ok &= check<GateUpSmallCfg>("gate/up few rows, gather on load", p);
    ok &= check<GateUpTinyCfg>("gate/up few rows, gather, streamed weights", p);
    release(p);
    Problem q = make(16, 150, 512, 392, 8, true, 0, 1.0f);
    ok &= check<GateUpTinyCfg>("gate/up few rows, streamed weights", q);
    ok &= check<DownTinyCfg>("down few rows, streamed weights", q);
    release(q);
  }
  {
    Problem p = make(7, 3001, 576, 392, 11, true, 0, 1.0f);
    ok &= check_nt<DgradCfg>("dgrad ragged", p, 1);
    ok &= check_nt<DgradCfg>("dgrad ragged, two segments", p, 2);
    ok &= check_tn<WgradCfg>("wgrad ragged", p, 0);
    ok &= check_tn<WgradDualCfg>("wgrad dual ragged", p, 0);
    release(p);
  }
  {
    Problem p = make(5, 2400, 512, 384, 12, true, 3, 1.0f);
    ok &= check_nt<DgradCfg>("dgrad gather on load", p, 1);
    ok &= check_tn<WgradDualGatherCfg>("wgrad dual, transposed operand gathered", p, 1);
    ok &= check_tn<WgradGatherCfg>("wgrad, other operand gathered", p, 2);
    release(p);
  }
  {
    Problem p = make(1, 777, 512, 520, 13, false, 0, 1.0f);
    ok &= check_nt<DgradCfg>("dgrad dense", p, 2, true);
    ok &= check_tn<WgradCfg>("wgrad dense", p, 0, true);
    ok &= check_tn<WgradDualCfg>("wgrad dual dense", p, 0, true);
    release(p);
  }
  {
    // the 4 x 16 block layout of the B tile, which the large configurations no longer use
    using GateUpNarrowCfg = DmaGemmCfg<256, 128, 64, 4, 2, true, 2, 16>;
    using DownNarrowCfg = DmaGemmCfg<256, 256, 64, 2, 4, false, 2, 16 + 64>;
    Problem p = make(7, 3001, 576, 392, 21, true, 0, 1.0f);
    ok &= check<GateUpNarrowCfg>("gate/up ragged, 4 x 16 blocks", p);
    ok &= check<DownNarrowCfg>("down ragged, 4 x 16 blocks", p);
    release(p);
  }
  {
    // the one-tile-per-workgroup kernel with the 256-row configurations (the library runs them persistently)
    g_one_tile_per_workgroup = true;
    Problem p = make(7, 3001, 576, 392, 24, true, 0, 1.0f);
    ok &= check<GateUpCfg>("gate/up ragged, one tile per workgroup", p);
    ok &= check<DownCfg>("down ragged, one tile per workgroup", p);
    release(p);
    Problem q = make(5, 2400, 512, 384, 25, true, 3, 1.0f);
    ok &= check<GateUpCfg>("gate/up gather, one tile per workgroup", q);
    release(q);
    g_one_tile_per_workgroup = false;
    Problem t = make(3, 700, 64, 136, 26, false, 0, 1.0f);  // a single k step per tile
    ok &= check<GateUpCfg>("gate/up one k step", t);
    ok &= check<DownCfg>("down one k step", t);
    release(t);
    Problem u = make(40, 70000, 128, 264, 27, true, 0, 1.0f);  // many more tiles than workgroups
    ok &= check<GateUpCfg>("gate/up many tiles per workgroup", u);
    ok &= check<DownCfg>("down many tiles per workgroup", u);
    release(u);
  }
  {
    Problem u = make(40, 70000, 128, 264, 28, true, 0, 1.0f);  // many more tiles than workgroups
    ok &= check_nt<DgradCfg>("dgrad many tiles per workgroup", u, 1);
    ok &= check_nt<DgradCfg>("dgrad many tiles per workgroup, two segments", u, 2);
    release(u);
    Problem v = make(9, 20000, 64, 520, 29, true, 3, 1.0f);  // one k step, gathered rows
    ok &= check_nt<DgradCfg>("dgrad one k step, gather on load", v, 1);
    release(v);
  }
  {
    Problem u = make(40, 30000, 520, 264, 30, true, 0, 1.0f);  // many more (group, tile) pairs than workgroups
    ok &= check_tn<WgradCfg>("wgrad many pairs per workgroup", u, 0);
    ok &= check_tn<WgradDualCfg>("wgrad dual many pairs per workgroup", u, 0);
    release(u);
    Problem v = make(70, 20000, 520, 264, 31, true, 3, 1.0f);  // the same with gathered operands and empty groups
    ok &= check_tn<WgradDualGatherCfg>("wgrad dual many pairs, transposed operand gathered", v, 1);
    ok &= check_tn<WgradGatherCfg>("wgrad many pairs, other operand gathered", v, 2);
    release(v);
    Problem w = make(256, 50000, 136, 264, 32, true, 0, 1.0f);  // the most groups, very unequal sizes
    ok &= check_tn<WgradCfg>("wgrad 256 unequal groups", w, 0);
    ok &= check_tn<WgradDualCfg>("wgrad dual 256 unequal groups", w, 0);
    release(w);
    Problem tiny = make(250, 7500, 256, 264, 49, false, 0, 1.0f);  // groups of about 30 rows: fewer k steps than stages
    ok &= check_tn<WgradCfg>("wgrad tiny groups", tiny, 0);
    ok &= check_tn<WgradDualCfg>("wgrad dual tiny groups", tiny, 0);
    release(tiny);
  }
  {
    // the stream kernel: 32-deep steps with four stages, and 64-deep steps with two
    g_stream = true;
    Problem p = make(7, 3001, 576, 392, 51, true, 0, 1.0f);
    ok &= check<GateUpStreamCfg>("stream gate/up ragged", p);
    ok &= check<DownStreamCfg>("stream down ragged", p);
    ok &= check<GateUpStream2Cfg>("stream 2 x 64 gate/up ragged", p);
    ok &= check<DownStream2Cfg>("stream 2 x 64 down ragged", p);
    release(p);
    Problem q = make(5, 2400, 512, 384, 52, true, 3, 1.0f);
    ok &= check<GateUpStreamCfg>("stream gate/up gather on load", q);
    ok &= check<GateUpStream2Cfg>("stream 2 x 64 gate/up gather on load", q);
    release(q);
    Problem r = make(1, 777, 512, 520, 53, false, 0, 1.0f);
    ok &= check<GateUpStreamCfg>("stream gate/up dense", r, true);
    ok &= check<DownStreamCfg>("stream down dense", r, true);
    release(r);
    Problem u = make(40, 70000, 256, 264, 54, true, 0, 1.0f);  // many more tiles than workgroups
    ok &= check<GateUpStreamCfg>("stream gate/up many tiles per workgroup", u);
    ok &= check<DownStreamCfg>("stream down many tiles per workgroup", u);
    ok &= check<DownStream2Cfg>("stream 2 x 64 down many tiles per workgroup", u);
    release(u);
    Problem v = make(33, 90000, 256, 392, 55, true, 4, 1.0f);  // the same with gathered rows (row map by LDS-DMA)
    ok &= check<GateUpStreamCfg>("stream gate/up many tiles, gather", v);
    ok &= check<GateUpStream2Cfg>("stream 2 x 64 gate/up many tiles, gather", v);
    g_chunk = 0;
    ok &= check<GateUpStreamCfg>("stream gate/up many tiles, gather, one workgroup per CU", v);
    g_chunk = -1;
    release(v);
    g_stream = false;
    // the transposed-B form of the stream kernel
    for (g_stream_nt = 1; g_stream_nt <= 3; ++g_stream_nt) {
    Problem w1 = make(7, 3001, 576, 392, 61, true, 0, 1.0f);  // ragged groups, N not a multiple of the tile
    ok &= check_nt<DgradCfg>("stream dgrad ragged", w1, 1);
    ok &= check_nt<DgradCfg>("stream dgrad ragged, two segments", w1, 2);
    release(w1);
    Problem w2 = make(5, 2400, 512, 384, 62, true, 3, 1.0f);
    ok &= check_nt<DgradCfg>("stream dgrad gather on load", w2, 1);
    release(w2);
    Problem w3 = make(1, 777, 512, 520, 63, false, 0, 1.0f);
    ok &= check_nt<DgradCfg>("stream dgrad dense, two segments", w3, 2, true);
    release(w3);
    Problem w4 = make(40, 70000, 256, 264, 64, true, 0, 1.0f);  // many more tiles than workgroups
    ok &= check_nt<DgradCfg>("stream dgrad many tiles per workgroup", w4, 1);
    ok &= check_nt<DgradCfg>("stream dgrad many tiles per workgroup, two segments", w4, 2);
    release(w4);
    Problem w5 = make(33, 90000, 128, 392, 65, true, 4, 1.0f);  // 4 k steps per segment: two segments just fill the pipeline
    ok &= check_nt<DgradCfg>("stream dgrad short segments, gather", w5, 2);
    release(w5);
    }
    g_stream_nt = 0;
  }
  }  // !nocheck
  if (ok && argc > 1 && !strcmp(argv[1], "time_stream")) {
    Problem g = make(64, 131072, 2048, 1408, 4, false, 8, 1.0f);  // rows gathered through a permutation, as in the layer
    Problem d = make(64, 131072, 1408, 2048, 5, false, 0, 1.0f);
    for (int rep = 0; rep < 3; ++rep) {
      g_stream = false;
      timeit<GateUpCfg>("gate/up library", g, 20);
      timeit<DownCfg>("down library", d, 20);
      g_stream = true;
      timeit<GateUpStreamCfg>("gate/up stream 4 x 32 (library)", g, 20);
      timeit<DownStreamCfg>("down stream 4 x 32", d, 20);
      timeit<GateUpStream2Cfg>("gate/up stream 2 x 64", g, 20);
      timeit<DownStream2Cfg>("down stream 2 x 64", d, 20);
      g_chunk = 0;
      timeit<GateUpStreamCfg>("gate/up stream 4 x 32, one wg per CU", g, 20);
      timeit<DownStreamCfg>("down stream 4 x 32, 4 tiles per wg", d, 20);
      g_chunk = -1;
      g_stream = false;
    }
    release(g); release(d);
    // a dense square problem: the steady-state loop without ragged tiles
    Problem sq = make(1, 8192, 8192, 8192, 6, false, 0, 1.0f);
    for (int rep = 0; rep < 2; ++rep) {
      g_stream = false;
      timeit<DownCfg>("8192^3 library", sq, 10);
      g_stream = true;
      timeit<DownStreamCfg>("8192^3 stream 4 x 32", sq, 10);
      timeit<DownStream2Cfg>("8192^3 stream 2 x 64", sq, 10);
      g_stream = false;
    }
    release(sq);
  }
  if (ok && argc > 1 && !strcmp(argv[1], "time_stream_nt")) {
    // the data-gradient products of the C3 backward pass: older kernel against the stream form
    const int rows = 131072, H = 2048, I = 1408, E = 64;
    Problem z = make(E, rows, H, I, 21, false, 0, 1.0f);   // Z = dYp @ Wd^T : A [rows, H], B [E, I, H]
    Problem x = make(E, rows, I, H, 22, false, 0, 1.0f);   // dXp = dG @ Wg^T + dU @ Wu^T : A [rows, I] twice, B [E, H, I] twice
    uint16_t* A1 = random_bf16((size_t)rows * I, 33, 1.0f);
    for (int rep = 0; rep < 3; ++rep) {
      const char* names[4] = {"older kernel", "stream 4 x 32, 2 x 4 waves", "stream 4 x 32, 4 x 2 waves", "stream 2 x 64, 2 x 4 waves"};
      for (g_stream_nt = 0; g_stream_nt <= 3; ++g_stream_nt) {
        char label[96];
        snprintf(label, sizeof label, "Z = dYp @ Wd^T, %s", names[g_stream_nt]);
        time_launches(label, 2.0 * rows * H * I, 10, [&] { launch_nt<DgradCfg>(z, nullptr, 1, false); });
        snprintf(label, sizeof label, "dXp (2 segments), %s", names[g_stream_nt]);
        time_launches(label, 4.0 * rows * H * I, 10, [&] { launch_nt<DgradCfg>(x, A1, 2, false); });
      }
      g_stream_nt = 0;
    }
    hipFree(A1);
    release(z); release(x);
  }
  if (ok && argc > 1 && !strcmp(argv[1], "time_c2_down")) {
    // the down projection of the second configuration: 16 groups of about 1024 rows, K = 2816, N = 1024 --
    // 288 tiles of 256 x 256 on 256 CUs (one full round and an eighth of a second one) against 576
    // tiles of 256 x 128 -- which looks 8 % faster when the launch is repeated back to back (operands and result,
    // 217 MB, stay in the memory-side cache) and is 15 % slower with the caches cold, as in a layer
    using Half = DmaGemmCfg<256, 128, 64, 4, 2, false, 2, 16 + 64 + 128 + 32768>;
    Problem d = make(16, 16384, 2816, 1024, 7, false, 0, 1.0f);
    ok &= check<Half>("down, 256 x 128 tiles", d);
    for (int rep = 0; rep < 3; ++rep) {
      timeit<DownCfg>("C2 down, 256 x 256 tiles (library)", d, 20);
      timeit<Half>("C2 down, 256 x 128 tiles", d, 20);
      timeit_cold<DownCfg>("C2 down, 256 x 256 tiles (library)", d, 20);
      timeit_cold<Half>("C2 down, 256 x 128 tiles", d, 20);
    }
    release(d);
    // the gate/up launch of the same configuration (gathered rows, K = 1024, N = 2816: 72 x 22 tiles of
    // 256 x 128 + 128, 6.2 per CU) with the stream kernel's workgroups holding 4 tiles (library), 3, 2, 1,
    // or one workgroup per CU walking its share (0)
    {
      Problem g2 = make(16, 16384, 1024, 2816, 6, false, 2, 1.0f);
      g_stream = true;
      for (int rep = 0; rep < 3; ++rep)
        for (int chunk : {-1, 0, 1, 2, 3}) {
          g_chunk = chunk;
          char name[64];
          snprintf(name, sizeof name, "C2 gate/up stream, %d tiles per workgroup", chunk < 0 ? 4 : chunk);
          timeit_cold<GateUpStreamCfg>(name, g2, 20);
        }
      g_chunk = -1;
      // the same launch with 64-deep steps in two stages, and with the older kernel
      for (int rep = 0; rep < 3; ++rep) {
        g_stream = true;
        timeit_cold<GateUpStreamCfg>("C2 gate/up stream 4 x 32 (library)", g2, 20);
        timeit_cold<GateUpStream2Cfg>("C2 gate/up stream 2 x 64", g2, 20);
        g_stream = false;
        timeit_cold<GateUpCfg>("C2 gate/up, older kernel", g2, 20);
      }
      g_stream = false;
      release(g2);
    }
    Problem d3 = make(64, 131072, 1408, 2048, 5, false, 0, 1.0f);
    for (int rep = 0; rep < 2; ++rep) {
      timeit<DownCfg>("C3 down, 256 x 256 tiles (library)", d3, 20);
      timeit<Half>("C3 down, 256 x 128 tiles", d3, 20);
    }
    release(d3);
  }
  if (ok && argc > 1 && !strcmp(argv[1], "time_prio")) {
    using Prio = DmaGemmCfg<256, 128, 32, 4, 2, true, 4, 16 + 128 + 32>;
    Problem g = make(64, 131072, 2048, 1408, 4, false, 8, 1.0f);
    g_stream = true;
    for (int rep = 0; rep < 3; ++rep) {
      timeit<GateUpStreamCfg>("gate/up stream", g, 20);
      timeit<Prio>("gate/up stream, wave priority around the MFMAs", g, 20);
    }
    g_stream = false;
    release(g);
  }
  if (ok && argc > 1 && !strcmp(argv[1], "time_ragged")) {
    // What the ragged last tile of every group costs: the C3 launches on groups of random sizes
    // (about 2048 +- 45 rows: 544 row tiles, 64 of them partly filled) and on 64 groups of exactly
    // 2048 rows (512 full row tiles).
    Problem g = make(64, 131072, 2048, 1408, 4, false, 8, 1.0f);
    Problem d = make(64, 131072, 1408, 2048, 5, false, 0, 1.0f);
    g_equal_groups = true;
    Problem ge = make(64, 131072, 2048, 1408, 4, false, 8, 1.0f);
    Problem de = make(64, 131072, 1408, 2048, 5, false, 0, 1.0f);
    g_equal_groups = false;
    for (int rep = 0; rep < 3; ++rep) {
      g_stream = true;
      timeit<GateUpStreamCfg>("gate/up stream, random group sizes", g, 20);
      timeit<GateUpStreamCfg>("gate/up stream, equal groups", ge, 20);
      g_stream = false;
      timeit<DownCfg>("down library, random group sizes", d, 20);
      timeit<DownCfg>("down library, equal groups", de, 20);
    }
    release(g); release(d); release(ge); release(de);
  }
  if (ok && argc > 1 && !strcmp(argv[1], "time_ablation")) {
    // What bounds the stream kernel: the same launch with parts of the k loop left out (results are
    // wrong by construction), on N(0,1) x N(0,0.05) operands and on all-zero operands.  Dense problems
    // (one group), one workgroup per CU.
    using Full = GateUpStreamCfg;
    using NoLoads = DmaGemmCfg<256, 128, 32, 4, 2, true, 4, 16 + 128 + 256>;
    using NoFrags = DmaGemmCfg<256, 128, 32, 4, 2, true, 4, 16 + 128 + 512>;
    using MfmaOnly = DmaGemmCfg<256, 128, 32, 4, 2, true, 4, 16 + 128 + 256 + 512>;
    using SqFull = DownStreamCfg;
    using SqNoLoads = DmaGemmCfg<256, 256, 32, 2, 4, false, 4, 16 + 128 + 32768 + 256>;
    using SqNoFrags = DmaGemmCfg<256, 256, 32, 2, 4, false, 4, 16 + 128 + 32768 + 512>;
    using SqMfmaOnly = DmaGemmCfg<256, 256, 32, 2, 4, false, 4, 16 + 128 + 32768 + 256 + 512>;
    using SameTile = DmaGemmCfg<256, 128, 32, 4, 2, true, 4, 16 + 128 + 1024>;
    using SqSameTile = DmaGemmCfg<256, 256, 32, 2, 4, false, 4, 16 + 128 + 32768 + 1024>;
    g_stream = true;
    g_chunk = 0;
    for (float scale : {1.0f, 0.0f}) {
      printf("-- operand data: %s\n", scale > 0 ? "N(0,1) activations, N(0,0.05) weights" : "all zeros");
      Problem gd = make(1, 131072, 2048, 1408, 4, false, 0, scale);
      timeit<Full>("gate/up dense: whole kernel", gd, 10);
      timeit<NoLoads>("gate/up dense: no operand loads", gd, 10);
      timeit<NoFrags>("gate/up dense: no fragment reads", gd, 10);
      timeit<MfmaOnly>("gate/up dense: MFMAs and barriers only", gd, 10);
      timeit<SameTile>("gate/up dense: loads of one cached k step", gd, 10);
      release(gd);
      Problem sq = make(1, 8192, 8192, 8192, 6, false, 0, scale);
      timeit<SqFull>("8192^3: whole kernel", sq, 10);
      timeit<SqNoLoads>("8192^3: no operand loads", sq, 10);
      timeit<SqNoFrags>("8192^3: no fragment reads", sq, 10);
      timeit<SqMfmaOnly>("8192^3: MFMAs and barriers only", sq, 10);
      timeit<SqSameTile>("8192^3: loads of one cached k step", sq, 10);
      release(sq);
    }
    g_chunk = -1;
    g_stream = false;
  }
  if (ok && argc > 1 && !strcmp(argv[1], "counters_stream")) {
    // a few launches of each kernel for a hardware-counter run (rocprofv3 --pmc ... -- gemm_check counters_stream nocheck)
    Problem g = make(64, 131072, 2048, 1408, 4, false, 8, 1.0f);
    Problem d = make(64, 131072, 1408, 2048, 5, false, 0, 1.0f);
    Problem sq = make(1, 8192, 8192, 8192, 6, false, 0, 1.0f);
    for (int rep = 0; rep < 12; ++rep) {
      g_stream = false;
      launch<GateUpCfg>(g, false);
      launch<DownCfg>(d, false);
      launch<DownCfg>(sq, false);
      g_stream = true;
      launch<GateUpStreamCfg>(g, false);
      launch<GateUpStream2Cfg>(g, false);
      launch<DownStreamCfg>(sq, false);
      g_stream = false;
    }
    CK(hipDeviceSynchronize());
    release(g); release(d); release(sq);
  }
  if (ok && argc > 1 && !strcmp(argv[1], "time_tn_stages")) {
    // the weight-gradient kernel with two stages of 64 rows, and three and four (the library's) of 32
    using Dual64x2 = WgradDualGatherCfg;
    using Dual32x3 = TnGemmCfg<256, 128, 4, 2, true, 16 + 32768, 32, 3>;
    using Single64x2 = WgradGatherCfg;
    using Single32x3 = TnGemmCfg<256, 256, 2, 4, false, 16 + 32768, 32, 3>;
    {
      Problem c = make(37, 50000, 512, 392, 41, false, 0, 1.0f);
      ok &= check_tn<Dual32x3>("wgrad dual, 3 stages of 32", c, 0);
      ok &= check_tn<Single32x3>("wgrad, 3 stages of 32", c, 0);
      release(c);
      Problem w = make(256, 60000, 256, 264, 43, true, 0, 1.0f);
      ok &= check_tn<Dual32x3>("wgrad dual, 3 stages of 32, unequal groups", w, 0);
      release(w);
      Problem d = make(1, 5000, 512, 392, 47, false, 0, 1.0f);
      ok &= check_tn<Single32x3>("wgrad, 3 stages of 32, dense", d, 0, true);
      release(d);
    }
    const int E = 64, T = 16384, topk = 8, H = 2048, I = 1408, rows = T * topk;
    Problem p = make(E, rows, H, I, 21, false, 0, 1.0f);
    uint16_t* D0 = random_bf16((size_t)rows * I, 31, 1.0f);
    uint16_t* D1 = random_bf16((size_t)rows * I, 32, 1.0f);
    uint16_t *C0, *C1;
    CK(hipMalloc(&C0, (size_t)E * H * I * 2)); CK(hipMalloc(&C1, (size_t)E * H * I * 2));
    Problem q = make(E, rows, I, H, 23, false, 0, 1.0f);
    uint16_t* dYp = random_bf16((size_t)rows * H, 37, 1.0f);
    for (int rep = 0; ok && rep < 3; ++rep) {
      time_launches("wgrad gate/up, 2 stages of 64", 4.0 * rows * H * I, 10, [&] { launch_tn<Dual64x2>(p, D0, D1, C0, C1, false, false, false); });
      time_launches("wgrad gate/up, 3 stages of 32", 4.0 * rows * H * I, 10, [&] { launch_tn<Dual32x3>(p, D0, D1, C0, C1, false, false, false); });
      time_launches("wgrad gate/up, 4 stages of 32 (library)", 4.0 * rows * H * I, 10, [&] { launch_tn<WgradDualCfg>(p, D0, D1, C0, C1, false, false, false); });
      time_launches("wgrad down, 2 stages of 64", 2.0 * rows * H * I, 10, [&] { launch_tn<Single64x2>(q, dYp, nullptr, C0, nullptr, false, false, false); });
      time_launches("wgrad down, 3 stages of 32", 2.0 * rows * H * I, 10, [&] { launch_tn<Single32x3>(q, dYp, nullptr, C0, nullptr, false, false, false); });
      time_launches("wgrad down, 4 stages of 32 (library)", 2.0 * rows * H * I, 10, [&] { launch_tn<WgradCfg>(q, dYp, nullptr, C0, nullptr, false, false, false); });
    }
    // what stands between the pairs of a workgroup: the same rows in half as many groups twice as
    // long (half the pairs, the same matrix work)
    Problem p2 = make(E / 2, rows, H, I, 21, false, 0, 1.0f);
    Problem q2 = make(E / 2, rows, I, H, 23, false, 0, 1.0f);
    for (int rep = 0; ok && rep < 2; ++rep) {
      time_launches("wgrad gate/up, 64 groups", 4.0 * rows * H * I, 10, [&] { launch_tn<WgradDualCfg>(p, D0, D1, C0, C1, false, false, false); });
      time_launches("wgrad gate/up, 32 groups", 4.0 * rows * H * I, 10, [&] { launch_tn<WgradDualCfg>(p2, D0, D1, C0, C1, false, false, false); });
      time_launches("wgrad down, 64 groups", 2.0 * rows * H * I, 10, [&] { launch_tn<WgradCfg>(q, dYp, nullptr, C0, nullptr, false, false, false); });
      time_launches("wgrad down, 32 groups", 2.0 * rows * H * I, 10, [&] { launch_tn<WgradCfg>(q2, dYp, nullptr, C0, nullptr, false, false, false); });
    }
    release(p2); release(q2);
    hipFree(D0); hipFree(D1); hipFree(C0); hipFree(C1); hipFree(dYp);
    release(p); release(q);
  }
  if (ok && argc > 1 && !strcmp(argv[1], "time_persistent")) {
    Problem g = make(64, 131072, 2048, 1408, 4, false, 0, 1.0f);
    Problem d = make(64, 131072, 1408, 2048, 5, false, 0, 1.0f);
    for (int rep = 0; rep < 3; ++rep) {
      g_one_tile_per_workgroup = true;
      timeit<GateUpCfg>("gate/up one tile per workgroup", g, 20);
      timeit<DownCfg>("down one tile per workgroup", d, 20);
      g_one_tile_per_workgroup = false;
      timeit<GateUpCfg>("gate/up persistent (library)", g, 20);
      timeit<DownCfg>("down persistent (library)", d, 20);
      for (int chunk : {0, 2, 4, 8}) {
        g_chunk = chunk;
        char name[64];
        snprintf(name, sizeof name, "gate/up %d tiles per workgroup", chunk);
        timeit<GateUpCfg>(name, g, 20);
        snprintf(name, sizeof name, "down %d tiles per workgroup", chunk);
        timeit<DownCfg>(name, d, 20);
      }
      g_chunk = -1;
    }
    release(g); release(d);
  }
  if (ok && argc > 1 && !strcmp(argv[1], "time_down")) {
    // The down projection at the shapes of the three large configurations -- 44, 22 and 12 k steps of 64
    // under a 256 x 256 result tile -- with the caches cold, as inside a layer: the library's kernel, the
    // stream kernel (four stages of 32 and two of 64), and the library's loop with the results written
    // straight from transposed accumulators instead of through LDS.
    using DownDirect = DmaGemmCfg<256, 256, 64, 2, 4, false, 2, 16 + 64 + 128 + 2048>;
    // Half-size tiles in workgroups of four waves, two workgroups to a CU (each SIMD then holds waves of two
    // tiles that are in different phases: one tile's epilogue and first loads run under the other's MFMAs)
    using Down256x128w4 = DmaGemmCfg<256, 128, 32, 4, 1, false, 2, 16 + 128 + 32768>;
    using Down256x128w4s3 = DmaGemmCfg<256, 128, 32, 4, 1, false, 3, 16 + 128 + 32768>;
    using Down128x256w4 = DmaGemmCfg<128, 256, 32, 2, 2, false, 2, 16 + 128 + 32768>;
    using Down128x256w4s3 = DmaGemmCfg<128, 256, 32, 2, 2, false, 3, 16 + 128 + 32768>;
    {
      Problem p = make(7, 3001, 576, 392, 71, true, 0, 1.0f);
      ok &= check<DownDirect>("down ragged, results from accumulators", p);
      ok &= check<Down256x128w4>("down ragged, 256 x 128, four waves", p);
      ok &= check<Down256x128w4s3>("down ragged, 256 x 128, four waves, 3 stages", p);
      ok &= check<Down128x256w4>("down ragged, 128 x 256, four waves", p);
      ok &= check<Down128x256w4s3>("down ragged, 128 x 256, four waves, 3 stages", p);
      release(p);
      Problem u = make(40, 70000, 128, 264, 72, true, 0, 1.0f);
      ok &= check<DownDirect>("down many tiles, results from accumulators", u);
      release(u);
    }
    struct Shape { const char* name; int E, rows, K, N; bool skew; };
    const Shape shapes[3] = {{"C2", 16, 16384, 2816, 1024, false}, {"C3", 64, 131072, 1408, 2048, false},
                             {"C4", 128, 131072, 768, 2048, true}};
    for (const Shape& sh : shapes) {
      Problem d = make(sh.E, sh.rows, sh.K, sh.N, 5, sh.skew, 0, 1.0f);
      char name[96];
      for (int rep = 0; ok && rep < 3; ++rep) {
        snprintf(name, sizeof name, "%s down, library", sh.name);
        timeit_cold<DownCfg>(name, d, 20);
        g_stream = true;
        snprintf(name, sizeof name, "%s down, stream 4 x 32", sh.name);
        timeit_cold<DownStreamCfg>(name, d, 20);
        snprintf(name, sizeof name, "%s down, stream 2 x 64", sh.name);
        timeit_cold<DownStream2Cfg>(name, d, 20);
        g_stream = false;
        snprintf(name, sizeof name, "%s down, results from accumulators", sh.name);
        timeit_cold<DownDirect>(name, d, 20);
        snprintf(name, sizeof name, "%s down, 256 x 128 x 32, 4 waves, 2 per CU", sh.name);
        timeit_cold<Down256x128w4>(name, d, 20);
        snprintf(name, sizeof name, "%s down, 256 x 128 x 32, 4 waves, 3 stages", sh.name);
        timeit_cold<Down256x128w4s3>(name, d, 20);
        snprintf(name, sizeof name, "%s down, 128 x 256 x 32, 4 waves, 2 per CU", sh.name);
        timeit_cold<Down128x256w4>(name, d, 20);
        snprintf(name, sizeof name, "%s down, 128 x 256 x 32, 4 waves, 3 stages", sh.name);
        timeit_cold<Down128x256w4s3>(name, d, 20);
      }
      release(d);
    }
  }
  if (ok && argc > 1 && (!strcmp(argv[1], "time_chunks") || !strcmp(argv[1], "counters_chunks"))) {
    // The routed gate/up launch of the third configuration with the stream kernel, its tiles cut into
    // workgroups of 1, 2, 4 (the library's), 8 tiles or one workgroup per CU for the whole launch (0), and,
    // at 4 tiles per workgroup, the tile order walked in groups of 2, 4 (the library's) or 8 m-tiles.
    // time_chunks: events around 20 launches, three rounds, alternating.  counters_chunks: 12 launches of
    // each for a hardware-counter or kernel-trace run (the variants differ in grid size or kernel name).
    using Group8 = DmaGemmCfg<256, 128, 32, 4, 2, true, 4, 16 + 128 + 8192>;
    using Group2 = DmaGemmCfg<256, 128, 32, 4, 2, true, 4, 16 + 128 + 16384>;
    const bool timing = !strcmp(argv[1], "time_chunks");
    Problem g = make(64, 131072, 2048, 1408, 4, false, 8, 1.0f);
    g_stream = true;
    if (timing) {
      ok &= check<Group8>("stream gate/up, groups of 8 m-tiles", g);
      ok &= check<Group2>("stream gate/up, groups of 2 m-tiles", g);
    }
    for (int rep = 0; ok && rep < (timing ? 3 : 12); ++rep) {
      for (int chunk : {0, 1, 2, 4, 8}) {
        g_chunk = chunk;
        char name[80];
        snprintf(name, sizeof name, "gate/up stream, %d tiles per workgroup", chunk);
        if (timing) timeit<GateUpStreamCfg>(name, g, 20); else launch<GateUpStreamCfg>(g, false);
      }
      g_chunk = 4;
      if (timing) {
        timeit<Group2>("gate/up stream, 4 tiles per workgroup, groups of 2 m-tiles", g, 20);
        timeit<Group8>("gate/up stream, 4 tiles per workgroup, groups of 8 m-tiles", g, 20);
      } else {
        launch<Group2>(g, false);
        launch<Group8>(g, false);
      }
    }
    CK(hipDeviceSynchronize());
    g_chunk = -1;
    g_stream = false;
    release(g);
  }
  if (ok && argc > 1 && !strcmp(argv[1], "time_backward")) time_backward();
  if (ok && argc > 1 && !strcmp(argv[1], "time_decode")) time_decode();
  if (ok && argc > 1 && !strcmp(argv[1], "time")) {
    for (float scale : {1.0f, 0.0f}) {
      printf("-- operand data: %s\n", scale > 0 ? "N(0,1) activations, N(0,0.05) weights" : "all zeros");
      Problem g = make(64, 131072, 2048, 1408, 4, false, 0, scale);
      timeit<GateUpCfg>("gate/up 64 groups", g, 20);
      release(g);
      Problem d = make(64, 131072, 1408, 2048, 5, false, 0, scale);
      timeit<DownCfg>("down 64 groups", d, 20);
      release(d);
    }
    time_backward();
    time_decode();
  }
  printf(ok ? "PASS\n" : "FAIL\n");
  return ok ? 0 : 1;
}
