// Stand-alone check of the grouped GEMM kernels (no Python, no torch), in the manner of the
// reference's rmsnorm_test.cu (src/jaxtitan/kernels/cuda/rmsnorm/rmsnorm_test.cu:126-149):
// deterministic inputs, an independent reference (one thread per output element, fp32
// accumulation in k order), a tolerance, and PASS / FAIL on stdout.
//
//   gemm_check            correctness on ragged groups, gather-on-load and the dense case
//   gemm_check time       + timing of the library's two configurations at the C3 shape,
//                           once on N(0,1)-like data and once on all-zero data
#include "grouped_gemm_dma.hpp"

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
static Problem make(int E, int rows, int K, int N, unsigned seed, bool skew, int top_k, float scale) {
  Problem p;
  p.E = E; p.rows = rows; p.K = K; p.N = N; p.top_k = top_k;
  std::mt19937 rng(seed);
  p.gs.assign(E, 0);
  for (int r = 0; r < rows; ++r) {
    int e = skew ? (int)(std::pow((double)(rng() % 10000) / 10000.0, 3.0) * E) : (int)(rng() % E);
    if (skew && e % 5 == 3) e = 0;
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

template <typename Cfg>
static void launch(Problem& p, bool dense) {
  auto kernel = grouped_gemm_dma_kernel<Cfg>;
  CK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                         (int)Cfg::SMEM_BYTES));
  const long mt = dense ? (p.rows + Cfg::BM - 1) / Cfg::BM
                        : (p.rows + Cfg::BM - 1) / Cfg::BM + (p.E < p.rows ? p.E : p.rows);
  const long nt = (p.N + Cfg::BN - 1) / Cfg::BN;
  kernel<<<(unsigned)gemm_grid(mt, nt), Cfg::NT, Cfg::SMEM_BYTES>>>(
      p.A, p.B0, Cfg::kDual ? p.B1 : nullptr, p.C, dense ? nullptr : p.dgs, dense ? nullptr : p.doff, p.E, p.rows,
      p.K, p.N, (int)mt, (int)nt, p.top_k > 0 ? p.dmap : nullptr, p.top_k > 0 ? p.top_k : 1, p.a_rows);
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
  for (int i = 0; i < 10; ++i) launch<Cfg>(p, false);
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

int main(int argc, char** argv) {
  bool ok = true;
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
    release(p);
  }
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
    // decode-sized batch: 8 rows per group, bound by streaming the expert matrices
    Problem g = make(64, 512, 2048, 1408, 8, false, 0, 1.0f);
    timeit<GateUpCfg>("gate/up 64 groups, 256-row tiles", g, 20);
    timeit<GateUpSmallCfg>("gate/up 64 groups, 64-row tiles", g, 20);
    release(g);
    Problem d = make(64, 512, 1408, 2048, 9, false, 0, 1.0f);
    timeit<DownCfg>("down 64 groups, 256-row tiles", d, 20);
    timeit<DownSmallCfg>("down 64 groups, 64-row tiles", d, 20);
    release(d);
  }
  printf(ok ? "PASS\n" : "FAIL\n");
  return ok ? 0 : 1;
}
