// Measurement aids: where the rate of the bf16 MFMA main loop goes (gfx950).  No counterpart in the reference and
// no part of any product path: the entry points below time stripped-down forms of the filtered-rank main loop of
// bf16 tables with d == 128 (rank128_kernel) for a given number of seconds and report the MFMA rate each sustains,
// so that a benchmark run can print the whole ladder from the same box and process:
//   kge_probe_mfma(count = 0, reads = 0)  the tile statement's 32 MFMAs on random bf16 operands held in registers
//   kge_probe_mfma(count = 1, reads = 0)  the same with the rank count between the MFMAs (5 VALU per MFMA)
//   kge_probe_mfma(count = 0 / 1, reads = 1)  the same with the entity fragments re-read from LDS every tile
//   kge_probe_walk                        the main loop itself over a caller's table (global -> LDS stages, barriers,
//                                         fragment reads, MFMAs) without the count
// and, for the top-k scan of int8 tables (topk_i8_filter_kernel):
//   kge_probe_i8_scan                     the scan over a caller's prepared table with thresholds of +inf: no tile
//                                         passes the bound, so what is timed is the hot loop alone (MFMAs, the test
//                                         of every tile, the walk), none of the parking and collecting of candidates
#include "kge_rank128.hip.h"
#include "kge_topk_i8.hip.h"

#include <string.h>

#include <vector>

namespace kge {
namespace {

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}
// about N(0, std): the sum of four uniforms, centred and scaled
__device__ __forceinline__ float probe_normal(uint32_t key, float std) {
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k) s += (float)(probe_hash(key * 4u + k) >> 8) * (1.0f / 16777216.0f);
  return (s - 2.0f) * 1.7320508f * std;
}
__device__ __forceinline__ bf16x8 probe_fragment(uint32_t key, float std) {
  f32x4 lo, hi;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    lo[j] = probe_normal(key * 8u + j, std);
    hi[j] = probe_normal(key * 8u + 4 + j, std);
  }
  return cvt_bf16x8(lo, hi);
}

// `iters` stages of two tile statements per wave, 8 waves per workgroup, two waves per SIMD, no barrier, no global
// traffic.  Operands: random bf16 of the scale of the benchmark's tables; with READS the entity fragments are read
// again from a random LDS buffer under every tile's last chain, as the main loop does.
template <bool COUNT, bool READS>
__global__ void __launch_bounds__(512, 2) probe_tile_kernel(int iters, uint32_t seed, int32_t* sink) {
  constexpr int ROW_BYTES = 256, TILE_BYTES = 32 * ROW_BYTES, STAGE_BYTES = 2 * TILE_BYTES;
  __shared__ __attribute__((aligned(1024))) unsigned char lds_e[QS_NBUF * STAGE_BYTES];
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  const uint32_t me = (seed * 0x9e3779b9u) ^ ((uint32_t)blockIdx.x * 512u + (uint32_t)tid);
  for (int i = tid; i < QS_NBUF * STAGE_BYTES / 16; i += 512)
    *(bf16x8*)(lds_e + 16 * i) = probe_fragment(probe_hash(seed ^ (uint32_t)i) + blockIdx.x, 0.05f);
  __syncthreads();
  bf16x8 qf[R128_NQT][8];
#pragma unroll
  for (int t = 0; t < R128_NQT; ++t) {
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      qf[t][s] = probe_fragment(probe_hash(me) + 64u * t + s, 0.005f);
      asm volatile("" : "+v"(qf[t][s]));
    }
  }
  bf16x8 ef[8];
  int fb[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    fb[s] = c * ROW_BYTES + (((2 * s + hf) ^ (c & 15)) << 4);
    ef[s] = *(const bf16x8*)(lds_e + fb[s]);
  }
  float thr[R128_NQT] = {1e-4f, -1e-4f, 2e-4f, 0.f};
  int32_t gt[R128_NQT] = {0, 0, 0, 0};
  float mn[R128_NQT] = {1e30f, 1e30f, 1e30f, 1e30f};
  r128_acc X;
#pragma unroll
  for (int i = 0; i < 16; ++i) X[i] = 0.f;
  for (int k = 0; k < iters; ++k) {
    r128_tile<TILE_BYTES, COUNT, READS>(qf, ef, fb, X, thr, gt, mn);
    r128_tile<STAGE_BYTES, COUNT, READS>(qf, ef, fb, X, thr, gt, mn);
  }
  asm volatile("s_waitcnt lgkmcnt(0)\ns_nop 7\ns_nop 7" : "+{v[224:239]}"(X)::"memory");
  int32_t keep = gt[0] + gt[1] + gt[2] + gt[3] + (mn[0] + mn[1] + mn[2] + mn[3] == 12345.f ? 1 : 0);
#pragma unroll
  for (int i = 0; i < 16; ++i) keep += X[i] == 54321.f ? 1 : 0;
  if (keep == 0x7fffffff) sink[0] = keep;  // (never: the results only have to be observable)
}

struct ProbeTimer {
  hipEvent_t e0 = nullptr, e1 = nullptr, e2 = nullptr;
  ~ProbeTimer() {
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (e2) (void)hipEventDestroy(e2);
  }
};

// launches `launch()` back to back for about `seconds` (wall clock, checked every few launches), and returns the
// average duration of a launch over the second half of them (the first half settles the clocks)
template <class F>
int probe_run(F&& launch, double seconds, hipStream_t st, double* ms_per_launch, int64_t* launches) {
  ProbeTimer t;
  KGE_HIP_CHECK(hipEventCreate(&t.e0));
  KGE_HIP_CHECK(hipEventCreate(&t.e1));
  KGE_HIP_CHECK(hipEventCreate(&t.e2));
  for (int i = 0; i < 3; ++i) launch();
  KGE_HIP_CHECK(hipStreamSynchronize(st));
  // size the run from a first timed group
  KGE_HIP_CHECK(hipEventRecord(t.e0, st));
  for (int i = 0; i < 4; ++i) launch();
  KGE_HIP_CHECK(hipEventRecord(t.e1, st));
  KGE_HIP_CHECK(hipEventSynchronize(t.e1));
  float ms4 = 0.f;
  KGE_HIP_CHECK(hipEventElapsedTime(&ms4, t.e0, t.e1));
  const double per = ms4 > 0.f ? ms4 / 4.0 : 1.0;
  int64_t n = (int64_t)(seconds * 1e3 / per);
  if (n < 8) n = 8;
  if (n > 200000) n = 200000;
  n &= ~(int64_t)1;
  KGE_HIP_CHECK(hipEventRecord(t.e0, st));
  for (int64_t i = 0; i < n / 2; ++i) launch();
  KGE_HIP_CHECK(hipEventRecord(t.e1, st));
  for (int64_t i = 0; i < n / 2; ++i) launch();
  KGE_HIP_CHECK(hipEventRecord(t.e2, st));
  KGE_HIP_CHECK(hipEventSynchronize(t.e2));
  KGE_LAUNCH_CHECK("probe kernel");
  float ms = 0.f;
  KGE_HIP_CHECK(hipEventElapsedTime(&ms, t.e1, t.e2));
  *ms_per_launch = (double)ms / (double)(n / 2);
  *launches = n;
  return KGE_OK;
}

}  // namespace
}  // namespace kge

using namespace kge;

extern "C" int kge_probe_mfma(int count, int reads, double seconds, double* tflops, double* ms_per_launch, void* stream) {
  clear_error();
  KGE_REQUIRE(seconds > 0.0 && seconds <= 30.0 && tflops, KGE_ERR_INVALID, "kge_probe_mfma: seconds=%g", seconds);
  hipStream_t st = (hipStream_t)stream;
  int32_t* sink = nullptr;
  KGE_HIP_CHECK(hipMalloc(&sink, 256));
  const int iters = 400;                                  // stages per wave and launch
  const dim3 grid(256), block(512);                       // one workgroup per CU
  auto launch = [&]() {
    if (count && reads) hipLaunchKernelGGL((probe_tile_kernel<true, true>), grid, block, 0, st, iters, 1u, sink);
    else if (count) hipLaunchKernelGGL((probe_tile_kernel<true, false>), grid, block, 0, st, iters, 1u, sink);
    else if (reads) hipLaunchKernelGGL((probe_tile_kernel<false, true>), grid, block, 0, st, iters, 1u, sink);
    else hipLaunchKernelGGL((probe_tile_kernel<false, false>), grid, block, 0, st, iters, 1u, sink);
  };
  double ms = 0.0;
  int64_t n = 0;
  const int rc = probe_run(launch, seconds, st, &ms, &n);
  (void)hipFree(sink);
  if (rc) return rc;
  const double flop = 256.0 * 8.0 * (double)iters * 64.0 * 32768.0;  // waves x stages x MFMAs per stage x 2 * 32 * 32 * 16
  *tflops = flop / (ms * 1e-3) / 1e12;
  if (ms_per_launch) *ms_per_launch = ms;
  return KGE_OK;
}

extern "C" int kge_probe_walk(const float* Q, const void* E, int64_t B, int64_t N, double seconds, double* tflops,
                              double* ms_per_launch, void* stream) {
  clear_error();
  KGE_REQUIRE(Q && E && B >= 1 && N >= 1 && tflops && seconds > 0.0 && seconds <= 30.0, KGE_ERR_INVALID,
              "kge_probe_walk: bad arguments");
  KGE_REQUIRE((((uintptr_t)Q | (uintptr_t)E) & 15) == 0, KGE_ERR_INVALID, "kge_probe_walk: Q and E must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  // thresholds (zeros), targets (zeros) and the three counters: the walk never counts, and writes nothing but what
  // the exact pass of the table's last stage adds to the counters
  char* buf = nullptr;
  const size_t bytes = (size_t)B * (4 + 8 + 12);
  KGE_HIP_CHECK(hipMalloc(&buf, bytes));
  hipError_t e = hipMemsetAsync(buf, 0, bytes, st);
  if (e != hipSuccess) {
    (void)hipFree(buf);
    return set_error(KGE_ERR_HIP, "kge_probe_walk: %s", hipGetErrorString(e));
  }
  RankArgs ea;
  ea.target = (const int64_t*)buf;
  ea.thr = (const float*)(buf + 8 * B);
  ea.n_gt = (int32_t*)(buf + 12 * B);
  ea.n_eq = ea.n_gt + B;
  ea.n_eql = ea.n_eq + B;
  ContractArgs a;
  memset(&a, 0, sizeof(a));
  a.Q = Q;
  a.E = E;
  a.B = B;
  a.N = N;
  a.e_begin = 0;
  a.e_end = N;
  a.d = 128;
  host::rank128_plan(B, N, &a.n_qgroups, &a.n_lanes, &a.chunk_rows, &a.n_chunks);
  const dim3 grid((unsigned)(8 * a.n_qgroups * a.n_lanes)), block(64 * host::R128_WG_WAVES);
  auto launch = [&]() { hipLaunchKernelGGL((rank128_kernel<host::R128_WG_WAVES, false>), grid, block, 0, st, a, ea); };
  double ms = 0.0;
  int64_t n = 0;
  const int rc = probe_run(launch, seconds, st, &ms, &n);
  (void)hipFree(buf);
  if (rc) return rc;
  *tflops = 2.0 * 128.0 * (double)B * (double)N / (ms * 1e-3) / 1e12;
  if (ms_per_launch) *ms_per_launch = ms;
  return KGE_OK;
}

extern "C" int kge_probe_i8_scan(const float* Q, const void* prepared, int64_t B, int64_t N, double seconds, double* pops,
                                 double* ms_per_launch, void* stream) {
  clear_error();
  KGE_REQUIRE(Q && prepared && B >= 1 && N >= 1 && N <= 0x7fffffffLL && pops && seconds > 0.0 && seconds <= 30.0,
              KGE_ERR_INVALID, "kge_probe_i8_scan: bad arguments");
  KGE_REQUIRE((((uintptr_t)Q | (uintptr_t)prepared) & 255) == 0, KGE_ERR_INVALID,
              "kge_probe_i8_scan: Q and the prepared table must be 256-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const host::TopkPreparedOffsets t = host::topk_prepared_offsets(N);
  // the queries as the scan reads them (int8 rows, four constants each), thresholds of +inf, candidate counters and
  // a token candidate buffer (nothing is ever written to it)
  auto up = [](size_t x) { return (x + 255) / 256 * 256; };
  const size_t o_qh = 0, o_qc = up((size_t)B * 128), o_tau = o_qc + up((size_t)B * 16), o_cnt = o_tau + up((size_t)B * 4),
               o_cand = o_cnt + up((size_t)B * 4), bytes = o_cand + up((size_t)B * 16 * 4);
  char* buf = nullptr;
  KGE_HIP_CHECK(hipMalloc(&buf, bytes));
  struct Free {
    char* p;
    ~Free() { (void)hipFree(p); }
  } guard{buf};
  KGE_HIP_CHECK(hipMemsetAsync(buf, 0, bytes, st));
  KGE_HIP_CHECK(hipMemsetAsync(buf + o_tau, 0x7f, (size_t)B * 4, st));  // 0x7f7f7f7f = 3.39e38: no bound reaches it ...
  {
    std::vector<float> inf((size_t)B, __builtin_inff());                    // ... and then +inf itself
    KGE_HIP_CHECK(hipMemcpyAsync(buf + o_tau, inf.data(), (size_t)B * 4, hipMemcpyHostToDevice, st));
    KGE_HIP_CHECK(hipStreamSynchronize(st));
  }
  hipLaunchKernelGGL(topk_i8_qprep_kernel, dim3((unsigned)((B + 3) / 4)), dim3(256), 0, st, Q, B, (int8_t*)(buf + o_qh),
                     (f32x4*)(buf + o_qc));
  KGE_LAUNCH_CHECK("topk_i8_qprep_kernel");
  ContractArgs a;
  memset(&a, 0, sizeof(a));
  a.Q = Q;
  a.B = B;
  a.N = N;
  a.e_begin = 0;
  a.e_end = N;
  a.d = 128;
  a.n_qgroups = (int)((B + TF_WG_QUERIES - 1) / TF_WG_QUERIES);
  a.n_lanes = 32 / a.n_qgroups;
  if (a.n_lanes < 1) a.n_lanes = 1;
  int64_t chunk = N / (8 * (int64_t)a.n_lanes * 4);
  chunk = (chunk + TF_STAGE_ROWS - 1) / TF_STAGE_ROWS * TF_STAGE_ROWS;
  if (chunk < TF_STAGE_ROWS) chunk = TF_STAGE_ROWS;
  if (chunk > 1024) chunk = 1024;
  a.chunk_rows = (int)chunk;
  a.n_chunks = (N + chunk - 1) / chunk;
  const int64_t nwg = 8 * (int64_t)a.n_qgroups * a.n_lanes;
  KGE_REQUIRE(nwg <= 0x7fffffffLL, KGE_ERR_INVALID, "kge_probe_i8_scan: grid too large");
  I8FilterArgs ea{(const float*)(buf + o_tau), nullptr, (int32_t*)(buf + o_cnt), (uint32_t*)(buf + o_cand), 16,
                  (const int8_t*)((const unsigned char*)prepared + t.requant), (const unsigned char*)prepared + t.rowmeta,
                  (const int8_t*)(buf + o_qh), (const f32x4*)(buf + o_qc)};
  auto launch = [&]() { hipLaunchKernelGGL(topk_i8_filter_kernel, dim3((unsigned)nwg), dim3(64 * TF_W), 0, st, a, ea); };
  double ms = 0.0;
  int64_t n = 0;
  const int rc = probe_run(launch, seconds, st, &ms, &n);
  if (rc) return rc;
  *pops = 2.0 * 128.0 * (double)B * (double)N / (ms * 1e-3) / 1e12;  // tera-operations per second
  if (ms_per_launch) *ms_per_launch = ms;
  return KGE_OK;
}

