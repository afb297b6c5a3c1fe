// Top-k over a per-row int8 table, d == 128: the scan as an integer filter.
//
// A round of kge_topk only has to find the entities whose score beats the query's threshold tau; nearly all of
// the B x N scores do not.  The scan therefore works on a bound that is cheap to form:
//   * once per call the table is written again with one scale per 32-row tile (topk_i8_requant_kernel):
//     s_e e_k = S (e'_k + rho_k), S the tile's largest |scale|, e'_k an int8, |rho_k| <= 0.501.  The sign of a
//     negative scale moves into e'; a row whose scale is tiny against its neighbours' becomes mostly zeros,
//     which costs the bound tightness but not validity;
//   * the query row is rounded to bf16 (qb, the operand of the exact score) and then quantised to int8,
//     qb_k = s_q qh_k + delta_k;  H' = sum_k e'_k qh_k is an exact int32 from the int8 MFMA (32x32x32, twice the
//     bf16 rate, and the rows go global -> LDS untouched);
//   * in exact arithmetic s_e sum_k e_k qb_k = S ( s_q H' + sum_k e'_k delta_k + sum_k rho_k qb_k ), and each of
//     the two residual sums is at most the product of the two vectors' Euclidean norms.  The exact score is
//     fl(s_e A) with A = fl(sum_k e_k qb_k) (fp32 accumulation: |A - sum| is at most 128 * 2^-23 * sum_k |e_k qb_k|
//     <= 1.9e-3 s_q L1(e), since |qb_k| <= 127 s_q; S L1(e) <= S (L1(e') + 64) <= S (11.32 |e'|_2 + 64)).  Hence
//       s_e A <= S ( s_q H' + m_q |e'|_2 + |rho|_2 |qb|_2 + 0.256 s_q ),      m_q = |delta|_2 + 0.0453 s_q
//     (0.0453 = 4e-3 * 11.32 and 0.256 = 4e-3 * 64: the rounding of the chain, and of this bound's own few
//     operations, with a factor two to spare).  |e'|_2 and |rho|_2 are the largest of the tile's rows, rounded up.
//     Per element nothing but the MFMA; per tile and lane the maximum of its 16 accumulators and six float
//     operations.  A tile none of whose lanes can beat its query's tau is passed over; in the others the
//     accumulators are compared with the threshold turned into an integer.
// An element that passes is only a candidate: its entity id goes to the query's candidate buffer, and its score
// is recomputed with the exact chain (the one kge_scores uses) before the selection compares it with tau.  So the
// filter decides nothing about the result, it only has to let every true candidate through.
//
// The tiles that do not pass as a whole are few, and in each of them one lane or two hold all the elements of
// interest.  Such a lane parks its 16 accumulators, its integer threshold and its position in a small queue of its
// wave; when 64 are waiting the wave works them off together, one lane per parked set.  (A tile most of whose lanes
// are of interest, as in the first rounds of a call when thresholds are loose, is worked off on the spot.)
//
// Pipeline: the persistent XCD-aware walk and the three-buffer global -> LDS ring of qstream_kernel, 64-row
// stages of 8 KB, one barrier per stage; a tile's test runs under the next tile's MFMA chain.  Candidate ids are
// parked in per-query LDS buckets and leave for global memory as one run per query when the workgroup ends.
#pragma once
#include "kge_contract.hip.h"

namespace kge {
// (the kernels below have internal linkage: the library's main source and its measurement aids both include this file)

typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;

struct I8FilterArgs {
  const float* tau;       // per query: the threshold candidates must beat (-inf: everything is a candidate)
  const int32_t* active;  // NULL = all queries; else only queries with active[b] != 0 collect
  int32_t* cnt;           // per query: candidates appended this round
  uint32_t* cand;         // [B, cap] candidate entity ids
  int32_t cap;
  const int8_t* Eq;              // the table with tile-common scales (topk_i8_requant_kernel)
  const unsigned char* rowmeta;  // one record per 64 table rows: per 32-row tile {S (negative: forced), max |e'|_2, max |rho|_2, 1 / S}
  const int8_t* qh;              // [B, 128] the queries as int8 (topk_i8_qprep_kernel)
  const f32x4* qc;               // [B] per query {s_q, m_q, |qb|_2, finite ? 1 : 0}
};

constexpr int TF_NQT = 4;                              // 32-query tiles per wave
constexpr int TF_W = 8;                                // waves per workgroup
constexpr int TF_WG_QUERIES = TF_W * 32 * TF_NQT;      // 1024
constexpr int TF_STAGE_ROWS = 64;
constexpr int TF_STAGE_BYTES = TF_STAGE_ROWS * 128;    // 8 KB of int8 rows
constexpr int TF_NBUF = 3;
constexpr int TF_BUCKET = 16;                          // candidate ids a query can park in LDS
constexpr int TF_VALU_PER_MFMA = 4;
static_assert(host::TOPK_ROWMETA_ROWS == TF_STAGE_ROWS && host::TOPK_ROWMETA_BYTES == 32, "record per stage");

// (a candidate id goes into its query's global buffer at the query's running count; a full buffer keeps a uniform
// sample of what arrives, and the query is repaired by a later rescan with its final threshold: tf_place below)
// The table with one scale per 32-row tile, and per 64 rows one record for the scan.  One workgroup per 64 rows:
// thread t takes 16 bytes of row (t >> 3) of each of the two tiles, so loads and stores are whole rows in order.
// A row past the table's end counts for nothing; a scale that is not finite forces its tile (the scan then takes
// all its rows as candidates).
static __global__ void __launch_bounds__(256) topk_i8_requant_kernel(const int8_t* E, const float* scale, int64_t N, int8_t* Eq,
                                                              unsigned char* meta) {
  __shared__ float s_max[2][4], s_bad[2][4], s_e2[2][4], s_r2[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t rec = blockIdx.x;
  float scv[2];
  u32x4 w[2];
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int64_t row = rec * 64 + it * 32 + (tid >> 3);
    const bool in = row < N;
    const float sc = in ? scale[row] : 0.f;
    w[it] = in ? *(const u32x4*)(E + row * 128 + 16 * (tid & 7)) : u32x4{0u, 0u, 0u, 0u};
    const bool bad = !(__builtin_fabsf(sc) <= 3.4028234e38f);
    scv[it] = bad ? 0.f : sc;
    float sM = __builtin_fabsf(scv[it]), fM = bad ? 1.f : 0.f;
#pragma unroll
    for (int o = 8; o <= 32; o <<= 1) {
      sM = __builtin_fmaxf(sM, __shfl_xor(sM, o, 64));
      fM = __builtin_fmaxf(fM, __shfl_xor(fM, o, 64));
    }
    if (lane == 0) {
      s_max[it][wave] = sM;
      s_bad[it][wave] = fM;
    }
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int64_t row = rec * 64 + it * 32 + (tid >> 3);
    const float S = __builtin_fmaxf(__builtin_fmaxf(s_max[it][0], s_max[it][1]), __builtin_fmaxf(s_max[it][2], s_max[it][3]));
    const float ratio = (S > 0.f) ? scv[it] / S : 0.f;  // |ratio| <= 1: the products below stay within +-127
    u32x4 o;
    int e2 = 0;       // sum of e'^2 over this thread's sixteen components (exact)
    float r2 = 0.f;   // sum of rho^2 as computed (the true rho differs by at most 2e-5 per component)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t pk = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const float x = (float)(int)(int8_t)(w[it][i] >> (8 * b));
        const float y = x * ratio;
        const float yr = __builtin_rintf(y);
        const int v = (int)yr;
        pk |= ((uint32_t)v & 0xffu) << (8 * b);
        e2 += v * v;
        r2 = __builtin_fmaf(y - yr, y - yr, r2);
      }
      o[i] = pk;
    }
    if (row < N) *(u32x4*)(Eq + row * 128 + 16 * (tid & 7)) = o;
#pragma unroll
    for (int s = 1; s <= 4; s <<= 1) {  // the eight threads of a row
      e2 += __shfl_xor(e2, s, 64);
      r2 += __shfl_xor(r2, s, 64);
    }
    float e2M = (float)e2;  // at most 128 * 127^2: exact
    float r2M = r2;
#pragma unroll
    for (int s = 8; s <= 32; s <<= 1) {  // the eight rows of a wave
      e2M = __builtin_fmaxf(e2M, __shfl_xor(e2M, s, 64));
      r2M = __builtin_fmaxf(r2M, __shfl_xor(r2M, s, 64));
    }
    if (lane == 0) {
      s_e2[it][wave] = e2M;
      s_r2[it][wave] = r2M;
    }
  }
  __syncthreads();
  if (tid < 2) {
    const float S = __builtin_fmaxf(__builtin_fmaxf(s_max[tid][0], s_max[tid][1]), __builtin_fmaxf(s_max[tid][2], s_max[tid][3]));
    const float E2 = __builtin_fmaxf(__builtin_fmaxf(s_e2[tid][0], s_e2[tid][1]), __builtin_fmaxf(s_e2[tid][2], s_e2[tid][3]));
    const float R2 = __builtin_fmaxf(__builtin_fmaxf(s_r2[tid][0], s_r2[tid][1]), __builtin_fmaxf(s_r2[tid][2], s_r2[tid][3]));
    const float F = __builtin_fmaxf(__builtin_fmaxf(s_bad[tid][0], s_bad[tid][1]), __builtin_fmaxf(s_bad[tid][2], s_bad[tid][3]));
    // (a scale so small that 1 / S overflows: the tile is forced, like one with a scale that is not finite)
    const float iS = S > 0.f ? 1.f / S : 0.f;
    const bool forced = F != 0.f || !(iS <= 3.4028234e38f);
    // norms rounded up: the square roots and the sums' own rounding (1e-5 relative), and for rho the difference
    // between the computed and the true residuals (128 components of at most 2e-5: 2.3e-4 on the norm)
    const f32x4 tc = {forced ? -S : S, __builtin_sqrtf(E2) * 1.00001f, __builtin_sqrtf(R2) * 1.00001f + 1e-3f,
                      forced ? 0.f : iS};
    *(f32x4*)(meta + rec * host::TOPK_ROWMETA_BYTES + 16 * tid) = tc;
  }
}

// The queries as the scan reads them, once per call.  One wave per query, two components per lane: the row rounded
// to bf16 (qb, the operand of the exact score), its largest magnitude and Euclidean norm, then qb_k = s_q qh_k + delta_k
// with qh_k an int8.  Per query {s_q, m_q = |delta|_2 + 0.0453 s_q, |qb|_2, kind} (norms rounded up).  kind 0: a row
// with a component that is not finite has no finite bound; the scan collects nothing for it (its scores are NaN or
// infinite anyway).  kind 2: components so large (about 1e34) that the bound's own arithmetic could overflow; the
// scan takes every row as a candidate for it.  kind 1: everything else.
constexpr float TF_NORM_MAX = 1e35f;  // m_q |e'|_2 + |rho|_2 |qb|_2 + s_q |H'| stays finite below this
static __global__ void __launch_bounds__(256) topk_i8_qprep_kernel(const float* Q, int64_t B, int8_t* qh, f32x4* qc) {
  const int lane = threadIdx.x & 63;
  const int64_t q = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (q >= B) return;
  const float* row = Q + q * 128;
  const float r0 = (float)(__bf16)row[2 * lane], r1 = (float)(__bf16)row[2 * lane + 1];
  float amax = __builtin_fmaxf(__builtin_fabsf(r0), __builtin_fabsf(r1));
  int bad = (r0 != r0 || r1 != r1) ? 1 : 0;  // fmax drops a NaN
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, o, 64));
    bad |= __shfl_xor(bad, o, 64);
  }
  const bool finite = !bad && amax <= 3.4028234e38f;
  const float s_q = finite ? amax / 127.f : 0.f;
  const float inv = (finite && amax > 0.f) ? 127.f / amax : 0.f;
  // the squares are taken of the components times 2^-ex (below 1 in magnitude: neither overflow nor underflow of
  // what matters), the norms scaled back after
  int ex = 0;
  if (finite) (void)__builtin_frexpf(amax, &ex);
  float d2 = 0.f, n2 = 0.f;
  uint32_t pk = 0;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const float r = finite ? (j ? r1 : r0) : 0.f;
    float h = __builtin_rintf(r * inv);
    h = __builtin_fminf(__builtin_fmaxf(h, -127.f), 127.f);
    const float dl = __builtin_ldexpf(__builtin_fmaf(-s_q, h, r), -ex);
    const float rl = __builtin_ldexpf(r, -ex);
    d2 = __builtin_fmaf(dl, dl, d2);
    n2 = __builtin_fmaf(rl, rl, n2);
    pk |= ((uint32_t)(int)h & 0xffu) << (8 * j);
  }
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    d2 += __shfl_xor(d2, o, 64);
    n2 += __shfl_xor(n2, o, 64);
  }
  ((uint16_t*)(qh + q * 128))[lane] = (uint16_t)pk;
  if (lane == 0) {
    // 1.0001: the roundings of the two sums of 128 squares and of the square roots
    const float dn = __builtin_ldexpf(__builtin_sqrtf(d2) * 1.0001f, ex);
    const float qn = __builtin_ldexpf(__builtin_sqrtf(n2) * 1.0001f, ex);
    const float mq = dn + 0.0453f * s_q;
    f32x4 c = {0.f, 0.f, 0.f, 0.f};
    if (finite) {
      if (mq <= TF_NORM_MAX && qn <= TF_NORM_MAX)
        c = f32x4{s_q, mq, qn, 1.f};
      else
        c[3] = 2.f;
    }
    qc[q] = c;
  }
}

constexpr int TF_QUEUE = 64;         // parked accumulator sets per wave
constexpr int TF_QUEUE_STRIDE = 20;  // dwords per set (19 used): five 16-byte pieces, written and read as such
constexpr int TF_DENSE_LANES = 16;   // a tile with more lanes of interest than this is worked off on the spot

// What the out-of-line slow paths need, as few scalars as will do (every argument travels in a register: a struct
// passed by value would go through the call frame in scratch memory, once per call and lane).
struct TfSink {
  uint32_t* bucket;  // LDS [TF_WG_QUERIES][TF_BUCKET] candidate ids parked per query
  int* bcnt;         // LDS [TF_WG_QUERIES]
  int32_t* cnt;      // global: per query, candidates appended this round
  uint32_t* cand;    // global [B, cap]
  int32_t cap;
  int32_t q_wg;      // first query of the workgroup
  uint32_t limit;    // entities >= limit are padding (ids stay below 2^31, a stage's padding rows below 2^31 + 64)
};

__device__ __forceinline__ void tf_place(const TfSink& k, int64_t q, int32_t slot, uint32_t e) {
  if (slot >= k.cap) {
    uint32_t h = (e * 2654435761u) ^ ((uint32_t)slot * 0x9e3779b9u);
    h ^= h >> 15; h *= 0x2c1b3c6du; h ^= h >> 12;
    const uint32_t r = h % (uint32_t)(slot + 1);
    slot = (r < (uint32_t)k.cap) ? (int32_t)r : -1;
  }
  if (slot >= 0) k.cand[q * k.cap + slot] = e;
}

// The elements among h[0..16) above thr, as candidates of local query `qlocal`: entity e_base + row_of(i, hf).
__device__ __forceinline__ void tf_collect(const int (&h)[16], int thr, bool on, int qlocal, int hf, uint32_t e_base,
                                           const TfSink& k) {
  uint32_t bits = 0;  // bit 15 - i: element i may beat the threshold (|thr| <= 2^30, |h| < 2^21: no wrap)
#pragma unroll
  for (int i = 0; i < 16; ++i) bits = __builtin_amdgcn_alignbit(bits, (uint32_t)(thr - h[i]), 31);
  if (!on) bits = 0;
  while (__builtin_amdgcn_ballot_w64(bits != 0) != 0) {
    if (bits != 0) {
      const int b = 31 - __builtin_clz(bits);
      bits &= ~(1u << b);
      const int i = 15 - b;
      const uint32_t e = e_base + (uint32_t)(((i >> 2) << 3) + (hf << 2) + (i & 3));
      if (e < k.limit) {
        const int idx = atomicAdd(&k.bcnt[qlocal], 1);
        if (idx < TF_BUCKET)
          k.bucket[qlocal * TF_BUCKET + idx] = e;
        else  // bucket full: straight to global memory
          tf_place(k, (int64_t)k.q_wg + qlocal, atomicAdd(&k.cnt[k.q_wg + qlocal], 1), e);
      }
    }
  }
}

// A tile most of whose lanes are of interest: every lane tests its own 16 elements.  Out of line (one copy).
// where = qlocal | hf << 16 | on << 17.
__device__ __attribute__((noinline)) void tf_dense(i32x16 h, int thr, uint32_t where, uint32_t e_base, uint32_t* bucket,
                                                   int* bcnt, int32_t* cnt, uint32_t* cand, int32_t cap, int32_t q_wg,
                                                   uint32_t limit) {
  int hh[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) hh[i] = h[i];
  const TfSink k{bucket, bcnt, cnt, cand, cap, q_wg, limit};
  tf_collect(hh, thr, ((where >> 17) & 1u) != 0u, (int)(where & 0xffffu), (int)((where >> 16) & 1u), e_base, k);
}

// The parked sets of a wave, one lane per set.  Out of line (one copy).
__device__ __attribute__((noinline)) void tf_drain(const uint32_t* queue, int n, uint32_t* bucket, int* bcnt, int32_t* cnt,
                                                   uint32_t* cand, int32_t cap, int32_t q_wg, uint32_t limit) {
  const int lane = threadIdx.x & 63;
  const bool on = lane < n;
  const u32x4* ent = (const u32x4*)(queue + (on ? lane : 0) * TF_QUEUE_STRIDE);
  int hh[16];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const u32x4 v = ent[p];
#pragma unroll
    for (int j = 0; j < 4; ++j) hh[4 * p + j] = (int)v[j];
  }
  const u32x4 tail = ent[4];
  const int thr = (int)tail[0];
  const uint32_t where = tail[1];
  const uint32_t e_base = tail[2];
  const TfSink k{bucket, bcnt, cnt, cand, cap, q_wg, limit};
  tf_collect(hh, thr, on, (int)(where & 0xffffu), (int)(where >> 16), e_base, k);
}

static __global__ void __launch_bounds__(64 * TF_W, 2) topk_i8_filter_kernel(ContractArgs a, I8FilterArgs ea) {
  constexpr int NQT = TF_NQT, W = TF_W, WQ = TF_WG_QUERIES;
  __shared__ __attribute__((aligned(1024))) unsigned char lds_e[TF_NBUF * TF_STAGE_BYTES];
  __shared__ __attribute__((aligned(16))) unsigned char meta_lds[TF_NBUF][host::TOPK_ROWMETA_BYTES];
  __shared__ uint32_t bucket[WQ * TF_BUCKET];
  __shared__ int bcnt[WQ];
  __shared__ __attribute__((aligned(16))) uint32_t queue[W][TF_QUEUE * TF_QUEUE_STRIDE];

  const int64_t wg = blockIdx.x;
  const int xcd = (int)(wg & 7);
  const int64_t slot = wg >> 3;
  const int qg = (int)(slot % a.n_qgroups);
  const int wlane = (int)(slot / a.n_qgroups);
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int d = 128;
  const int64_t q_wg = (int64_t)qg * WQ;
  const int ql0 = wave * (32 * NQT);
  const float INF = __uint_as_float(0x7f800000u);

  const int64_t c_first = xcd + 8 * (int64_t)wlane;
  const int64_t c_stride = 8 * (int64_t)a.n_lanes;
  if (c_first >= a.n_chunks) return;
  const int my_chunks = (int)((a.n_chunks - 1 - c_first) / c_stride) + 1;
  const int spc = a.chunk_rows / TF_STAGE_ROWS;
  const int64_t r_end = a.e_end;
  const int64_t row_first = a.e_begin + c_first * a.chunk_rows;
  const int64_t row_last_chunk = row_first + c_stride * (int64_t)(my_chunks - 1) * a.chunk_rows;
  int valid_last = (int)((r_end - row_last_chunk + TF_STAGE_ROWS - 1) / TF_STAGE_ROWS);
  valid_last = valid_last < spc ? valid_last : spc;
  const int n_st = (my_chunks - 1) * spc + valid_last;
  const int64_t chunk_skip = (c_stride - 1) * (int64_t)a.chunk_rows;

  for (int i = tid; i < WQ; i += 64 * W) bcnt[i] = 0;

  // ---- the queries of this lane: int8 fragments and the constants of the bound ------------------
  i32x4 qf[NQT][4];
  float sq[NQT], isq[NQT], cq[NQT], mq[NQT], nq[NQT], tau_lo[NQT];
#pragma unroll
  for (int t = 0; t < NQT; ++t) {
    const int64_t q = q_wg + ql0 + 32 * t + c;
    // the query's int8 fragments (k = 32 s + 16 hf + 0..15: sixteen consecutive bytes of its row) and constants
    f32x4 qcv = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      i32x4 w = {0, 0, 0, 0};
      if (q < a.B) w = *(const i32x4*)(ea.qh + q * d + 32 * s + 16 * hf);
      qf[t][s] = w;
    }
    if (q < a.B) qcv = ea.qc[q];
    const float s_q = qcv[0];
    const bool finite = qcv[3] != 0.f;
    const bool everything = qcv[3] == 2.f;  // no usable bound: s_q, m_q and the norm are 0 and the threshold -inf
    sq[t] = s_q;
    isq[t] = s_q > 0.f ? 1.f / s_q : 0.f;
    mq[t] = qcv[1];
    nq[t] = qcv[2];
    cq[t] = 0.256f * s_q;
    // a query with a non-finite component has no finite bound: it collects nothing (its scores are NaN or
    // infinite anyway)
    const bool on = q < a.B && finite && (ea.active == nullptr || ea.active[q] != 0);
    float th = INF;
    if (on) {
      th = ea.tau[q];
      if (th > -INF && th < INF) th = th - 1e-6f * __builtin_fabsf(th);  // the comparison's own rounding
      if (everything && th < INF) th = -INF;  // every bound (0 or more) passes, and so does every accumulator
    }
    tau_lo[t] = th;
  }

  // ---- staging: thread `tid` owns 16-byte slot `tid` of every stage -------------------------------
  // slot = row * 8 + (piece ^ ((row >> 1) & 7)): the 16 rows a fragment read touches at a time fall on distinct
  // bank groups.  Rows past the table's end repeat its last row (their entities are >= limit and are ignored).
  const int lrow = tid >> 3;
  const int lpiece = (tid & 7) ^ ((lrow >> 1) & 7);
  const unsigned char* Eb = (const unsigned char*)ea.Eq;
  auto stage_issue = [&](int64_t row0, int buf) {
    int64_t g = row0 + lrow;
    g = (g < r_end) ? g : r_end - 1;
    unsigned char* dst = lds_e + buf * TF_STAGE_BYTES + wave * 1024;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(Eb + g * 128 + lpiece * 16),
                                     (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    if (wave == 0 && lane < host::TOPK_ROWMETA_BYTES / 4)  // row0 is a multiple of 64: the stage's record
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(ea.rowmeta + (row0 >> 6) * host::TOPK_ROWMETA_BYTES + lane * 4),
          (__attribute__((address_space(3))) void*)&meta_lds[buf][0], 4, 0, 0);
  };
  int64_t issue_row = row_first;
  int issue_so = 0;
  auto issue_advance = [&]() {
    issue_row += TF_STAGE_ROWS;
    if (++issue_so == spc) {
      issue_so = 0;
      issue_row += chunk_skip;
    }
  };
  int foff[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) foff[s] = c * 128 + (((2 * s + hf) ^ ((c >> 1) & 7)) << 4);

  // ---- the test of one finished tile ------------------------------------------------------------
  // constants of the entity tile the finished accumulators belong to
  float m_S = 0.f, m_E2 = 0.f, m_R2 = 0.f, m_iS = 0.f;
  bool m_force = false;  // the same for the whole wave
  int64_t e_prev = r_end;
  auto tile_meta = [&](int buf, int et) {
    const f32x4 tc = *(const f32x4*)&meta_lds[buf][16 * et];
    m_S = __builtin_fabsf(tc[0]);
    m_E2 = tc[1];
    m_R2 = tc[2];
    m_force = (int)__builtin_amdgcn_readfirstlane(__float_as_uint(tc[0])) < 0;  // the sign of S: a forced tile
    m_iS = tc[3];
  };
  const TfSink sink{bucket, bcnt, ea.cnt, ea.cand, ea.cap, (int32_t)q_wg, (uint32_t)r_end};
  uint32_t* const wqueue = &queue[wave][0];
  int qn = 0;  // sets parked in this wave's queue (the same in every lane)
  auto tile_test = [&](int t, const i32x16& h) {
    int hm = h[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) hm = hm > h[i] ? hm : h[i];
    const float slack = __builtin_fmaf(mq[t], m_E2, __builtin_fmaf(m_R2, nq[t], cq[t]));
    const float Bd = m_S * __builtin_fmaf(sq[t], (float)hm, slack);
    const unsigned long long any = __builtin_amdgcn_ballot_w64(Bd > tau_lo[t]);
    if (__builtin_expect(any != 0 || m_force, 0)) {
      // The accumulators against the threshold as an integer: S (s_q H + slack) > tau  <=>  H > (tau / S - slack) / s_q,
      // lowered by its own rounding and kept inside +-2^30.
      // Where the bound does not depend on H (a tile of zero scales: 1 / S is stored as 0; a zero query: 1 / s_q is
      // held as 0) every H of such a tile or query is 0 and the formula gives x <= -1 or NaN: everything passes, as
      // it must when the bound has passed.  A NaN (0 times an infinite tau) falls to the lower clamp.
      float x = (tau_lo[t] * m_iS - slack) * isq[t];
      x = x - 1e-5f * __builtin_fabsf(x) - 1.f;
      bool mine = Bd > tau_lo[t];
      if (m_force) {  // the same for the whole wave
        x = (tau_lo[t] < INF) ? -INF : INF;
        mine = tau_lo[t] < INF;
      }
      const int thr = (int)__builtin_fminf(__builtin_fmaxf(x, -1073741824.f), 1073741824.f);
      const unsigned long long who = __builtin_amdgcn_ballot_w64(mine);
      const int n_new = __builtin_popcountll(who);
      const int qlocal = ql0 + 32 * t + c;
      if (n_new > TF_DENSE_LANES) {
        tf_dense(h, thr, (uint32_t)qlocal | ((uint32_t)hf << 16) | ((uint32_t)mine << 17), (uint32_t)e_prev, sink.bucket,
                 sink.bcnt, sink.cnt, sink.cand, sink.cap, sink.q_wg, sink.limit);
      } else if (n_new > 0) {
        if (qn + n_new > TF_QUEUE) {
          tf_drain(wqueue, qn, sink.bucket, sink.bcnt, sink.cnt, sink.cand, sink.cap, sink.q_wg, sink.limit);
          qn = 0;
        }
        if (mine) {
          const int at = qn + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(who >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)who, 0u));
          i32x4* ent = (i32x4*)(wqueue + at * TF_QUEUE_STRIDE);
          ent[0] = __builtin_shufflevector(h, h, 0, 1, 2, 3);
          ent[1] = __builtin_shufflevector(h, h, 4, 5, 6, 7);
          ent[2] = __builtin_shufflevector(h, h, 8, 9, 10, 11);
          ent[3] = __builtin_shufflevector(h, h, 12, 13, 14, 15);
          ent[4] = i32x4{thr, (int)((uint32_t)qlocal | ((uint32_t)hf << 16)), (int)(uint32_t)e_prev, 0};
        }
        qn += n_new;
      }
    }
  };

  // A barrier that orders nothing but the waves: the loads it guards are waited for explicitly.
  auto wg_barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };

  stage_issue(issue_row, 0);
  issue_advance();
  stage_issue(issue_row, 1);
  issue_advance();
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the cleared bucket counts
  wg_barrier();
  i32x4 ef[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) ef[s] = *(const i32x4*)(lds_e + foff[s]);

  // the first test has no tile to work on: e_prev past the limit keeps whatever it finds out of the buckets
  i32x16 acc_prev;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc_prev[i] = 0;
  int64_t row0 = row_first;
  int so = 0;

  auto run_stage = [&](auto bufc, int k) {
    constexpr int BUF = decltype(bufc)::value;
    constexpr int NEXT = (BUF + 1) % TF_NBUF, NEXT2 = (BUF + 2) % TF_NBUF;
#pragma unroll
    for (int et = 0; et < 2; ++et) {
      if (et == 1) {
        // stage k + 1 has landed for every wave, and everyone is done with the buffer of stage k - 1, which takes
        // the loads of stage k + 2
        wg_barrier();
        stage_issue(issue_row, NEXT2);
        if (k + 3 < n_st) issue_advance();
      }
      const int roff = (et == 0) ? BUF * TF_STAGE_BYTES + 4096 : NEXT * TF_STAGE_BYTES;
#pragma unroll
      for (int t = 0; t < NQT; ++t) {
        const int t_prev = (t + NQT - 1) % NQT;
        const bool refill = (t == NQT - 1);
        i32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(ef[s], qf[t][s], acc, 0, 0, 0);
          if (refill) ef[s] = *(const i32x4*)(lds_e + roff + foff[s]);
        }
        tile_test(t_prev, acc_prev);
        if (t == 0) {  // from here on the finished tiles belong to this entity tile
          tile_meta(BUF, et);
          e_prev = row0 + et * 32;
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, TF_VALU_PER_MFMA, 0);
          if (refill) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        acc_prev = acc;
      }
    }
    row0 += TF_STAGE_ROWS;
    if (++so == spc) {
      so = 0;
      row0 += chunk_skip;
    }
  };
  for (int k = 0;;) {
    run_stage(std::integral_constant<int, 0>{}, k);
    if (++k >= n_st) break;
    run_stage(std::integral_constant<int, 1>{}, k);
    if (++k >= n_st) break;
    run_stage(std::integral_constant<int, 2>{}, k);
    if (++k >= n_st) break;
  }
  tile_test(NQT - 1, acc_prev);
  if (qn > 0) tf_drain(wqueue, qn, sink.bucket, sink.bcnt, sink.cnt, sink.cand, sink.cap, sink.q_wg, sink.limit);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may land in LDS after the workgroup has gone

  // ---- the parked candidates of every query leave as one run ---------------------------------------
  // (sixteen lanes per query, so that the ids of a run are written side by side: whole lines, not one per id)
  __syncthreads();
  static_assert(TF_BUCKET == 16 && WQ % (4 * W) == 0, "one group of sixteen lanes per bucket");
  for (int i = tid >> 4; i < WQ; i += 4 * W) {
    const int64_t q = q_wg + i;
    const int j = tid & 15;
    int n = bcnt[i];
    n = n < TF_BUCKET ? n : TF_BUCKET;
    int32_t base = 0;
    if (j == 0 && n > 0 && q < a.B) base = atomicAdd(&ea.cnt[q], n);
    base = __shfl(base, lane & ~15, 64);
    if (j < n && q < a.B) tf_place(sink, q, base + j, bucket[i * TF_BUCKET + j]);
  }
}

}  // namespace kge
