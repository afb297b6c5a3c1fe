// Filtered-rank main loop for bf16 tables with d == 128, FOUR query tiles per wave (gfx950).
//
// The walk, stage ring, LDS layout, tiles and reduction order are those of qstream_kernel<RankFastEpi, 2, ...>
// (same fp32 bit pattern for every score, same counters); what differs is the register allocation, which is
// done by hand: with four 32-query tiles per wave every fragment read from LDS feeds four MFMAs instead of
// two (half the LDS -> register bytes per MFMA), and with 8-wave workgroups a workgroup covers 1024 queries
// (half the global -> LDS bytes per MFMA as well).  At two waves per SIMD the budget is 256 registers:
//   128 query fragments (4 tiles x 8 K steps x 4), 32 entity fragments (refilled in place by the reads that
//   fetch the next entity tile, each issued right behind the last MFMA that consumes its predecessor),
//   2 x 16 accumulators (one filling while the other is counted), 8 fragment addresses, and the epilogue's
//   thresholds, counters and temporaries.
// The compiler's allocation of the same dataflow needs about 330 (it keeps a second set of entity fragments
// and spills), so one entity tile (4 chains of 8 MFMAs, the deferred count of the previous 4 result tiles
// between them, 8 fragment reads) is ONE asm statement whose operands the compiler allocates and whose order
// is fixed here: MFMA, five VALU instructions of the previous tile's count, (fragment read), MFMA, ...
// The two accumulators are pinned to v[224:239] and v[240:255] because the count addresses their elements.
//
// Wait states the asm statement provides itself (the compiler's hazard recogniser does not look inside):
//   * `s_waitcnt lgkmcnt(0)` before the first MFMA: the fragment reads of the previous statement have landed;
//   * `s_nop 5` between the first MFMA of a chain and the first VALU read of the accumulator the previous chain
//     finished (the distance the compiler keeps for the same pair in qstream_kernel);
//   * a chain's MFMAs depend on each other through SrcC == vDst of the same opcode, which issues back to back;
//   * a fragment register is overwritten by a read issued after the MFMA that takes it as SrcA has issued
//     (an MFMA reads SrcA / SrcB as it issues; LDS data returns tens of cycles later).
#pragma once
#include "kge_contract.hip.h"

namespace kge {

constexpr int R128_NQT = 4;  // query tiles per wave

// ---- pieces of the asm text ---------------------------------------------------------------------------
// count of one pair of accumulator elements (registers `a0`, `a1`) against threshold TH into bits / minimum M
#define R128_PAIR_FIRST(a0, a1, TH, M)                 \
  "v_sub_f32 %[d0], " TH ", " a0 "\n"                  \
  "v_sub_f32 %[d1], " TH ", " a1 "\n"                  \
  "v_lshrrev_b32 %[bits], 31, %[d0]\n"                 \
  "v_min3_f32 " M ", " M ", |%[d0]|, |%[d1]|\n"        \
  "v_alignbit_b32 %[bits], %[bits], %[d1], 31\n"
#define R128_PAIR(a0, a1, TH, M)                       \
  "v_sub_f32 %[d0], " TH ", " a0 "\n"                  \
  "v_sub_f32 %[d1], " TH ", " a1 "\n"                  \
  "v_alignbit_b32 %[bits], %[bits], %[d0], 31\n"       \
  "v_min3_f32 " M ", " M ", |%[d0]|, |%[d1]|\n"        \
  "v_alignbit_b32 %[bits], %[bits], %[d1], 31\n"
#define R128_MFMA(ACC, E, Q, C) "v_mfma_f32_32x32x16_bf16 " ACC ", " E ", " Q ", " C "\n"
#define R128_READ(E, F) "ds_read_b128 " E ", " F " offset:%[roff]\n"
#define R128_NOREAD(E, F) ""
// one chain: accumulator NEW <- sum over the 8 K steps of ef[s] x q[s]; between its MFMAs the count of OLD
// (registers o0 .. o15) against TH into GT / M; READ: R128_READ in the chain that consumes the fragments last
#define R128_BCNT(GT) "v_bcnt_u32_b32 " GT ", %[bits], " GT "\n"
// (the measurement aids of kge_probe.hip build the same statement without the count or without the reads)
#define R128_NOPAIR(a0, a1, TH, M) ""
#define R128_NOBCNT(GT) ""
#define R128_CHAIN(NEW, Q0, Q1, Q2, Q3, Q4, Q5, Q6, Q7, o0, o1, o2, o3, o4, o5, o6, o7, o8, o9, o10, o11, o12, o13, \
                   o14, o15, TH, GT, M, READ, PAIR0, PAIR, BCNT)                                                     \
  R128_MFMA(NEW, "%[e0]", Q0, "0")                                                                                  \
  "s_nop 5\n"                                                                                                      \
  PAIR0(o0, o1, TH, M) READ("%[e0]", "%[f0]")                                                                       \
  R128_MFMA(NEW, "%[e1]", Q1, NEW) PAIR(o2, o3, TH, M) READ("%[e1]", "%[f1]")                                       \
  R128_MFMA(NEW, "%[e2]", Q2, NEW) PAIR(o4, o5, TH, M) READ("%[e2]", "%[f2]")                                       \
  R128_MFMA(NEW, "%[e3]", Q3, NEW) PAIR(o6, o7, TH, M) READ("%[e3]", "%[f3]")                                       \
  R128_MFMA(NEW, "%[e4]", Q4, NEW) PAIR(o8, o9, TH, M) READ("%[e4]", "%[f4]")                                       \
  R128_MFMA(NEW, "%[e5]", Q5, NEW) PAIR(o10, o11, TH, M) READ("%[e5]", "%[f5]")                                     \
  R128_MFMA(NEW, "%[e6]", Q6, NEW) PAIR(o12, o13, TH, M) READ("%[e6]", "%[f6]")                                     \
  R128_MFMA(NEW, "%[e7]", Q7, NEW) PAIR(o14, o15, TH, M)                                                            \
  BCNT(GT) READ("%[e7]", "%[f7]")
#define R128_X "v224", "v225", "v226", "v227", "v228", "v229", "v230", "v231", "v232", "v233", "v234", "v235", "v236", \
               "v237", "v238", "v239"
#define R128_Y "v240", "v241", "v242", "v243", "v244", "v245", "v246", "v247", "v248", "v249", "v250", "v251", "v252", \
               "v253", "v254", "v255"
#define R128_Q(t) "%[q" #t "0]", "%[q" #t "1]", "%[q" #t "2]", "%[q" #t "3]", "%[q" #t "4]", "%[q" #t "5]", "%[q" #t "6]", "%[q" #t "7]"
// one entity tile: on entry X holds the last result tile of the previous entity tile (query tile 3), not yet
// counted; every query tile has a running minimum of its own
#define R128_CHAIN_(...) R128_CHAIN(__VA_ARGS__)  // (expands the register lists before the chain counts its arguments)
#define R128_TILE_TEXT(READ, PAIR0, PAIR, BCNT)                                                   \
  "s_waitcnt lgkmcnt(0)\n"                                                                        \
  R128_CHAIN_("%[Y]", R128_Q(0), R128_X, "%[t3]", "%[g3]", "%[m3]", R128_NOREAD, PAIR0, PAIR, BCNT) \
  R128_CHAIN_("%[X]", R128_Q(1), R128_Y, "%[t0]", "%[g0]", "%[m0]", R128_NOREAD, PAIR0, PAIR, BCNT) \
  R128_CHAIN_("%[Y]", R128_Q(2), R128_X, "%[t1]", "%[g1]", "%[m1]", R128_NOREAD, PAIR0, PAIR, BCNT) \
  R128_CHAIN_("%[X]", R128_Q(3), R128_Y, "%[t2]", "%[g2]", "%[m2]", READ, PAIR0, PAIR, BCNT)
#define R128_TILE R128_TILE_TEXT(R128_READ, R128_PAIR_FIRST, R128_PAIR, R128_BCNT)

typedef __attribute__((ext_vector_type(16))) float r128_acc;

// ROFF: where the fragments of the next entity tile are, relative to the addresses in fb[].
// COUNT / READS: false only in the measurement aids (the statement without its count, without its fragment reads).
template <int ROFF, bool COUNT = true, bool READS = true>
__device__ __forceinline__ void r128_tile(const bf16x8 (&qf)[R128_NQT][8], bf16x8 (&ef)[8], const int (&foff)[8],
                                          r128_acc& X, const float (&thr)[R128_NQT], int32_t (&gt)[R128_NQT],
                                          float (&mn)[R128_NQT]) {
  float d0, d1;
  uint32_t bits;
  r128_acc Y;
#define R128_OPERANDS \
  : [X] "+{v[224:239]}"(X), [Y] "=&{v[240:255]}"(Y), [e0] "+v"(ef[0]), [e1] "+v"(ef[1]), [e2] "+v"(ef[2]), \
    [e3] "+v"(ef[3]), [e4] "+v"(ef[4]), [e5] "+v"(ef[5]), [e6] "+v"(ef[6]), [e7] "+v"(ef[7]), [g0] "+v"(gt[0]), \
    [g1] "+v"(gt[1]), [g2] "+v"(gt[2]), [g3] "+v"(gt[3]), [m0] "+v"(mn[0]), [m1] "+v"(mn[1]), [m2] "+v"(mn[2]), \
    [m3] "+v"(mn[3]), [d0] "=&v"(d0), [d1] "=&v"(d1), [bits] "=&v"(bits) \
  : [q00] "v"(qf[0][0]), [q01] "v"(qf[0][1]), [q02] "v"(qf[0][2]), [q03] "v"(qf[0][3]), [q04] "v"(qf[0][4]), \
    [q05] "v"(qf[0][5]), [q06] "v"(qf[0][6]), [q07] "v"(qf[0][7]), [q10] "v"(qf[1][0]), [q11] "v"(qf[1][1]), \
    [q12] "v"(qf[1][2]), [q13] "v"(qf[1][3]), [q14] "v"(qf[1][4]), [q15] "v"(qf[1][5]), [q16] "v"(qf[1][6]), \
    [q17] "v"(qf[1][7]), [q20] "v"(qf[2][0]), [q21] "v"(qf[2][1]), [q22] "v"(qf[2][2]), [q23] "v"(qf[2][3]), \
    [q24] "v"(qf[2][4]), [q25] "v"(qf[2][5]), [q26] "v"(qf[2][6]), [q27] "v"(qf[2][7]), [q30] "v"(qf[3][0]), \
    [q31] "v"(qf[3][1]), [q32] "v"(qf[3][2]), [q33] "v"(qf[3][3]), [q34] "v"(qf[3][4]), [q35] "v"(qf[3][5]), \
    [q36] "v"(qf[3][6]), [q37] "v"(qf[3][7]), [f0] "v"(foff[0]), [f1] "v"(foff[1]), [f2] "v"(foff[2]), \
    [f3] "v"(foff[3]), [f4] "v"(foff[4]), [f5] "v"(foff[5]), [f6] "v"(foff[6]), [f7] "v"(foff[7]), \
    [t0] "v"(thr[0]), [t1] "v"(thr[1]), [t2] "v"(thr[2]), [t3] "v"(thr[3]), [roff] "n"(ROFF)
  if constexpr (COUNT && READS) asm volatile(R128_TILE R128_OPERANDS);
  else if constexpr (READS) asm volatile(R128_TILE_TEXT(R128_READ, R128_NOPAIR, R128_NOPAIR, R128_NOBCNT) R128_OPERANDS);
  else if constexpr (COUNT) asm volatile(R128_TILE_TEXT(R128_NOREAD, R128_PAIR_FIRST, R128_PAIR, R128_BCNT) R128_OPERANDS);
  else asm volatile(R128_TILE_TEXT(R128_NOREAD, R128_NOPAIR, R128_NOPAIR, R128_NOBCNT) R128_OPERANDS);
#undef R128_OPERANDS
}

// W waves per workgroup (8: one workgroup per CU, 1024 queries; 4: two per CU, 512 queries each), two waves per SIMD.
// COUNT: false only in the measurement aid that times the walk without its count (kge_probe.hip).
template <int W, bool COUNT = true>
__global__ void __launch_bounds__(64 * W, 2) rank128_kernel(ContractArgs a, RankArgs ea) {
  constexpr int NQT = R128_NQT, KSTEPS = 8;
  constexpr int ROW_BYTES = 256;
  constexpr int STAGE_BYTES = QS_STAGE_ROWS * ROW_BYTES;
  constexpr int TILE_BYTES = 32 * ROW_BYTES;
  __shared__ __attribute__((aligned(1024))) unsigned char lds_e[QS_NBUF * STAGE_BYTES];

  const int64_t wg = blockIdx.x;
  const int xcd = (int)(wg & 7);
  const int64_t slot = wg >> 3;
  const int qg = (int)(slot % a.n_qgroups);
  const int wlane = (int)(slot / a.n_qgroups);
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t q0 = (int64_t)qg * (W * 32 * NQT) + wave * (32 * NQT);

  // chunks of this workgroup: first, stride, count; stages that hold at least one valid row
  const int64_t c_first = xcd + 8 * (int64_t)wlane;
  const int64_t c_stride = 8 * (int64_t)a.n_lanes;
  if (c_first >= a.n_chunks) return;
  const int my_chunks = (int)((a.n_chunks - 1 - c_first) / c_stride) + 1;
  const int spc = a.chunk_rows / QS_STAGE_ROWS;
  const int64_t r_end = a.e_end;
  const int64_t row_first = a.e_begin + c_first * a.chunk_rows;
  const int64_t row_last_chunk = row_first + c_stride * (int64_t)(my_chunks - 1) * a.chunk_rows;
  int valid_last = (int)((r_end - row_last_chunk + QS_STAGE_ROWS - 1) / QS_STAGE_ROWS);
  valid_last = valid_last < spc ? valid_last : spc;
  const int n_st = (my_chunks - 1) * spc + valid_last;
  const int64_t chunk_skip = (c_stride - 1) * (int64_t)a.chunk_rows;

  // query fragments: rows past the end of the batch read the batch's last row (no branch) and are zeroed
  bf16x8 qf[NQT][KSTEPS];
#pragma unroll
  for (int t = 0; t < NQT; ++t) {
    const int64_t q = q0 + 32 * t + c;
    const bool live = q < a.B;
    const f32x4* src = (const f32x4*)(a.Q + (live ? q : a.B - 1) * 128 + 8 * hf);
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      f32x4 lo = src[4 * s], hi = src[4 * s + 1];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        lo[j] = live ? lo[j] : 0.f;
        hi[j] = live ? hi[j] : 0.f;
      }
      qf[t][s] = cvt_bf16x8(lo, hi);
    }
    // one tile's loads at a time (64 fp32 registers in flight, not 256): the fragments are pinned here
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) asm volatile("" : "+v"(qf[t][s]));
  }
  float thr[NQT];
  int32_t gt[NQT];
#pragma unroll
  for (int t = 0; t < NQT; ++t) {
    const int64_t q = q0 + 32 * t + c;
    thr[t] = (q < a.B) ? ea.thr[q] : __uint_as_float(0x7fc00000u);  // NaN never compares
    gt[t] = 0;
  }
  // running minimum of |threshold - score| per query tile over the stage being counted (0: an exact tie)
  constexpr float INF = __builtin_inff();
  float mn[NQT] = {INF, INF, INF, INF};

  // this lane's share of a stage (as in qstream_kernel): rows lrow + RPI * j, always the same swizzled piece
  constexpr int LPR = 16, RPW = 4, RPI = RPW * W, NLD = QS_STAGE_ROWS / RPI;
  const int lrow = wave * RPW + lane / LPR;
  const int lpiece = (lane % LPR) ^ (lrow & 15);
  const unsigned char* Eb = (const unsigned char*)a.E;
  uint32_t voff[NLD];
#pragma unroll
  for (int j = 0; j < NLD; ++j) voff[j] = (uint32_t)((lrow + RPI * j) * ROW_BYTES + lpiece * 16);
  auto stage_issue = [&](int64_t row0, int bufo) {  // bufo: byte offset of the stage buffer
    unsigned char* dst = lds_e + bufo + wave * 1024;
    if (__builtin_expect(row0 + QS_STAGE_ROWS <= r_end, 1)) {
      const unsigned char* src = Eb + row0 * ROW_BYTES;  // wave-uniform
#pragma unroll
      for (int j = 0; j < NLD; ++j)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + voff[j]),
                                         (__attribute__((address_space(3))) void*)(dst + j * (RPI * ROW_BYTES)), 16, 0, 0);
    } else {
#pragma unroll
      for (int j = 0; j < NLD; ++j) {
        int64_t g = row0 + lrow + RPI * j;
        g = (g < r_end) ? g : r_end - 1;  // rows past the end repeat the last row; the exact pass ignores them
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(Eb + g * ROW_BYTES + lpiece * 16),
                                         (__attribute__((address_space(3))) void*)(dst + j * (RPI * ROW_BYTES)), 16, 0, 0);
      }
    }
  };
  int64_t issue_row = row_first;
  int issue_so = 0;
  auto issue_advance = [&]() {
    issue_row += QS_STAGE_ROWS;
    if (++issue_so == spc) {
      issue_so = 0;
      issue_row += chunk_skip;
    }
  };

  // fragment addresses of this lane: fb[s] points into the buffer the next refill reads from
  const int fswz = c * ROW_BYTES;
  int fb[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) fb[s] = fswz + (((2 * s + hf) ^ (c & 15)) << 4);

  // nothing to count before the first tile: scores of -inf are never greater than, never equal to a threshold
  r128_acc X;
#pragma unroll
  for (int i = 0; i < 16; ++i) X[i] = __uint_as_float(0xff800000u);

  auto wg_barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    // (the builtin, not an asm statement: the compiler's own wait-count bookkeeping must see that nothing older than
    // this point is outstanding, or it waits for the global -> LDS loads of stage k + 2 at the top of every stage)
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };

  stage_issue(issue_row, 0);
  issue_advance();
  stage_issue(issue_row, STAGE_BYTES);
  issue_advance();
  wg_barrier();
  bf16x8 ef[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) ef[s] = *(const bf16x8*)(lds_e + fb[s]);

  // The exact pass over one stage for the query tiles in `tiles` (bit t: tile t): those tiles formed again from the
  // intact buffer; ties, and rows past the end of the table (the fast count has already counted every element that
  // is strictly greater, padding rows included).  Everything it needs beyond the query fragments is formed inside the
  // branch from an opaque lane number, so that nothing of it is kept in a register across the main loop; the entity
  // fragments are dead across it (it ends by reading them again), which leaves it their registers.
  auto fix_stage = [&](uint32_t tiles, int bufo, int next_read_o, int64_t rows0) __attribute__((always_inline)) {
    // The tile statement before this one has left fragment reads in flight into ef[]'s registers, which are free
    // for this path's own values from here on: they must have landed before anything here is written.
    int ln;
    asm volatile("s_waitcnt lgkmcnt(0)\n\tv_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln)::"memory");
    __builtin_amdgcn_sched_barrier(0);
    const int lc = ln & 31, lhf = ln >> 5;
    const int sw = (lc & 15) ^ lhf;  // piece 2 s + hf of row c sits at slot (2 s) ^ sw
    const int row_end = (int)((r_end - rows0 > 64) ? 64 : r_end - rows0);  // rows of this stage that exist
#pragma unroll 1
    for (int it = 0; it < 2 * NQT; ++it) {
      const int t = it >> 1, et = it & 1;
      if (!((tiles >> t) & 1u)) continue;
      const unsigned char* base = lds_e + bufo + et * TILE_BYTES + lc * ROW_BYTES;
      f32x16 acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
      auto chain = [&](const bf16x8 (&q)[KSTEPS]) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) acc = mfma_bf16(*(const bf16x8*)(base + (((2 * s) ^ sw) << 4)), q[s], acc);
      };
      if (t == 0) chain(qf[0]);
      else if (t == 1) chain(qf[1]);
      else if (t == 2) chain(qf[2]);
      else chain(qf[3]);
      const float th = t == 0 ? thr[0] : t == 1 ? thr[1] : t == 2 ? thr[2] : thr[3];
      const int64_t q = q0 + 32 * t + lc;
      const int64_t tgd = (q < a.B) ? ea.target[q] - rows0 : -1;
      const int tg_row = (int)(tgd < -1 ? -1 : tgd > 64 ? 64 : tgd);  // the target's row in this stage, clamped
      int32_t dg = 0, eq = 0, eql = 0;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int r = et * 32 + ((i >> 2) << 3) + (lhf << 2) + (i & 3);
        const bool in = r < row_end, tie = acc[i] == th;
        eq += (in && tie) ? 1 : 0;
        eql += (in && tie && r < tg_row) ? 1 : 0;
        dg -= (!in && acc[i] > th) ? 1 : 0;
      }
      gt[0] += t == 0 ? dg : 0;
      gt[1] += t == 1 ? dg : 0;
      gt[2] += t == 2 ? dg : 0;
      gt[3] += t == 3 ? dg : 0;
      if (eq) atomicAdd(&ea.n_eq[q], eq);
      if (eql) atomicAdd(&ea.n_eql[q], eql);
    }
    // the entity fragments the next tile statement multiplies (the ones it was about to use, read again)
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s)
      ef[s] = *(const bf16x8*)(lds_e + next_read_o + lc * ROW_BYTES + (((2 * s) ^ sw) << 4));
  };
  // bit t: query tile t met an exact tie in the stage just counted (wave-uniform); resets that minimum
  auto tie_bit = [&](float& m, int t) -> uint32_t {
    const unsigned long long tie = __builtin_amdgcn_ballot_w64(m == 0.f);
    m = INF;
    return tie != 0 ? (1u << t) : 0u;
  };

  int64_t row0 = row_first, prev_row0 = row_first;
  int so = 0;
  int cur_o = 0, prev_o = 2 * STAGE_BYTES;  // byte offsets of the buffers of stage k and stage k - 1 (= of stage k + 2)
  uint32_t dirty = 0;                       // query tiles 0..2 of the previous stage that need the exact pass
  for (int k = 0; k < n_st; ++k) {
    // first entity tile; the fragments of the second are fetched under its last chain
    r128_tile<TILE_BYTES, COUNT>(qf, ef, fb, X, thr, gt, mn);
    // every tile of the previous stage has been counted by now (query tile 3 of its second entity tile by the
    // statement above), and its buffer is intact until this wave passes the barrier below: the place for that
    // stage's exact pass, if it needs one
    if (k > 0) {
      dirty |= tie_bit(mn[3], 3);
      if (prev_row0 + QS_STAGE_ROWS > r_end) dirty = 15u;
      if (dirty) fix_stage(dirty, prev_o, cur_o + TILE_BYTES, prev_row0);
    }
    // stage k + 1 has landed for every wave, and everyone is done with the buffer of stage k - 1
    wg_barrier();
    // stage k + 2 (past the last stage: the last stage's rows once more, into a buffer nobody reads)
    stage_issue(issue_row, prev_o);
    if (k + 3 < n_st) issue_advance();
    const int next_o = (cur_o == 2 * STAGE_BYTES) ? 0 : cur_o + STAGE_BYTES;
    const int step = next_o - cur_o;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) fb[s] += step;
    // second entity tile; the fragments of the next stage's first tile are fetched under its last chain
    r128_tile<0, COUNT>(qf, ef, fb, X, thr, gt, mn);
    dirty = tie_bit(mn[0], 0) | tie_bit(mn[1], 1) | tie_bit(mn[2], 2);
    prev_o = cur_o;
    cur_o = next_o;
    prev_row0 = row0;
    row0 += QS_STAGE_ROWS;
    if (++so == spc) {
      so = 0;
      row0 += chunk_skip;
    }
  }
  // after the last stage: the count of its last result tile (query tile 3), then its exact pass if needed
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\ns_nop 7\ns_nop 7" : "+{v[224:239]}"(X)::"memory");
  {
    const float th = thr[NQT - 1];
    uint32_t bits = 0;
    float m = mn[NQT - 1];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float dd = th - X[i];
      bits = __builtin_amdgcn_alignbit(bits, __float_as_uint(dd), 31);
      m = __builtin_fminf(m, __builtin_fabsf(dd));
    }
    mn[NQT - 1] = m;
    gt[NQT - 1] += __builtin_popcount(bits);
  }
  dirty |= tie_bit(mn[3], 3);
  if (prev_row0 + QS_STAGE_ROWS > r_end) dirty = 15u;
  if (dirty) fix_stage(dirty, prev_o, prev_o, prev_row0);
  {
    int ln;  // (formed here, so that neither it nor the addresses below are kept in registers across the main loop)
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
      const int64_t q = q0 + 32 * t + (ln & 31);
      const int32_t g = gt[t] + __shfl_xor(gt[t], 32, 64);  // both halves of the wave hold the same query
      if (ln < 32 && q < a.B && thr[t] == thr[t] && g) atomicAdd(&ea.n_gt[q], g);
    }
  }
}

}  // namespace kge
