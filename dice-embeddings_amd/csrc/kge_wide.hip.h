// qwide_kernel: bf16 or per-row int8 table, 256 < d <= 512 (gfx950).  The persistent walk of qstream_kernel with the
// whole query row of ONE 32-query tile per wave in registers (32 fragments at d = 512: the 128 registers that hold
// four tiles at d = 128) and the entity rows streamed through LDS in stages of one 32-row tile (three buffers):
// a score is ONE chain of d / 16 MFMAs on one accumulator, k ascending, as everywhere else, so the bits are those of
// the other kernels.  The eight entity fragments a wave holds cover 128 columns (a segment); each is replaced, right
// after the MFMA that consumed it, by the fragment of the same rows 128 columns on, and under the last segment by
// the first segment of the next stage.  Eight waves (256 queries) share every stage, so a workgroup fetches an eighth
// of a kilobyte from L2 per MFMA (kchunk_kernel, which served these widths before: half a kilobyte, and the fp32
// queries again for every entity tile).  Table rows narrower than the LDS row class (PAD) leave the row's tail zero
// in LDS; a class is 24 or 32 K steps (d <= 384, d <= 512).
// bf16 rows go global -> LDS directly, two stages ahead.  int8 rows are widened to bf16 (exactly) on the way: each
// thread keeps its 32 bytes of the stage after next in registers for one stage, then converts and stores them; the
// fp32 row scales ride along in LDS and a finished tile's scores are multiplied by them, as in the other int8 kernels.
#pragma once
#include "kge_contract.hip.h"

namespace kge {

constexpr int QW_WG_WAVES = 8;
constexpr int QW_WG_QUERIES = QW_WG_WAVES * 32;
constexpr int QW_ROW_BYTES = 1040;     // an LDS row: 512 bf16 (64 pieces of 16 bytes) and 16 bytes that nobody reads:
                                       // the 16 lanes of a fragment read that go together, one row each at the same
                                       // column, then fall into 16 different groups of four banks
constexpr int QW_STAGE_ROWS = 32;
constexpr int QW_STAGE_BYTES = QW_STAGE_ROWS * QW_ROW_BYTES;
constexpr int QW_NBUF = 3;

template <int EDT, template <int> class EpiT, int KSTEPS, bool PAD>
__global__ void __launch_bounds__(64 * QW_WG_WAVES, 2) qwide_kernel(ContractArgs a, typename EpiT<1>::Args ea) {
  using Epi = EpiT<1>;
  static_assert(EDT == KGE_BF16 || EDT == KGE_I8, "bf16 or int8 rows");
  constexpr bool I8 = (EDT == KGE_I8);
  static_assert(KSTEPS == 24 || KSTEPS == 32, "three or four segments of eight K steps");
  static_assert(!Epi::DEFER, "the epilogue runs after its tile's chain");
  constexpr int FR = 8;  // entity fragments a wave holds: a segment of 16 FR columns (4: no register left over is
                         // needed any more, and the rank at d = 512 runs 2 - 3 % slower: a read has four MFMAs to land)
  constexpr int NSEG = KSTEPS / FR;
  constexpr int d = 16 * KSTEPS;
  const int dq = PAD ? a.d : d;                         // elements of a query row and of a table row in memory
  const int64_t row_stride = (I8 ? 1 : 2) * (int64_t)dq;  // bytes of a table row in memory
  __shared__ __attribute__((aligned(1024))) unsigned char lds_e[QW_NBUF * QW_STAGE_BYTES];
  __shared__ __attribute__((aligned(16))) float lds_sc[I8 ? QW_NBUF : 1][QW_STAGE_ROWS];

  const int64_t wg = blockIdx.x;
  const int xcd = (int)(wg & 7);
  const int64_t slot = wg >> 3;
  const int qg = (int)(slot % a.n_qgroups);
  const int wlane = (int)(slot / a.n_qgroups);
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t q0 = (int64_t)qg * QW_WG_QUERIES + wave * 32;

  // chunks of this workgroup: first, stride, count; stages that hold at least one valid row
  const int64_t c_first = xcd + 8 * (int64_t)wlane;
  const int64_t c_stride = 8 * (int64_t)a.n_lanes;
  if (c_first >= a.n_chunks) return;
  const int my_chunks = (int)((a.n_chunks - 1 - c_first) / c_stride) + 1;
  const int spc = a.chunk_rows / QW_STAGE_ROWS;  // stages per chunk
  const int64_t r_end = a.e_end;
  const int64_t row_first = a.e_begin + c_first * a.chunk_rows;
  const int64_t row_last_chunk = row_first + c_stride * (int64_t)(my_chunks - 1) * a.chunk_rows;
  int valid_last = (int)((r_end - row_last_chunk + QW_STAGE_ROWS - 1) / QW_STAGE_ROWS);
  valid_last = valid_last < spc ? valid_last : spc;
  const int n_st = (my_chunks - 1) * spc + valid_last;
  const int64_t chunk_skip = (c_stride - 1) * (int64_t)a.chunk_rows;

  // the query row of this lane's column as MFMA fragments (rounded to bf16 once)
  bf16x8 qf[KSTEPS];
  {
    const int64_t q = q0 + c;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = 16 * s + 8 * hf;
      f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
      if (q < a.B && (!PAD || k < dq)) {
        const f32x4* src = (const f32x4*)(a.Q + q * dq + k);
        lo = src[0];
        hi = src[1];
      }
      qf[s] = cvt_bf16x8(lo, hi);
      // (one fragment at a time: with every fp32 load of the row in flight at once, the 128 registers of the
      // finished fragments and the 256 of the loads do not fit, and fragments would live in scratch memory)
      if (s % 4 == 3) asm volatile("" : "+v"(qf[s - 3]), "+v"(qf[s - 2]), "+v"(qf[s - 1]), "+v"(qf[s]));
    }
  }
  Epi epi;
  epi.init(ea, q0, c, hf, a.B);
  __shared__ typename Epi::Shared epi_sh;
  epi.bind(&epi_sh);

  // bf16: this lane's share of a stage is piece `lane` (16 bytes) of the rows wave + 8 j, j = 0..3: one wave-wide
  // load is one row, 1 KB in a piece.  int8: this thread's share is piece tid % 32 (16 bytes, 16 elements) of the rows
  // tid / 32 + 16 j, j = 0, 1.  In the table's last, partial stage the rows past the end repeat its last row (the
  // epilogues ignore them).
  constexpr int NLD = QW_STAGE_ROWS / QW_WG_WAVES;
  const unsigned char* Eb = (const unsigned char*)a.E;
  if constexpr (PAD) {
    for (int i = tid * 16; i < QW_NBUF * QW_STAGE_BYTES; i += 64 * QW_WG_WAVES * 16) *(u32x4*)(lds_e + i) = u32x4{0u, 0u, 0u, 0u};
    __syncthreads();  // no load may land before the zeros do
  }
  const bool lane_on = !PAD || (I8 ? 16 * (tid & 31) : 8 * lane) < dq;  // (a lane past the row's end fetches nothing: its piece stays zero)
  const uint32_t voff = I8 ? (uint32_t)((tid >> 5) * (int)row_stride + (tid & 31) * 16) : (uint32_t)(wave * (int)row_stride + lane * 16);
  u32x4 held[I8 ? 2 : 1];  // int8: the rows on their way into LDS
  float held_sc = 0.f;
  auto stage_issue = [&](int64_t row0, int buf_o) {
    if constexpr (I8) {
      const bool full = row0 + QW_STAGE_ROWS <= r_end;  // (uniform)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        int64_t g = row0 + (tid >> 5) + 16 * j;
        g = (full || g < r_end) ? g : r_end - 1;
        if (lane_on) held[j] = *(const u32x4*)(Eb + g * row_stride + (tid & 31) * 16);
      }
      if (tid < QW_STAGE_ROWS) {
        int64_t g = row0 + tid;
        g = (g < r_end) ? g : r_end - 1;
        held_sc = a.scale[g];
      }
    } else {
      unsigned char* dst = lds_e + buf_o + wave * QW_ROW_BYTES;
      if (!lane_on) return;
      if (__builtin_expect(row0 + QW_STAGE_ROWS <= r_end, 1)) {
        const unsigned char* src = Eb + row0 * row_stride;  // wave-uniform
#pragma unroll
        for (int j = 0; j < NLD; ++j)
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + j * QW_WG_WAVES * row_stride + voff),
                                           (__attribute__((address_space(3))) void*)(dst + j * (QW_WG_WAVES * QW_ROW_BYTES)), 16, 0, 0);
      } else {
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
          int64_t g = row0 + wave + QW_WG_WAVES * j;
          g = (g < r_end) ? g : r_end - 1;
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(Eb + g * row_stride + lane * 16),
                                           (__attribute__((address_space(3))) void*)(dst + j * (QW_WG_WAVES * QW_ROW_BYTES)), 16, 0, 0);
        }
      }
    }
  };
  // int8: what stage_issue fetched goes into the buffer at byte offset buf_o (number buf_n)
  auto stage_store = [&](int buf_o, int buf_n) {
    if constexpr (I8) {
      if (lane_on) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          unsigned char* dst = lds_e + buf_o + ((tid >> 5) + 16 * j) * QW_ROW_BYTES + (tid & 31) * 32;
          *(u32x4*)dst = i8x8_to_bf16x8(held[j][0], held[j][1]);
          *(u32x4*)(dst + 16) = i8x8_to_bf16x8(held[j][2], held[j][3]);
        }
      }
      if (tid < QW_STAGE_ROWS) lds_sc[buf_n][tid] = held_sc;
    }
  };
  // the stage the next issue fetches (two ahead of the one being multiplied) and its position in its chunk
  int64_t issue_row = row_first;
  int issue_so = 0;
  auto issue_advance = [&]() {
    issue_row += QW_STAGE_ROWS;
    if (++issue_so == spc) {
      issue_so = 0;
      issue_row += chunk_skip;
    }
  };

  // fragment address of this lane inside a buffer: K step s of segment g is 32 s + 256 g bytes further on
  const int fbase = c * QW_ROW_BYTES + 16 * hf;

  float sc_dummy[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) sc_dummy[i] = 1.f;

  // bf16: a barrier that orders nothing but the waves: the loads it guards are waited for explicitly, and the
  // compiler is kept from moving LDS accesses across it.  int8: the stage went into LDS with ordinary stores.
  auto wg_barrier = [&]() {
    if constexpr (I8) {
      __syncthreads();
    } else {
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  stage_issue(issue_row, 0);
  stage_store(0, 0);
  issue_advance();
  stage_issue(issue_row, QW_STAGE_BYTES);
  stage_store(QW_STAGE_BYTES, 1);
  issue_advance();
  wg_barrier();
  if constexpr (I8) {  // the stage after next waits in registers
    stage_issue(issue_row, 0);
    if (3 < n_st) issue_advance();
  }
  bf16x8 ef[FR];
#pragma unroll
  for (int s = 0; s < FR; ++s) ef[s] = *(const bf16x8*)(lds_e + fbase + 32 * s);

  int64_t row0 = row_first;
  int so = 0;
  int cur_o = 0, next_o = QW_STAGE_BYTES, next2_o = 2 * QW_STAGE_BYTES;
  int cur_n = 0, next_n = 1, next2_n = 2;  // (int8: the buffers' numbers, for the row scales)
#pragma unroll 1
  for (int k = 0; k < n_st; ++k) {
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    const unsigned char* cur = lds_e + cur_o + fbase;
#pragma unroll
    for (int g = 0; g < NSEG - 1; ++g) {
#pragma unroll
      for (int s = 0; s < FR; ++s) {
        acc = Epi::SWAP ? mfma_bf16(qf[FR * g + s], ef[s], acc) : mfma_bf16(ef[s], qf[FR * g + s], acc);
        ef[s] = *(const bf16x8*)(cur + 32 * s + 32 * FR * (g + 1));
      }
      // the order the scheduler is asked for: every MFMA followed by the read that replaces the fragment it consumed
#pragma unroll
      for (int s = 0; s < FR; ++s) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
    if (Epi::STAGE_HOOK) {
      epi.stage_mark();
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    // stage k + 1 has landed for every wave, and everyone is done with the buffer of stage k - 1
    wg_barrier();
    if (Epi::STAGE_HOOK) epi.stage_end();
    // bf16: stage k + 2 is requested (past the last stage: the last stage's rows once more, into a buffer nobody
    // reads).  int8: stage k + 2, requested a stage ago, is stored and stage k + 3 requested.
    stage_store(next2_o, next2_n);
    stage_issue(issue_row, next2_o);
    if (k + (I8 ? 4 : 3) < n_st) issue_advance();
    float sc16[16];
    float sc_col = 1.f;
    if constexpr (I8) {  // the row scales of this stage's tile: fetched under the last segment
      if (Epi::SWAP) {
        sc_col = lds_sc[cur_n][c];
      } else {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 v = *(const f32x4*)&lds_sc[cur_n][8 * g + 4 * hf];
          sc16[4 * g] = v[0];
          sc16[4 * g + 1] = v[1];
          sc16[4 * g + 2] = v[2];
          sc16[4 * g + 3] = v[3];
        }
      }
    }
    const unsigned char* nxt = lds_e + next_o + fbase;
#pragma unroll
    for (int s = 0; s < FR; ++s) {
      acc = Epi::SWAP ? mfma_bf16(qf[FR * (NSEG - 1) + s], ef[s], acc) : mfma_bf16(ef[s], qf[FR * (NSEG - 1) + s], acc);
      ef[s] = *(const bf16x8*)(nxt + 32 * s);
    }
#pragma unroll
    for (int s = 0; s < FR; ++s) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    if constexpr (I8) epi.template tile<true>(0, acc, sc16, sc_col, row0, r_end);
    else epi.template tile<false>(0, acc, sc_dummy, 1.f, row0, r_end);
    row0 += QW_STAGE_ROWS;
    if (++so == spc) {
      so = 0;
      row0 += chunk_skip;
    }
    const int t = cur_o, tn = cur_n;
    cur_o = next_o;
    next_o = next2_o;
    next2_o = t;
    cur_n = next_n;
    next_n = next2_n;
    next2_n = tn;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may land in LDS after the workgroup has gone
  epi.finish();
}

}  // namespace kge
