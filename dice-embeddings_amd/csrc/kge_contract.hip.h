// Query x all-entity contraction on MFMA with fused epilogues (gfx950).
//
// All main loops run on the bf16 MFMA (32x32x16) and share one epilogue interface:
//   qreg_async_kernel   bf16 table, d <= 256 (LDS rows of 64, 128 or 256 elements, narrower table rows zero-padded
//                       there): persistent, queries register-resident, entity rows global -> LDS
//   qstream_kernel      the same with a deeper pipeline and the epilogue inside the MFMA chain (filtered rank, scores)
//   qreg_i8_kernel      per-row int8 table, the same widths and walk, rows widened to bf16 on the way into LDS
//   kchunk_kernel       bf16 / int8 with d > 256: K in chunks of 64 through LDS
//   ksplit_kernel       fp32 tables, any d: every operand as three bf16 parts, six part products per product
// Reduction order of one score is fixed (k ascending in steps of the MFMA depth, nothing else), so
// every kernel that forms dot(Q[b], E[e]) with these helpers produces the same fp32 bit pattern.
//
// Orientation: by default the entity tile is the MFMA "A" operand (rows) and the query tile the "B"
// operand (columns), so each lane owns ONE query per tile (column = lane % 32) and 16 entities:
// per-query epilogue state (threshold, counters) lives in one register per lane.  Epilogues that
// write scores set SWAP so that consecutive lanes hold consecutive entities (coalesced stores).
#pragma once
#include "kge_internal.h"

namespace kge {

struct ContractArgs {
  const float* Q;
  const void* E;
  const float* scale;
  int64_t B, N;
  int64_t e_begin, e_end;  // entity rows scanned by this launch
  int64_t n_chunks;
  int d;
  int chunk_rows;
  int n_qgroups;
  int n_lanes;  // persistent kernels: entity-chunk lanes per (XCD, query group)
  // ksplit_kernel only: row strides of Q and E in elements (0: d), and the length of the K range one
  // workgroup sums (0: all of d; otherwise a multiple of 32, and blockIdx.y selects the range)
  int ldq, lde;
  int k_split_len;
  // ksplit_kernel only: 0, or the number of K ranges (a multiple of 8) of a launch whose grid is flat: range y is
  // dealt to XCD y % 8, so that the workgroups that read one range of a K-major operand share an L2
  int k_split_xcd;
  int persistent;  // host side: the decomposition above is that of a persistent kernel (checked at launch)
};

__device__ __forceinline__ f32x16 mfma_bf16(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 cvt_bf16x8(f32x4 lo, f32x4 hi) {
  bf16x8 r;
  r[0] = (__bf16)lo[0]; r[1] = (__bf16)lo[1]; r[2] = (__bf16)lo[2]; r[3] = (__bf16)lo[3];
  r[4] = (__bf16)hi[0]; r[5] = (__bf16)hi[1]; r[6] = (__bf16)hi[2]; r[7] = (__bf16)hi[3];
  return r;
}

// fp32 through the bf16 MFMA: x = x1 + x2 + x3 with three bf16 parts (8 + 8 + 8 mantissa bits: exact
// unless the residual underflows), and a product x * y is taken as the six leading part products
//   x1 y1, x1 y2, x2 y1, x1 y3, x2 y2, x3 y1      (the dropped ones are below 2^-24 of x y)
// each exact in fp32 and summed by the MFMA's fp32 accumulator.  SPLIT_A / SPLIT_B give the parts of
// the two operands for product p; every kernel that forms a score uses this order.
constexpr int SPLIT_PRODUCTS = 6;
__device__ constexpr int SPLIT_A[SPLIT_PRODUCTS] = {0, 0, 1, 0, 1, 2};
__device__ constexpr int SPLIT_B[SPLIT_PRODUCTS] = {0, 1, 0, 2, 1, 0};
// One pair: round both to bf16 (nearest even, one packed instruction), return the packed pair and leave the
// residuals in r0, r1 (exact: a residual fits fp32).
__device__ __forceinline__ uint32_t split_step(float& r0, float& r1) {
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  const uint32_t pk = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{r0, r1}, bf16x2));
  r0 = r0 - __uint_as_float(pk << 16);
  r1 = r1 - __uint_as_float(pk & 0xffff0000u);
  return pk;
}
__device__ __forceinline__ void split3_bf16x8(f32x4 lo, f32x4 hi, bf16x8 (&s)[3]) {
  float r[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
  for (int part = 0; part < 3; ++part) {
    u32x4 w;
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = split_step(r[2 * j], r[2 * j + 1]);
    s[part] = __builtin_bit_cast(bf16x8, w);
  }
}
// the same split for four values
__device__ __forceinline__ void split3_bf16x4(f32x4 v, bf16x4 (&s)[3]) {
  float r[4] = {v[0], v[1], v[2], v[3]};
#pragma unroll
  for (int part = 0; part < 3; ++part) {
    uint32_t w[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) w[j] = split_step(r[2 * j], r[2 * j + 1]);
    s[part] = __builtin_bit_cast(bf16x4, w);
  }
}

// two int8 (bytes `lo`,`hi` of w selected by shift) -> packed pair of bf16; exact for |v| <= 127
__device__ __forceinline__ uint32_t i8x2_to_bf16x2(uint32_t w, int shift) {
  float f0 = (float)(int)(int8_t)(w >> shift);
  float f1 = (float)(int)(int8_t)(w >> (shift + 8));
  return (__float_as_uint(f0) >> 16) | (__float_as_uint(f1) & 0xffff0000u);
}
__device__ __forceinline__ u32x4 i8x8_to_bf16x8(uint32_t w0, uint32_t w1) {
  u32x4 r;
  r[0] = i8x2_to_bf16x2(w0, 0);
  r[1] = i8x2_to_bf16x2(w0, 16);
  r[2] = i8x2_to_bf16x2(w1, 0);
  r[3] = i8x2_to_bf16x2(w1, 16);
  return r;
}

// XCD-aware decomposition of a flat workgroup id: hardware deals consecutive ids round-robin over
// the 8 XCDs, so ids with the same (id % 8) share an L2.  Consecutive slots on one XCD walk the
// query groups of ONE entity chunk, which keeps that chunk's rows hot in that XCD's L2.
// contract_grid_wgs() (host) gives the matching grid size.
__device__ __forceinline__ bool decompose_wg(const ContractArgs& a, int& qg, int64_t& chunk, int64_t wg = blockIdx.x) {
  if (a.n_chunks < 8) {  // too few chunks to give every XCD one: plain order, so that all XCDs get work
    qg = (int)(wg % a.n_qgroups);
    chunk = wg / a.n_qgroups;
    return chunk < a.n_chunks;
  }
  const int xcd = (int)(wg & 7);
  const int64_t slot = wg >> 3;
  qg = (int)(slot % a.n_qgroups);
  chunk = (slot / a.n_qgroups) * 8 + xcd;
  return chunk < a.n_chunks;
}

// ============================================================================================
// Epilogues.  tile<HAS_SCALE>(qt, acc, sc16, sc_col, e_base, limit): `acc` is one finished 32x32
// tile; without SWAP acc[i] = score(entity e_base + row_of(i,hf), query of this lane in tile qt);
// with SWAP acc[i] = score(query row_of(i,hf) of tile qt, entity e_base + c).  Entities >= limit
// are padding.  sc16[i] / sc_col are the int8 row scales of the entities this lane holds.
// ============================================================================================

struct StoreArgs {
  float* S;
  const float* bias;
  int64_t ldS;
  int64_t split_stride;  // K-split launches: partial result of range y goes to S + y * split_stride
  int64_t row_limit;     // StoreTEpi: entity rows from this one on are not stored (0: no such limit)
};
// The transposed result, S[e * ldS + q]: lanes along the queries, so a wave writes runs of 128 bytes of one entity's
// row (fp32 tables, no bias).  For products whose "entity" side is the larger matrix (dE = G^T Q as the rows of G
// against the rows of Q: the result row is an entity's).
template <int NQT>
struct StoreTEpi {
  static constexpr bool SWAP = false;
  static constexpr bool STAGE_HOOK = false;
  static constexpr bool DEFER = false;
  using Args = StoreArgs;
  struct Shared {
    int unused;
  };
  Args a;
  int64_t q0, B;
  int c, hf;
  __device__ void init(const Args& args, int64_t q0_, int c_, int hf_, int64_t B_) {
    a = args; q0 = q0_; c = c_; hf = hf_; B = B_;
  }
  __device__ void bind(Shared*) {}
  __device__ void stage_mark() {}
  __device__ void stage_end() {}
  template <bool HAS_SCALE>
  __device__ __forceinline__ void tile(int qt, const f32x16& acc, const float* sc16, float sc_col, int64_t e_base,
                                       int64_t limit) {
    static_assert(!HAS_SCALE, "fp32 tables only");
    const int64_t q = q0 + 32 * qt + c;
    if (q >= B) return;
    const int64_t lim = (a.row_limit && a.row_limit < limit) ? a.row_limit : limit;
    float* p = a.S + q;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int64_t e = e_base + row_of(i, hf);
      if (e < lim) p[e * a.ldS] = acc[i];
    }
  }
  __device__ void finish() {}
};
template <int NQT>
struct StoreEpi {
  static constexpr bool SWAP = true;
  static constexpr bool STAGE_HOOK = false;
  static constexpr bool DEFER = false;
  using Args = StoreArgs;
  struct Shared {
    float bias[8 * 32 * NQT];  // per wave: the biases of its 32 * NQT queries (up to 8 waves per workgroup)
  };
  Args a;
  const float* lb;  // this wave's slice of Shared::bias
  int64_t q0, B;
  int c, hf;
  __device__ void init(const Args& args, int64_t q0_, int c_, int hf_, int64_t B_) {
    a = args; q0 = q0_; c = c_; hf = hf_; B = B_;
    a.S += (int64_t)blockIdx.y * a.split_stride;
  }
  __device__ void bind(Shared* sh) {
    float* mine = sh->bias + (threadIdx.x >> 6) * (32 * NQT);
    for (int j = (threadIdx.x & 63); j < 32 * NQT; j += 64) {
      const int64_t q = q0 + j;
      mine[j] = (a.bias && q < B) ? a.bias[q] : 0.f;
    }
    lb = mine;
    __syncthreads();
  }
  __device__ void stage_mark() {}
  __device__ void stage_end() {}
  template <bool HAS_SCALE>
  __device__ __forceinline__ void tile(int qt, const f32x16& acc, const float* sc16, float sc_col, int64_t e_base,
                                       int64_t limit) {
    const int64_t e = e_base + c;
    if (e >= limit) return;
    const int64_t qrow = q0 + 32 * qt + 4 * hf;  // query row of acc[0]; acc[4g + r] is row qrow + 8g + r
    float* p = a.S + qrow * a.ldS + e;
    if (q0 + 32 * qt + 32 <= B) {  // the same for the wave: every query row of the tile exists (no test per element)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 b4 = *(const f32x4*)(lb + 32 * qt + 8 * g + 4 * hf);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = acc[4 * g + r];
          if (HAS_SCALE) v *= sc_col;
          p[(int64_t)(8 * g + r) * a.ldS] = v + b4[r];
        }
      }
    } else {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 b4 = *(const f32x4*)(lb + 32 * qt + 8 * g + 4 * hf);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = acc[4 * g + r];
          if (HAS_SCALE) v *= sc_col;
          v += b4[r];
          if (qrow + 8 * g + r < B) p[(int64_t)(8 * g + r) * a.ldS] = v;
        }
      }
    }
  }
  __device__ void finish() {}
};

// First round of kge_topk: every row scanned is a candidate (no threshold yet), so the scores go out as packed
// keys in row order, cand[q, e - e_begin], lanes along the entity index (whole lines per store), instead of
// through the candidate queues, which that many candidates would flush sixty times per workgroup.  A score that
// no threshold admits (NaN, -inf: the rounds admit what beats the k-th best, -inf at the start) leaves key 0 (empty).
struct TopkFirstArgs {
  unsigned long long* cand;  // [B, cap]
  int64_t cap;
  int64_t e_begin;
};
template <int NQT>
struct TopkFirstEpi {
  static constexpr bool SWAP = true;
  static constexpr bool STAGE_HOOK = false;
  static constexpr bool DEFER = false;
  using Args = TopkFirstArgs;
  struct Shared {
    int unused;
  };
  Args a;
  int64_t q0, B;
  int c, hf;
  __device__ void init(const Args& args, int64_t q0_, int c_, int hf_, int64_t B_) {
    a = args; q0 = q0_; c = c_; hf = hf_; B = B_;
  }
  __device__ void bind(Shared*) {}
  __device__ void stage_mark() {}
  __device__ void stage_end() {}
  template <bool HAS_SCALE>
  __device__ __forceinline__ void tile(int qt, const f32x16& acc, const float* sc16, float sc_col, int64_t e_base,
                                       int64_t limit) {
    const int64_t e = e_base + c;
    if (e >= limit) return;
    const int64_t qrow = q0 + 32 * qt + 4 * hf;  // query row of acc[0]; acc[4g + r] is row qrow + 8g + r
    unsigned long long* p = a.cand + qrow * a.cap + (e - a.e_begin);
    const unsigned long long id_part = (unsigned long long)(0xffffffffu - (uint32_t)e);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = acc[4 * g + r];
        if (HAS_SCALE) v *= sc_col;
        const unsigned long long key =
            (v > __uint_as_float(0xff800000u)) ? (((unsigned long long)f32_to_ordered(v) << 32) | id_part) : 0ull;
        if (qrow + 8 * g + r < B) p[(int64_t)(8 * g + r) * a.cap] = key;
      }
    }
  }
  __device__ void finish() {}
};

struct RankArgs {
  const float* thr;  // raw target score per query
  const int64_t* target;
  int32_t* n_gt;
  int32_t* n_eq;
  int32_t* n_eql;
};
template <int NQT>
struct RankEpi {
  static constexpr bool SWAP = false;
  static constexpr bool STAGE_HOOK = false;
  static constexpr bool DEFER = false;
  struct Shared {
    int unused;
  };
  __device__ void bind(Shared*) {}
  __device__ void stage_mark() {}
  __device__ void stage_end() {}
  using Args = RankArgs;
  Args a;
  float thr[NQT];
  int32_t tgt[NQT];
  int32_t gt[NQT], eq[NQT], eql[NQT];
  int64_t q0, B;
  int c, hf;
  __device__ void init(const Args& args, int64_t q0_, int c_, int hf_, int64_t B_) {
    a = args; q0 = q0_; c = c_; hf = hf_; B = B_;
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
      const int64_t q = q0 + 32 * t + c;
      thr[t] = (q < B) ? a.thr[q] : __uint_as_float(0x7fc00000u);  // NaN never compares
      tgt[t] = (q < B) ? (int32_t)a.target[q] : -1;
      gt[t] = eq[t] = eql[t] = 0;
    }
  }
  // Rare path (padding rows in the tile, or some lane saw an exact tie).  Out of line and free of
  // `this` so that the epilogue state stays in registers and the hot loop stays one basic block.
  // Returns the corrections (d_gt, eq, eq_lower) for one lane.
  struct Fix {
    int32_t dg, eq, eql;
  };
  static __device__ __attribute__((noinline)) Fix tile_fix(f32x16 s, float th, int32_t tg, int64_t e_base,
                                                           int64_t limit, int hf) {
    Fix f{0, 0, 0};
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int64_t e = e_base + row_of(i, hf);
      if (e < limit) {
        if (s[i] == th) {
          f.eq += 1;
          f.eql += (e < (int64_t)tg) ? 1 : 0;
        }
      } else {
        f.dg -= (s[i] > th) ? 1 : 0;  // the fast path counted this padding row
      }
    }
    return f;
  }
  // Hot path, VALU only (no compare-to-mask / scalar round trips, which stall on this hardware):
  // d = thr - s is exact in sign and is zero only for an exact tie; the sign bits are shifted into
  // one register (v_alignbit) and counted once per tile, min |d| detects ties.
  template <bool HAS_SCALE>
  __device__ __forceinline__ void tile(int qt, const f32x16& acc, const float* sc16, float sc_col, int64_t e_base,
                                       int64_t limit) {
    const float th = thr[qt];
    f32x16 s;
    uint32_t bits = 0;
    float mn = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i += 2) {
      s[i] = HAS_SCALE ? acc[i] * sc16[i] : acc[i];
      s[i + 1] = HAS_SCALE ? acc[i + 1] * sc16[i + 1] : acc[i + 1];
      const float d0 = th - s[i], d1 = th - s[i + 1];
      bits = __builtin_amdgcn_alignbit(bits, __float_as_uint(d0), 31);
      bits = __builtin_amdgcn_alignbit(bits, __float_as_uint(d1), 31);
      mn = (i == 0) ? __builtin_fminf(__builtin_fabsf(d0), __builtin_fabsf(d1))
                    : __builtin_fminf(__builtin_fminf(mn, __builtin_fabsf(d0)), __builtin_fabsf(d1));
    }
    gt[qt] += __builtin_popcount(bits);
    const unsigned long long tie = __builtin_amdgcn_ballot_w64(mn == 0.f);
    if (__builtin_expect(tie != 0 || e_base + 32 > limit, 0)) {
      const Fix f = tile_fix(s, th, tgt[qt], e_base, limit, hf);
      gt[qt] += f.dg;
      eq[qt] += f.eq;
      eql[qt] += f.eql;
    }
  }
  __device__ void finish() {
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
      const int64_t q = q0 + 32 * t + c;
      // both halves of the wave hold the same query: fold them, lanes < 32 publish
      int32_t g = gt[t] + __shfl_xor(gt[t], 32, 64);
      int32_t e = eq[t] + __shfl_xor(eq[t], 32, 64);
      int32_t l = eql[t] + __shfl_xor(eql[t], 32, 64);
      if (hf == 0 && q < B && thr[t] == thr[t]) {  // a NaN threshold (invalid target) publishes nothing
        if (g) atomicAdd(&a.n_gt[q], g);
        if (e) atomicAdd(&a.n_eq[q], e);
        if (l) atomicAdd(&a.n_eql[q], l);
      }
    }
  }
};

// The rank epilogue of qstream_kernel.  The hot path has no branch at all: the exact-tie test of a tile only
// feeds a running minimum of |threshold - score| per stage buffer, padding rows are counted like any other,
// and the kernel asks once per stage whether anything in it needs the exact treatment (a tie, or rows past
// the end of the table); if so it forms that stage's tiles again and hands them to tile_slow().  Ties other
// than a target with itself are rare and padding only exists in the last stage of the table, so the second
// pass costs a fraction of a percent, and the main loop stays straight-line code.
template <int NQT>
struct RankFastEpi {
  static constexpr bool SWAP = false;
  static constexpr bool STAGE_HOOK = false;
  static constexpr bool DEFER = true;
  static constexpr int SLOTS = 3;  // stage buffers in flight: one running minimum each
  struct Shared {
    int unused;
  };
  __device__ void bind(Shared*) {}
  __device__ void stage_mark() {}
  __device__ void stage_end() {}
  using Args = RankArgs;
  Args a;
  float thr[NQT];
  int32_t gt[NQT];
  float mn[SLOTS];
  int64_t q0, B;
  int c, hf;
  __device__ void init(const Args& args, int64_t q0_, int c_, int hf_, int64_t B_) {
    a = args; q0 = q0_; c = c_; hf = hf_; B = B_;
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
      const int64_t q = q0 + 32 * t + c;
      thr[t] = (q < B) ? a.thr[q] : __uint_as_float(0x7fc00000u);  // NaN never compares
      gt[t] = 0;
    }
#pragma unroll
    for (int j = 0; j < SLOTS; ++j) mn[j] = __uint_as_float(0x7f800000u);
  }
  // d = thr - s is exact in sign and is zero only for an exact tie; the sign bits are shifted into one register
  // (v_alignbit) and counted once per tile.  `slot`: the buffer of the stage the tile belongs to.
  __device__ __forceinline__ void tile_fast(int slot, int qt, const f32x16& acc) {
    const float th = thr[qt];
    uint32_t bits = 0;
    float m = mn[slot];
#pragma unroll
    for (int i = 0; i < 16; i += 2) {
      const float d0 = th - acc[i], d1 = th - acc[i + 1];
      bits = __builtin_amdgcn_alignbit(bits, __float_as_uint(d0), 31);
      bits = __builtin_amdgcn_alignbit(bits, __float_as_uint(d1), 31);
      m = __builtin_fminf(__builtin_fminf(m, __builtin_fabsf(d0)), __builtin_fabsf(d1));
    }
    mn[slot] = m;
    gt[qt] += __builtin_popcount(bits);
  }
  // wave-uniform: does the stage whose tiles went to `slot` need the exact pass?  Resets the slot.
  __device__ __forceinline__ bool stage_dirty(int slot, bool padded) {
    const unsigned long long tie = __builtin_amdgcn_ballot_w64(mn[slot] == 0.f);
    mn[slot] = __uint_as_float(0x7f800000u);
    return tie != 0 || padded;
  }
  // one tile of a stage formed again: ties and padding rows, exactly (the hot path has already counted every
  // element whose score is strictly greater, padding rows included).  Out of line and fed with scalars only, so
  // that nothing of it (addresses of the target / tie counters) is kept in registers across the main loop.
  static __device__ __attribute__((noinline)) int32_t slow_impl(f32x16 s, float th, int64_t q, int64_t B,
                                                               const int64_t* target, int32_t* n_eq, int32_t* n_eql,
                                                               int64_t e_base, int64_t limit, int hf) {
    const int32_t tg = (q < B) ? (int32_t)target[q] : -1;
    const typename RankEpi<NQT>::Fix f = RankEpi<NQT>::tile_fix(s, th, tg, e_base, limit, hf);
    if (q < B && th == th) {
      if (f.eq) atomicAdd(&n_eq[q], f.eq);
      if (f.eql) atomicAdd(&n_eql[q], f.eql);
    }
    return f.dg;
  }
  __device__ __forceinline__ void tile_slow(int qt, const f32x16& s, int64_t e_base, int64_t limit) {
    gt[qt] += slow_impl(s, thr[qt], q0 + 32 * qt + c, B, a.target, a.n_eq, a.n_eql, e_base, limit, hf);
  }
  // after a barrier: the thresholds pass through an opaque no-op, so that no epilogue arithmetic of a tile
  // scheduled after the barrier is moved (and its results kept in registers) to before it
  __device__ __forceinline__ void touch() {
#pragma unroll
    for (int t = 0; t < NQT; ++t) asm volatile("" : "+v"(thr[t]));
  }
  __device__ void finish() {
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
      const int64_t q = q0 + 32 * t + c;
      const int32_t g = gt[t] + __shfl_xor(gt[t], 32, 64);  // both halves of the wave hold the same query
      if (hf == 0 && q < B && thr[t] == thr[t] && g) atomicAdd(&a.n_gt[q], g);
    }
  }
};

struct TopkArgs {
  const float* tau;          // per query: k-th best score so far (-inf while fewer than k known)
  const int32_t* active;     // NULL = all queries; else only queries with active[b] != 0 collect
  int32_t* cnt;              // per query: candidates appended this round
  unsigned long long* cand;  // [B, cap] packed (ordered score << 32 | 0xffffffff - entity)
  int32_t cap;
};
// Repair scans: a candidate is what ranks above the packed key of the query's k-th best (0: none yet), i.e. a higher
// score or an equal score at a lower entity id.  (Its own epilogue type, so that the scans of the ordinary rounds
// carry nothing of it.)
struct TopkKeyArgs : TopkArgs {
  const unsigned long long* kth;
};
constexpr int TOPK_LQ = 512;   // candidates a workgroup parks in LDS between flushes
template <int NQT, bool BYKEY>
struct TopkEpiT {
  static constexpr bool SWAP = false;
  static constexpr bool STAGE_HOOK = true;
  static constexpr bool DEFER = false;
  using Args = typename std::conditional<BYKEY, TopkKeyArgs, TopkArgs>::type;
  // Candidates are parked in LDS (cheap atomics) and moved to the per-query global buffers in bulk
  // at stage boundaries, so the hot loop never waits for a global atomic's round trip.
  struct Shared {
    int n;
    int snap[2];  // n as thread 0 saw it just before a stage barrier (by stage parity): the same value for every wave
    int q[TOPK_LQ];
    unsigned long long key[TOPK_LQ];
  };
  Args a;
  Shared* sh;
  int par;  // parity of the stage barriers passed so far
  float tau[NQT];
  int64_t q0, B;
  int c, hf;
  __device__ void init(const Args& args, int64_t q0_, int c_, int hf_, int64_t B_) {
    a = args; q0 = q0_; c = c_; hf = hf_; B = B_;
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
      const int64_t q = q0 + 32 * t + c;
      const bool on = q < B && (a.active == nullptr || a.active[q] != 0);
      float th = on ? a.tau[q] : __uint_as_float(0x7f800000u);  // +inf: nothing qualifies
      if constexpr (BYKEY) {
        // ties with the k-th best must reach collect(): the hot path tests against a threshold they beat
        if (on) th = just_below(th);
      }
      tau[t] = th;
    }
  }
  __device__ void bind(Shared* s) {
    sh = s;
    par = 0;
    if (threadIdx.x == 0) {
      s->n = 0;
      s->snap[0] = s->snap[1] = 0;
    }
    __syncthreads();
  }
  // One candidate into its query's global buffer.  A full buffer keeps a uniform sample of what
  // arrives (reservoir sampling): the query is repaired by a later rescan, and the threshold derived
  // from the kept entries tightens geometrically whatever order the entities come in.
  static __device__ __forceinline__ void publish(int64_t q, unsigned long long key, int32_t* cnt,
                                                 unsigned long long* cand, int32_t cap) {
    int32_t slot = atomicAdd(&cnt[q], 1);
    if (slot >= cap) {
      const uint32_t e = 0xffffffffu - (uint32_t)(key & 0xffffffffull);
      uint32_t h = (e * 2654435761u) ^ ((uint32_t)slot * 0x9e3779b9u);
      h ^= h >> 15; h *= 0x2c1b3c6du; h ^= h >> 12;
      const uint32_t r = h % (uint32_t)(slot + 1);
      slot = (r < (uint32_t)cap) ? (int32_t)r : -1;
    }
    if (slot >= 0) cand[q * cap + slot] = key;
  }
  // Rare path: some element of the tile beats its query's threshold.  Out of line, so it stays out of
  // the hot loop's register budget.
  static __device__ __attribute__((noinline)) void collect(f32x16 s, float th, int64_t q, int64_t e_base, int64_t limit,
                                                           int hf, Shared* sh, int32_t* cnt, unsigned long long* cand,
                                                           int32_t cap, const unsigned long long* kth) {
    unsigned long long kk = 0ull;
    if constexpr (BYKEY) {
      bool any = false;  // (a lane past the batch's end has th = +inf: it must not read kth[q])
#pragma unroll
      for (int i = 0; i < 16; ++i) any = any || s[i] > th;
      if (any) kk = kth[q];
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int64_t e = e_base + row_of(i, hf);
      const unsigned long long key =
          ((unsigned long long)f32_to_ordered(s[i]) << 32) | (unsigned long long)(0xffffffffu - (uint32_t)e);
      const bool admit = BYKEY ? (s[i] > th && key > kk) : (s[i] > th);
      if (admit && e < limit) {
        const int idx = atomicAdd(&sh->n, 1);
        if (idx < TOPK_LQ) {
          sh->q[idx] = (int)q;
          sh->key[idx] = key;
        } else {
          publish(q, key, cnt, cand, cap);  // LDS queue full: go to global memory directly
        }
      }
    }
  }
  template <bool HAS_SCALE>
  __device__ __forceinline__ void tile(int qt, const f32x16& acc, const float* sc16, float sc_col, int64_t e_base,
                                       int64_t limit) {
    const float th = tau[qt];
    f32x16 s;
    float mx = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i += 2) {
      s[i] = HAS_SCALE ? acc[i] * sc16[i] : acc[i];
      s[i + 1] = HAS_SCALE ? acc[i + 1] * sc16[i + 1] : acc[i + 1];
      mx = (i == 0) ? __builtin_fmaxf(s[i], s[i + 1]) : __builtin_fmaxf(__builtin_fmaxf(mx, s[i]), s[i + 1]);
    }
    const unsigned long long hit = __builtin_amdgcn_ballot_w64(mx > th);
    if (__builtin_expect(hit != 0, 0))
      collect(s, th, q0 + 32 * qt + c, e_base, limit, hf, sh, a.cnt, a.cand, a.cap, key_ptr());
  }
  __device__ __forceinline__ const unsigned long long* key_ptr() const {
    if constexpr (BYKEY) return a.kth;
    else return nullptr;
  }
  // Empties the LDS queue.  Every wave of the workgroup is inside (nobody appends meanwhile).
  __device__ void flush() {
    const int n = sh->n;
    const int m = n < TOPK_LQ ? n : TOPK_LQ;
    for (int i = threadIdx.x; i < m; i += blockDim.x) publish(sh->q[i], sh->key[i], a.cnt, a.cand, a.cap);
    __syncthreads();
    if (threadIdx.x == 0) sh->n = 0;
    __syncthreads();
  }
  // Stage boundaries: stage_mark() before the workgroup's barrier, stage_end() after it.  The decision to
  // flush (queue at least half full) is taken on the count thread 0 recorded before the barrier, so every
  // wave takes the same branch even if a fast wave is already appending again.  Two slots, used in turn: a
  // slot is rewritten two barriers later, which no wave can reach before every wave has read it.
  __device__ void stage_mark() {
    if (threadIdx.x == 0) sh->snap[par] = sh->n;
  }
  __device__ void stage_end() {
    const int n = sh->snap[par];
    par ^= 1;
    if (n >= TOPK_LQ / 2) flush();
  }
  __device__ void finish() {
    __syncthreads();
    flush();
  }
};

template <int NQT>
using TopkEpi = TopkEpiT<NQT, false>;
template <int NQT>
using TopkKeyEpi = TopkEpiT<NQT, true>;

using host::BCE_SLOTS;  // the accumulator is spread: same-address double atomics serialise
struct BceArgs {
  const float* bias;
  double* sums;  // [0, BCE_SLOTS) partial sums of softplus(s), [BCE_SLOTS, 2 BCE_SLOTS) partial sums of s
  int32_t want_s;
};
template <int NQT>
struct BceEpi {
  static constexpr bool SWAP = false;
  static constexpr bool STAGE_HOOK = false;
  static constexpr bool DEFER = false;
  struct Shared {
    int unused;
  };
  __device__ void bind(Shared*) {}
  __device__ void stage_mark() {}
  __device__ void stage_end() {}
  using Args = BceArgs;
  Args a;
  float bias[NQT];
  bool valid[NQT];
  double sp, ss;
  int hf;
  __device__ void init(const Args& args, int64_t q0, int c, int hf_, int64_t B) {
    a = args; hf = hf_;
    sp = 0.0; ss = 0.0;
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
      const int64_t q = q0 + 32 * t + c;
      valid[t] = q < B;
      bias[t] = (valid[t] && a.bias) ? a.bias[q] : 0.f;
    }
  }
  template <bool HAS_SCALE>
  __device__ __forceinline__ void tile(int qt, const f32x16& acc, const float* sc16, float sc_col, int64_t e_base,
                                       int64_t limit) {
    if (!valid[qt]) return;
    // softplus(s) = max(s, 0) + log(1 + exp(-|s|)).  The sixteen logarithms of a lane's elements are taken as one:
    // the factors 1 + exp(-|s|) lie in (1, 2], their product stays below 2^16 and carries a relative error of at
    // most sixteen roundings, which after the logarithm is an absolute 1e-6 on a sum of order 10.
    float tpos = 0.f, tss = 0.f, prod = 1.f;
    if (e_base + 32 <= limit) {  // the same for the wave: no row of the tile is padding (one branch, no masks)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float s = acc[i];
        if (HAS_SCALE) s *= sc16[i];
        s += bias[qt];
        const float e = __expf(-fabsf(s));
        prod = __builtin_fmaf(prod, e, prod);  // prod * (1 + e) in one rounding
        tpos += fmaxf(s, 0.f);
        tss += s;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float s = acc[i];
        if (HAS_SCALE) s *= sc16[i];
        s += bias[qt];
        const bool ok = e_base + row_of(i, hf) < limit;
        const float e = __expf(-fabsf(s));
        prod = __builtin_fmaf(prod, ok ? e : 0.f, prod);
        tpos += ok ? fmaxf(s, 0.f) : 0.f;
        tss += ok ? s : 0.f;
      }
    }
    sp += (double)(tpos + __logf(prod));
    ss += (double)tss;
  }
  __device__ void finish() {
    double x = sp, y = ss;
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      x += __shfl_xor(x, o, 64);
      y += __shfl_xor(y, o, 64);
    }
    if ((threadIdx.x & 63) == 0) {
      const int slot = (int)((blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) & (BCE_SLOTS - 1));
      atomicAdd(&a.sums[slot], x);
      if (a.want_s) atomicAdd(&a.sums[BCE_SLOTS + slot], y);
    }
  }
};

// Backward of the multi-hot BCE step: g = (sigmoid(s) - y') * inv_bn for the dense part of y' (the
// known tails are subtracted afterwards from the CSR), written as G [B, ldG] and, when GT is given, also as its
// transpose GT [N, ldT] (the operands of the two gradient contractions when they take row-major operands only), plus
// the loss sums of BceEpi and the row sums of g (the gradient of the per-query bias).
struct GradArgs {
  const float* bias;
  double* sums;      // as BceArgs::sums
  float* G;
  float* GT;         // may be null
  float* dbias;      // [B], zero-initialised; may be null
  int64_t ldG, ldT;
  float inv_bn;      // upstream gradient / (B * N)
  float uniform;     // label smoothing: the 1/N every label carries, times inv_bn (0 without smoothing)
  int32_t want_s;
};
template <int NQT>
struct GradEpi {
  static constexpr bool SWAP = true;
  static constexpr bool STAGE_HOOK = false;
  static constexpr bool DEFER = false;
  using Args = GradArgs;
  struct Shared {
    float bias[8 * 32 * NQT];
  };
  Args a;
  const float* lb;
  float rowsum[NQT][16];
  double sp, ss;
  int64_t q0, B;
  int c, hf;
  __device__ void init(const Args& args, int64_t q0_, int c_, int hf_, int64_t B_) {
    a = args; q0 = q0_; c = c_; hf = hf_; B = B_;
    sp = 0.0; ss = 0.0;
#pragma unroll
    for (int t = 0; t < NQT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) rowsum[t][i] = 0.f;
  }
  __device__ void bind(Shared* sh) {
    float* mine = sh->bias + (threadIdx.x >> 6) * (32 * NQT);
    for (int j = (threadIdx.x & 63); j < 32 * NQT; j += 64) {
      const int64_t q = q0 + j;
      mine[j] = (a.bias && q < B) ? a.bias[q] : 0.f;
    }
    lb = mine;
    __syncthreads();
  }
  __device__ void stage_mark() {}
  __device__ void stage_end() {}
  template <bool HAS_SCALE>
  __device__ __forceinline__ void tile(int qt, const f32x16& acc, const float* sc16, float sc_col, int64_t e_base,
                                       int64_t limit) {
    const int64_t e = e_base + c;
    if (e >= limit) return;
    const int64_t qrow = q0 + 32 * qt + 4 * hf;  // query row of acc[0]; acc[4g + r] is row qrow + 8g + r
    float* pg = a.G + qrow * a.ldG + e;
    float* pt = a.GT + e * a.ldT + qrow;
    const bool full = q0 + 32 * qt + 32 <= B;  // the same for the wave: one branch, no test per element
    float tpos = 0.f, tss = 0.f, prod = 1.f;  // one logarithm for the sixteen elements, as in BceEpi
    if (full) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 b4 = *(const f32x4*)(lb + 32 * qt + 8 * g + 4 * hf);
        f32x4 out;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = acc[4 * g + r];
          if (HAS_SCALE) v *= sc_col;
          v += b4[r];
          const float ex = __expf(-fabsf(v));                       // in (0, 1]
          const float sig = (v >= 0.f ? 1.0f : ex) / (1.0f + ex);    // sigmoid without overflow
          const float gr = sig * a.inv_bn - a.uniform;
          prod = __builtin_fmaf(prod, ex, prod);
          tpos += fmaxf(v, 0.f);
          tss += v;
          out[r] = gr;
          rowsum[qt][4 * g + r] += gr;
          __builtin_nontemporal_store(gr, &pg[(int64_t)(8 * g + r) * a.ldG]);  // (streamed: the table stays in L2)
        }
        if (a.GT) *(f32x4*)(pt + 8 * g) = out;
      }
    } else {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 b4 = *(const f32x4*)(lb + 32 * qt + 8 * g + 4 * hf);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = acc[4 * g + r];
          if (HAS_SCALE) v *= sc_col;
          v += b4[r];
          const bool ok = qrow + 8 * g + r < B;
          const float ex = __expf(-fabsf(v));
          const float sig = (v >= 0.f ? 1.0f : ex) / (1.0f + ex);
          const float gr = ok ? sig * a.inv_bn - a.uniform : 0.f;
          prod = __builtin_fmaf(prod, ok ? ex : 0.f, prod);
          tpos += ok ? fmaxf(v, 0.f) : 0.f;
          tss += ok ? v : 0.f;
          rowsum[qt][4 * g + r] += gr;
          if (ok) {
            __builtin_nontemporal_store(gr, &pg[(int64_t)(8 * g + r) * a.ldG]);  // (streamed: the table stays in L2)
            if (a.GT) pt[8 * g + r] = gr;
          }
        }
      }
    }
    sp += (double)(tpos + __logf(prod));
    ss += (double)tss;
  }
  __device__ void finish() {
    double x = sp, y = ss;
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      x += __shfl_xor(x, o, 64);
      y += __shfl_xor(y, o, 64);
    }
    if ((threadIdx.x & 63) == 0) {
      const int slot = (int)((blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) & (BCE_SLOTS - 1));
      atomicAdd(&a.sums[slot], x);
      if (a.want_s) atomicAdd(&a.sums[BCE_SLOTS + slot], y);
    }
    if (a.dbias) {
#pragma unroll
      for (int t = 0; t < NQT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float v = rowsum[t][i];
#pragma unroll
          for (int o = 16; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);  // over the 32 entity columns of this half
          const int64_t q = q0 + 32 * t + 8 * (i >> 2) + 4 * hf + (i & 3);
          if (c == 0 && q < B) atomicAdd(&a.dbias[q], v);
        }
    }
  }
};

// Smallest and largest raw score of every query over all entities (the per-row min-max
// normalisation of ensemble evaluation needs them before any score can be combined).
struct MinMaxArgs {
  uint32_t* kmin;  // [B] order-preserving keys (f32_to_ordered), combined with atomicMin
  uint32_t* kmax;  // [B] combined with atomicMax
};
template <int NQT>
struct MinMaxEpi {
  static constexpr bool SWAP = false;
  static constexpr bool STAGE_HOOK = false;
  static constexpr bool DEFER = false;
  struct Shared {
    int unused;
  };
  __device__ void bind(Shared*) {}
  __device__ void stage_mark() {}
  __device__ void stage_end() {}
  using Args = MinMaxArgs;
  Args a;
  float lo[NQT], hi[NQT];
  int64_t q0, B;
  int c, hf;
  __device__ void init(const Args& args, int64_t q0_, int c_, int hf_, int64_t B_) {
    a = args; q0 = q0_; c = c_; hf = hf_; B = B_;
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
      lo[t] = __uint_as_float(0x7f800000u);
      hi[t] = __uint_as_float(0xff800000u);
    }
  }
  template <bool HAS_SCALE>
  __device__ __forceinline__ void tile(int qt, const f32x16& acc, const float* sc16, float sc_col, int64_t e_base,
                                       int64_t limit) {
    const bool full = e_base + 32 <= limit;  // uniform: one branch per tile, not a 64-bit compare per element
    float l = lo[qt], h = hi[qt];
    if (full) {
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const float s0 = HAS_SCALE ? acc[i] * sc16[i] : acc[i];
        const float s1 = HAS_SCALE ? acc[i + 1] * sc16[i + 1] : acc[i + 1];
        l = __builtin_fminf(__builtin_fminf(l, s0), s1);
        h = __builtin_fmaxf(__builtin_fmaxf(h, s0), s1);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float s = HAS_SCALE ? acc[i] * sc16[i] : acc[i];
        if (e_base + row_of(i, hf) < limit) {
          l = __builtin_fminf(l, s);
          h = __builtin_fmaxf(h, s);
        }
      }
    }
    lo[qt] = l;
    hi[qt] = h;
  }
  __device__ void finish() {
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
      // the two halves of the wave hold different entity rows of the same query
      const float l = __builtin_fminf(lo[t], __shfl_xor(lo[t], 32, 64));
      const float h = __builtin_fmaxf(hi[t], __shfl_xor(hi[t], 32, 64));
      const int64_t q = q0 + 32 * t + c;
      if (hf == 0 && q < B && l <= h) {
        atomicMin(&a.kmin[q], f32_to_ordered(l));
        atomicMax(&a.kmax[q], f32_to_ordered(h));
      }
    }
  }
};

constexpr int QREG_NQT = 2;            // 32-query tiles per wave in the d <= 128 forms of the persistent kernels

// ============================================================================================
// qreg_async_kernel: bf16 tables up to 256 elements wide (written for d == 128).  Queries live in registers as MFMA
// fragments; entity rows go from global memory straight into LDS (global_load_lds_dwordx4: no staging
// registers, no ds_write), in 128-row stages, and each wave prefetches the next stage while it computes the
// current one.
//
// LDS layout of a stage: row r is 256 B = 16 pieces of 16 B; piece p of row r sits in slot
// r*16 + (p ^ (r & 15)).  A direct-to-LDS load writes 64 consecutive slots per wave, so the swizzle
// is applied on the global side (which piece a lane fetches); fragment reads (ds_read_b128 of piece
// 2s+hf for rows c..c+15 at a time) then hit 16 distinct 16-byte bank groups.
// ============================================================================================
#ifndef KGE_QA_NQT
#define KGE_QA_NQT 2
#endif
#ifndef KGE_QA_WAVES
#define KGE_QA_WAVES 2
#endif
constexpr int QA_NQT = KGE_QA_NQT;                // 32-query tiles per wave
constexpr int QA_WAVES_PER_SIMD = KGE_QA_WAVES;   // occupancy the register budget is sized for
#ifndef KGE_QA_WG_WAVES
#define KGE_QA_WG_WAVES 8
#endif
constexpr int QA_WG_WAVES = KGE_QA_WG_WAVES;      // waves per workgroup (4 or 8)
constexpr int QA_WG_QUERIES = QA_WG_WAVES * 32 * QA_NQT;
constexpr int QA_WGS_PER_CU = 4 * QA_WAVES_PER_SIMD / QA_WG_WAVES;
constexpr int QA_STAGE_ROWS = 128;
constexpr int QA_BUF_BYTES = QA_STAGE_ROWS * 256;

// Work decomposition: persistent workgroups.  Flat id -> (xcd = id % 8, query group, lane); the
// workgroup keeps its query group for its whole life and walks the entity chunks
// xcd + 8 * (lane + n_lanes * i), i = 0, 1, ...  All query groups of a (xcd, lane) pair walk the same
// chunks in the same order, so a chunk is pulled from HBM once and shared through that XCD's L2.
// Stages run back to back across chunk boundaries (the prefetch never drains).
// NQT query tiles per wave and KSTEPS K steps of 16 per score: (QA_NQT, 8) for d == 128; (1, 16) for d == 256 (512-byte
// rows, two 64 KB stage buffers, the next tile's fragments read straight into the registers of the current ones);
// (QA_NQT, 4) for d == 64.
// PAD: the table's rows are narrower than the LDS rows (a.d < 16 * KSTEPS, a.d % 8 == 0): a row is fetched with its
// own stride, the 16-byte pieces past a.d are never written and stay the zeros the buffers start with, and the
// queries' fragments are zero there as well, so the chain adds exact zeros after the row's last K step.
template <template <int> class EpiT, int NQT = QA_NQT, int KSTEPS = 8, bool PAD = false>
__global__ void __launch_bounds__(64 * QA_WG_WAVES, QA_WAVES_PER_SIMD) qreg_async_kernel(ContractArgs a, typename EpiT<NQT>::Args ea) {
  using Epi = EpiT<NQT>;
  constexpr int d = 16 * KSTEPS;
  constexpr int ROW_BYTES = 2 * d;
  const int dq = PAD ? a.d : d;              // elements of a query row and of a table row in memory
  const int64_t row_stride = 2 * (int64_t)dq;  // bytes of a table row in memory
  constexpr int BUF_BYTES = QA_STAGE_ROWS * ROW_BYTES;
  constexpr int TILE_BYTES = 32 * ROW_BYTES;
  constexpr bool INPLACE = (KSTEPS > 8);  // no second set of fragment registers
  __shared__ __attribute__((aligned(1024))) unsigned char lds_e[2 * BUF_BYTES];

  const int64_t wg = blockIdx.x;
  const int xcd = (int)(wg & 7);
  const int64_t slot = wg >> 3;
  const int qg = (int)(slot % a.n_qgroups);
  const int wlane = (int)(slot / a.n_qgroups);
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t q0 = (int64_t)qg * (QA_WG_WAVES * 32 * NQT) + wave * (32 * NQT);

  // chunks of this workgroup: first, stride, count
  const int64_t c_first = xcd + 8 * (int64_t)wlane;
  const int64_t c_stride = 8 * (int64_t)a.n_lanes;
  if (c_first >= a.n_chunks) return;
  const int my_chunks = (int)((a.n_chunks - 1 - c_first) / c_stride) + 1;
  const int spc = a.chunk_rows / QA_STAGE_ROWS;  // stages per chunk
  const int total_stages = my_chunks * spc;
  const int64_t r_end = a.e_end;
  auto stage_row = [&](int k) -> int64_t {
    const int ci = k / spc, so = k - ci * spc;
    return a.e_begin + (c_first + c_stride * ci) * a.chunk_rows + (int64_t)so * QA_STAGE_ROWS;
  };

  bf16x8 qf[NQT][KSTEPS];
#pragma unroll
  for (int t = 0; t < NQT; ++t) {
    const int64_t q = q0 + 32 * t + c;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = 16 * s + 8 * hf;
      f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
      if (q < a.B && (!PAD || k < dq)) {
        const f32x4* src = (const f32x4*)(a.Q + q * dq + k);
        lo = src[0];
        hi = src[1];
      }
      qf[t][s] = cvt_bf16x8(lo, hi);
    }
  }
  Epi epi;
  epi.init(ea, q0, c, hf, a.B);
  __shared__ typename Epi::Shared epi_sh;
  epi.bind(&epi_sh);

  // this lane's share of a stage: rows lrow + RPI * j, always the same swizzled piece (RPI is a multiple of 16)
  constexpr int LPR = ROW_BYTES / 16;             // lanes (16-byte pieces) per row
  constexpr int RPW = 64 / LPR;                   // rows one wave-wide load instruction covers (1 KB)
  constexpr int RPI = RPW * QA_WG_WAVES;          // rows one workgroup-wide load instruction covers
  constexpr int NLD = QA_STAGE_ROWS / RPI;        // load instructions per lane per stage
  static_assert(RPI % 16 == 0 && QA_STAGE_ROWS % RPI == 0, "stage / workgroup shape");
  constexpr int SWZ = LPR < 16 ? LPR - 1 : 15;  // the swizzle permutes the low four bits of the piece index (all of
                                                // them in a row of fewer than sixteen pieces)
  const int lrow = wave * RPW + lane / LPR;
  const int lpiece = (lane % LPR) ^ (lrow & SWZ);
  const bool lane_on = !PAD || 8 * lpiece < dq;  // (a lane fetches the same piece of every row it handles)
  const unsigned char* Eb = (const unsigned char*)a.E;
  if constexpr (PAD) {
    for (int i = tid * 16; i < 2 * BUF_BYTES; i += 64 * QA_WG_WAVES * 16) *(u32x4*)(lds_e + i) = u32x4{0u, 0u, 0u, 0u};
    __syncthreads();  // no load may land before the zeros do
  }
  auto stage_issue = [&](int64_t row0, int buf) {
    unsigned char* dst = lds_e + buf * BUF_BYTES + wave * 1024;
    if (!lane_on) return;
    if (row0 + QA_STAGE_ROWS <= r_end) {
      const unsigned char* src = Eb + (row0 + lrow) * row_stride + lpiece * 16;
#pragma unroll
      for (int j = 0; j < NLD; ++j)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + j * (RPI * row_stride)),
                                         (__attribute__((address_space(3))) void*)(dst + j * (RPI * ROW_BYTES)), 16, 0, 0);
    } else {
#pragma unroll
      for (int j = 0; j < NLD; ++j) {
        int64_t g = row0 + lrow + RPI * j;
        g = (g < r_end) ? g : r_end - 1;  // padding rows repeat the last valid row; the epilogue ignores them
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(Eb + g * row_stride + lpiece * 16),
                                         (__attribute__((address_space(3))) void*)(dst + j * (RPI * ROW_BYTES)), 16, 0, 0);
      }
    }
  };

  // fragment addresses of this lane inside a stage buffer (row c of e-tile 0)
  int foff[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) foff[s] = c * ROW_BYTES + (((2 * s + hf) ^ (c & SWZ)) << 4);

  constexpr int ET = QA_STAGE_ROWS / 32;
  f32x16 acc_prev;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc_prev[i] = 0.f;
  float sc_dummy[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) sc_dummy[i] = 1.f;
  int64_t e_prev = r_end;  // "nothing to do" for the first epilogue: a tile entirely past the limit

  int64_t row_next = stage_row(0);
  stage_issue(row_next, 0);
  for (int st = 0; st < total_stages; ++st) {
    const int buf = st & 1;
    const int64_t row0 = row_next;
    if (row0 >= r_end) break;  // only the trailing stages of the table's last chunk can be empty
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (Epi::STAGE_HOOK) epi.stage_mark();
    __syncthreads();  // stage st has landed for every wave; everyone is done reading the other buffer
    if (Epi::STAGE_HOOK) epi.stage_end();
    if (st + 1 < total_stages) {
      row_next = stage_row(st + 1);
      if (row_next < r_end) stage_issue(row_next, buf ^ 1);
    }
    const unsigned char* base = lds_e + buf * BUF_BYTES;
    bf16x8 ef[KSTEPS];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) ef[s] = *(const bf16x8*)(base + foff[s]);
#pragma unroll
    for (int et = 0; et < ET; ++et) {
#pragma unroll
      for (int t = 0; t < NQT; ++t) {
        const int t_prev = (t + NQT - 1) % NQT;
        const bool refill = (t == NQT - 1) && (et + 1 < ET);
        bf16x8 efn[INPLACE ? 1 : KSTEPS];
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          acc = Epi::SWAP ? mfma_bf16(qf[t][s], ef[s], acc) : mfma_bf16(ef[s], qf[t][s], acc);
          // last use of fragment s for this e-tile: fetch the next e-tile's fragment into its place
          if (refill) {
            if constexpr (INPLACE) ef[s] = *(const bf16x8*)(base + (et + 1) * TILE_BYTES + foff[s]);
            else efn[s] = *(const bf16x8*)(base + (et + 1) * TILE_BYTES + foff[s]);
          }
        }
        epi.template tile<false>(t_prev, acc_prev, sc_dummy, 1.f, e_prev, r_end);
        if (refill) {
          if constexpr (!INPLACE) {
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) ef[s] = efn[s];
          }
        }
        acc_prev = acc;
        e_prev = row0 + et * 32;
      }
    }
  }
  epi.template tile<false>(NQT - 1, acc_prev, sc_dummy, 1.f, e_prev, r_end);
  epi.finish();
}

// ============================================================================================
// qstream_kernel: bf16 table, d == 128, the persistent walk, tiles, swizzled LDS rows and reduction
// order of qreg_async_kernel with a deeper pipeline:
//   * entity rows go global -> LDS in 64-row stages through a ring of three buffers: the loads of stage
//     k + 2 are issued while stage k is multiplied, so a load has two stages to land;
//   * one barrier per stage, between the stage's two entity tiles, and it waits for nothing but the
//     global -> LDS loads it guards; the fragments of the next entity tile (of this stage or the next)
//     are fetched under the last MFMA chain of the current one, so no wave waits for LDS after a barrier;
//   * NQT query tiles per wave reuse every fragment read;
//   * everything between two barriers is straight-line code (loads are issued unconditionally with clamped
//     rows, the epilogue defers its rare cases to a per-stage check), scheduled as one MFMA, a few VALU
//     instructions of the previous tile's epilogue, one fragment read, and so on.
// W waves per workgroup, OCC waves per SIMD: a workgroup covers W * 32 * NQT queries.
// ============================================================================================
constexpr int QS_STAGE_ROWS = 64;
constexpr int QS_STAGE_BYTES = QS_STAGE_ROWS * 256;
constexpr int QS_NBUF = 3;
// VALU instructions of the previous tile's epilogue asked for behind each MFMA (an MFMA takes two of the eight
// issue slots of its 32 cycles; about 42 epilogue instructions per 8 MFMAs: five per MFMA measured best of 4..8)
constexpr int QS_VALU_PER_MFMA = 5;

// KSTEPS: K steps of 16 per score (8: d == 128; 16: d == 256, rows of 512 bytes, one query tile per wave; 4: d == 64).
// PAD: rows narrower than the LDS rows, as in qreg_async_kernel.
template <template <int> class EpiT, int NQT, int W, int OCC, int KSTEPS = 8, bool PAD = false>
__global__ void __launch_bounds__(64 * W, OCC) qstream_kernel(ContractArgs a, typename EpiT<NQT>::Args ea) {
  using Epi = EpiT<NQT>;
  constexpr int d = 16 * KSTEPS;
  constexpr int ROW_BYTES = 2 * d;                      // a bf16 row in LDS
  const int dq = PAD ? a.d : d;                         // elements of a query row and of a table row in memory
  const int64_t row_stride = 2 * (int64_t)dq;           // bytes of a table row in memory
  constexpr int STAGE_BYTES = QS_STAGE_ROWS * ROW_BYTES;
  constexpr int TILE_BYTES = 32 * ROW_BYTES;            // one 32-row entity tile of a stage
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
  const int spc = a.chunk_rows / QS_STAGE_ROWS;  // stages per chunk
  const int64_t r_end = a.e_end;
  const int64_t row_first = a.e_begin + c_first * a.chunk_rows;
  const int64_t row_last_chunk = row_first + c_stride * (int64_t)(my_chunks - 1) * a.chunk_rows;
  int valid_last = (int)((r_end - row_last_chunk + QS_STAGE_ROWS - 1) / QS_STAGE_ROWS);
  valid_last = valid_last < spc ? valid_last : spc;
  const int n_st = (my_chunks - 1) * spc + valid_last;
  const int64_t chunk_skip = (c_stride - 1) * (int64_t)a.chunk_rows;

  bf16x8 qf[NQT][KSTEPS];
#pragma unroll
  for (int t = 0; t < NQT; ++t) {
    const int64_t q = q0 + 32 * t + c;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = 16 * s + 8 * hf;
      f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
      if (q < a.B && (!PAD || k < dq)) {
        const f32x4* src = (const f32x4*)(a.Q + q * dq + k);
        lo = src[0];
        hi = src[1];
      }
      qf[t][s] = cvt_bf16x8(lo, hi);
    }
  }
  Epi epi;
  epi.init(ea, q0, c, hf, a.B);
  __shared__ typename Epi::Shared epi_sh;
  epi.bind(&epi_sh);

  // this lane's share of a stage: rows lrow + RPI * j, always the same swizzled piece (RPI is a multiple of 16).
  // A full stage is a scalar base plus per-lane offsets that never change; in the table's last, partial stage the
  // rows past the end repeat its last row (the epilogues ignore them).
  constexpr int LPR = ROW_BYTES / 16;   // lanes (16-byte pieces) per row
  constexpr int RPW = 64 / LPR;         // rows one wave-wide load instruction covers (1 KB)
  constexpr int RPI = RPW * W;
  constexpr int NLD = QS_STAGE_ROWS / RPI;
  static_assert(RPI % 16 == 0 && QS_STAGE_ROWS % RPI == 0, "stage / workgroup shape");
  constexpr int SWZ = LPR < 16 ? LPR - 1 : 15;  // the swizzle permutes the low four bits of the piece index (all of
                                                // them in a row of fewer than sixteen pieces)
  const int lrow = wave * RPW + lane / LPR;
  const int lpiece = (lane % LPR) ^ (lrow & SWZ);
  const bool lane_on = !PAD || 8 * lpiece < dq;  // (a lane fetches the same piece of every row it handles)
  const unsigned char* Eb = (const unsigned char*)a.E;
  if constexpr (PAD) {
    for (int i = tid * 16; i < QS_NBUF * STAGE_BYTES; i += 64 * W * 16) *(u32x4*)(lds_e + i) = u32x4{0u, 0u, 0u, 0u};
    __syncthreads();  // no load may land before the zeros do
  }
  uint32_t voff[NLD];
#pragma unroll
  for (int j = 0; j < NLD; ++j) voff[j] = (uint32_t)((lrow + RPI * j) * (int)row_stride + lpiece * 16);
  auto stage_issue = [&](int64_t row0, int buf) {
    unsigned char* dst = lds_e + buf * STAGE_BYTES + wave * 1024;
    if (!lane_on) return;
    if (__builtin_expect(row0 + QS_STAGE_ROWS <= r_end, 1)) {
      const unsigned char* src = Eb + row0 * row_stride;  // wave-uniform
#pragma unroll
      for (int j = 0; j < NLD; ++j)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + voff[j]),
                                         (__attribute__((address_space(3))) void*)(dst + j * (RPI * ROW_BYTES)), 16, 0, 0);
    } else {
#pragma unroll
      for (int j = 0; j < NLD; ++j) {
        int64_t g = row0 + lrow + RPI * j;
        g = (g < r_end) ? g : r_end - 1;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(Eb + g * row_stride + lpiece * 16),
                                         (__attribute__((address_space(3))) void*)(dst + j * (RPI * ROW_BYTES)), 16, 0, 0);
      }
    }
  };
  // the stage the next issue fetches (two ahead of the one being multiplied) and its position in its chunk
  int64_t issue_row = row_first;
  int issue_so = 0;
  auto issue_advance = [&]() {
    issue_row += QS_STAGE_ROWS;
    if (++issue_so == spc) {
      issue_so = 0;
      issue_row += chunk_skip;
    }
  };

  // fragment addresses of this lane inside buffer 0 (row c of entity tile 0)
  int foff[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) foff[s] = c * ROW_BYTES + (((2 * s + hf) ^ (c & SWZ)) << 4);

  // the first epilogue has no tile to work on: e_prev past the limit says so to the branching epilogues, scores of
  // -inf (never greater than, never equal to a threshold) to the deferring one
  f32x16 acc_prev;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc_prev[i] = Epi::DEFER ? __uint_as_float(0xff800000u) : 0.f;
  float sc_dummy[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) sc_dummy[i] = 1.f;
  int64_t e_prev = r_end;

  // A barrier that orders nothing but the waves: the loads it guards are waited for explicitly, and the
  // compiler is kept from moving LDS accesses across it.
  auto wg_barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);  // nothing is scheduled across: no epilogue value is kept alive over the wait
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };

  stage_issue(issue_row, 0);
  issue_advance();
  stage_issue(issue_row, 1);
  issue_advance();
  wg_barrier();
  bf16x8 ef[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) ef[s] = *(const bf16x8*)(lds_e + foff[s]);

  int64_t row0 = row_first, prev_row0 = row_first;
  int so = 0;
  // a stage's tiles formed again from its buffer, for the exact pass of a deferring epilogue
  auto fix_stage = [&](auto bufc, int64_t rows0) {
    if constexpr (Epi::DEFER) {
      constexpr int BUF = decltype(bufc)::value;
      for (int et = 0; et < 2; ++et) {
#pragma unroll
        for (int t = 0; t < NQT; ++t) {
          f32x16 acc;
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
          for (int s = 0; s < KSTEPS; ++s) {
            const bf16x8 f = *(const bf16x8*)(lds_e + BUF * STAGE_BYTES + et * TILE_BYTES + foff[s]);
            acc = mfma_bf16(f, qf[t][s], acc);
          }
          epi.tile_slow(t, acc, rows0 + et * 32, r_end);
        }
      }
    }
  };
  auto bufc_prev = [](auto bufc) { return std::integral_constant<int, (decltype(bufc)::value + QS_NBUF - 1) % QS_NBUF>{}; };
  auto run_stage = [&](auto bufc, int k) {
    constexpr int BUF = decltype(bufc)::value;
    constexpr int NEXT = (BUF + 1) % QS_NBUF, NEXT2 = (BUF + 2) % QS_NBUF, PREV = NEXT2;
#pragma unroll
    for (int et = 0; et < 2; ++et) {
      if (et == 1) {
        if constexpr (Epi::DEFER) {
          // every tile of the previous stage has been through the epilogue by now, and its buffer is intact
          // until this wave passes the barrier below: the place for that stage's exact pass, if it needs one
          if (k > 0 && epi.stage_dirty(PREV, prev_row0 + QS_STAGE_ROWS > r_end)) fix_stage(bufc_prev(bufc), prev_row0);
        }
        if (Epi::STAGE_HOOK) {
          epi.stage_mark();
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
        // stage k + 1 has landed for every wave, and everyone is done with the buffer of stage k - 1
        wg_barrier();
        if constexpr (Epi::DEFER) epi.touch();
        if (Epi::STAGE_HOOK) epi.stage_end();
        // stage k + 2 (past the last stage: the last stage's rows once more, into a buffer nobody reads)
        stage_issue(issue_row, NEXT2);
        if (k + 3 < n_st) issue_advance();
      }
      // where the next entity tile's fragments come from: the second tile of this stage, or the first of the next
      const int roff = (et == 0) ? BUF * STAGE_BYTES + TILE_BYTES : NEXT * STAGE_BYTES;
#pragma unroll
      for (int t = 0; t < NQT; ++t) {
        const int t_prev = (t + NQT - 1) % NQT;
        const bool refill = (t == NQT - 1);
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          acc = Epi::SWAP ? mfma_bf16(qf[t][s], ef[s], acc) : mfma_bf16(ef[s], qf[t][s], acc);
          if (refill) ef[s] = *(const bf16x8*)(lds_e + roff + foff[s]);  // last use of fragment s: fetch its successor
        }
        if constexpr (Epi::DEFER) {
          epi.tile_fast((et == 0 && t == 0) ? PREV : BUF, t_prev, acc_prev);  // the stage the finished tile belongs to
        } else {
          epi.template tile<false>(t_prev, acc_prev, sc_dummy, 1.f, e_prev, r_end);
        }
        // the order the scheduler is asked for: each MFMA of this chain, then a share of the previous tile's
        // epilogue, then (in a refilling chain) the read that replaces the fragment the MFMA consumed
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, QS_VALU_PER_MFMA, 0);
          if (refill) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        acc_prev = acc;
        e_prev = row0 + et * 32;
      }
    }
    prev_row0 = row0;
    row0 += QS_STAGE_ROWS;
    if (++so == spc) {
      so = 0;
      row0 += chunk_skip;
    }
  };
  // after the last stage: the epilogue of its last tile, then (deferring epilogues) its exact pass
  auto tail = [&](auto bufc) {
    if constexpr (Epi::DEFER) {
      constexpr int BUF = decltype(bufc)::value;
      epi.tile_fast(BUF, NQT - 1, acc_prev);
      if (epi.stage_dirty(BUF, prev_row0 + QS_STAGE_ROWS > r_end)) fix_stage(bufc, prev_row0);
    } else {
      epi.template tile<false>(NQT - 1, acc_prev, sc_dummy, 1.f, e_prev, r_end);
    }
  };
  for (int k = 0;;) {
    run_stage(std::integral_constant<int, 0>{}, k);
    if (++k >= n_st) { tail(std::integral_constant<int, 0>{}); break; }
    run_stage(std::integral_constant<int, 1>{}, k);
    if (++k >= n_st) { tail(std::integral_constant<int, 1>{}); break; }
    run_stage(std::integral_constant<int, 2>{}, k);
    if (++k >= n_st) { tail(std::integral_constant<int, 2>{}); break; }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may land in LDS after the workgroup has gone
  epi.finish();
}

// ============================================================================================
// qreg_i8_kernel: per-row int8 table, d == 128.  Same persistent work decomposition, 128-row
// stages, swizzled LDS layout, tiles and reduction order as qreg_async_kernel.  Rows cannot go
// straight into LDS because they are widened to bf16 (exactly) on the way: each thread keeps its
// share of the next stage in registers while the current stage is consumed, then converts and
// stores it.  The fp32 row scales of a stage ride along in LDS.
// ============================================================================================
#ifndef KGE_I8_WG_WAVES
#define KGE_I8_WG_WAVES 8
#endif
constexpr int I8_WG_WAVES = KGE_I8_WG_WAVES;
constexpr int I8_WG_QUERIES = I8_WG_WAVES * 32 * QREG_NQT;
constexpr int I8_WGS_PER_CU = 8 / I8_WG_WAVES;  // 2 waves per SIMD

// NQT query tiles per wave and KSTEPS K steps of 16 per score: (2, 8) for d == 128; (1, 16) for d == 256, whose rows are
// 512 bytes of bf16 in LDS (64 KB per stage buffer) and whose queries still fit the register file one tile per wave;
// (2, 4) for d == 64.
// PAD: rows narrower than the LDS rows (a.d < 16 * KSTEPS, a.d % 16 == 0): the pieces past a.d are stored as zeros.
template <template <int> class EpiT, int NQT = QREG_NQT, int KSTEPS = 8, bool PAD = false>
__global__ void __launch_bounds__(64 * I8_WG_WAVES, 2) qreg_i8_kernel(ContractArgs a, typename EpiT<NQT>::Args ea) {
  using Epi = EpiT<NQT>;
  constexpr int d = 16 * KSTEPS;
  constexpr int ROW_BYTES = 2 * d;                      // a row widened to bf16, in LDS
  const int dq = PAD ? a.d : d;                         // elements (and bytes) of a table row in memory
  constexpr int BUF_BYTES = QA_STAGE_ROWS * ROW_BYTES;
  constexpr int PPR = d / 16;                           // 16-byte pieces of int8 per row
  constexpr int SWZ = 2 * PPR < 16 ? 2 * PPR - 1 : 15;  // swizzled bits of the index of a row's 16-byte bf16 pieces
  __shared__ __attribute__((aligned(1024))) unsigned char lds_e[2 * BUF_BYTES];
  __shared__ __attribute__((aligned(16))) float lds_sc[2][QA_STAGE_ROWS];
  constexpr int NT = 64 * I8_WG_WAVES;
  constexpr int NPIECE = QA_STAGE_ROWS * PPR / NT;  // 16-byte pieces of int8 a thread stages per stage

  const int64_t wg = blockIdx.x;
  const int xcd = (int)(wg & 7);
  const int64_t slot = wg >> 3;
  const int qg = (int)(slot % a.n_qgroups);
  const int wlane = (int)(slot / a.n_qgroups);
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t q0 = (int64_t)qg * (I8_WG_WAVES * 32 * NQT) + wave * (32 * NQT);

  const int64_t c_first = xcd + 8 * (int64_t)wlane;
  const int64_t c_stride = 8 * (int64_t)a.n_lanes;
  if (c_first >= a.n_chunks) return;
  const int my_chunks = (int)((a.n_chunks - 1 - c_first) / c_stride) + 1;
  const int spc = a.chunk_rows / QA_STAGE_ROWS;
  const int total_stages = my_chunks * spc;
  const int64_t r_end = a.e_end;
  auto stage_row = [&](int k) -> int64_t {
    const int ci = k / spc, so = k - ci * spc;
    return a.e_begin + (c_first + c_stride * ci) * a.chunk_rows + (int64_t)so * QA_STAGE_ROWS;
  };

  bf16x8 qf[NQT][KSTEPS];
#pragma unroll
  for (int t = 0; t < NQT; ++t) {
    const int64_t q = q0 + 32 * t + c;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = 16 * s + 8 * hf;
      f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
      if (q < a.B && (!PAD || k < dq)) {
        const f32x4* src = (const f32x4*)(a.Q + q * dq + k);
        lo = src[0];
        hi = src[1];
      }
      qf[t][s] = cvt_bf16x8(lo, hi);
    }
  }
  Epi epi;
  epi.init(ea, q0, c, hf, a.B);
  __shared__ typename Epi::Shared epi_sh;
  epi.bind(&epi_sh);

  // staging: 128 rows x d bytes in pieces of 16 int8; thread handles pieces tid + NT j
  u32x4 stage[NPIECE];
  float stage_sc = 0.f;
  const int8_t* Eb = (const int8_t*)a.E;
  auto stage_load = [&](int64_t row0) {
#pragma unroll
    for (int j = 0; j < NPIECE; ++j) {
      const int idx = tid + NT * j, row = idx / PPR, piece = idx % PPR;
      int64_t g = row0 + row;
      g = (g < r_end) ? g : r_end - 1;  // padding rows repeat the last valid row; epilogues ignore them
      stage[j] = u32x4{0u, 0u, 0u, 0u};
      if (!PAD || 16 * piece < dq) stage[j] = *(const u32x4*)(Eb + g * dq + piece * 16);
    }
    if (tid < QA_STAGE_ROWS) {
      int64_t g = row0 + tid;
      g = (g < r_end) ? g : r_end - 1;
      stage_sc = a.scale[g];
    }
  };
  auto stage_store = [&](int buf) {
    unsigned char* base = lds_e + buf * BUF_BYTES;
#pragma unroll
    for (int j = 0; j < NPIECE; ++j) {
      const int idx = tid + NT * j, row = idx / PPR, piece = idx % PPR;
      const int p0 = 2 * piece, sw = row & SWZ;  // (the swizzle permutes the low four bits of the piece index)
      *(u32x4*)(base + row * ROW_BYTES + ((p0 ^ sw) << 4)) = i8x8_to_bf16x8(stage[j][0], stage[j][1]);
      *(u32x4*)(base + row * ROW_BYTES + (((p0 + 1) ^ sw) << 4)) = i8x8_to_bf16x8(stage[j][2], stage[j][3]);
    }
    if (tid < QA_STAGE_ROWS) lds_sc[buf][tid] = stage_sc;
  };

  int foff[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) foff[s] = c * ROW_BYTES + (((2 * s + hf) ^ (c & SWZ)) << 4);

  constexpr int ET = QA_STAGE_ROWS / 32;
  // A tile's epilogue runs right after its MFMA chain (deferring it under the next chain, as the bf16
  // path does, does not fit the register budget next to the row scales).
  float sc16[16] = {};
  float sc_col = 1.f;

  int64_t row_next = stage_row(0);
  stage_load(row_next);
  stage_store(0);
  __syncthreads();
  for (int st = 0; st < total_stages; ++st) {
    const int buf = st & 1;
    const int64_t row0 = row_next;
    if (row0 >= r_end) break;
    bool have_next = false;
    if (st + 1 < total_stages) {
      row_next = stage_row(st + 1);
      have_next = row_next < r_end;
      if (have_next) stage_load(row_next);
    } else {
      row_next = r_end;
    }
    const unsigned char* base = lds_e + buf * BUF_BYTES;
#pragma unroll
    for (int et = 0; et < ET; ++et) {
      bf16x8 ef[KSTEPS];
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) ef[s] = *(const bf16x8*)(base + et * (32 * ROW_BYTES) + foff[s]);
#pragma unroll
      for (int t = 0; t < NQT; ++t) {
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
          acc = Epi::SWAP ? mfma_bf16(qf[t][s], ef[s], acc) : mfma_bf16(ef[s], qf[t][s], acc);
        if (t == 0) {  // row scales of this entity tile: fetched under the first chain
          if (Epi::SWAP) {
            sc_col = lds_sc[buf][et * 32 + c];
          } else {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              const f32x4 v = *(const f32x4*)&lds_sc[buf][et * 32 + 8 * g + 4 * hf];
              sc16[4 * g] = v[0];
              sc16[4 * g + 1] = v[1];
              sc16[4 * g + 2] = v[2];
              sc16[4 * g + 3] = v[3];
            }
          }
        }
        epi.template tile<true>(t, acc, sc16, sc_col, row0 + et * 32, r_end);
      }
    }
    if (have_next) stage_store(buf ^ 1);
    if (Epi::STAGE_HOOK) epi.stage_mark();
    __syncthreads();
    if (Epi::STAGE_HOOK) epi.stage_end();
  }
  epi.finish();
}

// ============================================================================================
// ksplit_kernel: fp32 tables on the bf16 MFMA (split3_bf16x8).  256 entities x 128 queries per
// workgroup of 8 waves (each wave 64 x 64), K in chunks of 32.  Both operands are loaded as fp32 into
// registers while the previous chunk is multiplied, split into their three bf16 parts and stored as
// three planes per operand in LDS; per 16-wide K step a wave reads 12 fragments and issues 24 MFMAs.
// Chain order per score: K steps of 16 ascending, inside a step the six products in SPLIT order.
//
// LDS plane layout: row r is 64 B = 4 pieces of 16 B (8 bf16); piece p sits in slot
// r*4 + (p ^ ((r >> 2) & 3)), so the 16 rows a fragment read touches at a time spread over all banks.
// ============================================================================================
constexpr int KS_NQT = 2;
using host::KS_WG_QUERIES;
using host::KS_TILE_ROWS;
constexpr int KS_KC = 32;
constexpr int KS_E_PLANE = KS_TILE_ROWS * 64;
constexpr int KS_Q_PLANE = KS_WG_QUERIES * 64;
constexpr int KS_STAGE_BYTES = 3 * KS_E_PLANE + 3 * KS_Q_PLANE;

// KMAJ (bit 0: the entity operand, bit 1: the query operand; VEC only): that operand is given K-MAJOR, X[k][row] with
// the rows contiguous (row pitch lde / ldq), as the backward of a contraction meets its operands (dQ = G E sums over
// the rows of E, dE = G^T Q over the rows of both).  Its plane in LDS is then K-major too, [32 k][rows] bf16, filled
// with 8-byte stores of four neighbouring rows at one k (32-byte segment s of the row of k kept at s ^ 2 (k & 3), which
// spreads a fragment read's four k rows over all banks), and a fragment is two transposing reads
// (ds_read_b64_tr_b16: within 16 lanes, lane j receives element j % 4 of the 8 bytes that lanes j / 4 + 4 i
// addressed, i = 0..3), each giving a lane its row at four consecutive k.  Same products in the same order as the
// row-major form.  The K-major operand's row count and pitch must be multiples of 4 and its base 16-byte aligned.
template <template <int> class EpiT, bool VEC, int KMAJ>
__device__ __forceinline__ void ksplit_body(const ContractArgs& a, const typename EpiT<KS_NQT>::Args& ea) {
  using Epi = EpiT<KS_NQT>;
  static_assert(KMAJ == 0 || VEC, "K-major operands are loaded 16 bytes at a time");
  constexpr bool KE = (KMAJ & 1) != 0, KQ = (KMAJ & 2) != 0;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * KS_STAGE_BYTES];

  int qg;
  int64_t chunk;
  int64_t wg_flat = blockIdx.x;
  int k_range = (int)blockIdx.y;
  if (a.k_split_xcd) {  // flat grid: consecutive ids go round the XCDs, and an XCD keeps to its K ranges
    const int64_t per_range = a.n_chunks * a.n_qgroups, slot = wg_flat >> 3;
    k_range = (int)(wg_flat & 7) + 8 * (int)(slot / per_range);
    wg_flat = slot % per_range;
  }
  if (!decompose_wg(a, qg, chunk, wg_flat)) return;
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int we = wave >> 1, wq = wave & 1;
  const int ldq = a.ldq ? a.ldq : a.d, lde = a.lde ? a.lde : a.d;
  const int k_off = a.k_split_len ? k_range * a.k_split_len : 0;
  const int d = (a.k_split_len && a.d - k_off > a.k_split_len) ? a.k_split_len : a.d - k_off;  // K range of this workgroup
  const int64_t q_base = (int64_t)qg * KS_WG_QUERIES;
  const int64_t q0 = q_base + 64 * wq;
  Epi epi;
  epi.init(ea, q0, c, hf, a.B);
  if constexpr (std::is_same<Epi, StoreEpi<KS_NQT>>::value) {
    if (a.k_split_xcd) epi.a.S += (int64_t)k_range * epi.a.split_stride;  // (blockIdx.y is 0 in a flat grid)
  }
  __shared__ typename Epi::Shared epi_sh;
  epi.bind(&epi_sh);

  const int64_t r0 = a.e_begin + chunk * a.chunk_rows;
  const int64_t r1 = (r0 + a.chunk_rows < a.e_end) ? r0 + a.chunk_rows : a.e_end;
  const int nkc = (d + KS_KC - 1) / KS_KC;
  const int n_et = (int)((r1 - r0 + KS_TILE_ROWS - 1) / KS_TILE_ROWS);
  const int n_it = n_et * nkc;
  const float* Ef = (const float*)a.E + (KE ? (int64_t)k_off * lde : (int64_t)k_off);

  // Staging: a chunk is 384 rows (256 entity rows, then 128 query rows) of 128 B, taken in six passes of
  // 64 rows; in pass g thread tid takes 16 B piece (tid & 7) of row 64 g + tid / 8, so eight neighbouring
  // lanes read one whole 128 B line.  Loads are branch-free so that all six stay in flight: rows past the
  // end repeat the last valid row (epilogues ignore them), columns past d are read from a clamped address
  // and zeroed when stored.  Pass g of chunk i+2 is loaded right after pass g of chunk i+1 has been split
  // and stored, both while chunk i is multiplied: one register set, and a whole iteration for a load to land.
  const int s_row = tid >> 3, s_piece = tid & 7;
  const int64_t q_last = a.B - 1, e_last = r1 - 1;
  const float* q_ptr[2];
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    int64_t qr = q_base + 64 * g + s_row;
    qr = qr < q_last ? qr : q_last;
    q_ptr[g] = a.Q + k_off + qr * ldq;
  }
  // K-major operands: pass g of the entity operand is k rows 8 g + wave of the chunk, lane l the four rows 4 l ..;
  // pass g of the query operand k rows 16 (g - 4) + tid / 32, four rows 4 (tid % 32) ..  A quad of rows past the
  // operand's end is read from the last quad inside the pitch instead (its scores are never stored).
  const int ke_kk = wave, ke_mq = lane, kq_kk = tid >> 5, kq_mq = tid & 31;
  int64_t kq_col = q_base + 4 * kq_mq;
  if (KQ) kq_col = (kq_col + 4 <= ldq) ? kq_col : ldq - 4;
  const float* Qk = a.Q + (int64_t)k_off * ldq;
  int st_k0 = 0, ld_k0 = 0;  // first k of the staged chunk, of the chunk being loaded
  f32x4 staged[6];             // passes 0..3: entity rows, 4..5: query rows
  int st_valid = 0;            // how many of this thread's four columns of the staged chunk are inside d
  int ld_valid = 0, ld_k = 0;  // the same, and the first column, for the chunk being loaded
  int ld_kc = 0;               // K chunk and first row of the tile the next loads fetch
  int64_t ld_row = KE ? r0 : r0 + s_row;
  auto load_begin = [&]() {
    ld_k = ld_kc * KS_KC + 4 * s_piece;
    ld_valid = d - ld_k;
    ld_k0 = ld_kc * KS_KC;
  };
  auto load_pass = [&](int g) {
    const float* row_ptr;
    if (KE && g < 4) {
      const int k = ld_k0 + 8 * g + ke_kk;
      int64_t col = ld_row + 4 * ke_mq;
      col = (col + 4 <= r1) ? col : r1 - 4;
      staged[g] = *(const f32x4*)(Ef + (int64_t)(k < d ? k : 0) * lde + col);
      return;
    }
    if (KQ && g >= 4) {
      const int k = ld_k0 + 16 * (g - 4) + kq_kk;
      staged[g] = *(const f32x4*)(Qk + (int64_t)(k < d ? k : 0) * ldq + kq_col);
      return;
    }
    if (g < 4) {
      int64_t er = ld_row + 64 * g;
      er = er < e_last ? er : e_last;
      row_ptr = Ef + er * lde;
    } else {
      row_ptr = q_ptr[g - 4];
    }
    if constexpr (VEC) {
      staged[g] = *(const f32x4*)(row_ptr + (ld_k < d ? ld_k : 0));
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) staged[g][j] = row_ptr[ld_k + j < d ? ld_k + j : 0];
    }
  };
  auto load_end = [&]() {
    const bool wrap = (ld_kc == nkc - 1);
    ld_kc = wrap ? 0 : ld_kc + 1;
    ld_row += wrap ? KS_TILE_ROWS : 0;
    st_valid = ld_valid;
    st_k0 = ld_k0;
  };
  // 8-byte half (s_piece & 1) of 16-byte piece (s_piece >> 1); rows 64 g + s_row share the swizzle of s_row
  const int st_off = s_row * 64 + ((((s_piece >> 1) ^ ((s_row >> 2) & 3)) << 4) | ((s_piece & 1) << 3));
  auto store_pass = [&](int buf, int g) {
    if ((KE && g < 4) || (KQ && g >= 4)) {
      const bool e_side = g < 4;
      const int kk = e_side ? 8 * g + ke_kk : 16 * (g - 4) + kq_kk, mq = e_side ? ke_mq : kq_mq;
      const int pitch = e_side ? 2 * KS_TILE_ROWS : 2 * KS_WG_QUERIES, plane = e_side ? KS_E_PLANE : KS_Q_PLANE;
      unsigned char* base = lds + buf * KS_STAGE_BYTES + (e_side ? 0 : 3 * KS_E_PLANE) + kk * pitch +
                            ((((mq >> 2) ^ (2 * (kk & 3))) << 5) | ((mq & 3) << 3));
      f32x4 v = staged[g];
      const bool live = st_k0 + kk < d;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = live ? v[j] : 0.f;
      bf16x4 s[3];
      split3_bf16x4(v, s);
#pragma unroll
      for (int part = 0; part < 3; ++part) *(bf16x4*)(base + part * plane) = s[part];
      return;
    }
    unsigned char* base = lds + buf * KS_STAGE_BYTES + st_off +
                          (g < 4 ? g * 4096 : 3 * KS_E_PLANE + (g - 4) * 4096);
    const int plane = g < 4 ? KS_E_PLANE : KS_Q_PLANE;
    f32x4 v = staged[g];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = (j < st_valid) ? v[j] : 0.f;
    bf16x4 s[3];
    split3_bf16x4(v, s);
#pragma unroll
    for (int part = 0; part < 3; ++part) *(bf16x4*)(base + part * plane) = s[part];
  };

  // fragment offsets of this lane inside a plane (row c of a 32-row tile), per K step of the chunk
  int foff[KS_KC / 16];
#pragma unroll
  for (int ks = 0; ks < KS_KC / 16; ++ks) foff[ks] = c * 64 + (((2 * ks + hf) ^ ((c >> 2) & 3)) << 4);
  // K-major planes: this lane's address inside a 32-row tile for the transposing reads of K step 0, first half (k rows
  // 8 hf + (lane % 16) / 4, rows 16 ((lane / 16) % 2) + 4 (lane % 4) ..); per row pitch: the tile's first segment is
  // added before the swizzle, so the two parts are kept apart
  const int tr_k = 8 * hf + ((lane & 15) >> 2);
  const int tr_seg = (lane >> 4) & 1, tr_in = (lane & 3) << 3;
  auto tr_fragment = [&](const unsigned char* plane_base, int pitch, int row0, int ks) -> bf16x8 {
    typedef __attribute__((ext_vector_type(4))) short s16x4;
    const int seg = ((row0 >> 4) + tr_seg) ^ (2 * (tr_k & 3));
    const unsigned char* p0 = plane_base + (16 * ks + tr_k) * pitch + (seg << 5) + tr_in;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p0));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p0 + 4 * pitch));
    typedef __attribute__((ext_vector_type(8))) short s16x8;
    return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int te = 0; te < 2; ++te)
#pragma unroll
    for (int tq = 0; tq < 2; ++tq)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[te][tq][i] = 0.f;

  if (n_it > 0) {
    load_begin();
#pragma unroll
    for (int g = 0; g < 6; ++g) load_pass(g);
    load_end();
    load_begin();
#pragma unroll
    for (int g = 0; g < 6; ++g) {
      store_pass(0, g);
      load_pass(g);  // past the last chunk the clamped addresses still point into the tables
    }
    load_end();
  }
  __syncthreads();
  int kc = 0;
  int64_t et0 = r0;
  for (int it = 0; it < n_it; ++it) {
    const int buf = it & 1;
    const unsigned char* be = lds + buf * KS_STAGE_BYTES + (64 * we) * 64;
    const unsigned char* bq = lds + buf * KS_STAGE_BYTES + 3 * KS_E_PLANE + (64 * wq) * 64;
    bf16x8 fe[2][3][2], fq[2][3][2];
    auto read_step = [&](int ks) {
#pragma unroll
      for (int part = 0; part < 3; ++part)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          if constexpr (KE)
            fe[ks][part][t] = tr_fragment(lds + buf * KS_STAGE_BYTES + part * KS_E_PLANE, 2 * KS_TILE_ROWS, 64 * we + 32 * t, ks);
          else
            fe[ks][part][t] = *(const bf16x8*)(be + part * KS_E_PLANE + t * 2048 + foff[ks]);
          if constexpr (KQ)
            fq[ks][part][t] = tr_fragment(lds + buf * KS_STAGE_BYTES + 3 * KS_E_PLANE + part * KS_Q_PLANE,
                                          2 * KS_WG_QUERIES, 64 * wq + 32 * t, ks);
          else
            fq[ks][part][t] = *(const bf16x8*)(bq + part * KS_Q_PLANE + t * 2048 + foff[ks]);
        }
    };
    // The iteration in six slices, fenced so that each keeps its share of the work: eight of the chunk's
    // 48 MFMAs, and the split + store of one staged pass of chunk it+1 followed by the load of that pass of
    // chunk it+2.  Unconditional on purpose (no branches inside the iteration): after the last chunk this
    // stores and loads a chunk nobody reads.
    read_step(0);
    load_begin();
#pragma unroll
    for (int sl = 0; sl < 6; ++sl) {
      if (sl == 2) read_step(1);
      store_pass(buf ^ 1, sl);
      load_pass(sl);
#pragma unroll
      for (int m = 8 * sl; m < 8 * sl + 8; ++m) {
        const int ks = m / 24, p = (m % 24) / 4, te = (m >> 1) & 1, tq = m & 1;
        acc[te][tq] = Epi::SWAP ? mfma_bf16(fq[ks][SPLIT_B[p]][tq], fe[ks][SPLIT_A[p]][te], acc[te][tq])
                                : mfma_bf16(fe[ks][SPLIT_A[p]][te], fq[ks][SPLIT_B[p]][tq], acc[te][tq]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    load_end();
    if (kc == nkc - 1) {  // this entity tile is complete
      float sc16[16];
#pragma unroll
      for (int te = 0; te < 2; ++te) {
        const int64_t e_base = et0 + 64 * we + 32 * te;
        if (e_base < r1) {
#pragma unroll
          for (int tq = 0; tq < 2; ++tq) epi.template tile<false>(tq, acc[te][tq], sc16, 1.f, e_base, r1);
        }
#pragma unroll
        for (int tq = 0; tq < 2; ++tq)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[te][tq][i] = 0.f;
      }
      kc = 0;
      et0 += KS_TILE_ROWS;
      if (Epi::STAGE_HOOK) epi.stage_mark();
      __syncthreads();
      if (Epi::STAGE_HOOK) epi.stage_end();
    } else {
      ++kc;
      __syncthreads();
    }
  }
  epi.finish();
}

template <template <int> class EpiT, bool VEC>
__global__ void __launch_bounds__(512, 2) ksplit_kernel(ContractArgs a, typename EpiT<KS_NQT>::Args ea) {
  ksplit_body<EpiT, VEC, 0>(a, ea);
}
// the same with K-major operands (KMAJ = 1: the entity operand, 3: both)
template <template <int> class EpiT, int KMAJ>
__global__ void __launch_bounds__(512, 2) ksplit_kmajor_kernel(ContractArgs a, typename EpiT<KS_NQT>::Args ea) {
  ksplit_body<EpiT, true, KMAJ>(a, ea);
}

// ============================================================================================
// kchunk_kernel: bf16 or per-row int8 table of any width (d % 8 == 0); used for d > 256, where the queries no
// longer fit the register file of the persistent kernels.  int8 rows are widened to bf16 (exactly) on the way into
// LDS and a finished tile's scores are multiplied by the row scales, as in the other int8 kernels.  The shape of ksplit_kernel with one part per operand:
// 256 entities x 128 queries per workgroup of 8 waves (64 x 64 per wave), K in chunks of 64, both operands
// staged through registers into double-buffered LDS (the fp32 queries are rounded to bf16 on the way, as in
// the other bf16 kernels), one MFMA per 32 x 32 x 16 block.  Reduction order per score: K ascending in steps of
// 16, as everywhere else.
//
// LDS row: 128 B = 8 pieces of 16 B (8 bf16); piece p of row r sits in slot r*8 + (p ^ (r & 7)).
// ============================================================================================
constexpr int KB_KC = 64;
constexpr int KB_E_PLANE = KS_TILE_ROWS * 128;
constexpr int KB_Q_PLANE = KS_WG_QUERIES * 128;
constexpr int KB_STAGE_BYTES = KB_E_PLANE + KB_Q_PLANE;

template <int EDT, template <int> class EpiT>
__global__ void __launch_bounds__(512, 2) kchunk_kernel(ContractArgs a, typename EpiT<KS_NQT>::Args ea) {
  static_assert(EDT == KGE_BF16 || EDT == KGE_I8, "bf16 or int8 rows");
  constexpr bool I8 = (EDT == KGE_I8);
  using Epi = EpiT<KS_NQT>;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * KB_STAGE_BYTES];

  int qg;
  int64_t chunk;
  if (!decompose_wg(a, qg, chunk)) return;
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int we = wave >> 1, wq = wave & 1;
  const int d = a.d;
  const int64_t q_base = (int64_t)qg * KS_WG_QUERIES;
  const int64_t q0 = q_base + 64 * wq;
  Epi epi;
  epi.init(ea, q0, c, hf, a.B);
  __shared__ typename Epi::Shared epi_sh;
  epi.bind(&epi_sh);

  const int64_t r0 = a.e_begin + chunk * a.chunk_rows;
  const int64_t r1 = (r0 + a.chunk_rows < a.e_end) ? r0 + a.chunk_rows : a.e_end;
  const int nkc = (d + KB_KC - 1) / KB_KC;
  const int n_et = (int)((r1 - r0 + KS_TILE_ROWS - 1) / KS_TILE_ROWS);
  const int n_it = n_et * nkc;
  const unsigned char* Eb = (const unsigned char*)a.E;
  constexpr int ESZ = I8 ? 1 : 2;  // bytes per table element

  // Staging (branch-free, clamped addresses, zeroing at store time): entity rows as pieces of 8 elements (16 bytes
  // of bf16, or 8 bytes of int8 that become 16 bytes of bf16 when stored),
  // 4 passes of 64 rows (8 lanes read one 128 B line); query rows as fp32, 4 passes of 32 rows (16 lanes read
  // 256 B of one row), rounded to bf16 when stored.
  const int e_row = tid >> 3, e_piece = tid & 7;
  const int q_row = tid >> 4, q_piece = tid & 15;  // q_piece: which 4 of the chunk's 64 columns
  const int64_t q_last = a.B - 1, e_last = r1 - 1;
  const float* q_ptr[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    int64_t qr = q_base + 32 * g + q_row;
    qr = qr < q_last ? qr : q_last;
    q_ptr[g] = a.Q + qr * d;
  }
  u32x4 se[4];
  f32x4 sq[4];
  bool st_e_ok = false, st_q_ok = false, ld_e_ok = false, ld_q_ok = false;
  bool st_tail = false, ld_tail = false;  // (uniform) the chunk reaches past d: only then is anything masked
  int ld_kc = 0;
  int64_t ld_row = r0 + e_row;
  // the rows of the entity tile being requested, as pointers: recomputed when the tile changes, not per chunk
  const unsigned char* e_ptr[4];
  auto tile_rows = [&]() {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      int64_t er = ld_row + 64 * g;
      er = er < e_last ? er : e_last;
      e_ptr[g] = Eb + er * d * ESZ;
    }
  };
  tile_rows();
  auto chunk_load = [&]() {
    const int ke = ld_kc * KB_KC + 8 * e_piece, kq = ld_kc * KB_KC + 4 * q_piece;
    ld_e_ok = ke < d;  // d % 8 == 0: a piece is inside d or outside as a whole
    ld_q_ok = kq < d;
    ld_tail = (ld_kc + 1) * KB_KC > d;
    const int e_col = (ld_e_ok ? ke : 0) * ESZ;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const unsigned char* src = e_ptr[g] + e_col;
      if (I8) {
        const u32x2 w = *(const u32x2*)src;
        se[g] = u32x4{w[0], w[1], 0u, 0u};
      } else {
        se[g] = *(const u32x4*)src;
      }
      sq[g] = *(const f32x4*)(q_ptr[g] + (ld_q_ok ? kq : 0));
    }
    if (ld_kc == nkc - 1) {  // (uniform)
      ld_kc = 0;
      ld_row += KS_TILE_ROWS;
      tile_rows();
    } else {
      ++ld_kc;
    }
  };
  const int e_off = e_row * 128 + ((e_piece ^ (e_row & 7)) << 4);
  const int q_off = q_row * 128 + ((((q_piece >> 1) ^ (q_row & 7)) << 4) | ((q_piece & 1) << 3));
  auto chunk_store = [&](int buf) {
    unsigned char* base = lds + buf * KB_STAGE_BYTES;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x4 v = I8 ? i8x8_to_bf16x8(se[g][0], se[g][1]) : se[g];
      f32x4 w = sq[g];
      if (__builtin_expect(st_tail, 0)) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = st_e_ok ? v[j] : 0u;
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = st_q_ok ? w[j] : 0.f;
      }
      *(u32x4*)(base + g * 8192 + e_off) = v;
      bf16x4 b;
      b[0] = (__bf16)w[0]; b[1] = (__bf16)w[1]; b[2] = (__bf16)w[2]; b[3] = (__bf16)w[3];
      *(bf16x4*)(base + KB_E_PLANE + g * 4096 + q_off) = b;
    }
  };

  int foff[KB_KC / 16];
#pragma unroll
  for (int ks = 0; ks < KB_KC / 16; ++ks) foff[ks] = c * 128 + (((2 * ks + hf) ^ (c & 7)) << 4);

  f32x16 acc[2][2];
#pragma unroll
  for (int te = 0; te < 2; ++te)
#pragma unroll
    for (int tq = 0; tq < 2; ++tq)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[te][tq][i] = 0.f;

  if (n_it > 0) {
    chunk_load();
    st_e_ok = ld_e_ok;
    st_q_ok = ld_q_ok;
    st_tail = ld_tail;
    chunk_store(0);
    chunk_load();  // past the last chunk the clamped addresses still point into the tables
  }
  __syncthreads();
  int kc = 0;
  int64_t et0 = r0;
  for (int it = 0; it < n_it; ++it) {
    const int buf = it & 1;
    // chunk it+1 (loaded during the previous iteration) goes to the other buffer, then chunk it+2 is requested
    st_e_ok = ld_e_ok;
    st_q_ok = ld_q_ok;
    st_tail = ld_tail;
    chunk_store(buf ^ 1);
    chunk_load();
    const unsigned char* be = lds + buf * KB_STAGE_BYTES + (64 * we) * 128;
    const unsigned char* bq = lds + buf * KB_STAGE_BYTES + KB_E_PLANE + (64 * wq) * 128;
    const int k_left = d - kc * KB_KC;
#pragma unroll
    for (int ks = 0; ks < KB_KC / 16; ++ks) {
      if (ks * 16 >= k_left) break;  // uniform: whole K steps past d are skipped, as in the other kernels
      bf16x8 fe[2], fq[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        fe[t] = *(const bf16x8*)(be + t * 4096 + foff[ks]);
        fq[t] = *(const bf16x8*)(bq + t * 4096 + foff[ks]);
      }
#pragma unroll
      for (int te = 0; te < 2; ++te)
#pragma unroll
        for (int tq = 0; tq < 2; ++tq)
          acc[te][tq] = Epi::SWAP ? mfma_bf16(fq[tq], fe[te], acc[te][tq]) : mfma_bf16(fe[te], fq[tq], acc[te][tq]);
    }
    if (kc == nkc - 1) {  // this entity tile is complete
      float sc16[16];
#pragma unroll
      for (int te = 0; te < 2; ++te) {
        const int64_t e_base = et0 + 64 * we + 32 * te;
        if (e_base < r1) {
          float sc_col = 1.f;
          if (I8) {  // the scales of the rows this lane holds (rows past the chunk's end: its last row's, ignored)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int64_t er = e_base + row_of(i, hf);
              sc16[i] = a.scale[er < e_last ? er : e_last];
            }
            const int64_t ec = e_base + c;
            sc_col = a.scale[ec < e_last ? ec : e_last];
          }
#pragma unroll
          for (int tq = 0; tq < 2; ++tq) epi.template tile<I8>(tq, acc[te][tq], sc16, sc_col, e_base, r1);
        }
#pragma unroll
        for (int tq = 0; tq < 2; ++tq)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[te][tq][i] = 0.f;
      }
      kc = 0;
      et0 += KS_TILE_ROWS;
      if (Epi::STAGE_HOOK) epi.stage_mark();
      __syncthreads();
      if (Epi::STAGE_HOOK) epi.stage_end();
    } else {
      ++kc;
      __syncthreads();
    }
  }
  epi.finish();
}

}  // namespace kge
