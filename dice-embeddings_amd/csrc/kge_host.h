// Host-side logic of the library that needs no GPU: argument rules, workspace layouts, the packed keys and
// counters the kernels exchange, and a sequential model of the kernel that plans the filter correction.
//
// Plain C++17 with no HIP dependency: hipcc includes it into the device library, and g++ builds it (with
// -fsanitize=address,undefined) into the CPU test driver tests/host_model_test.cpp, so that every layout and
// every packed field is exercised with bounds checks where there is no GPU.
#pragma once
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>

#include <vector>

#include "../../include/kge_hip.h"

#if defined(__HIPCC__)
#define KGE_HD __host__ __device__
#else
#define KGE_HD
#endif

namespace kge {
namespace host {

// ---- sizes shared by host and kernels -------------------------------------------------------------------
constexpr int SORT_MAX = 8192;           // queries per sub-batch of the filter correction
constexpr int WORK_MAX = 16 * SORT_MAX;  // upper bound on work items per sub-batch (bounds the slice count only)
constexpr int SLICE_MIN = 128;           // shortest slice of a filter row
constexpr int SLICE_PREF = 256;          // slices of a large sub-batch are at least this long (fewer, longer work items)
constexpr int SLICE_PREF_ITEMS = 4096;   // ... as long as that still leaves about this many work items
constexpr int PLAN_SLOTS = 2 * SORT_MAX; // hash table of the plan kernel: load factor <= 0.5
constexpr int PLAN_HASH_SHIFT = 18;      // 32 - log2(PLAN_SLOTS)
static_assert(PLAN_SLOTS == (1 << (32 - PLAN_HASH_SHIFT)), "hash width");
constexpr int TOPK_CAP = 4096;           // candidates a query can collect in one round
constexpr int TOPK_MAX_K = 1024;
constexpr int TOPK_FIRST_ROWS = 1024;    // first round takes everything: must not exceed TOPK_CAP
constexpr int BCE_SLOTS = 128;
constexpr int KS_WG_QUERIES = 128;       // workgroup shape of the fp32 contraction (also sizes the backward's K split)
constexpr int KS_TILE_ROWS = 256;

// Work decomposition of the four-tile filtered-rank main loop (bf16 tables, d == 128): 8-wave workgroups of
// 4 x 32 queries per wave, one per CU; the workgroups resident on one XCD (32) are shared out among the query
// groups; chunks of at most 512 rows (2442 chunks of 1024 rows over 64 workgroup lanes leave 39 to some lanes and
// 38 to others: 2 % of the launch idle at its end; at 512 it is under 1 %), at least 4 per workgroup.
constexpr int R128_WG_WAVES = 8;
constexpr int R128_WG_QUERIES = R128_WG_WAVES * 32 * 4;
constexpr int R128_MAX_CHUNK = 512;
inline void rank128_plan(int64_t B, int64_t rows, int* n_qgroups, int* n_lanes, int* chunk_rows, int64_t* n_chunks) {
  int g = (int)((B + R128_WG_QUERIES - 1) / R128_WG_QUERIES);
  if (g < 1) g = 1;
  int lanes = 32 / g;
  if (lanes < 1) lanes = 1;
  int64_t chunk = rows / (8 * (int64_t)lanes * 4);
  chunk = (chunk + 127) / 128 * 128;
  if (chunk < 128) chunk = 128;
  if (chunk > R128_MAX_CHUNK) chunk = R128_MAX_CHUNK;
  *n_qgroups = g;
  *n_lanes = lanes;
  *chunk_rows = (int)chunk;
  *n_chunks = (rows + chunk - 1) / chunk;
}

struct Status {
  int code = KGE_OK;
  char msg[256] = "";
  bool ok() const { return code == KGE_OK; }
};
#define KGE_HOST_FAIL(st, c, ...)                      \
  do {                                                 \
    (st).code = (c);                                   \
    snprintf((st).msg, sizeof((st).msg), __VA_ARGS__); \
    return (st);                                       \
  } while (0)

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// ---- argument rules of every contraction entry point ---------------------------------------------------
inline Status contract_rules(const char* who, const void* Q, const void* E, int dtype, const void* scale, int64_t B,
                             int64_t d, int64_t N) {
  Status st;
  if (!(B >= 0 && N >= 1)) KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: B=%lld N=%lld", who, (long long)B, (long long)N);
  if (N > 0x7fffffffLL) KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: N=%lld exceeds int32 entity ids", who, (long long)N);
  if (B > (1 << 24)) KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: B=%lld exceeds 2^24", who, (long long)B);
  if (!(B == 0 || (Q && E))) KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: null Q or E", who);
  if ((((uintptr_t)Q | (uintptr_t)E) & 15) != 0)
    KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: Q and E must be 16-byte aligned", who);
  switch (dtype) {
    case KGE_F32:
      if (!(d >= 1 && d <= 65536)) KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: d=%lld", who, (long long)d);
      break;
    case KGE_BF16:
      if (!(d >= 8 && d % 8 == 0))
        KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: bf16 tables need d %% 8 == 0, got %lld", who, (long long)d);
      if (d > 65536) KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: d=%lld", who, (long long)d);
      break;
    case KGE_I8:
      if (!(d >= 16 && d % 16 == 0))
        KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: int8 tables need d %% 16 == 0, got %lld", who, (long long)d);
      if (d > 65536) KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: d=%lld", who, (long long)d);
      if (!scale) KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: int8 tables need per-row scales", who);
      break;
    default: KGE_HOST_FAIL(st, KGE_ERR_INVALID, "%s: unknown dtype %d", who, dtype);
  }
  return st;
}

// ---- workspace layouts ------------------------------------------------------------------------------------
// thresholds [B]; per query the leader of its filter group (`lead`, -1: none) and per leader whether its group holds
// different query vectors (`mixed`); then one plan (member keys, group ends, group records, 4 counters) per
// sub-batch of SORT_MAX queries
struct RankWsOffsets {
  size_t thr, lead, mixed, plans, total;
  size_t plan_stride, skey, gend, work, meta;  // of one plan: stride between plans, offsets inside a plan
  int64_t n_plans;
};
inline RankWsOffsets rank_ws_offsets(int64_t B) {
  RankWsOffsets o{};
  size_t off = 0;
  auto take = [&](size_t bytes) {
    const size_t at = off;
    off = align_up(off + bytes, 256);
    return at;
  };
  o.n_plans = (B + SORT_MAX - 1) / SORT_MAX;
  if (o.n_plans < 1) o.n_plans = 1;
  o.thr = take((size_t)B * 4);
  o.lead = take((size_t)B * 4);
  o.mixed = take((size_t)B * 4);
  o.plans = off;
  o.skey = 0;
  o.gend = align_up((size_t)SORT_MAX * 8, 256);
  o.work = o.gend + align_up((size_t)SORT_MAX * 4, 256);
  o.meta = o.work + align_up((size_t)SORT_MAX * 8, 256);
  o.plan_stride = o.meta + 256;
  o.total = o.plans + (size_t)o.n_plans * o.plan_stride;
  return o;
}

// tau: k-th best score per query (kth: the k-th best as a packed key, 0 while fewer than k are known); tau_scan: the threshold the next scan admits candidates with (tau, or a tighter
// guess that the selection verifies); list: the best k so far as packed keys; cand: this round's candidates as packed
// keys; cand_id: this round's candidates as entity ids (int8 filter scan, scored exactly before they are ranked);
// requant: the int8 table written again with one scale per 32-row tile, N x 128 bytes, and rowmeta: one
// TOPK_ROWMETA_BYTES record per TOPK_ROWMETA_ROWS table rows (both for the int8 filter scan)
constexpr int TOPK_ROWMETA_ROWS = 64;
constexpr int TOPK_ROWMETA_BYTES = 32;  // per 32-row tile {scale (negative: forced), max |e'|_2, max |rho|_2, 1 / scale}
constexpr int TOPK_REQUANT_D = 128;
constexpr int64_t TOPK_FILTER_MIN_ROWS = 65536;  // rounds of at most this many rows skip the int8 filter scan
// qh / qc: the queries as the int8 filter scan reads them (TOPK_REQUANT_D int8 per query, and per query the four
// constants of its bound), written once per call.
struct TopkWsOffsets {
  size_t tau, tau_scan, cnt, list_len, dirty, n_dirty, kth, list, cand, cand_id, qh, qc, rowmeta, requant, total;
  int64_t kpad;
};
// the prepared form of an int8 table (what kge_topk_prepare writes): rowmeta records, then the requantised rows
struct TopkPreparedOffsets {
  size_t rowmeta, requant, total;
};
inline TopkPreparedOffsets topk_prepared_offsets(int64_t N) {
  TopkPreparedOffsets o{};
  o.rowmeta = 0;
  o.requant = align_up((size_t)((N + TOPK_ROWMETA_ROWS - 1) / TOPK_ROWMETA_ROWS) * TOPK_ROWMETA_BYTES, 256);
  o.total = o.requant + align_up((size_t)N * TOPK_REQUANT_D, 256);
  return o;
}
// with_table: the workspace also holds the prepared form of the table (a call that was not handed one)
inline TopkWsOffsets topk_ws_offsets(int64_t B, int64_t N, int64_t k, bool with_table = true) {
  TopkWsOffsets o{};
  size_t off = 0;
  auto take = [&](size_t bytes) {
    const size_t at = off;
    off = align_up(off + bytes, 256);
    return at;
  };
  o.kpad = (k + 7) / 8 * 8;
  o.tau = take((size_t)B * 4);
  o.tau_scan = take((size_t)B * 4);
  o.cnt = take((size_t)B * 4);
  o.list_len = take((size_t)B * 4);
  o.dirty = take((size_t)B * 4);
  o.n_dirty = take(4);
  o.kth = take((size_t)B * 8);
  o.list = take((size_t)B * (size_t)o.kpad * 8);
  o.cand = take((size_t)B * TOPK_CAP * 8);
  o.cand_id = take((size_t)B * TOPK_CAP * 4);
  o.qh = take((size_t)B * TOPK_REQUANT_D);
  o.qc = take((size_t)B * 16);
  if (with_table) {
    const TopkPreparedOffsets t = topk_prepared_offsets(N);
    const size_t base = take(t.total);
    o.rowmeta = base + t.rowmeta;
    o.requant = base + t.requant;
  } else {
    o.rowmeta = o.requant = off;
  }
  o.total = off;
  return o;
}

// The threshold a scan of `n_next` more rows may use once `ranked` rows are ranked: the j-th best score so far, j as
// small as the order statistics allow.  Of the best k of all ranked + n_next rows, the number X that are among
// the rows already ranked is hypergeometric (rows in exchangeable order), mean k rho, variance below
// k rho (1 - rho), rho = ranked / (ranked + n_next); the j-th best so far is below the final k-th best whenever
// j > X.  Five standard deviations: a query in a few million falls short (the selection notices, and the query is
// scanned again with its k-th best).
inline int64_t topk_speculative_rank(int64_t k, int64_t ranked, int64_t n_next) {
  if (n_next <= 0 || ranked <= 0) return k;
  const double rho = (double)ranked / ((double)ranked + (double)n_next);
  const double mean = (double)k * rho, var = (double)k * rho * (1.0 - rho);
  double sd = 0.0;
  for (double lo = 0.0, hi = var + 1.0; hi - lo > 1e-9;) {  // sqrt without <cmath>: bisection on [0, var + 1]
    sd = 0.5 * (lo + hi);
    if (sd * sd < var) lo = sd; else hi = sd;
  }
  int64_t j = (int64_t)(mean + 5.0 * sd) + 2;
  if (j < 1) j = 1;
  return j < k ? j : k;
}

// how many times the ranked prefix grows per round of kge_topk.  Larger factors were measured and are no faster,
// with or without the guessed thresholds: every round costs a launch of the persistent scan, a selection and the gaps
// between them, but a scan with a looser threshold spends more time in its slow paths and hands more candidates to
// the selection (k = 100, N = 10M through the int8 filter: x4 11.9 ms, x8 12.1, x16 12.7 per call; k = 10, N = 2.5M,
// bf16: x4 3.00 ms, x8 3.04, x16 3.03).
inline int64_t topk_growth(int64_t k) { return k <= 256 ? 4 : 2; }

constexpr int BCE_POS_SLOTS = 128;  // partial sums over the positives (one atomic per workgroup, spread)
inline size_t bce_ws_bytes() { return (2 * BCE_SLOTS + BCE_POS_SLOTS) * sizeof(double) + 128; }

struct BwdPlan {
  int64_t ldG, ldT;  // row strides of G [B, ldG] (a multiple of 32) and GT [N, ldT] (a multiple of 4)
  int k_splits, k_split_len;
  bool kmajor;  // d a multiple of 4: the gradient contractions read G, E and Q where they lie (no GT, ET, QT)
  size_t off_G, off_GT, off_ET, off_QT, off_part, total;
};
inline BwdPlan bwd_plan(int64_t B, int64_t d, int64_t N) {
  BwdPlan p{};
  p.ldG = (N + 31) / 32 * 32;  // rows start on 128-byte lines: a wave's run of 32 gradients is one whole line
  p.ldT = (B + 3) / 4 * 4;
  // dQ = G . E sums over N: split so that about 256 workgroups run
  const int64_t tiles = ((B + KS_WG_QUERIES - 1) / KS_WG_QUERIES) * ((d + KS_TILE_ROWS - 1) / KS_TILE_ROWS);
  int64_t splits = (256 + tiles - 1) / tiles;
  if (splits > 64) splits = 64;
  if (splits < 1) splits = 1;
  const int64_t len = ((N + splits - 1) / splits + 31) / 32 * 32;
  p.k_split_len = (int)len;
  p.k_splits = (int)((N + len - 1) / len);
  auto up = [](size_t x) { return (x + 255) / 256 * 256; };
  size_t off = up(bce_ws_bytes());
  p.off_G = off;     off += up((size_t)B * p.ldG * sizeof(float));
  p.kmajor = d % 4 == 0;
  p.off_GT = off;    off += p.kmajor ? 0 : up((size_t)N * p.ldT * sizeof(float));
  p.off_ET = off;    off += p.kmajor ? 0 : up((size_t)d * p.ldG * sizeof(float));
  p.off_QT = off;    off += p.kmajor ? 0 : up((size_t)d * p.ldT * sizeof(float));
  p.off_part = off;  off += up((size_t)p.k_splits * B * d * sizeof(float));
  p.total = off;
  return p;
}

// ---- vocabulary keys: ((a * range_b + b) << vbits) | v ----------------------------------------------------
KGE_HD inline int bits_for(int64_t range) {  // bits needed for values in [0, range)
  int b = 1;
  while (b < 63 && (1LL << b) < range) ++b;
  return b;
}
struct CsrKeyLayout {
  int vbits, key_bits;
  bool fits;                   // key_bits <= 62: room for the `invalid` marker one bit above every valid key
  unsigned long long invalid;  // key of a triple with an id outside its range (sorts last)
};
KGE_HD inline CsrKeyLayout csr_key_layout(int64_t range_a, int64_t range_b, int64_t range_v) {
  CsrKeyLayout l;
  l.vbits = bits_for(range_v);
  l.key_bits = bits_for(range_a) + bits_for(range_b) + l.vbits;  // a * range_b + b < 2^(bits_a + bits_b)
  l.fits = l.key_bits <= 62;
  l.invalid = l.fits ? 1ull << l.key_bits : 0ull;
  return l;
}
KGE_HD inline unsigned long long csr_pack_key(int64_t a, int64_t b, int64_t v, int64_t range_b, int vbits) {
  return ((unsigned long long)(a * range_b + b) << vbits) | (unsigned long long)v;
}
inline Status csr_build_rules(int64_t n, int col_a, int col_b, int col_v, int64_t range_a, int64_t range_b,
                              int64_t range_v) {
  Status st;
  if (!(n >= 0 && n < (1LL << 31))) KGE_HOST_FAIL(st, KGE_ERR_INVALID, "kge_csr_build: n=%lld outside [0, 2^31)", (long long)n);
  if (!(col_a >= 0 && col_a < 3 && col_b >= 0 && col_b < 3 && col_v >= 0 && col_v < 3 && col_a != col_b &&
        col_a != col_v && col_b != col_v))
    KGE_HOST_FAIL(st, KGE_ERR_INVALID, "kge_csr_build: columns (%d, %d, %d) are not a permutation of 0..2", col_a, col_b,
                  col_v);
  if (!(range_a >= 1 && range_b >= 1 && range_v >= 1 && range_v <= (1LL << 31)))
    KGE_HOST_FAIL(st, KGE_ERR_INVALID, "kge_csr_build: ranges (%lld, %lld, %lld) must be positive and values fit int32",
                  (long long)range_a, (long long)range_b, (long long)range_v);
  if (!csr_key_layout(range_a, range_b, range_v).fits)
    KGE_HOST_FAIL(st, KGE_ERR_UNSUPPORTED, "kge_csr_build: (%lld x %lld) pairs x %lld values do not fit a 62-bit key",
                  (long long)range_a, (long long)range_b, (long long)range_v);
  return st;
}

// ---- the plan of the filter correction --------------------------------------------------------------------
// A sub-batch of at most SORT_MAX queries is grouped by filter row; every group's row is cut into slices of
// `slice` entries, one work item each.  One exclusive scan over the group leaders carries three counters in
// one 64-bit word: groups (bits 48..63), members (bits 32..47), slices (bits 0..31).  All three stay inside
// their fields: at most SORT_MAX groups and members, and at most WORK_MAX slices (plan_slice_length).
KGE_HD inline uint32_t plan_hash(int64_t row) { return ((uint32_t)row * 2654435761u) >> PLAN_HASH_SHIFT; }
KGE_HD inline unsigned long long plan_pack(unsigned long long members, unsigned long long slices) {
  return (1ull << 48) | (members << 32) | slices;
}
KGE_HD inline int plan_groups(unsigned long long v) { return (int)(v >> 48); }
KGE_HD inline int plan_members(unsigned long long v) { return (int)((v >> 32) & 0xffffull); }
KGE_HD inline unsigned int plan_slices(unsigned long long v) { return (unsigned int)(v & 0xffffffffull); }
// slice length for a sub-batch whose groups' rows hold `total` entries together: at least SLICE_MIN, a multiple
// of 32, and long enough that sum over groups of ceil(len / slice) <= total / slice + SORT_MAX <= WORK_MAX
KGE_HD inline int plan_slice_length(unsigned long long total) {
  const unsigned long long room = (unsigned long long)(WORK_MAX - SORT_MAX);
  unsigned long long sl = (total + room - 1) / room;
  sl = (sl + 31) & ~31ull;
  if (sl < (unsigned long long)SLICE_MIN) sl = SLICE_MIN;
  // a work item costs a chain of dependent loads whatever its length: a sub-batch with plenty of entries takes longer
  // slices (measured at 1.5M entries per 4096 queries: 142 -> 125 us with 256 instead of 128), a small one keeps
  // short slices so that its few entries still spread over the chip (50k entries per 1024 queries: 32 -> 37 us at 256)
  unsigned long long pref = ((total / SLICE_PREF_ITEMS) + 31) & ~31ull;
  if (pref > (unsigned long long)SLICE_PREF) pref = SLICE_PREF;
  if (sl < pref) sl = pref;
  return (int)(sl > 0x7fffffe0ull ? 0x7fffffe0ull : sl);
}
// member key of the plan: filter row << 24 | position of the query in its sub-batch
KGE_HD inline unsigned long long plan_member_key(int64_t row, int pos_in_batch) {
  return ((unsigned long long)row << 24) | (unsigned long long)pos_in_batch;
}
KGE_HD inline int64_t plan_key_row(unsigned long long key) { return (int64_t)(key >> 24); }
KGE_HD inline int plan_key_pos(unsigned long long key) { return (int)(key & 0xffffffull); }

// What plan_fix_kernel writes, computed sequentially in the kernel's own order (thread t owns the queries
// t, t + 1024, ...; the scan runs over threads, then over a thread's queries).  Every index and every packed
// field is checked; `error` names the first violation.
struct PlanModel {
  std::vector<unsigned long long> skey;
  std::vector<int32_t> gend, work;
  int32_t meta[3] = {0, 0, 0};
  const char* error = nullptr;
};
inline PlanModel plan_fix_model(const int64_t* csr_row, int nb, int64_t n_rows, const int64_t* row_ptr) {
  PlanModel m;
  m.skey.assign(SORT_MAX, ~0ull);
  m.gend.assign(SORT_MAX, -1);
  m.work.assign(2 * SORT_MAX, -1);
  auto fail = [&](const char* what) {
    if (!m.error) m.error = what;
  };
  if (nb < 0 || nb > SORT_MAX) {
    fail("sub-batch larger than SORT_MAX");
    return m;
  }
  constexpr int THREADS = 1024, QPT = SORT_MAX / THREADS;
  std::vector<int32_t> tab_row(PLAN_SLOTS, 0), tab_cnt(PLAN_SLOTS, 0);
  std::vector<int64_t> my_row(SORT_MAX, -1), len(SORT_MAX, 0);
  std::vector<int> my_slot(SORT_MAX, -1), my_pos(SORT_MAX, -1);
  for (int i = 0; i < nb; ++i) {
    const int64_t r = csr_row[i];
    my_row[i] = (r >= 0 && r < n_rows) ? r : -1;
  }
  // (1) claim slots, take tickets (any interleaving of the threads gives the same groups; tickets differ)
  for (int i = 0; i < nb; ++i) {
    if (my_row[i] < 0) continue;
    if (my_row[i] + 1 > 0x7fffffffLL) fail("filter row + 1 does not fit the 32-bit slot key");
    const int32_t key = (int32_t)my_row[i] + 1;
    uint32_t h = plan_hash(my_row[i]);
    int probes = 0;
    for (;;) {
      if (h >= (uint32_t)PLAN_SLOTS) fail("hash outside the table");
      if (tab_row[h] == 0) tab_row[h] = key;
      if (tab_row[h] == key) break;
      h = (h + 1) & (PLAN_SLOTS - 1);
      if (++probes > PLAN_SLOTS) {
        fail("hash table full");
        return m;
      }
    }
    my_slot[i] = (int)h;
    my_pos[i] = tab_cnt[h]++;
  }
  unsigned long long total = 0;
  for (int i = 0; i < nb; ++i)
    if (my_pos[i] == 0) {
      const int64_t l = row_ptr[my_row[i] + 1] - row_ptr[my_row[i]];
      if (l < 0) fail("row_ptr not ascending");
      len[i] = l;
      total += (unsigned long long)l;
    }
  // (2) slice length
  const int slice = plan_slice_length(total);
  if (slice < SLICE_MIN || slice % 32 != 0) fail("slice length");
  // (3) exclusive scan of the packed counters in the kernel's order
  unsigned long long base = 0;
  for (int t = 0; t < THREADS; ++t)
    for (int j = 0; j < QPT; ++j) {
      const int i = t + THREADS * j;
      if (i >= nb || my_pos[i] != 0) continue;
      const unsigned long long n = (unsigned long long)((len[i] + slice - 1) / slice);
      if (n == 0) {
        tab_cnt[my_slot[i]] = -1;  // empty filter row: nothing to take out for this group
        continue;
      }
      if (n > 0xffffffffull) fail("slices of one group overflow 32 bits");
      const unsigned long long members = (unsigned long long)tab_cnt[my_slot[i]];
      if (members > 0xffffull) fail("members of one group overflow their 16-bit field");
      const unsigned long long val = plan_pack(members, n);
      const int g = plan_groups(base), first = plan_members(base);
      if (g < 0 || g >= SORT_MAX) fail("group index outside the plan");
      if (first < 0 || first + (int)members > SORT_MAX) fail("member positions outside the plan");
      if (m.error) return m;
      m.work[2 * g] = first;
      m.work[2 * g + 1] = (int32_t)plan_slices(base);
      m.gend[first] = first + (int)members;
      tab_cnt[my_slot[i]] = first;
      const unsigned long long next = base + val;
      if (plan_groups(next) != g + 1 || plan_members(next) != first + (int)members ||
          (unsigned long long)plan_slices(next) != (unsigned long long)plan_slices(base) + n)
        fail("a packed counter carried into its neighbour");
      base = next;
    }
  m.meta[0] = (int32_t)plan_slices(base);
  m.meta[1] = slice;
  m.meta[2] = plan_groups(base);
  if ((unsigned long long)plan_slices(base) > (unsigned long long)WORK_MAX) fail("more work items than WORK_MAX");
  // (4) members to their positions
  for (int i = 0; i < nb; ++i) {
    if (my_slot[i] < 0) continue;
    const int first = tab_cnt[my_slot[i]];
    if (first < 0) continue;
    const int at = first + my_pos[i];
    if (at < 0 || at >= SORT_MAX) {
      fail("member written outside the plan");
      return m;
    }
    m.skey[at] = plan_member_key(my_row[i], i);
    if (plan_key_row(m.skey[at]) != my_row[i] || plan_key_pos(m.skey[at]) != i) fail("member key does not round-trip");
  }
  return m;
}

}  // namespace host
}  // namespace kge
