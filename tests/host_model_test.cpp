// CPU test driver of the library's host logic (dice-embeddings_amd/csrc/kge_host.h), built by
// tests/test_host_logic.py with g++ -fsanitize=address,undefined.  No GPU, no HIP.
//
// Covers: argument rules, workspace layouts (disjoint, aligned, inside the reported size), vocabulary key packing,
// and the sequential model of the filter-correction plan on the cases that stress its packed fields.
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <array>
#include <tuple>
#include <map>
#include <random>
#include <set>

#include "../dice-embeddings_amd/csrc/kge_host.h"

using namespace kge::host;

static int g_checks = 0;
#define CHECK(cond)                                                      \
  do {                                                                   \
    ++g_checks;                                                          \
    if (!(cond)) {                                                       \
      fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);  \
      exit(1);                                                           \
    }                                                                    \
  } while (0)

static void test_contract_rules() {
  alignas(16) static float buf[64];
  CHECK(contract_rules("t", buf, buf, KGE_F32, nullptr, 4, 7, 10).ok());
  CHECK(contract_rules("t", buf, buf, KGE_F32, nullptr, 0, 1, 1).ok());
  CHECK(contract_rules("t", nullptr, nullptr, KGE_F32, nullptr, 0, 1, 1).ok());           // empty batch: no pointers needed
  CHECK(contract_rules("t", nullptr, buf, KGE_F32, nullptr, 1, 1, 1).code == KGE_ERR_INVALID);
  CHECK(contract_rules("t", buf, buf, KGE_F32, nullptr, 1, 0, 1).code == KGE_ERR_INVALID);
  CHECK(contract_rules("t", buf, buf, KGE_F32, nullptr, 1, 8, 0).code == KGE_ERR_INVALID);
  CHECK(contract_rules("t", buf, buf, KGE_F32, nullptr, -1, 8, 5).code == KGE_ERR_INVALID);
  CHECK(contract_rules("t", buf, buf, KGE_F32, nullptr, 1, 8, 1LL << 31).code == KGE_ERR_INVALID);
  CHECK(contract_rules("t", buf, buf, KGE_F32, nullptr, (1 << 24) + 1, 8, 5).code == KGE_ERR_INVALID);
  CHECK(contract_rules("t", buf + 1, buf, KGE_F32, nullptr, 1, 8, 5).code == KGE_ERR_INVALID);   // misaligned
  CHECK(contract_rules("t", buf, buf, KGE_BF16, nullptr, 1, 12, 5).code == KGE_ERR_INVALID);
  CHECK(contract_rules("t", buf, buf, KGE_BF16, nullptr, 1, 136, 5).ok());
  CHECK(contract_rules("t", buf, buf, KGE_I8, buf, 1, 128, 5).ok());
  CHECK(contract_rules("t", buf, buf, KGE_I8, nullptr, 1, 128, 5).code == KGE_ERR_INVALID);
  CHECK(contract_rules("t", buf, buf, KGE_I8, buf, 1, 144, 5).ok());
  CHECK(contract_rules("t", buf, buf, KGE_I8, buf, 1, 65552, 5).code == KGE_ERR_INVALID);
  CHECK(contract_rules("t", buf, buf, KGE_I8, buf, 1, 24, 5).code == KGE_ERR_INVALID);
  CHECK(contract_rules("t", buf, buf, 7, nullptr, 1, 8, 5).code == KGE_ERR_INVALID);
  const Status st = contract_rules("kge_scores", buf, buf, KGE_BF16, nullptr, 1, 12, 5);
  CHECK(strstr(st.msg, "kge_scores") && strstr(st.msg, "12"));
}

static void check_disjoint(std::vector<std::pair<size_t, size_t>> parts, size_t total) {
  std::sort(parts.begin(), parts.end());
  size_t end = 0;
  for (auto& p : parts) {
    CHECK(p.first % 256 == 0);
    CHECK(p.first >= end);
    end = p.first + p.second;
  }
  CHECK(end <= total);
}

static void test_layouts() {
  for (int64_t B : {1LL, 2LL, 63LL, 4096LL, 8192LL, 8193LL, 65536LL, (1LL << 24)}) {
    const RankWsOffsets r = rank_ws_offsets(B);
    std::vector<std::pair<size_t, size_t>> parts = {{r.thr, (size_t)B * 4}, {r.lead, (size_t)B * 4}, {r.mixed, (size_t)B * 4}};
    CHECK(r.n_plans * (int64_t)SORT_MAX >= B && (r.n_plans - 1) * (int64_t)SORT_MAX < std::max<int64_t>(B, 1));
    for (int64_t s = 0; s < r.n_plans; ++s) {
      const size_t base = r.plans + (size_t)s * r.plan_stride;
      parts.push_back({base + r.skey, (size_t)SORT_MAX * 8});
      parts.push_back({base + r.gend, (size_t)SORT_MAX * 4});
      parts.push_back({base + r.work, (size_t)SORT_MAX * 8});
      parts.push_back({base + r.meta, 16});
    }
    check_disjoint(parts, r.total);
    for (int64_t k : {1LL, 7LL, 8LL, 100LL, 1024LL}) {
      for (int64_t N : {1LL, 63LL, 64LL, 65LL, 10000000LL}) {
        const TopkWsOffsets t = topk_ws_offsets(B, N, k);
        CHECK(t.kpad >= k && t.kpad % 8 == 0 && t.kpad < k + 8);
        const size_t n_rec = (size_t)((N + TOPK_ROWMETA_ROWS - 1) / TOPK_ROWMETA_ROWS);
        CHECK((int64_t)n_rec * TOPK_ROWMETA_ROWS >= N);
        check_disjoint({{t.tau, (size_t)B * 4}, {t.tau_scan, (size_t)B * 4}, {t.cnt, (size_t)B * 4},
                        {t.list_len, (size_t)B * 4}, {t.dirty, (size_t)B * 4}, {t.n_dirty, 4}, {t.kth, (size_t)B * 8},
                        {t.list, (size_t)B * t.kpad * 8}, {t.cand, (size_t)B * TOPK_CAP * 8},
                        {t.cand_id, (size_t)B * TOPK_CAP * 4}, {t.qh, (size_t)B * TOPK_REQUANT_D},
                        {t.qc, (size_t)B * 16}, {t.rowmeta, n_rec * TOPK_ROWMETA_BYTES},
                        {t.requant, (size_t)N * TOPK_REQUANT_D}}, t.total);
        // a call that is handed the prepared table keeps none in its workspace
        const TopkWsOffsets u = topk_ws_offsets(B, N, k, false);
        CHECK(u.total <= t.total && u.qc + (size_t)B * 16 <= u.total && u.qh == t.qh && u.cand_id == t.cand_id);
        const TopkPreparedOffsets pr = topk_prepared_offsets(N);
        check_disjoint({{pr.rowmeta, n_rec * TOPK_ROWMETA_BYTES}, {pr.requant, (size_t)N * TOPK_REQUANT_D}}, pr.total);
        CHECK(t.total - u.total >= pr.total);
      }
    }
  }
  // the rank whose score a scan may use as its threshold: between the expected number of survivors and k
  for (int64_t k : {1LL, 10LL, 100LL, 1000LL}) {
    CHECK(topk_speculative_rank(k, 0, 1000) == k && topk_speculative_rank(k, 1000, 0) == k);
    int64_t prev = 0;
    for (int64_t ranked : {1024LL, 4096LL, 1LL << 20}) {
      const int64_t j = topk_speculative_rank(k, ranked, 3 * ranked);
      CHECK(j >= 1 && j <= k && 4 * j >= k);             // never below the mean k / 4
      CHECK(prev == 0 || j == prev);                     // depends on the ratio only
      prev = j;
    }
    CHECK(topk_speculative_rank(k, 1 << 20, 1) == k || k > 20);   // almost nothing left to scan: nearly all survive
  }
  CHECK(topk_speculative_rank(100, 4096, 3 * 4096) == 48);        // 25 + 5 sqrt(18.75) = 46.65 -> 48
  // the static scratch array of kge_rank_filtered_static holds the layout of its largest batch
  CHECK(rank_ws_offsets(KGE_RANK_STATIC_MAX_B).total <= KGE_RANK_STATIC_SCRATCH_BYTES);
  CHECK(TOPK_FIRST_ROWS <= TOPK_CAP);
  for (auto bdn : {std::array<int64_t, 3>{1, 1, 1}, {2048, 256, 40943}, {5, 7, 3}, {4096, 128, 1 << 24}}) {
    const BwdPlan p = bwd_plan(bdn[0], bdn[1], bdn[2]);
    CHECK(p.ldG % 4 == 0 && p.ldG >= bdn[2] && p.ldT % 4 == 0 && p.ldT >= bdn[0]);
    CHECK(p.k_splits >= 1 && p.k_splits <= 64 && p.k_split_len % 32 == 0);
    CHECK((int64_t)p.k_splits * p.k_split_len >= bdn[2]);                       // the splits cover the summed index
    CHECK((int64_t)(p.k_splits - 1) * p.k_split_len < bdn[2]);                  // and none of them is empty
    // the transposed copies exist only where the contractions cannot read G, E and Q in place (d not a multiple of 4)
    CHECK(p.kmajor == (bdn[1] % 4 == 0));
    const size_t copies = p.kmajor ? 0 : 1;
    check_disjoint({{0, bce_ws_bytes()}, {p.off_G, (size_t)bdn[0] * p.ldG * 4},
                    {p.off_GT, copies * bdn[2] * p.ldT * 4}, {p.off_ET, copies * bdn[1] * p.ldG * 4},
                    {p.off_QT, copies * bdn[1] * p.ldT * 4}, {p.off_part, (size_t)p.k_splits * bdn[0] * bdn[1] * 4}},
                   p.total);
  }
}

static void test_csr_keys() {
  CHECK(bits_for(1) == 1 && bits_for(2) == 1 && bits_for(3) == 2 && bits_for(1LL << 31) == 31 && bits_for((1LL << 31) + 1) == 32);
  std::mt19937_64 rng(7);
  for (auto r : {std::array<int64_t, 3>{135, 46, 135}, {2500000, 37, 2500000}, {1, 1, 1}, {1LL << 20, 1LL << 20, 1LL << 22}}) {
    const CsrKeyLayout l = csr_key_layout(r[0], r[1], r[2]);
    CHECK(l.fits);
    unsigned long long largest = csr_pack_key(r[0] - 1, r[1] - 1, r[2] - 1, r[1], l.vbits);
    CHECK(largest < l.invalid);                                                  // `invalid` sorts after every valid key
    for (int it = 0; it < 200; ++it) {
      const int64_t a = rng() % r[0], b = rng() % r[1], v = rng() % r[2];
      const unsigned long long k = csr_pack_key(a, b, v, r[1], l.vbits);
      CHECK((int64_t)(k & ((1ull << l.vbits) - 1)) == v);
      CHECK((int64_t)(k >> l.vbits) == a * r[1] + b);
      // order of keys = order of (a, b, v)
      const int64_t a2 = rng() % r[0], b2 = rng() % r[1], v2 = rng() % r[2];
      const unsigned long long k2 = csr_pack_key(a2, b2, v2, r[1], l.vbits);
      CHECK((k < k2) == (std::make_tuple(a, b, v) < std::make_tuple(a2, b2, v2)));
    }
  }
  CHECK(!csr_key_layout(1LL << 31, 1LL << 31, 2).fits);
  CHECK(csr_build_rules(10, 0, 1, 2, 5, 5, 5).ok());
  CHECK(csr_build_rules(10, 0, 0, 2, 5, 5, 5).code == KGE_ERR_INVALID);
  CHECK(csr_build_rules(10, 0, 1, 2, 1LL << 31, 1LL << 31, 2).code == KGE_ERR_UNSUPPORTED);
  CHECK(csr_build_rules(1LL << 31, 0, 1, 2, 5, 5, 5).code == KGE_ERR_INVALID);
  CHECK(csr_build_rules(10, 0, 1, 2, 5, 5, (1LL << 31) + 1).code == KGE_ERR_INVALID);
}

// the plan must partition the queries with a filter row into groups of equal row, positions contiguous, and the
// work list must cover every slice of every group exactly once
static void check_plan(const std::vector<int64_t>& csr_row, int64_t n_rows, const std::vector<int64_t>& row_ptr) {
  const int nb = (int)csr_row.size();
  const PlanModel m = plan_fix_model(csr_row.data(), nb, n_rows, row_ptr.data());
  if (m.error) fprintf(stderr, "plan model: %s\n", m.error);
  CHECK(m.error == nullptr);
  const int n_work = m.meta[0], slice = m.meta[1], n_groups = m.meta[2];
  CHECK(slice >= SLICE_MIN && slice % 32 == 0 && n_work >= 0 && n_work <= WORK_MAX && n_groups >= 0 && n_groups <= SORT_MAX);
  std::map<int64_t, std::set<int>> want;  // filter row -> queries, rows with entries only
  for (int i = 0; i < nb; ++i) {
    const int64_t r = csr_row[i];
    if (r >= 0 && r < n_rows && row_ptr[r + 1] > row_ptr[r]) want[r].insert(i);
  }
  CHECK((int)want.size() == n_groups);
  long long work_seen = 0;
  std::set<int64_t> rows_seen;
  int members_seen = 0;
  for (int g = 0; g < n_groups; ++g) {
    const int first = m.work[2 * g], w0 = m.work[2 * g + 1];
    CHECK(first >= 0 && first < SORT_MAX && w0 == work_seen);
    const int end = m.gend[first];
    CHECK(end > first && end <= SORT_MAX);
    const int64_t row = plan_key_row(m.skey[first]);
    CHECK(want.count(row) && rows_seen.insert(row).second);
    std::set<int> got;
    for (int i = first; i < end; ++i) {
      CHECK(plan_key_row(m.skey[i]) == row);
      got.insert(plan_key_pos(m.skey[i]));
    }
    CHECK(got == want[row]);
    members_seen += end - first;
    const int64_t len = row_ptr[row + 1] - row_ptr[row];
    work_seen += (len + slice - 1) / slice;
    if (g + 1 < n_groups) CHECK(m.work[2 * (g + 1)] == end);                     // groups are packed back to back
  }
  CHECK(work_seen == n_work);
  size_t expect_members = 0;
  for (auto& kv : want) expect_members += kv.second.size();
  CHECK((size_t)members_seen == expect_members);
}

static std::vector<int64_t> ptr_of(const std::vector<int64_t>& lens) {
  std::vector<int64_t> p(lens.size() + 1, 0);
  for (size_t i = 0; i < lens.size(); ++i) p[i + 1] = p[i] + lens[i];
  return p;
}

static void test_plan() {
  // all of a full sub-batch in ONE group (the member field carries 8192)
  check_plan(std::vector<int64_t>(SORT_MAX, 3), 5, ptr_of({1, 2, 3, 70000, 5}));
  // 8192 singleton groups (the group field carries 8192), short rows: one slice each
  {
    std::vector<int64_t> rows(SORT_MAX), lens(SORT_MAX, 3);
    for (int i = 0; i < SORT_MAX; ++i) rows[i] = SORT_MAX - 1 - i;
    check_plan(rows, SORT_MAX, ptr_of(lens));
  }
  // one 50,000-entry row among ordinary ones, unknown pairs (-1), out-of-range rows, empty rows
  {
    std::vector<int64_t> lens(1000, 4);
    lens[17] = 50000;
    lens[18] = 0;
    std::vector<int64_t> rows(4096);
    std::mt19937 rng(3);
    for (auto& r : rows) r = (int64_t)(rng() % 1100) - 50;  // some < 0, some >= n_rows
    for (int i = 0; i < 40; ++i) rows[i * 7] = 17;
    rows[5] = 18;
    check_plan(rows, 1000, ptr_of(lens));
  }
  // total filter length that pushes the work list to its bound: 8192 groups whose rows need many slices each
  {
    std::vector<int64_t> rows(SORT_MAX), lens(SORT_MAX);
    for (int i = 0; i < SORT_MAX; ++i) {
      rows[i] = i;
      lens[i] = 1919 + (i % 3);  // ~15 slices of 128 each -> about 122,880 + 8192 work items before the slice grows
    }
    check_plan(rows, SORT_MAX, ptr_of(lens));
    for (auto& l : lens) l = 50000;  // 410M entries: the slice length grows instead of the work list
    check_plan(rows, SORT_MAX, ptr_of(lens));
    for (auto& l : lens) l = (1LL << 31) - 1;  // the longest rows an int32 column index allows
    check_plan(rows, SORT_MAX, ptr_of(lens));
  }
  // slice length: monotone, a multiple of 32, never below SLICE_MIN, and the bound on work items holds
  unsigned long long prev = 0;
  for (unsigned long long total : {0ull, 1ull, 127ull, 128ull, 15728640ull, 15728641ull, 1ull << 32, 1ull << 44, ~0ull >> 1}) {
    const unsigned long long sl = (unsigned long long)plan_slice_length(total);
    CHECK(sl >= (unsigned long long)SLICE_MIN && sl % 32 == 0 && sl >= prev);
    if (sl < 0x7fffffe0ull) CHECK(total / sl + SORT_MAX <= (unsigned long long)WORK_MAX);
    prev = sl;
  }
  // small and empty sub-batches
  check_plan({}, 4, ptr_of({1, 1, 1, 1}));
  check_plan({2}, 4, ptr_of({1, 1, 300, 1}));
  check_plan({-1, -1, 9}, 4, ptr_of({1, 1, 300, 1}));
  // randomised: group sizes and row lengths from heavy-tailed distributions
  std::mt19937 rng(11);
  for (int it = 0; it < 20; ++it) {
    const int n_rows = 1 + rng() % 3000, nb = 1 + rng() % SORT_MAX;
    std::vector<int64_t> lens(n_rows);
    for (auto& l : lens) l = (rng() % 10 == 0) ? rng() % 60000 : rng() % 9;
    std::vector<int64_t> rows(nb);
    for (auto& r : rows) r = (rng() % 4 == 0) ? (int64_t)(rng() % 8) : (int64_t)(rng() % (n_rows + 20)) - 10;
    check_plan(rows, n_rows, ptr_of(lens));
  }
}

int main() {
  test_contract_rules();
  test_layouts();
  test_csr_keys();
  test_plan();
  printf("host logic ok: %d checks\n", g_checks);
  return 0;
}
