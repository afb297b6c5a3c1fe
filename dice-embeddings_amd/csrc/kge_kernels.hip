// Entry points of the contraction path: materialised scores, fused filtered rank, fused top-k and
// fused multi-hot BCE, plus the small helper kernels around the two MFMA main loops.
#include "kge_contract.hip.h"
#include "kge_rank128.hip.h"
#include "kge_wide.hip.h"
#include "kge_topk_i8.hip.h"

#include <string.h>

#include <mutex>
#include <utility>
#include <vector>

namespace kge {

// ---- thread-local error text --------------------------------------------------------------
static thread_local char g_err[512] = "";
int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
void clear_error() { g_err[0] = 0; }

// ---- optional timing of the contraction launches (measurement aid) ------------------------
static std::mutex g_prof_mu;
static bool g_prof_on = false;
static std::vector<std::pair<hipEvent_t, hipEvent_t>> g_prof_events;
static char g_prof_kernel[160] = "";  // the main loop most recently bracketed, as dispatched

namespace {

// ============================================================================================
// One 32x32 tile straight from global memory: entity rows as A, query rows as B, in the same
// reduction order as the two main loops.  Lane (c, hf) supplies entity row `e_row` and query row
// `q_row` (either may be -1: a zero row).  Used where rows are gathered (targets, filter lists).
// ============================================================================================
template <int EDT>
__device__ __forceinline__ f32x16 chain_direct(const void* E, int d, int64_t e_row, const float* Q, int64_t q_row,
                                               int hf) {
  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  if (EDT == KGE_F32) {
    // fp32 rows on the bf16 MFMA: both rows split into three bf16 parts, six products per K step of 16
    // (the order of ksplit_kernel).  Four K steps per trip: all sixteen loads are issued first.
    const bool e_ok = e_row >= 0, q_ok = q_row >= 0;
    const float* e_ptr = (const float*)E + (e_ok ? e_row : 0) * d;
    const float* q_ptr = Q + (q_ok ? q_row : 0) * d;
    const bool vec_ok = (d & 3) == 0;
    const int nks = (d + 15) >> 4;
    // Branch-free loads (a missing row or a column past d reads a clamped address and is zeroed after), so
    // that the sixteen loads of a trip of four K steps are in flight together.
    auto load_trip = [&](int ks0, f32x4 (&fe)[4][2], f32x4 (&fq)[4][2]) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int k = (ks0 + u) * 16 + 8 * hf + 4 * h;
          if (vec_ok) {
            const int kk = (k < d) ? k : 0;
            fe[u][h] = *(const f32x4*)(e_ptr + kk);
            fq[u][h] = *(const f32x4*)(q_ptr + kk);
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int kk = (k + j < d) ? k + j : 0;
              fe[u][h][j] = e_ptr[kk];
              fq[u][h][j] = q_ptr[kk];
            }
          }
        }
      }
    };
    auto mul_trip = [&](int ks0, f32x4 (&fe)[4][2], f32x4 (&fq)[4][2]) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (ks0 + u < nks) {  // uniform: whole K steps past d are skipped (they would only add zeros)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int k = (ks0 + u) * 16 + 8 * hf + 4 * h;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const bool in = k + j < d;
              fe[u][h][j] = (in && e_ok) ? fe[u][h][j] : 0.f;
              fq[u][h][j] = (in && q_ok) ? fq[u][h][j] : 0.f;
            }
          }
          bf16x8 se[3], sq[3];
          split3_bf16x8(fe[u][0], fe[u][1], se);
          split3_bf16x8(fq[u][0], fq[u][1], sq);
#pragma unroll
          for (int p = 0; p < SPLIT_PRODUCTS; ++p) acc = mfma_bf16(se[SPLIT_A[p]], sq[SPLIT_B[p]], acc);
        }
      }
    };
    // (Issuing the next trip's loads before this trip is multiplied was measured slower: the second register
    // set costs the gather kernels more in occupancy than the overlap returns.)
    for (int ks0 = 0; ks0 < nks; ks0 += 4) {
      f32x4 fe[4][2], fq[4][2];
      load_trip(ks0, fe, fq);
      mul_trip(ks0, fe, fq);
    }
  } else {
    for (int s0 = 0; s0 < d; s0 += 128)  // eight K steps per trip (one trip for d <= 128)
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int k = s0 + 16 * s + 8 * hf;
      u32x4 ev = {0u, 0u, 0u, 0u};
      f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
      if (k < d) {
        if (e_row >= 0) {
          if (EDT == KGE_BF16) {
            ev = *(const u32x4*)((const uint16_t*)E + e_row * d + k);
          } else {
            const u32x2 w = *(const u32x2*)((const int8_t*)E + e_row * d + k);
            ev = i8x8_to_bf16x8(w[0], w[1]);
          }
        }
        if (q_row >= 0) {
          const f32x4* src = (const f32x4*)(Q + q_row * d + k);
          lo = src[0];
          hi = src[1];
        }
      }
      bf16x8 ef = __builtin_bit_cast(bf16x8, ev);
      acc = mfma_bf16(ef, cvt_bf16x8(lo, hi), acc);
    }
  }
  return acc;
}

// A member that is not its group's leader compares its vector with the leader's: the two halves of the wave
// take alternate 16-byte pieces of the row (alternate words when the rows are not 16-byte aligned).
__device__ __forceinline__ void group_vector_check(const ContractArgs& a, int64_t q, int hf, const int32_t* lead,
                                                   int32_t* mixed) {
  const int32_t l = lead[q];
  if (l >= 0 && (int64_t)l != q) {
    const uint32_t* x = (const uint32_t*)a.Q + q * a.d;
    const uint32_t* y = (const uint32_t*)a.Q + (int64_t)l * a.d;
    bool differs = false;
    if ((a.d & 3) == 0 && ((uintptr_t)a.Q & 15) == 0) {
#pragma unroll 4
      for (int64_t k = hf * 4; k < a.d; k += 8) {
        const uint4 u = *(const uint4*)(x + k), w = *(const uint4*)(y + k);
        differs = differs || u.x != w.x || u.y != w.y || u.z != w.z || u.w != w.w;
      }
    } else {
      for (int64_t k = hf; k < a.d; k += 2) differs = differs || x[k] != y[k];
    }
    if (differs) mixed[l] = 1;
  }
}

// ---- raw score of each query's target (the rank threshold) + counter initialisation ---------
// and, when the batch is filtered, the check the filter correction relies on: the correction scores a slice of a
// filter row once per group of queries that share the row, with the query vector of the group's leader.  A member
// whose vector differs from the leader's, in any bit, marks the group `mixed`; such a group is corrected one
// distinct vector at a time.  (Queries built from the same (head, relation) pair share row and vector.)
template <int EDT>
__global__ void __launch_bounds__(256) target_score_kernel(ContractArgs a, const int64_t* target, const float* bias,
                                                          float* thr, float* target_score, int32_t* n_gt,
                                                          int32_t* n_eq, int32_t* n_eql, const int32_t* lead,
                                                          int32_t* mixed) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  // With a filter the launch holds two sets of workgroups: the first forms the thresholds, the second makes the
  // group check for the same queries at the same time on other CUs (both are short chains of dependent loads; one
  // after the other in the same wave they would simply add up).
  const int64_t n_score_wgs = (a.B + 127) / 128;
  const bool check_role = (int64_t)blockIdx.x >= n_score_wgs;
  const int64_t q = (((int64_t)blockIdx.x - (check_role ? n_score_wgs : 0)) * 4 + wave) * 32 + c;
  if (check_role) {
    if (lead != nullptr && q < a.B) group_vector_check(a, q, hf, lead, mixed);
    return;
  }
  const int64_t t = (q < a.B) ? target[q] : -1;
  const bool ok = t >= 0 && t < a.N;
  f32x16 acc = chain_direct<EDT>(a.E, a.d, ok ? t : -1, a.Q, (q < a.B) ? q : -1, hf);
  // diagonal element (entity row c, query column c)
  const int isel = ((c >> 3) << 2) | (c & 3);
  float v = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i)
    if (i == isel) v = acc[i];
  if (hf == ((c >> 2) & 1) && q < a.B) {
    float raw = __uint_as_float(0x7fc00000u);
    if (ok) raw = (EDT == KGE_I8) ? v * a.scale[t] : v;
    thr[q] = raw;
    target_score[q] = raw + (bias ? bias[q] : 0.f);
    n_gt[q] = 0;
    n_eq[q] = ok ? -1 : 0;  // the main pass counts the target as tying with itself
    n_eql[q] = 0;
  }
}

// the one-vector-per-group check alone (a call whose thresholds were formed earlier, for many batches at once)
__global__ void __launch_bounds__(256) group_check_kernel(ContractArgs a, const int32_t* lead, int32_t* mixed) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  const int64_t q = ((int64_t)blockIdx.x * 4 + wave) * 32 + c;
  if (q < a.B) group_vector_check(a, q, hf, lead, mixed);
}

// ---- scores of given entities per query: the same chain, nothing else ------------------------------
// entity [B * group]: query b is scored against entity[b * group .. b * group + group - 1]
// (group = 1: forward_triples; group = k: forward_k_vs_sample)
template <int EDT>
__global__ void __launch_bounds__(256) triple_score_kernel(ContractArgs a, const int64_t* target, const float* bias,
                                                          float* out, int64_t group) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  const int64_t i = ((int64_t)blockIdx.x * 4 + wave) * 32 + c;
  const int64_t total = a.B * group;
  const int64_t q = (i < total) ? i / group : -1;
  const int64_t t = (i < total) ? target[i] : -1;
  const bool ok = t >= 0 && t < a.N;
  f32x16 acc = chain_direct<EDT>(a.E, a.d, ok ? t : -1, a.Q, q, hf);
  const int isel = ((c >> 3) << 2) | (c & 3);  // diagonal element (entity row c, query column c)
  float v = 0.f;
#pragma unroll
  for (int k = 0; k < 16; ++k)
    if (k == isel) v = acc[k];
  if (hf == ((c >> 2) & 1) && i < total) {
    float raw = __uint_as_float(0x7fc00000u);  // NaN for an id outside the table
    if (ok) raw = (EDT == KGE_I8) ? v * a.scale[t] : v;
    out[i] = raw + (bias ? bias[q] : 0.f);
  }
}

// ---- (head, relation) -> filter row: binary search in the sorted key array -----------------------
__global__ void csr_lookup_kernel(const int64_t* hr, int64_t B, const int64_t* keys, int64_t n_rows,
                                  int64_t num_relations, int64_t* csr_row) {
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  const int64_t key = hr[2 * b] * num_relations + hr[2 * b + 1];
  int64_t lo = 0, hi = n_rows;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (keys[mid] < key) lo = mid + 1; else hi = mid;
  }
  csr_row[b] = (lo < n_rows && keys[lo] == key) ? lo : -1;
}

// ---- group the queries of one sub-batch by filter row and plan the correction work -----------
// One workgroup, no sort: (1) every query claims the slot of its filter row in an LDS hash table
// (compare-and-swap on the row number) and takes a ticket from the slot's counter; the query with
// ticket 0 leads the group and fetches the row's length; (2) total filter length -> slice length
// (chosen so that there are at most WORK_MAX work items); (3) one exclusive scan over the leaders
// of three packed counters gives every group its index, the position of its first member and the
// index of its first work item; (4) members are written to their positions.  A group is the set of
// queries of the sub-batch that share a filter row (= the same (head, relation) pair, hence the
// same query vector); work item w is slice w - first of the group found by binary search in the
// group records.
using host::SORT_MAX;    // queries per sub-batch
using host::PLAN_SLOTS;  // hash table size: load factor <= 0.5

struct FixPlan {
  unsigned long long* skey;  // [SORT_MAX] csr_row << 24 | position in sub-batch, the members of a group adjacent
  int32_t* gend;             // [SORT_MAX] for a group's first position: one past its last position
  int32_t* work;             // [SORT_MAX][2] per group: (first position, index of its first work item)
  int32_t* meta;             // [0] work items, [1] slice length, [2] groups
  int32_t* lead;             // [B] per query: index of the first member of its group (itself for a leader), -1: no group
  int32_t* mixed;            // [B] per leader: set when some member of its group holds another query vector
};

__global__ void __launch_bounds__(1024) plan_fix_kernel(const int64_t* csr_row, int64_t b0, int nb, int64_t n_rows,
                                                       const int64_t* row_ptr, FixPlan plan) {
  __shared__ int32_t tab_row[PLAN_SLOTS];  // filter row + 1 that owns the slot, 0 = free
  __shared__ int32_t tab_cnt[PLAN_SLOTS];  // members of the slot's group; later: position of its first member
  __shared__ unsigned long long part[1024];
  __shared__ unsigned long long s_total;
  __shared__ int s_slice;
  constexpr int QPT = SORT_MAX / 1024;     // queries per thread
  const int tid = threadIdx.x;
  for (int i = tid; i < PLAN_SLOTS; i += 1024) {
    tab_row[i] = 0;
    tab_cnt[i] = 0;
  }
  if (tid == 0) s_total = 0;
  // the filter rows of this thread's queries (independent loads, all in flight together)
  int64_t my_row[QPT];
#pragma unroll
  for (int j = 0; j < QPT; ++j) {
    const int i = tid + 1024 * j;
    int64_t r = -1;
    if (i < nb) r = csr_row[b0 + i];
    my_row[j] = (r >= 0 && r < n_rows) ? r : -1;
  }
  __syncthreads();
  // (1) claim slots, take tickets
  int my_slot[QPT], my_pos[QPT];
#pragma unroll
  for (int j = 0; j < QPT; ++j) {
    my_slot[j] = -1;
    my_pos[j] = -1;
    if (my_row[j] >= 0) {
      const int32_t key = (int32_t)my_row[j] + 1;
      uint32_t h = host::plan_hash(my_row[j]);
      for (;;) {
        const int32_t old = atomicCAS(&tab_row[h], 0, key);
        if (old == 0 || old == key) break;
        h = (h + 1) & (PLAN_SLOTS - 1);
      }
      my_slot[j] = (int)h;
      my_pos[j] = atomicAdd(&tab_cnt[h], 1);
    }
  }
  // leaders fetch their row's length (unconditional loads of a valid row keep them in flight together)
  int64_t len[QPT];
  unsigned long long my_total = 0;
#pragma unroll
  for (int j = 0; j < QPT; ++j) {
    const bool lead = my_pos[j] == 0;
    const int64_t rr = lead ? my_row[j] : 0;
    const int64_t l = row_ptr[rr + 1] - row_ptr[rr];
    len[j] = lead ? l : 0;
    my_total += (unsigned long long)len[j];
  }
  if (my_total) atomicAdd(&s_total, my_total);
  __syncthreads();
  // (2) slice length: at least SLICE_MIN, large enough that extra slices fit the work list
  if (tid == 0) s_slice = host::plan_slice_length(s_total);
  __syncthreads();
  const int slice = s_slice;
  // (3) per leader with work: groups (bits 48..), members (bits 32..47), slices (bits 0..31)
  unsigned long long val[QPT];
  unsigned long long local = 0;
#pragma unroll
  for (int j = 0; j < QPT; ++j) {
    const unsigned long long n = (unsigned long long)((len[j] + slice - 1) / slice);  // an empty row needs no work
    val[j] = (n > 0) ? host::plan_pack((unsigned long long)tab_cnt[my_slot[j]], n) : 0;
    local += val[j];
  }
  part[tid] = local;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {
    const unsigned long long v = (tid >= off) ? part[tid - off] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  unsigned long long base = part[tid] - local;
#pragma unroll
  for (int j = 0; j < QPT; ++j) {
    if (val[j]) {
      const int g = host::plan_groups(base), first = host::plan_members(base);
      plan.work[2 * g] = first;
      plan.work[2 * g + 1] = (int)host::plan_slices(base);
      plan.gend[first] = first + tab_cnt[my_slot[j]];
      tab_cnt[my_slot[j]] = first;  // only this leader reads or writes its group's slot in this phase
      tab_row[my_slot[j]] = tid + 1024 * j;  // the slot's row number has done its work: now the leader's index
    } else if (my_pos[j] == 0) {
      tab_cnt[my_slot[j]] = -1;     // empty filter row: nothing to take out for this group
    }
    base += val[j];
  }
  if (tid == 1023) {
    plan.meta[0] = (int)host::plan_slices(part[1023]);
    plan.meta[1] = slice;
    plan.meta[2] = host::plan_groups(part[1023]);
  }
  __syncthreads();
  // (4) members to their positions; every query learns its group's leader (for the check that a group's members
  // hold one and the same query vector, which the kernel that forms the thresholds makes)
#pragma unroll
  for (int j = 0; j < QPT; ++j) {
    const int i = tid + 1024 * j;
    int32_t leader = -1;
    if (my_slot[j] >= 0) {
      const int first = tab_cnt[my_slot[j]];
      if (first >= 0) {
        plan.skey[first + my_pos[j]] = host::plan_member_key(my_row[j], i);
        leader = (int32_t)b0 + tab_row[my_slot[j]];
      }
    }
    if (i < nb) {
      plan.lead[b0 + i] = leader;
      plan.mixed[b0 + i] = 0;
    }
  }
}

// ---- take the filtered entities back out of the counters ------------------------------------
// Work item = (group of queries sharing a filter row, slice of that row).  The slice's entity scores
// are formed once per distinct query vector of the group (gathered rows, same MFMA chain as the main
// loop), then every query holding that vector compares them with its own threshold.  Queries built from
// the same (head, relation) pair share both the row and the vector, so a group normally takes one round;
// a caller that hands one filter row to different query vectors gets one round per distinct vector
// (vectors are compared bit for bit against the round's leader).
constexpr int FIX_CAP = 2048;
constexpr int FIX_ITEMS = 16;  // work items a workgroup resolves side by side
// ROWS256 (bf16 tables with d == 128: rows of 256 bytes): the slice's rows are gathered the way the main loop
// streams them, 16 lanes per row straight into LDS (whole 128-byte lines per request) in the swizzled stage
// layout, and the MFMA fragments are read from there; the generic path reads every row 16 bytes per lane at
// a stride, which costs four requests per line.
template <int EDT, bool ROWS256>
__global__ void __launch_bounds__(256) filter_fix_kernel(ContractArgs a, FixPlan plan, int64_t b0,
                                                        const int64_t* row_ptr, const int32_t* col,
                                                        const int64_t* target, const float* thr, int32_t* n_gt,
                                                        int32_t* n_eq, int32_t* n_eql) {
  constexpr int CAP = ROWS256 ? 512 : FIX_CAP;  // entities per pass (the staged rows leave less LDS for the scores)
  __shared__ float s_s[CAP];
  __shared__ float s_sc[EDT == KGE_I8 ? CAP : 1];
  __shared__ int32_t s_e[CAP];
  __shared__ int32_t s_cnt[3 * 256];
  __shared__ unsigned char s_state[SORT_MAX];  // per member of a group: 0 = waiting, 1 = in this round, 2 = done
  __shared__ __attribute__((aligned(1024))) unsigned char s_rows[ROWS256 ? 4 * 8192 : 16];  // per wave: one 32-row tile
  __shared__ int s_next;                       // first member still waiting after this round
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 31, hf = lane >> 5;
  const int n_work = plan.meta[0];
  const int64_t slice = plan.meta[1];
  const int n_groups = plan.meta[2];
  // This workgroup's work items are w = blockIdx.x + k * gridDim.x.  Up to FIX_ITEMS of them at a time are
  // resolved by one thread each, side by side (group by binary search, then the group's row and extent),
  // so that their chains of dependent loads overlap instead of running once per item.
  __shared__ int32_t it_i0[FIX_ITEMS], it_m[FIX_ITEMS], it_mixed[FIX_ITEMS];
  __shared__ int64_t it_z0[FIX_ITEMS], it_z1[FIX_ITEMS];
  for (int k0 = 0; blockIdx.x + (int64_t)k0 * gridDim.x < n_work; k0 += FIX_ITEMS) {
    __syncthreads();
    if (tid < FIX_ITEMS) {
      const int64_t w = blockIdx.x + (int64_t)(k0 + tid) * gridDim.x;
      if (w < n_work) {
        int lo = 0, hi = n_groups;  // last group whose first work item is <= w: in [lo, hi)
        // fifteen pivots per step, their loads in flight together: a sixteenth of the range is left (a search
        // that halves the range is a chain of log2(n_groups) dependent loads at the head of every workgroup)
        while (hi - lo > 16) {
          const int step = (hi - lo) >> 4;
          int first[15];
#pragma unroll
          for (int j = 0; j < 15; ++j) first[j] = plan.work[2 * (lo + step * (j + 1)) + 1];
          int le = 0;  // pivots whose first work item is <= w: a prefix
#pragma unroll
          for (int j = 0; j < 15; ++j) le += (first[j] <= (int64_t)w) ? 1 : 0;
          const int nlo = lo + step * le, nhi = (le < 15) ? lo + step * (le + 1) : hi;
          lo = nlo;
          hi = nhi;
        }
        while (hi - lo > 1) {
          const int mid = (lo + hi) >> 1;
          if (plan.work[2 * mid + 1] <= w) lo = mid; else hi = mid;
        }
        const int i0 = plan.work[2 * lo];
        const int64_t z = w - plan.work[2 * lo + 1];
        const unsigned long long key = plan.skey[i0];
        const int64_t row = host::plan_key_row(key);
        const int64_t L0 = row_ptr[row], L1 = row_ptr[row + 1];
        const int64_t z0 = L0 + z * slice;
        it_i0[tid] = i0;
        it_m[tid] = plan.gend[i0] - i0;
        it_mixed[tid] = plan.mixed[b0 + host::plan_key_pos(key)];
        it_z0[tid] = z0;
        it_z1[tid] = (z0 + slice < L1) ? z0 + slice : L1;
      }
    }
    __syncthreads();
  for (int kk = 0; kk < FIX_ITEMS && blockIdx.x + (int64_t)(k0 + kk) * gridDim.x < n_work; ++kk) {
    const int i0 = it_i0[kk];
    const int m = it_m[kk];
    const int64_t z0 = it_z0[kk], z1 = it_z1[kk];
    // threads per member in the compare phase: spread a small group over the whole workgroup
    int tpm = 1;
    while (tpm * 2 * m <= 256) tpm *= 2;
    const int sub = tid % tpm, mslot = tid / tpm, mstep = 256 / tpm;
    // a group whose members all hold the leader's query vector (the check is made once per group, by the kernel
    // that forms the thresholds) takes one round; a mixed group one round per distinct vector
    const bool rounds = m > 1 && it_mixed[kk] != 0;
    if (rounds) {
      for (int i = tid; i < m; i += 256) s_state[i] = 0;
    }
    // `lead` is the first member not yet served
    for (int lead = 0; lead < m;) {
      const int64_t bq = b0 + (int64_t)host::plan_key_pos(plan.skey[i0 + lead]);
      if (rounds) {
        // members whose query vector equals the leader's, bit for bit, join this round
        __syncthreads();
        if (tid == 0) s_next = m;
        __syncthreads();
        const uint32_t* ql = (const uint32_t*)(a.Q + bq * a.d);
        for (int mbase = lead; mbase < m; mbase += mstep) {
          const int mi = mbase + mslot;
          bool same = true;
          if (mi < m && s_state[mi] == 0 && mi != lead) {
            const uint32_t* qm = (const uint32_t*)(a.Q + (b0 + (int64_t)host::plan_key_pos(plan.skey[i0 + mi])) * a.d);
            for (int k = sub; k < a.d; k += tpm) same = same && (qm[k] == ql[k]);
          }
          // all threads of a member agree before anyone writes its state
          if (tpm > 1) {
#pragma unroll
            for (int o = 1; o < 64; o <<= 1)
              if (o < tpm) same = __shfl_xor((int)same, o, 64) != 0 && same;
          }
          if (tpm > 64) {  // a member spread over several waves (m == 1 never comes here): meet in LDS
            s_cnt[tid] = same ? 1 : 0;
            __syncthreads();
            bool all = true;
            for (int t = (tid / tpm) * tpm; t < (tid / tpm) * tpm + tpm; t += 64) all = all && s_cnt[t] != 0;
            same = all;
            __syncthreads();
          }
          if (mi < m && sub == 0 && s_state[mi] == 0) {
            if (same) s_state[mi] = 1;
            else atomicMin(&s_next, mi);
          }
        }
        __syncthreads();
      }
      // the threshold and target of this thread's member of the first compare batch (nearly always the only batch):
      // two dependent loads, issued here so that they travel while the slice's rows are gathered
      int64_t pre_b = 0, pre_t = 0;
      float pre_th = 0.f;
      if (lead + mslot < m) {
        pre_b = b0 + (int64_t)host::plan_key_pos(plan.skey[i0 + lead + mslot]);
        pre_th = thr[pre_b];
        pre_t = target[pre_b];
      }
      for (int64_t pass = z0; pass < z1; pass += CAP) {
        const int n_here = (int)((z1 - pass < CAP) ? z1 - pass : CAP);
        const int ntile = (n_here + 31) >> 5;
        if constexpr (ROWS256) {
          // the round's query vector as MFMA fragments (the same one in every column)
          bf16x8 qfrag[8];
#pragma unroll
          for (int sft = 0; sft < 8; ++sft) {
            const f32x4* src = (const f32x4*)(a.Q + bq * 128 + 16 * sft + 8 * hf);
            qfrag[sft] = cvt_bf16x8(src[0], src[1]);
          }
          const int wv = __builtin_amdgcn_readfirstlane(wave);
          unsigned char* stage = s_rows + wv * 8192;
          const unsigned char* Eb = (const unsigned char*)a.E;
          for (int tile = wv; tile < ntile; tile += 4) {
            const int j0 = tile * 32 + c;
            const int32_t e0 = (j0 < n_here) ? col[pass + j0] : -1;
            const bool ok0 = e0 >= 0 && (int64_t)e0 < a.N;
            if (hf == 0) s_e[j0] = ok0 ? e0 : -1;
            // lane l fetches piece (l & 15) ^ (row & 15) of row 4 j + l / 16 of the tile; an entry that is not a
            // valid entity id fetches row 0 instead (its score is ignored: s_e says -1)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const int row = 4 * j + (lane >> 4);
              const int32_t e = s_e[tile * 32 + row];
              const int64_t er = e >= 0 ? (int64_t)e : 0;
              __builtin_amdgcn_global_load_lds(
                  (const __attribute__((address_space(1))) void*)(Eb + er * 256 + (((lane & 15) ^ (row & 15)) << 4)),
                  (__attribute__((address_space(3))) void*)(stage + j * 1024), 16, 0, 0);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            f32x16 acc;
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
            for (int sft = 0; sft < 8; ++sft) {
              const bf16x8 ef = *(const bf16x8*)(stage + c * 256 + (((2 * sft + hf) ^ (c & 15)) << 4));
              acc = mfma_bf16(ef, qfrag[sft], acc);
            }
            if (c == 0) {
#pragma unroll
              for (int i = 0; i < 16; ++i) s_s[tile * 32 + row_of(i, hf)] = acc[i];
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the fragments are read before the next tile's rows land
          }
        } else {
        // two tiles per trip so that both row gathers are in flight before the first MFMA chain
        for (int tile = wave; tile < ntile; tile += 8) {
          const int j0 = tile * 32 + c, j1 = (tile + 4) * 32 + c;
          const int32_t e0 = (j0 < n_here) ? col[pass + j0] : -1;
          const int32_t e1 = (j1 < n_here) ? col[pass + j1] : -1;
          const bool ok0 = e0 >= 0 && (int64_t)e0 < a.N, ok1 = e1 >= 0 && (int64_t)e1 < a.N;
          const bool two = tile + 4 < ntile;  // uniform per wave
          f32x16 acc0 = chain_direct<EDT>(a.E, a.d, ok0 ? (int64_t)e0 : -1, a.Q, bq, hf);
          f32x16 acc1;
          if (two) acc1 = chain_direct<EDT>(a.E, a.d, ok1 ? (int64_t)e1 : -1, a.Q, bq, hf);
          if (c == 0) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s_s[tile * 32 + row_of(i, hf)] = acc0[i];
            if (two) {
#pragma unroll
              for (int i = 0; i < 16; ++i) s_s[(tile + 4) * 32 + row_of(i, hf)] = acc1[i];
            }
          }
          if (hf == 0) {
            s_e[j0] = ok0 ? e0 : -1;
            if (EDT == KGE_I8) s_sc[j0] = ok0 ? a.scale[e0] : 1.f;
            if (two) {
              s_e[j1] = ok1 ? e1 : -1;
              if (EDT == KGE_I8) s_sc[j1] = ok1 ? a.scale[e1] : 1.f;
            }
          }
        }
        }
        __syncthreads();
        // compare phase: `tpm` threads share one query; their partial counts meet in LDS so that each
        // query receives ONE global atomic per counter (hundreds of same-address atomics serialise)
        for (int mbase = lead; mbase < m; mbase += mstep) {
          const int mi = mbase + mslot;
          const bool mine = mi < m && (!rounds || s_state[mi] == 1);
          s_cnt[tid] = 0;
          s_cnt[256 + tid] = 0;
          s_cnt[512 + tid] = 0;
          __syncthreads();
          int64_t b = 0;
          if (mine) {
            const bool pre = mbase == lead;
            b = pre ? pre_b : b0 + (int64_t)host::plan_key_pos(plan.skey[i0 + mi]);
            const float th = pre ? pre_th : thr[b];
            const int64_t t = pre ? pre_t : target[b];
            int32_t g = 0, eq = 0, eql = 0;
            for (int j = sub; j < n_here; j += tpm) {
              const int32_t e = s_e[j];
              float s = s_s[j];
              if (EDT == KGE_I8) s *= s_sc[j];
              if (e >= 0 && (int64_t)e != t) {
                g += (s > th) ? 1 : 0;
                if (s == th) {
                  eq += 1;
                  eql += ((int64_t)e < t) ? 1 : 0;
                }
              }
            }
            if (tpm == 1) {
              s_cnt[mslot] = g;
              s_cnt[256 + mslot] = eq;
              s_cnt[512 + mslot] = eql;
            } else {
              if (g) atomicAdd(&s_cnt[mslot], g);
              if (eq) atomicAdd(&s_cnt[256 + mslot], eq);
              if (eql) atomicAdd(&s_cnt[512 + mslot], eql);
            }
          }
          __syncthreads();
          if (mine && sub == 0) {
            const int32_t g = s_cnt[mslot], eq = s_cnt[256 + mslot], eql = s_cnt[512 + mslot];
            if (g) atomicSub(&n_gt[b], g);
            if (eq) atomicSub(&n_eq[b], eq);
            if (eql) atomicSub(&n_eql[b], eql);
          }
          __syncthreads();
        }
      }
      if (!rounds) break;
      // this round's members are done; the next round is led by the first member still waiting
      __syncthreads();
      for (int i = lead + tid; i < m; i += 256)
        if (s_state[i] == 1) s_state[i] = 2;
      lead = s_next;
    }
  }
  }
}

// ---- top-k bookkeeping ------------------------------------------------------------------------
using host::TOPK_CAP;         // candidates a query can collect in one round
using host::TOPK_MAX_K;
using host::TOPK_FIRST_ROWS;  // first round takes everything: must not exceed TOPK_CAP

struct TopkWs {
  float* tau;       // k-th best score so far (-inf while fewer than k are known)
  float* tau_scan;  // what the next scan admits candidates with: tau, or the tighter guess of select_finish
  int32_t* cnt;
  int32_t* list_len;
  int32_t* dirty;
  int32_t* n_dirty;
  unsigned long long* kth;   // per query: its k-th best as a packed key (0 while fewer than k are known)
  unsigned long long* list;  // [B, kpad]
  unsigned long long* cand;  // [B, TOPK_CAP] packed keys
  uint32_t* cand_id;         // [B, TOPK_CAP] entity ids (int8 filter scan; scored into `cand` before they are ranked)
  unsigned char* rowmeta;    // int8 filter scan: per 64 table rows one record
  int8_t* requant;           // int8 filter scan: the table with one scale per 32-row tile
  int8_t* qh;                // int8 filter scan: the queries as int8
  f32x4* qc;                 // int8 filter scan: per query the constants of its bound
  int64_t kpad;
};

// `prepared`: the table's prepared form is in the caller's hands (kge_topk_prepare); the workspace then holds none
size_t topk_ws_layout(int64_t B, int64_t N, int64_t k, void* base, TopkWs* ws, const void* prepared = nullptr,
                      bool with_table = true) {
  const host::TopkWsOffsets o = host::topk_ws_offsets(B, N, k, with_table);
  if (ws) {
    char* p = (char*)base;
    ws->tau = (float*)(p + o.tau);
    ws->tau_scan = (float*)(p + o.tau_scan);
    ws->cnt = (int32_t*)(p + o.cnt);
    ws->list_len = (int32_t*)(p + o.list_len);
    ws->dirty = (int32_t*)(p + o.dirty);
    ws->n_dirty = (int32_t*)(p + o.n_dirty);
    ws->kth = (unsigned long long*)(p + o.kth);
    ws->list = (unsigned long long*)(p + o.list);
    ws->cand = (unsigned long long*)(p + o.cand);
    ws->cand_id = (uint32_t*)(p + o.cand_id);
    ws->qh = (int8_t*)(p + o.qh);
    ws->qc = (f32x4*)(p + o.qc);
    if (with_table) {
      ws->rowmeta = (unsigned char*)(p + o.rowmeta);
      ws->requant = (int8_t*)(p + o.requant);
    } else {
      const host::TopkPreparedOffsets t = host::topk_prepared_offsets(N);
      ws->rowmeta = (unsigned char*)prepared + t.rowmeta;
      ws->requant = (int8_t*)((unsigned char*)prepared + t.requant);
    }
    ws->kpad = o.kpad;
  }
  return o.total;
}

// `first_rows`: the rows of the first round, whose scan writes one key per row into every query's candidate buffer
__global__ void topk_init_kernel(TopkWs w, int64_t B, int32_t first_rows) {
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b < B) {
    w.tau[b] = __uint_as_float(0xff800000u);  // -inf
    w.tau_scan[b] = __uint_as_float(0xff800000u);
    w.cnt[b] = first_rows;
    w.list_len[b] = 0;
    w.dirty[b] = 0;
    w.kth[b] = 0;
  }
  if (b == 0) *w.n_dirty = 0;
}

// Merge a query's kept list with this round's candidates, keep the best k, publish the new
// threshold.  In `rescan` mode (only queries flagged dirty) the list entries that rank above the old k-th best (by
// key: a higher score, or the same score and a lower entity id) are dropped first: the rescan finds all of them again.
// Bitonic sort, descending, of 64 * KPL keys held by one wave: element i = lane * KPL + s sits in
// v[s] of `lane`.  Exchanges at distance < KPL stay inside a lane's registers; larger distances are
// a lane shuffle.  No LDS, no barriers.
template <int KPL>
__device__ __forceinline__ void wave_sort_desc(unsigned long long (&v)[KPL], int lane) {
  constexpr int N = 64 * KPL;
#pragma unroll
  for (int kk = 2; kk <= N; kk <<= 1) {
#pragma unroll
    for (int j = kk >> 1; j > 0; j >>= 1) {
      if (j < KPL) {
#pragma unroll
        for (int s = 0; s < KPL; ++s) {
          if ((s & j) == 0) {
            // element index i = lane * KPL + s; the pair is ordered "larger first" iff (i & kk) == 0
            const bool down = (kk < KPL) ? ((s & kk) == 0) : (((lane * KPL) & kk) == 0);
            const unsigned long long x = v[s], y = v[s | j];
            const unsigned long long hi = x > y ? x : y, lo = x > y ? y : x;
            v[s] = down ? hi : lo;
            v[s | j] = down ? lo : hi;
          }
        }
      } else {
        const int jl = j / KPL;
        const bool lower = (lane & jl) == 0;
        const bool down = ((lane * KPL) & kk) == 0;  // kk > j >= KPL: a function of the lane only
        const bool keep_max = lower == down;
#pragma unroll
        for (int s = 0; s < KPL; ++s) {
          const unsigned long long x = v[s];
          const unsigned long long y = __shfl_xor(x, jl, 64);
          const unsigned long long hi = x > y ? x : y, lo = x > y ? y : x;
          v[s] = keep_max ? hi : lo;
        }
      }
    }
  }
}

// Two launches cover a round.  First one wave per query, keys in registers (wave_sort_desc), for the
// queries with at most SELECT_SMALL entries to rank, which is nearly all of them; then four waves
// per query with the keys in LDS and room for a full candidate buffer for the rest.  A query ranked
// by the first launch has its candidate count reset, so the second one skips it.
constexpr int SELECT_SMALL = 1024;

// `th_used`: the threshold this round's scan admitted candidates with.  When it was a guess above the k-th best
// (th_used > tau_old), the round is complete only if the merged k-th best still beats it: every entity above the
// merged k-th best was then admitted.  Otherwise the query is flagged and scanned again at the end with its k-th best.
// `spec_key`: the key at rank j_spec - 1 of the merged list (0: none): the next scan's guess is just below its score.
__device__ __forceinline__ void select_finish(const TopkWs& w, int64_t b, int k, int rescan, bool over, int new_len,
                                              bool have_tau, unsigned long long kth_key, float tau_old, float th_used,
                                              unsigned long long spec_key) {
  const float NINF = __uint_as_float(0xff800000u);
  w.list_len[b] = new_len;
  const float tau = ordered_to_f32((uint32_t)(kth_key >> 32));
  const float tau_new = have_tau ? tau : NINF;
  w.tau[b] = tau_new;
  w.kth[b] = have_tau ? kth_key : 0ull;
  float guess = tau_new;
  if (have_tau && spec_key != 0) {
    // just below the score at that rank, so that its ties are admitted too
    const float below = just_below(ordered_to_f32((uint32_t)(spec_key >> 32)));
    if (below > guess) guess = below;  // never below the k-th best; NaN leaves it
  }
  w.tau_scan[b] = rescan ? tau_new : guess;
  w.cnt[b] = 0;
  const bool short_of_guess = th_used > tau_old && !(have_tau && tau > th_used);
  if (!rescan) {
    if ((over || short_of_guess) && !w.dirty[b]) {
      w.dirty[b] = 1;
      atomicAdd(w.n_dirty, 1);
    }
  } else if (!over) {
    w.dirty[b] = 0;
    atomicSub(w.n_dirty, 1);
  }
}

// Int8 filter scan: this round's candidates of every query are entity ids that passed a bound.  Their exact scores,
// by the chain every score of an int8 table goes through, as packed keys into `cand`; 0 where the score does not
// beat the threshold the scan worked with (the bound lets more through than that).  A wave takes 32 candidates of
// one query at a time; grid (B, y): the waves of the y blocks of a query share its candidates out.
__global__ void __launch_bounds__(256) topk_rescore_kernel(TopkWs w, ContractArgs a) {
  const int lane = threadIdx.x & 63, c = lane & 31, hf = lane >> 5;
  const int64_t b = blockIdx.x;
  const int raw = w.cnt[b];
  const int nc = raw < TOPK_CAP ? raw : TOPK_CAP;
  const float th = w.tau_scan[b];
  const uint32_t* ids = w.cand_id + b * TOPK_CAP;
  unsigned long long* out = w.cand + b * TOPK_CAP;
  const int wid = blockIdx.y * 4 + (threadIdx.x >> 6), nw = gridDim.y * 4;
  if (32 * wid >= nc) return;
  // The query row as MFMA fragments, once per wave (d == 128 here: the filter scan exists for that width only):
  // every tile multiplies the same row, and re-reading it per tile costs eight times the bytes of the gathered rows.
  bf16x8 qfrag[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const f32x4* src = (const f32x4*)(a.Q + b * 128 + 16 * s + 8 * hf);
    qfrag[s] = cvt_bf16x8(src[0], src[1]);
  }
  for (int j0 = 32 * wid; j0 < nc; j0 += 32 * nw) {
    const int j = j0 + c;
    const int64_t e = (j < nc) ? (int64_t)ids[j] : -1;
    const bool ok = e >= 0 && e < a.N;
    // the chain of chain_direct<KGE_I8> (K steps of 16 ascending, the row widened to bf16 exactly)
    u32x2 wv[8];
#pragma unroll
    for (int s = 0; s < 8; ++s)
      wv[s] = ok ? *(const u32x2*)((const int8_t*)a.E + e * 128 + 16 * s + 8 * hf) : u32x2{0u, 0u};
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s)
      acc = mfma_bf16(__builtin_bit_cast(bf16x8, i8x8_to_bf16x8(wv[s][0], wv[s][1])), qfrag[s], acc);
    const int isel = ((c >> 3) << 2) | (c & 3);  // diagonal element (entity row c, query column c)
    float v = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (i == isel) v = acc[i];
    if (hf == ((c >> 2) & 1) && j < nc) {
      unsigned long long key = 0;
      if (ok) {
        const float sc = v * a.scale[e];
        if (sc > th) key = ((unsigned long long)f32_to_ordered(sc) << 32) | (unsigned long long)(0xffffffffu - (uint32_t)e);
      }
      out[j] = key;
    }
  }
}

// `packed` (LDS, or null): this round's candidates with the empty slots taken out, `nc` of them; otherwise the
// candidates are read from the query's buffer as they lie.
template <int KPL>
__device__ __forceinline__ void select_in_registers(const TopkWs& w, int64_t b, int k, int rescan, int len, int nc,
                                                    float tau_old, float th_used, int j_spec, int lane,
                                                    const unsigned long long* packed = nullptr) {
  const unsigned long long kth_old = w.kth[b];  // (every lane reads it before lane 0 publishes the new one below)
  unsigned long long v[KPL];
#pragma unroll
  for (int s = 0; s < KPL; ++s) {
    const int i = lane * KPL + s;
    unsigned long long key = 0;
    if (i < len) {
      key = w.list[b * w.kpad + i];
      if (rescan && key > kth_old) key = 0;
    } else if (i < len + nc) {
      key = packed ? packed[i - len] : w.cand[b * TOPK_CAP + (i - len)];
    }
    v[s] = key;
  }
  wave_sort_desc<KPL>(v, lane);
  int valid = 0;
#pragma unroll
  for (int s = 0; s < KPL; ++s) valid += v[s] != 0 ? 1 : 0;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) valid += __shfl_xor(valid, o, 64);
  const int new_len = valid < k ? valid : k;
  unsigned long long kth = 0, spec = 0;  // the keys at positions k - 1 and j_spec - 1, if this lane holds them
#pragma unroll
  for (int s = 0; s < KPL; ++s) {
    const int i = lane * KPL + s;
    if (i < new_len) w.list[b * w.kpad + i] = v[s];
    if (i == k - 1) kth = v[s];
    if (i == j_spec - 1 && i < new_len) spec = v[s];
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {  // one lane at most holds each
    kth |= __shfl_xor(kth, o, 64);
    spec |= __shfl_xor(spec, o, 64);
  }
  if (lane == 0)
    select_finish(w, b, k, rescan, false, new_len, new_len == k, kth, tau_old, th_used, spec);
}

// Merge a query's kept list with this round's candidates, keep the best k, publish the new
// threshold.  In `rescan` mode (only queries flagged dirty) list entries above the old threshold
// are dropped first: the rescan finds all of them again.
// `sparse`: the candidates come from the int8 filter scan, whose exact rescoring leaves a zero where a candidate did
// not beat the threshold (most of them).  The keys that remain are packed in LDS first, so that the sorting network
// is chosen by what there is to sort.
constexpr int SELECT_PACKED = 512;  // packed candidates the one-wave selection keeps in LDS
__global__ void __launch_bounds__(64) topk_select_wave_kernel(TopkWs w, int k, int rescan, int j_spec, int sparse) {
  __shared__ unsigned long long packed[SELECT_PACKED];
  const int lane = threadIdx.x;
  const int64_t b = blockIdx.x;
  if (rescan && !w.dirty[b]) return;
  const int len = w.list_len[b];
  const int raw = w.cnt[b];
  if (raw > TOPK_CAP || len + raw > SELECT_SMALL) return;  // left to topk_select_kernel
  const float tau_old = w.tau[b];
  const float th_used = rescan ? tau_old : w.tau_scan[b];
  int nc = raw;
  const unsigned long long* from = nullptr;
  if (sparse && len + raw > 128) {
    int n = 0;  // packed so far (the same in every lane)
    for (int j0 = 0; j0 < raw; j0 += 64) {
      const int j = j0 + lane;
      const unsigned long long key = (j < raw) ? w.cand[b * TOPK_CAP + j] : 0ull;
      const unsigned long long has = __builtin_amdgcn_ballot_w64(key != 0);
      const int at = n + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(has >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)has, 0u));
      if (key != 0 && at < SELECT_PACKED) packed[at] = key;
      n += __builtin_popcountll(has);
    }
    if (n <= SELECT_PACKED) {  // (more than that: sorted as they lie, zeros included)
      nc = n;
      from = packed;
      __syncthreads();  // (one wave; the branch is the same for all of it)
    }
  }
  // (the network's cost grows faster than the number of keys: short lists, the usual case for small k, take a small one)
  if (len + nc <= 128)
    select_in_registers<2>(w, b, k, rescan, len, nc, tau_old, th_used, j_spec, lane, from);
  else if (len + nc <= 256)
    select_in_registers<4>(w, b, k, rescan, len, nc, tau_old, th_used, j_spec, lane, from);
  else if (len + nc <= 512)
    select_in_registers<8>(w, b, k, rescan, len, nc, tau_old, th_used, j_spec, lane, from);
  else
    select_in_registers<16>(w, b, k, rescan, len, nc, tau_old, th_used, j_spec, lane, from);
}

__global__ void __launch_bounds__(256) topk_select_kernel(TopkWs w, int k, int rescan, int j_spec) {
  extern __shared__ unsigned long long keys[];
  __shared__ int s_valid;
  const int tid = threadIdx.x;
  const int64_t b = blockIdx.x;
  if (rescan && !w.dirty[b]) return;
  const int len = w.list_len[b];
  const int raw = w.cnt[b];
  const int nc = raw < TOPK_CAP ? raw : TOPK_CAP;
  const bool over = raw > TOPK_CAP;
  const float tau_old = w.tau[b];
  const unsigned long long kth_old = w.kth[b];
  const float th_used = rescan ? tau_old : w.tau_scan[b];
  const int n = len + nc;
  if (n <= SELECT_SMALL) return;  // ranked by topk_select_wave_kernel (which reset the candidate count)
  int npad = 2;
  while (npad < n) npad <<= 1;
  if (tid == 0) s_valid = 0;
  for (int i = tid; i < npad; i += 256) {
    unsigned long long key = 0;
    if (i < len) {
      key = w.list[b * w.kpad + i];
      if (rescan && key > kth_old) key = 0;
    } else if (i < n) {
      key = w.cand[b * TOPK_CAP + (i - len)];
    }
    keys[i] = key;
  }
  __syncthreads();
  for (int kk = 2; kk <= npad; kk <<= 1) {
    for (int j = kk >> 1; j > 0; j >>= 1) {
      for (int i = tid; i < npad; i += 256) {
        const int ixj = i ^ j;
        if (ixj > i) {
          const bool down = (i & kk) == 0;
          const unsigned long long x = keys[i], y = keys[ixj];
          if ((x < y) == down) {
            keys[i] = y;
            keys[ixj] = x;
          }
        }
      }
      __syncthreads();
    }
  }
  for (int i = tid; i < npad; i += 256)
    if (keys[i] != 0 && (i + 1 == npad || keys[i + 1] == 0)) s_valid = i + 1;
  __syncthreads();
  const int n_valid = s_valid;
  const int new_len = n_valid < k ? n_valid : k;
  for (int i = tid; i < new_len; i += 256) w.list[b * w.kpad + i] = keys[i];
  if (tid == 0)
    select_finish(w, b, k, rescan, over, new_len, new_len == k, keys[k - 1], tau_old, th_used,
                  (j_spec >= 1 && j_spec <= new_len) ? keys[j_spec - 1] : 0ull);
}

__global__ void topk_output_kernel(TopkWs w, int64_t B, int k, const float* bias, int apply_sigmoid,
                                   float* out_scores, int64_t* out_idx) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= B * k) return;
  const int64_t b = i / k;
  const int j = (int)(i % k);
  float s = __uint_as_float(0x7fc00000u);
  int64_t e = -1;
  if (j < w.list_len[b]) {
    const unsigned long long key = w.list[b * w.kpad + j];
    s = ordered_to_f32((uint32_t)(key >> 32));
    e = (int64_t)(0xffffffffu - (uint32_t)(key & 0xffffffffull));
    if (bias) s += bias[b];
    if (apply_sigmoid) s = 1.0f / (1.0f + expf(-s));
  }
  out_scores[i] = s;
  out_idx[i] = e;
}

// ---- row minimum / maximum ----------------------------------------------------------------------
__global__ void minmax_init_kernel(uint32_t* kmin, uint32_t* kmax, int64_t B) {
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b < B) {
    kmin[b] = 0xffffffffu;
    kmax[b] = 0u;
  }
}
__global__ void minmax_final_kernel(uint32_t* kmin, uint32_t* kmax, const float* bias, int64_t B) {
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b < B) {
    const float add = bias ? bias[b] : 0.f;
    ((float*)kmin)[b] = ordered_to_f32(kmin[b]) + add;
    ((float*)kmax)[b] = ordered_to_f32(kmax[b]) + add;
  }
}

// ---- BCE helpers --------------------------------------------------------------------------------
// accumulators: BCE_SLOTS partial sums of softplus(s), BCE_SLOTS of s, then BCE_POS_SLOTS of the sum over the positives
using host::BCE_POS_SLOTS;
__global__ void bce_init_kernel(double* sums) {
  for (int i = threadIdx.x; i < 2 * BCE_SLOTS + BCE_POS_SLOTS; i += blockDim.x) sums[i] = 0.0;
}

// sum of the logits of the positive (query, tail) pairs.  Grid (queries, BCE_POS_SPLIT): a workgroup is sixteen
// groups of sixteen lanes, and positive j of a query's row goes to group j mod (16 * BCE_POS_SPLIT) of that query's
// workgroups.  The usual row of one or two positives is a single chain of dependent loads (row -> extent -> tail ->
// embedding row) that runs beside every other query's; a row of hundreds is shared out over 64 groups.  One atomic per
// workgroup that found work, spread over a few addresses: thousands of double-precision atomics on one address
// would serialise.
constexpr int BCE_POS_SPLIT = 4;
template <int EDT>
__global__ void __launch_bounds__(256) bce_pos_kernel(ContractArgs a, const float* bias, const int64_t* csr_row,
                                                     const int64_t* row_ptr, const int32_t* col, int64_t n_rows,
                                                     double* sums) {
  __shared__ double s_part[16];
  const int tid = threadIdx.x, grp = tid >> 4, sub = tid & 15;
  const int64_t q = blockIdx.x;
  const int64_t row = csr_row[q];
  if (row < 0 || row >= n_rows) return;
  const int64_t j0 = row_ptr[row], j1 = row_ptr[row + 1];
  const int slot = (int)blockIdx.y * 16 + grp;
  if (j0 + (int64_t)blockIdx.y * 16 >= j1) return;  // nothing for this workgroup (the same for all of it)
  const float bq = bias ? bias[q] : 0.f;
  const float* qv = a.Q + q * a.d;
  double local = 0.0;  // every lane of a group holds the same sum
  for (int64_t j = j0 + slot; j < j1; j += 16 * BCE_POS_SPLIT) {
    const int64_t e = col[j];
    if (e < 0 || e >= a.N) continue;  // uniform across the group
    float dot = 0.f;
    for (int k = sub; k < a.d; k += 16) {
      float x;
      float qk = qv[k];
      if (EDT == KGE_F32) {
        x = ((const float*)a.E)[e * a.d + k];
      } else {
        qk = (float)(__bf16)qk;
        if (EDT == KGE_BF16)
          x = __uint_as_float((uint32_t)((const uint16_t*)a.E)[e * a.d + k] << 16);
        else
          x = (float)((const int8_t*)a.E)[e * a.d + k];
      }
      dot = fmaf(qk, x, dot);
    }
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) dot += __shfl_xor(dot, o, 64);
    if (EDT == KGE_I8) dot *= a.scale[e];
    local += (double)(dot + bq);
  }
  if (sub == 0) s_part[grp] = local;
  __syncthreads();
  if (tid == 0) {
    double t = 0.0;
#pragma unroll
    for (int g = 0; g < 16; ++g) t += s_part[g];
    if (t != 0.0) atomicAdd(&sums[2 * BCE_SLOTS + ((blockIdx.x + blockIdx.y) & (BCE_POS_SLOTS - 1))], t);
  }
}

// one wave: the partial sums are read side by side (one thread reading 384 doubles in turn is a chain of its own)
__global__ void bce_final_kernel(const double* sums, double B, double N, float eps, float* loss) {
  const int lane = threadIdx.x;
  if (blockIdx.x != 0 || lane >= 64) return;
  double t = 0.0, s = 0.0, pos = 0.0;
  for (int i = lane; i < BCE_SLOTS; i += 64) {
    t += sums[i];
    s += sums[BCE_SLOTS + i];
  }
  for (int i = lane; i < BCE_POS_SLOTS; i += 64) pos += sums[2 * BCE_SLOTS + i];
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    t += __shfl_xor(t, o, 64);
    s += __shfl_xor(s, o, 64);
    pos += __shfl_xor(pos, o, 64);
  }
  if (lane == 0) {
    if (eps != 0.f)
      t -= (1.0 - (double)eps) * pos + s / N;
    else
      t -= pos;
    loss[0] = (float)(t / (B * N));
  }
}

// ---- backward of the BCE step: helpers -------------------------------------------------------------
__global__ void fill_zero_kernel(float* p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0.f;
}

// out[c, r] = in[r, c] for a rows x cols matrix (row strides ld_in, ld_out), 32 x 32 tiles through LDS
__global__ void __launch_bounds__(256) transpose_kernel(const float* in, int64_t rows, int64_t cols, int64_t ld_in,
                                                       float* out, int64_t ld_out) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  const int64_t c0 = (int64_t)blockIdx.x * 32, r0 = (int64_t)blockIdx.y * 32;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t r = r0 + ty + 8 * j, c = c0 + tx;
    tile[ty + 8 * j][tx] = (r < rows && c < cols) ? in[r * ld_in + c] : 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t c = c0 + ty + 8 * j, r = r0 + tx;
    if (c < cols && r < rows) out[c * ld_out + r] = tile[tx][ty + 8 * j];
  }
}

// the known tails: y = 1 there, so `pos` is subtracted from both copies of the gradient and from the row sums
__global__ void __launch_bounds__(256) grad_pos_kernel(const int64_t* csr_row, const int64_t* row_ptr,
                                                      const int32_t* col, int64_t n_rows, int64_t B, int64_t N, float* G,
                                                      int64_t ldG, float* GT, int64_t ldT, float* dbias, float pos) {
  for (int64_t q = blockIdx.x; q < B; q += gridDim.x) {
    const int64_t row = csr_row[q];
    if (row < 0 || row >= n_rows) continue;
    const int64_t j0 = row_ptr[row], j1 = row_ptr[row + 1];
    int n_valid = 0;
    for (int64_t j = j0 + threadIdx.x; j < j1; j += blockDim.x) {
      const int64_t e = col[j];
      if (e < 0 || e >= N) continue;
      G[q * ldG + e] -= pos;  // a row's tails are distinct: no two threads touch one element
      if (GT) GT[e * ldT + q] -= pos;
      ++n_valid;
    }
    if (dbias && n_valid) atomicAdd(&dbias[q], -pos * (float)n_valid);
  }
}

// out[i] = sum over y of partial[y][i], y ascending
__global__ void reduce_splits_kernel(const float* partial, int n_splits, int64_t n, float* out) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    float v = 0.f;
    for (int y = 0; y < n_splits; ++y) v += partial[(int64_t)y * n + i];
    out[i] = v;
  }
}

// ============================================================================================
// host side
// ============================================================================================
int check_contract(const char* who, const float* Q, const void* E, int dtype, const float* scale, int64_t B,
                   int64_t d, int64_t N) {
  const host::Status st = host::contract_rules(who, Q, E, dtype, scale, B, d, N);
  return st.ok() ? KGE_OK : set_error(st.code, "%s", st.msg);
}

// bf16 and int8 tables up to 256 elements wide run the persistent kernels, instantiated for LDS rows of 64, 128 or 256
// elements; a table whose rows are narrower than the LDS row of its class takes the PAD form of the same kernel
// (the row's tail stays zero in LDS: d = 200 runs at 0.78 of the d = 256 rate per useful product, against half of
// it in kchunk_kernel; below 64 a tile is bound by its epilogue, not by its K steps, and d = 32 runs at the
// scores-per-second of d = 64).  The 256 class keeps ONE query tile per wave (256-query workgroups): the 16 query
// fragments of a 512-byte row still fit the register file beside the 16 entity fragments.  In the 64 and 256
// classes the filtered rank and kge_scores take the streaming kernel, which runs the previous tile's epilogue inside
// the MFMA chain and suits a short branch-free one (the deferred rank count, a plain store) and not the branching or
// long ones (top-k and row extrema 10 % slower there, BCE twice as slow); those take qreg_async_kernel, epilogue
// after the chain.  Wider tables: kchunk_kernel.
struct RowClass {
  int lds_d;  // elements of an LDS row: 64, 128, 256; 0: wider than any persistent kernel's
  bool pad;   // the table's rows are narrower than that
};
static inline RowClass row_class(int64_t d) {
  const int w = d <= 64 ? 64 : d <= 128 ? 128 : d <= 256 ? 256 : 0;
  return RowClass{w, w != 0 && d != w};
}
constexpr int QS256_WG_QUERIES = QA_WG_WAVES * 32;
// bf16 and int8 tables of 257..512 elements: the query row of one tile per wave in registers, entity rows through LDS
// in segments of 128 columns (qwide_kernel)
static inline bool wide_query_rows(int dtype, int64_t d) { return (dtype == KGE_BF16 || dtype == KGE_I8) && d > 256 && d <= 512; }
template <template <int> class EpiT>
constexpr bool stream256_epilogue() {
  return std::is_same<EpiT<2>, RankEpi<2>>::value || std::is_same<EpiT<2>, StoreEpi<2>>::value;
}
ContractArgs make_args(const float* Q, const void* E, int dtype, const float* scale, int64_t B, int64_t d,
                       int64_t N, int64_t e_begin, int64_t e_end) {
  ContractArgs a;
  a.Q = Q;
  a.E = E;
  a.scale = scale;
  a.B = B;
  a.N = N;
  a.e_begin = e_begin;
  a.e_end = e_end;
  a.d = (int)d;
  a.ldq = a.lde = 0;
  a.k_split_len = 0;
  a.k_split_xcd = 0;
  a.persistent = 0;
  const RowClass rc = row_class(d);
  const bool fast_bf16 = dtype == KGE_BF16 && rc.lds_d != 0;  // (persistent whatever the epilogue)
  const bool fast_i8 = dtype == KGE_I8 && rc.lds_d != 0;
  const bool wide_q = wide_query_rows(dtype, d);  // qwide_kernel: persistent, one 32-query tile per wave
  const bool wide_bf16 = (dtype == KGE_BF16 || dtype == KGE_I8) && rc.lds_d == 0 && !wide_q;  // kchunk_kernel: the workgroup shape of the split kernel
  const int wgq = (dtype == KGE_F32 || wide_bf16) ? KS_WG_QUERIES : wide_q ? QW_WG_QUERIES : rc.lds_d == 256 ? QS256_WG_QUERIES
                  : fast_bf16 ? QA_WG_QUERIES : I8_WG_QUERIES;
  a.n_qgroups = (int)((B + wgq - 1) / wgq);
  if (a.n_qgroups < 1) a.n_qgroups = 1;
  const int64_t rows = e_end - e_begin;
  a.n_lanes = 1;
  if (fast_bf16 || fast_i8 || wide_q) {
    // persistent paths: the workgroups resident on one XCD (32 CUs x workgroups per CU) are shared out
    // among the query groups
    a.n_lanes = 32 * (wide_q ? 1 : fast_bf16 ? QA_WGS_PER_CU : I8_WGS_PER_CU) / a.n_qgroups;
    if (a.n_lanes < 1) a.n_lanes = 1;
    int64_t chunk = rows / (8 * (int64_t)a.n_lanes * 4);  // aim for >= 4 chunks per workgroup
    chunk = (chunk + QA_STAGE_ROWS - 1) / QA_STAGE_ROWS * QA_STAGE_ROWS;
    if (chunk < QA_STAGE_ROWS) chunk = QA_STAGE_ROWS;
    if (chunk > 1024) chunk = 1024;
    a.chunk_rows = (int)chunk;
    a.n_chunks = (rows + chunk - 1) / chunk;
    a.persistent = 1;
    return a;
  }
  // non-persistent paths (the split kernel and kchunk_kernel: 8-wave workgroups of 256 entity rows, one per CU): one
  // workgroup per (query group, chunk), `resident` workgroups at a time; choose the chunk length whose last round of
  // workgroups is fullest, preferring longer chunks (less per-workgroup set-up) among near-equal candidates.
  const int tile = KS_TILE_ROWS;
  const int max_chunk = 1024;
  const int64_t resident = 256;
  int64_t best_chunk = tile;
  double best_eff = -1.0;
  for (int64_t chunk = tile; chunk <= max_chunk; chunk += tile) {
    const int64_t n_chunks = (rows + chunk - 1) / chunk;
    const int64_t wgs = (n_chunks < 8) ? n_chunks * a.n_qgroups : (n_chunks + 7) / 8 * 8 * a.n_qgroups;
    const int64_t rounds = (wgs + resident - 1) / resident;
    const double eff = (double)rows * a.n_qgroups / ((double)rounds * (double)resident * (double)chunk);
    if (eff > best_eff + 0.02) {
      best_eff = eff;
      best_chunk = chunk;
    } else if (eff > best_eff - 0.02 && rounds >= 2) {
      best_chunk = chunk;  // about as full, fewer and longer workgroups
      if (eff > best_eff) best_eff = eff;
    }
  }
  a.chunk_rows = (int)best_chunk;
  a.n_chunks = (rows + best_chunk - 1) / best_chunk;
  return a;
}

// workgroups of a non-persistent contraction launch: what decompose_wg() expects
static int64_t contract_grid_wgs(const ContractArgs& a) {
  return (a.n_chunks < 8) ? a.n_chunks * a.n_qgroups : (a.n_chunks + 7) / 8 * 8 * a.n_qgroups;
}

// HIP events around a main-loop launch while kge_profile_begin() is in effect (the bench's per-launch timing)
struct LaunchTimer {
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  hipStream_t st = nullptr;
  bool timed = false;
  int begin(hipStream_t stream) {
    st = stream;
    {
      std::lock_guard<std::mutex> lk(g_prof_mu);
      timed = g_prof_on;
    }
    if (timed) {
      KGE_HIP_CHECK(hipEventCreate(&ev0));
      KGE_HIP_CHECK(hipEventCreate(&ev1));
      KGE_HIP_CHECK(hipEventRecord(ev0, st));
    }
    return KGE_OK;
  }
  int end(const char* kernel) {
    if (timed) {
      KGE_HIP_CHECK(hipEventRecord(ev1, st));
      std::lock_guard<std::mutex> lk(g_prof_mu);
      g_prof_events.emplace_back(ev0, ev1);
      snprintf(g_prof_kernel, sizeof(g_prof_kernel), "%s", kernel);
    }
    return KGE_OK;
  }
};

template <template <int> class EpiT>
constexpr const char* epilogue_name() {
  using E = EpiT<2>;
  return std::is_same<E, StoreEpi<2>>::value ? "StoreEpi" : std::is_same<E, StoreTEpi<2>>::value ? "StoreTEpi"
       : std::is_same<E, RankEpi<2>>::value ? "RankEpi"
       : std::is_same<E, TopkEpi<2>>::value ? "TopkEpi" : std::is_same<E, TopkKeyEpi<2>>::value ? "TopkKeyEpi"
       : std::is_same<E, TopkFirstEpi<2>>::value ? "TopkFirstEpi" : std::is_same<E, BceEpi<2>>::value ? "BceEpi"
       : std::is_same<E, GradEpi<2>>::value ? "GradEpi" : std::is_same<E, MinMaxEpi<2>>::value ? "MinMaxEpi" : "?";
}

template <template <int> class EpiT, class EArgs>
int launch_contract(int dtype, const ContractArgs& a, const EArgs& ea, hipStream_t st, const char* name) {
  if (a.B == 0 || a.e_end <= a.e_begin) return KGE_OK;
  const RowClass rc = row_class(a.d);
  const bool fast_bf16 = dtype == KGE_BF16 && rc.lds_d != 0;
  const bool fast_i8 = dtype == KGE_I8 && rc.lds_d != 0;
  const bool wide_q = wide_query_rows(dtype, a.d);
  const bool persistent = fast_bf16 || fast_i8 || wide_q;
  const bool pad = rc.pad;
  // (make_args and this function both decide, from the table, between the persistent and the tiled kernels; a plan
  // made for the other kind would be read as garbage, so the two must not drift apart)
  KGE_REQUIRE((a.persistent != 0) == persistent, KGE_ERR_INVALID, "%s: work decomposition planned for another kernel", name);
  const int64_t nwg = persistent ? 8 * (int64_t)a.n_qgroups * a.n_lanes : contract_grid_wgs(a);
  KGE_REQUIRE(nwg <= 0x7fffffffLL, KGE_ERR_INVALID, "%s: grid of %lld workgroups too large", name, (long long)nwg);
  const bool f32_split = (dtype == KGE_F32);
  const bool wide_bf16 = (dtype == KGE_BF16 || dtype == KGE_I8) && rc.lds_d == 0 && !wide_q;
  dim3 grid((unsigned)nwg), block(fast_i8 ? 64 * I8_WG_WAVES : wide_q ? 64 * QW_WG_WAVES : persistent ? 64 * QA_WG_WAVES : 512);
  LaunchTimer timer;
  if (int trc = timer.begin(st)) return trc;
  char kname[160];  // the kernel as dispatched below, for kge_profile_kernel()
  const char* epi = epilogue_name<EpiT>();
  const bool rows_aligned = (a.d % 4 == 0) && (((uintptr_t)a.E | (uintptr_t)a.Q) % 16 == 0);
  if (f32_split) snprintf(kname, sizeof(kname), "ksplit_kernel<%s, %s>", epi, rows_aligned ? "true" : "false");
  else if (wide_bf16) snprintf(kname, sizeof(kname), "kchunk_kernel<%s, %s>", dtype == KGE_BF16 ? "KGE_BF16" : "KGE_I8", epi);
  if (f32_split && rows_aligned)
    hipLaunchKernelGGL((ksplit_kernel<EpiT, true>), grid, block, 0, st, a, ea);
  else if (f32_split)
    hipLaunchKernelGGL((ksplit_kernel<EpiT, false>), grid, block, 0, st, a, ea);
  else if (wide_bf16 && dtype == KGE_BF16)
    hipLaunchKernelGGL((kchunk_kernel<KGE_BF16, EpiT>), grid, block, 0, st, a, ea);
  else if (wide_bf16)
    hipLaunchKernelGGL((kchunk_kernel<KGE_I8, EpiT>), grid, block, 0, st, a, ea);
  else if (wide_q) {
    const int ks = a.d <= 384 ? 24 : 32;
    const bool wpad = a.d != 16 * ks;
    snprintf(kname, sizeof(kname), "qwide_kernel<%s, %s, %d, %s>", dtype == KGE_BF16 ? "KGE_BF16" : "KGE_I8", epi, ks,
             wpad ? "true" : "false");
    auto go = [&](auto edt) {
      constexpr int EDT = decltype(edt)::value;
      if (ks == 24 && !wpad) hipLaunchKernelGGL((qwide_kernel<EDT, EpiT, 24, false>), grid, block, 0, st, a, ea);
      else if (ks == 24) hipLaunchKernelGGL((qwide_kernel<EDT, EpiT, 24, true>), grid, block, 0, st, a, ea);
      else if (!wpad) hipLaunchKernelGGL((qwide_kernel<EDT, EpiT, 32, false>), grid, block, 0, st, a, ea);
      else hipLaunchKernelGGL((qwide_kernel<EDT, EpiT, 32, true>), grid, block, 0, st, a, ea);
    };
    if (dtype == KGE_BF16) go(std::integral_constant<int, KGE_BF16>{});
    else go(std::integral_constant<int, KGE_I8>{});
  }
  else if (fast_bf16) {
    // the rank epilogue has a branch-free form for the deeper-pipelined kernel (same workgroup shape, same counts)
    constexpr bool is_rank = std::is_same<EpiT<2>, RankEpi<2>>::value;
    auto go = [&](auto nqt, auto ksteps, auto padc, auto streamed) {
      constexpr int NQT = decltype(nqt)::value, KS = decltype(ksteps)::value;
      constexpr bool PAD = decltype(padc)::value, STREAMED = decltype(streamed)::value;
      if constexpr (is_rank || STREAMED)
        snprintf(kname, sizeof(kname), "qstream_kernel<%s, %d, %d, %d, %d, %s>", is_rank ? "RankFastEpi" : epi, NQT, QA_WG_WAVES,
                 QA_WAVES_PER_SIMD, KS, PAD ? "true" : "false");
      else
        snprintf(kname, sizeof(kname), "qreg_async_kernel<%s, %d, %d, %s>", epi, NQT, KS, PAD ? "true" : "false");
      if constexpr (is_rank)
        hipLaunchKernelGGL((qstream_kernel<RankFastEpi, NQT, QA_WG_WAVES, QA_WAVES_PER_SIMD, KS, PAD>), grid, block, 0, st, a, ea);
      else if constexpr (STREAMED)
        hipLaunchKernelGGL((qstream_kernel<EpiT, NQT, QA_WG_WAVES, QA_WAVES_PER_SIMD, KS, PAD>), grid, block, 0, st, a, ea);
      else
        hipLaunchKernelGGL((qreg_async_kernel<EpiT, NQT, KS, PAD>), grid, block, 0, st, a, ea);
    };
    using std::integral_constant;
    constexpr bool s256 = stream256_epilogue<EpiT>();
    if (rc.lds_d == 128 && !pad) go(integral_constant<int, QA_NQT>{}, integral_constant<int, 8>{}, std::false_type{}, std::false_type{});
    else if (rc.lds_d == 128) go(integral_constant<int, QA_NQT>{}, integral_constant<int, 8>{}, std::true_type{}, std::false_type{});
    else if (rc.lds_d == 64 && !pad) go(integral_constant<int, QA_NQT>{}, integral_constant<int, 4>{}, std::false_type{}, std::false_type{});
    else if (rc.lds_d == 64) go(integral_constant<int, QA_NQT>{}, integral_constant<int, 4>{}, std::true_type{}, std::false_type{});
    else if (!pad) go(integral_constant<int, 1>{}, integral_constant<int, 16>{}, std::false_type{}, integral_constant<bool, s256>{});
    else go(integral_constant<int, 1>{}, integral_constant<int, 16>{}, std::true_type{}, integral_constant<bool, s256>{});
  }
  else {
    snprintf(kname, sizeof(kname), "qreg_i8_kernel<%s, %d, %d, %s>", epi, rc.lds_d == 256 ? 1 : QREG_NQT, rc.lds_d / 16,
             pad ? "true" : "false");
    if (rc.lds_d == 128 && !pad) hipLaunchKernelGGL((qreg_i8_kernel<EpiT, QREG_NQT, 8, false>), grid, block, 0, st, a, ea);
    else if (rc.lds_d == 128) hipLaunchKernelGGL((qreg_i8_kernel<EpiT, QREG_NQT, 8, true>), grid, block, 0, st, a, ea);
    else if (rc.lds_d == 64 && !pad) hipLaunchKernelGGL((qreg_i8_kernel<EpiT, QREG_NQT, 4, false>), grid, block, 0, st, a, ea);
    else if (rc.lds_d == 64) hipLaunchKernelGGL((qreg_i8_kernel<EpiT, QREG_NQT, 4, true>), grid, block, 0, st, a, ea);
    else if (!pad) hipLaunchKernelGGL((qreg_i8_kernel<EpiT, 1, 16, false>), grid, block, 0, st, a, ea);
    else hipLaunchKernelGGL((qreg_i8_kernel<EpiT, 1, 16, true>), grid, block, 0, st, a, ea);
  }
  KGE_LAUNCH_CHECK(name);
  if (int trc = timer.end(kname)) return trc;
  return KGE_OK;
}

// The filtered-rank main loop of bf16 tables with d == 128: four query tiles per wave (rank128_kernel), when the batch
// fills its 1024-query workgroups about as well as it fills the 512-query ones of the two-tile kernel.
bool rank128_applies(int dtype, int64_t d, int64_t B) {
  if (dtype != KGE_BF16 || d != 128) return false;
  const int64_t slots4 = (B + host::R128_WG_QUERIES - 1) / host::R128_WG_QUERIES * host::R128_WG_QUERIES;
  const int64_t slots2 = (B + QA_WG_QUERIES - 1) / QA_WG_QUERIES * QA_WG_QUERIES;
  return slots4 * 10 <= slots2 * 11;  // at most a tenth more query slots than the two-tile kernel would multiply
}
int launch_rank128(const ContractArgs& base, const RankArgs& ea, hipStream_t st, const char* name) {
  if (base.B == 0 || base.e_end <= base.e_begin) return KGE_OK;
  // At most 16,384 queries per launch: the query groups of a launch share the workgroup slots of an XCD, and with
  // more than sixteen of them a group is left with a single walk over its XCD's share of the table, 32 such walks
  // drift apart and the rows stop being shared through the L2 (C4's table, 32,768 queries: 27.9 against 24.0 ms).
  constexpr int64_t MAX_QUERIES = 16384;
  LaunchTimer timer;
  if (int trc = timer.begin(st)) return trc;
  for (int64_t s = 0; s < base.B; s += MAX_QUERIES) {
    ContractArgs a = base;
    RankArgs eb = ea;
    a.B = base.B - s < MAX_QUERIES ? base.B - s : MAX_QUERIES;
    a.Q = base.Q + s * 128;
    eb.thr += s;
    eb.target += s;
    eb.n_gt += s;
    eb.n_eq += s;
    eb.n_eql += s;
    host::rank128_plan(a.B, a.e_end - a.e_begin, &a.n_qgroups, &a.n_lanes, &a.chunk_rows, &a.n_chunks);
    const int64_t nwg = 8 * (int64_t)a.n_qgroups * a.n_lanes;
    KGE_REQUIRE(nwg <= 0x7fffffffLL, KGE_ERR_INVALID, "%s: grid of %lld workgroups too large", name, (long long)nwg);
    hipLaunchKernelGGL((rank128_kernel<host::R128_WG_WAVES>), dim3((unsigned)nwg), dim3(64 * host::R128_WG_WAVES), 0, st, a, eb);
    KGE_LAUNCH_CHECK(name);
  }
  if (int trc = timer.end("rank128_kernel<8>")) return trc;
  return KGE_OK;
}

// ksplit_kernel alone (fp32 operands), with row strides and an optional split of K over grid.y.
// kmaj (StoreEpi only): bit 0 / bit 1: the entity / query operand is K-major (ksplit_kmajor_kernel).
template <template <int> class EpiT, class EArgs>
int launch_ksplit(const ContractArgs& a, const EArgs& ea, unsigned k_splits, hipStream_t st, const char* name,
                  int kmaj = 0) {
  if (a.B == 0 || a.e_end <= a.e_begin) return KGE_OK;
  const int64_t nwg = contract_grid_wgs(a);
  KGE_REQUIRE(nwg <= 0x7fffffffLL && k_splits >= 1 && k_splits <= 65535, KGE_ERR_INVALID,
              "%s: grid of %lld x %u workgroups too large", name, (long long)nwg, k_splits);
  const int ldq = a.ldq ? a.ldq : a.d, lde = a.lde ? a.lde : a.d;
  const bool rows_aligned = (ldq % 4 == 0) && (lde % 4 == 0) && (((uintptr_t)a.E | (uintptr_t)a.Q) % 16 == 0) &&
                            (a.k_split_len % 4 == 0);
  dim3 grid((unsigned)nwg, k_splits), block(512);
  LaunchTimer timer;
  if (int trc = timer.begin(st)) return trc;
  if constexpr (std::is_same<EpiT<KS_NQT>, StoreEpi<KS_NQT>>::value || std::is_same<EpiT<KS_NQT>, StoreTEpi<KS_NQT>>::value) {
    if (kmaj) {
      // a K-major operand: whole quads of rows, 16-byte aligned (the caller chooses this form only then)
      KGE_REQUIRE(rows_aligned && (a.e_end - a.e_begin) % 4 == 0 && a.e_begin % 4 == 0 && (kmaj == 1 || kmaj == 3),
                  KGE_ERR_INVALID, "%s: K-major operands need aligned quads of rows", name);
      // K ranges in eights with few entity chunks: a flat grid that keeps every range on one XCD (the workgroups of
      // a range read the same rows of the K-major entity operand)
      ContractArgs ax = a;
      if (k_splits % 8 == 0 && a.n_chunks < 8 && nwg * k_splits <= 0x7fffffffLL) {
        ax.k_split_xcd = (int)k_splits;
        grid = dim3((unsigned)(nwg * k_splits), 1);
      }
      if (kmaj == 1) hipLaunchKernelGGL((ksplit_kmajor_kernel<EpiT, 1>), grid, block, 0, st, ax, ea);
      else hipLaunchKernelGGL((ksplit_kmajor_kernel<EpiT, 3>), grid, block, 0, st, ax, ea);
      KGE_LAUNCH_CHECK(name);
      char kname[160];
      snprintf(kname, sizeof(kname), "ksplit_kmajor_kernel<%s, %d>", epilogue_name<EpiT>(), kmaj);
      if (int trc = timer.end(kname)) return trc;
      return KGE_OK;
    }
  }
  if (rows_aligned)
    hipLaunchKernelGGL((ksplit_kernel<EpiT, true>), grid, block, 0, st, a, ea);
  else
    hipLaunchKernelGGL((ksplit_kernel<EpiT, false>), grid, block, 0, st, a, ea);
  KGE_LAUNCH_CHECK(name);
  char kname[160];
  snprintf(kname, sizeof(kname), "ksplit_kernel<%s, %s>", epilogue_name<EpiT>(), rows_aligned ? "true" : "false");
  if (int trc = timer.end(kname)) return trc;
  return KGE_OK;
}

#define KGE_DISPATCH_DTYPE(dtype, KERNEL, grid, block, shmem, st, ...)                       \
  do {                                                                                       \
    if ((dtype) == KGE_F32)                                                                  \
      hipLaunchKernelGGL((KERNEL<KGE_F32>), grid, block, shmem, st, __VA_ARGS__);            \
    else if ((dtype) == KGE_BF16)                                                            \
      hipLaunchKernelGGL((KERNEL<KGE_BF16>), grid, block, shmem, st, __VA_ARGS__);           \
    else                                                                                     \
      hipLaunchKernelGGL((KERNEL<KGE_I8>), grid, block, shmem, st, __VA_ARGS__);             \
  } while (0)

struct RankWs {
  float* thr;
  FixPlan plan;
};
// plan `sub` of the workspace laid out at `base` (one plan per sub-batch of SORT_MAX queries)
size_t rank_ws_layout(int64_t B, void* base, RankWs* ws, int64_t sub = 0) {
  const host::RankWsOffsets o = host::rank_ws_offsets(B);
  if (ws) {
    char* p = (char*)base;
    char* pl = p + o.plans + (size_t)sub * o.plan_stride;
    ws->thr = (float*)(p + o.thr);
    ws->plan.skey = (unsigned long long*)(pl + o.skey);
    ws->plan.gend = (int32_t*)(pl + o.gend);
    ws->plan.work = (int32_t*)(pl + o.work);
    ws->plan.meta = (int32_t*)(pl + o.meta);
    ws->plan.lead = (int32_t*)(p + o.lead);
    ws->plan.mixed = (int32_t*)(p + o.mixed);
  }
  return o.total;
}

}  // namespace
}  // namespace kge

using namespace kge;

extern "C" const char* kge_last_error(void) { return g_err; }
extern "C" int kge_abi_version(void) { return KGE_ABI_VERSION; }

extern "C" int kge_profile_begin(void) {
  clear_error();
  std::lock_guard<std::mutex> lk(g_prof_mu);
  for (auto& p : g_prof_events) {
    (void)hipEventDestroy(p.first);
    (void)hipEventDestroy(p.second);
  }
  g_prof_events.clear();
  g_prof_on = true;
  return KGE_OK;
}

extern "C" int kge_profile_end(double* total_ms, int64_t* launches) {
  clear_error();
  std::vector<std::pair<hipEvent_t, hipEvent_t>> evs;
  {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof_on = false;
    evs.swap(g_prof_events);
  }
  double total = 0.0;
  int rc = KGE_OK;
  for (auto& p : evs) {
    float ms = 0.f;
    hipError_t e = hipEventSynchronize(p.second);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, p.first, p.second);
    if (e != hipSuccess) rc = set_error(KGE_ERR_HIP, "kge_profile_end: %s", hipGetErrorString(e));
    total += ms;
    (void)hipEventDestroy(p.first);
    (void)hipEventDestroy(p.second);
  }
  if (total_ms) *total_ms = total;
  if (launches) *launches = (int64_t)evs.size();
  return rc;
}

extern "C" const char* kge_profile_kernel(void) {
  static thread_local char out[160];
  std::lock_guard<std::mutex> lk(g_prof_mu);
  snprintf(out, sizeof(out), "%s", g_prof_kernel);
  return out;
}

extern "C" int kge_scores(const float* Q, const float* bias, const void* E, int dtype, const float* scale, int64_t B,
                          int64_t d, int64_t N, float* S, int64_t ldS, void* stream) {
  clear_error();
  int rc = check_contract("kge_scores", Q, E, dtype, scale, B, d, N);
  if (rc) return rc;
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(S && ldS >= N, KGE_ERR_INVALID, "kge_scores: S is null or ldS=%lld < N=%lld", (long long)ldS,
              (long long)N);
  ContractArgs a = make_args(Q, E, dtype, scale, B, d, N, 0, N);
  StoreArgs ea{S, bias, ldS, 0};
  return launch_contract<StoreEpi>(dtype, a, ea, (hipStream_t)stream, "kge_scores");
}

extern "C" int kge_triple_scores(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                                 int64_t B, int64_t d, int64_t N, const int64_t* entity, float* out, void* stream) {
  clear_error();
  int rc = check_contract("kge_triple_scores", Q, E, dtype, scale, B, d, N);
  if (rc) return rc;
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(entity && out, KGE_ERR_INVALID, "kge_triple_scores: null entity or output pointer");
  ContractArgs a = make_args(Q, E, dtype, scale, B, d, N, 0, N);
  dim3 grid((unsigned)((B + 127) / 128)), block(256);
  hipStream_t st = (hipStream_t)stream;
  KGE_DISPATCH_DTYPE(dtype, triple_score_kernel, grid, block, 0, st, a, entity, bias, out, (int64_t)1);
  KGE_LAUNCH_CHECK("triple_score_kernel");
  return KGE_OK;
}

extern "C" int kge_sample_scores(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                                 int64_t B, int64_t d, int64_t N, const int64_t* entity, int64_t k, float* out,
                                 void* stream) {
  clear_error();
  int rc = check_contract("kge_sample_scores", Q, E, dtype, scale, B, d, N);
  if (rc) return rc;
  KGE_REQUIRE(k >= 0, KGE_ERR_INVALID, "kge_sample_scores: k=%lld", (long long)k);
  if (B == 0 || k == 0) return KGE_OK;
  KGE_REQUIRE(entity && out, KGE_ERR_INVALID, "kge_sample_scores: null entity or output pointer");
  const int64_t total = B * k;
  KGE_REQUIRE((total + 127) / 128 <= 0x7fffffffLL, KGE_ERR_INVALID, "kge_sample_scores: B * k = %lld too large",
              (long long)total);
  ContractArgs a = make_args(Q, E, dtype, scale, B, d, N, 0, N);
  dim3 grid((unsigned)((total + 127) / 128)), block(256);
  hipStream_t st = (hipStream_t)stream;
  KGE_DISPATCH_DTYPE(dtype, triple_score_kernel, grid, block, 0, st, a, entity, bias, out, k);
  KGE_LAUNCH_CHECK("triple_score_kernel");
  return KGE_OK;
}

extern "C" int kge_csr_lookup(const int64_t* hr, int64_t B, const int64_t* keys, int64_t n_rows,
                              int64_t num_relations, int64_t* csr_row, void* stream) {
  clear_error();
  KGE_REQUIRE(B >= 0 && n_rows >= 0 && num_relations >= 1, KGE_ERR_INVALID, "kge_csr_lookup: B=%lld n_rows=%lld R=%lld",
              (long long)B, (long long)n_rows, (long long)num_relations);
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(hr && csr_row && (keys || n_rows == 0), KGE_ERR_INVALID, "kge_csr_lookup: null pointer argument");
  hipLaunchKernelGGL(csr_lookup_kernel, dim3((unsigned)((B + 255) / 256)), dim3(256), 0, (hipStream_t)stream, hr, B, keys,
                     n_rows, num_relations, csr_row);
  KGE_LAUNCH_CHECK("csr_lookup_kernel");
  return KGE_OK;
}

extern "C" size_t kge_rank_workspace_bytes(int64_t B) { return rank_ws_layout(B < 1 ? 1 : B, nullptr, nullptr); }

namespace {
// argument checks shared by the two filtered-rank entry points
int check_rank_args(const char* who, const float* Q, const void* E, int dtype, const float* scale, int64_t B, int64_t d,
                    int64_t N, const int64_t* target, const int64_t* csr_row, const int64_t* row_ptr, const int32_t* col,
                    int64_t n_rows, const int32_t* n_greater, const int32_t* n_equal, const int32_t* n_equal_lower,
                    const float* target_score) {
  int rc = check_contract(who, Q, E, dtype, scale, B, d, N);
  if (rc) return rc;
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(target && n_greater && n_equal && n_equal_lower && target_score, KGE_ERR_INVALID,
              "%s: null target or output pointer", who);
  KGE_REQUIRE(!csr_row || (row_ptr && col && n_rows >= 0), KGE_ERR_INVALID, "%s: csr_row given without row_ptr / col", who);
  KGE_REQUIRE(n_rows < 0x7fffffffLL, KGE_ERR_INVALID, "%s: n_rows=%lld too large", who, (long long)n_rows);
  return KGE_OK;
}

// the launches of a filtered-rank call; `ws_base` is a caller's workspace or the library's static scratch.
// Order: the plan of every sub-batch (it only needs the filter rows, and tells every query its group's leader),
// thresholds + counters + the one-vector-per-group check, the main loop, the filter correction of every sub-batch.
int rank_filtered_launch(const char* who, const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                         int64_t B, int64_t d, int64_t N, const int64_t* target, const int64_t* csr_row,
                         const int64_t* row_ptr, const int32_t* col, int64_t n_rows, int32_t* n_greater, int32_t* n_equal,
                         int32_t* n_equal_lower, float* target_score, void* ws_base, hipStream_t st,
                         const float* thr_in = nullptr, bool one_vector_per_row = false) {
  ContractArgs a = make_args(Q, E, dtype, scale, B, d, N, 0, N);
  const bool filtered = csr_row != nullptr && n_rows > 0;
  RankWs ws;
  rank_ws_layout(B, ws_base, &ws);
  if (thr_in) ws.thr = const_cast<float*>(thr_in);  // formed (and the counters initialised) by kge_rank_thresholds
  if (filtered) {
    for (int64_t b0 = 0, sub = 0; b0 < B; b0 += SORT_MAX, ++sub) {
      const int nb = (int)((B - b0 < SORT_MAX) ? B - b0 : SORT_MAX);
      RankWs wsub;
      rank_ws_layout(B, ws_base, &wsub, sub);
      hipLaunchKernelGGL(plan_fix_kernel, dim3(1), dim3(1024), 0, st, csr_row, b0, nb, n_rows, row_ptr, wsub.plan);
      KGE_LAUNCH_CHECK("plan_fix_kernel");
    }
  }
  if (!thr_in) {
    dim3 grid((unsigned)((B + 127) / 128 * (filtered ? 2 : 1))), block(256);  // (second half: the group check)
    KGE_DISPATCH_DTYPE(dtype, target_score_kernel, grid, block, 0, st, a, target, bias, ws.thr, target_score,
                       n_greater, n_equal, n_equal_lower, filtered ? (const int32_t*)ws.plan.lead : (const int32_t*)nullptr,
                       ws.plan.mixed);
    KGE_LAUNCH_CHECK("target_score_kernel");
  } else if (filtered && !one_vector_per_row) {
    hipLaunchKernelGGL(group_check_kernel, dim3((unsigned)((B + 127) / 128)), dim3(256), 0, st, a,
                       (const int32_t*)ws.plan.lead, ws.plan.mixed);
    KGE_LAUNCH_CHECK("group_check_kernel");
  }
  RankArgs ea{ws.thr, target, n_greater, n_equal, n_equal_lower};
  int rc = rank128_applies(dtype, d, B) ? launch_rank128(a, ea, st, who) : launch_contract<RankEpi>(dtype, a, ea, st, who);
  if (rc) return rc;
  if (filtered) {
    for (int64_t b0 = 0, sub = 0; b0 < B; b0 += SORT_MAX, ++sub) {
      RankWs wsub;
      rank_ws_layout(B, ws_base, &wsub, sub);
      dim3 grid(2048), block(256);
      if (dtype == KGE_F32)
        hipLaunchKernelGGL((filter_fix_kernel<KGE_F32, false>), grid, block, 0, st, a, wsub.plan, b0, row_ptr, col, target,
                           ws.thr, n_greater, n_equal, n_equal_lower);
      else if (dtype == KGE_BF16 && d == 128)
        hipLaunchKernelGGL((filter_fix_kernel<KGE_BF16, true>), grid, block, 0, st, a, wsub.plan, b0, row_ptr, col, target,
                           ws.thr, n_greater, n_equal, n_equal_lower);
      else if (dtype == KGE_BF16)
        hipLaunchKernelGGL((filter_fix_kernel<KGE_BF16, false>), grid, block, 0, st, a, wsub.plan, b0, row_ptr, col, target,
                           ws.thr, n_greater, n_equal, n_equal_lower);
      else
        hipLaunchKernelGGL((filter_fix_kernel<KGE_I8, false>), grid, block, 0, st, a, wsub.plan, b0, row_ptr, col, target,
                           ws.thr, n_greater, n_equal, n_equal_lower);
      KGE_LAUNCH_CHECK("filter_fix_kernel");
    }
  }
  return KGE_OK;
}
}  // namespace

extern "C" int kge_rank_filtered(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                                 int64_t B, int64_t d, int64_t N, const int64_t* target, const int64_t* csr_row,
                                 const int64_t* row_ptr, const int32_t* col, int64_t n_rows, int32_t* n_greater,
                                 int32_t* n_equal, int32_t* n_equal_lower, float* target_score, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  clear_error();
  int rc = check_rank_args("kge_rank_filtered", Q, E, dtype, scale, B, d, N, target, csr_row, row_ptr, col, n_rows,
                           n_greater, n_equal, n_equal_lower, target_score);
  if (rc) return rc;
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(workspace && workspace_bytes >= kge_rank_workspace_bytes(B), KGE_ERR_WORKSPACE,
              "kge_rank_filtered: workspace of %zu bytes, need %zu", workspace_bytes, kge_rank_workspace_bytes(B));
  KGE_REQUIRE(((uintptr_t)workspace & 7) == 0, KGE_ERR_WORKSPACE, "kge_rank_filtered: workspace must be 8-byte aligned");
  return rank_filtered_launch("kge_rank_filtered", Q, bias, E, dtype, scale, B, d, N, target, csr_row, row_ptr, col,
                              n_rows, n_greater, n_equal, n_equal_lower, target_score, workspace, (hipStream_t)stream);
}

// ---- thresholds of many batches at once, and the rank call that takes them ------------------------------
extern "C" int kge_rank_thresholds(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                                   int64_t B, int64_t d, int64_t N, const int64_t* target, float* thr,
                                   int32_t* n_greater, int32_t* n_equal, int32_t* n_equal_lower, float* target_score,
                                   void* stream) {
  clear_error();
  int rc = check_rank_args("kge_rank_thresholds", Q, E, dtype, scale, B, d, N, target, nullptr, nullptr, nullptr, 0,
                           n_greater, n_equal, n_equal_lower, target_score);
  if (rc) return rc;
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(thr != nullptr, KGE_ERR_INVALID, "kge_rank_thresholds: null threshold array");
  KGE_REQUIRE((B + 127) / 128 <= 0x7fffffffLL, KGE_ERR_INVALID, "kge_rank_thresholds: B=%lld too large", (long long)B);
  ContractArgs a = make_args(Q, E, dtype, scale, B, d, N, 0, N);
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)((B + 127) / 128)), block(256);
  KGE_DISPATCH_DTYPE(dtype, target_score_kernel, grid, block, 0, st, a, target, bias, thr, target_score, n_greater,
                     n_equal, n_equal_lower, (const int32_t*)nullptr, (int32_t*)nullptr);
  KGE_LAUNCH_CHECK("target_score_kernel");
  return KGE_OK;
}

extern "C" int kge_rank_filtered_with_thresholds(const float* Q, const void* E, int dtype, const float* scale, int64_t B,
                                                 int64_t d, int64_t N, const int64_t* target, const float* thr,
                                                 const int64_t* csr_row, const int64_t* row_ptr, const int32_t* col,
                                                 int64_t n_rows, int one_vector_per_row, int32_t* n_greater,
                                                 int32_t* n_equal, int32_t* n_equal_lower, void* workspace,
                                                 size_t workspace_bytes, void* stream) {
  clear_error();
  float dummy = 0.f;  // (target_score was written by kge_rank_thresholds; the argument check only wants a non-null pointer)
  int rc = check_rank_args("kge_rank_filtered_with_thresholds", Q, E, dtype, scale, B, d, N, target, csr_row, row_ptr,
                           col, n_rows, n_greater, n_equal, n_equal_lower, &dummy);
  if (rc) return rc;
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(thr != nullptr, KGE_ERR_INVALID, "kge_rank_filtered_with_thresholds: null threshold array");
  KGE_REQUIRE(workspace && workspace_bytes >= kge_rank_workspace_bytes(B), KGE_ERR_WORKSPACE,
              "kge_rank_filtered_with_thresholds: workspace of %zu bytes, need %zu", workspace_bytes,
              kge_rank_workspace_bytes(B));
  KGE_REQUIRE(((uintptr_t)workspace & 7) == 0, KGE_ERR_WORKSPACE,
              "kge_rank_filtered_with_thresholds: workspace must be 8-byte aligned");
  return rank_filtered_launch("kge_rank_filtered_with_thresholds", Q, nullptr, E, dtype, scale, B, d, N, target, csr_row,
                              row_ptr, col, n_rows, n_greater, n_equal, n_equal_lower, nullptr, workspace,
                              (hipStream_t)stream, thr, one_vector_per_row != 0);
}

// ---- the same call for callers that cannot allocate ---------------------------------------------------
// The workspace of kge_rank_filtered (thresholds, the plan of the filter correction) lives in a file-scope
// device array instead of caller memory.  Every GPU the library runs on holds its own copy of the array at its
// own address until the process ends; the address is looked up once per device and only that pointer is ever
// handed to a kernel.  All calls on one GPU share the array: calls that overlap on one GPU race.
static __device__ __align__(256) unsigned char scratch[KGE_RANK_STATIC_SCRATCH_BYTES];

namespace {
constexpr int SCRATCH_MAX_DEVICES = 64;
std::mutex g_scratch_mu;
unsigned char* g_scratch_ptr[SCRATCH_MAX_DEVICES] = {};

// device address of `scratch` on the current device (looked up on the first call on that device)
int scratch_on_current_device(unsigned char** out) {
  int dev = -1;
  KGE_HIP_CHECK(hipGetDevice(&dev));
  KGE_REQUIRE(dev >= 0 && dev < SCRATCH_MAX_DEVICES, KGE_ERR_UNSUPPORTED, "device ordinal %d outside [0, %d)", dev,
              SCRATCH_MAX_DEVICES);
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    KGE_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    KGE_REQUIRE(p != nullptr, KGE_ERR_HIP, "hipGetSymbolAddress returned a null address for the scratch array");
    g_scratch_ptr[dev] = (unsigned char*)p;
  }
  *out = g_scratch_ptr[dev];
  return KGE_OK;
}
}  // namespace

extern "C" int kge_rank_static_init(void) {
  clear_error();
  unsigned char* base = nullptr;
  return scratch_on_current_device(&base);
}

extern "C" int kge_rank_filtered_static(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                                        int64_t B, int64_t d, int64_t N, const int64_t* target, const int64_t* csr_row,
                                        const int64_t* row_ptr, const int32_t* col, int64_t n_rows, int32_t* n_greater,
                                        int32_t* n_equal, int32_t* n_equal_lower, float* target_score, void* stream) {
  clear_error();
  int rc = check_rank_args("kge_rank_filtered_static", Q, E, dtype, scale, B, d, N, target, csr_row, row_ptr, col, n_rows,
                           n_greater, n_equal, n_equal_lower, target_score);
  if (rc) return rc;
  KGE_REQUIRE(B <= KGE_RANK_STATIC_MAX_B, KGE_ERR_WORKSPACE,
              "kge_rank_filtered_static: B=%lld exceeds the %d queries the static scratch array holds; split the batch "
              "or call kge_rank_filtered with a workspace", (long long)B, KGE_RANK_STATIC_MAX_B);
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(rank_ws_layout(B, nullptr, nullptr) <= sizeof(scratch), KGE_ERR_WORKSPACE,
              "kge_rank_filtered_static: internal layout of %zu bytes exceeds the scratch array",
              rank_ws_layout(B, nullptr, nullptr));
  unsigned char* base = nullptr;
  rc = scratch_on_current_device(&base);
  if (rc) return rc;
  // the scratch array used is the current device's: the operands must live there too (where the runtime cannot say,
  // e.g. under a capture mode that refuses the query, the rule stays the caller's to keep)
  {
    int cur = -1;
    KGE_HIP_CHECK(hipGetDevice(&cur));
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, Q) == hipSuccess) {
      KGE_REQUIRE(attr.device == cur, KGE_ERR_INVALID,
                  "kge_rank_filtered_static: Q lives on device %d, the current device is %d", attr.device, cur);
    } else {
      (void)hipGetLastError();
    }
  }
  // nothing in the scratch needs clearing: thresholds, leaders and the mixed-group flags are written for every
  // query and every sub-batch's plan is rebuilt before anything reads it, so what an earlier call left behind is
  // never read
  return rank_filtered_launch("kge_rank_filtered_static", Q, bias, E, dtype, scale, B, d, N, target, csr_row, row_ptr,
                              col, n_rows, n_greater, n_equal, n_equal_lower, target_score, base, (hipStream_t)stream);
}

extern "C" size_t kge_topk_workspace_bytes(int64_t B, int64_t N, int64_t k) {
  if (B < 1) B = 1;
  if (N < 1) N = 1;
  if (k < 1) k = 1;
  if (k > TOPK_MAX_K) k = TOPK_MAX_K;
  return topk_ws_layout(B, N, k, nullptr, nullptr);
}

namespace {
// does a table of this storage and width have a prepared form for top-k?
bool topk_has_prepared_form(int dtype, int64_t d) { return dtype == KGE_I8 && d == host::TOPK_REQUANT_D; }

int topk_prepare_launch(const void* E, const float* scale, int64_t N, unsigned char* rowmeta, int8_t* requant,
                        hipStream_t st) {
  const int64_t n_rec = (N + host::TOPK_ROWMETA_ROWS - 1) / host::TOPK_ROWMETA_ROWS;
  hipLaunchKernelGGL(topk_i8_requant_kernel, dim3((unsigned)n_rec), dim3(256), 0, st, (const int8_t*)E, scale, N, requant,
                     rowmeta);
  KGE_LAUNCH_CHECK("topk_i8_requant_kernel");
  return KGE_OK;
}

int topk_impl(const char* who, const float* Q, const float* bias, const void* E, int dtype, const float* scale, int64_t B,
              int64_t d, int64_t N, int64_t k, float* out_scores, int64_t* out_idx, int apply_sigmoid,
              const void* prepared, void* workspace, hipStream_t st);
}  // namespace

extern "C" size_t kge_topk_prepared_bytes(int dtype, int64_t d, int64_t N) {
  if (!topk_has_prepared_form(dtype, d) || N < 1) return 0;
  return host::topk_prepared_offsets(N).total;
}

extern "C" int kge_topk_prepare(const void* E, int dtype, const float* scale, int64_t d, int64_t N, void* prepared,
                                size_t prepared_bytes, void* stream) {
  clear_error();
  KGE_REQUIRE(topk_has_prepared_form(dtype, d), KGE_ERR_UNSUPPORTED,
              "kge_topk_prepare: tables of dtype %d with d=%lld have no prepared form (int8 with d = %d does)", dtype,
              (long long)d, host::TOPK_REQUANT_D);
  KGE_REQUIRE(N >= 1 && N <= 0x7fffffffLL, KGE_ERR_INVALID, "kge_topk_prepare: N=%lld", (long long)N);
  KGE_REQUIRE(E && scale && prepared, KGE_ERR_INVALID, "kge_topk_prepare: null pointer argument");
  KGE_REQUIRE((((uintptr_t)E | (uintptr_t)prepared) & 15) == 0, KGE_ERR_INVALID,
              "kge_topk_prepare: E and prepared must be 16-byte aligned");
  KGE_REQUIRE(prepared_bytes >= kge_topk_prepared_bytes(dtype, d, N), KGE_ERR_WORKSPACE,
              "kge_topk_prepare: buffer of %zu bytes, need %zu", prepared_bytes, kge_topk_prepared_bytes(dtype, d, N));
  const host::TopkPreparedOffsets t = host::topk_prepared_offsets(N);
  return topk_prepare_launch(E, scale, N, (unsigned char*)prepared + t.rowmeta,
                             (int8_t*)((unsigned char*)prepared + t.requant), (hipStream_t)stream);
}

extern "C" size_t kge_topk_prepared_workspace_bytes(int64_t B, int64_t N, int64_t k) {
  if (B < 1) B = 1;
  if (N < 1) N = 1;
  if (k < 1) k = 1;
  if (k > TOPK_MAX_K) k = TOPK_MAX_K;
  return topk_ws_layout(B, N, k, nullptr, nullptr, nullptr, false);
}

extern "C" int kge_topk(const float* Q, const float* bias, const void* E, int dtype, const float* scale, int64_t B,
                        int64_t d, int64_t N, int64_t k, float* out_scores, int64_t* out_idx, int apply_sigmoid,
                        void* workspace, size_t workspace_bytes, void* stream) {
  clear_error();
  int rc = check_contract("kge_topk", Q, E, dtype, scale, B, d, N);
  if (rc) return rc;
  KGE_REQUIRE(k >= 1 && k <= N, KGE_ERR_INVALID, "kge_topk: k=%lld outside [1, N=%lld]", (long long)k, (long long)N);
  KGE_REQUIRE(k <= TOPK_MAX_K, KGE_ERR_UNSUPPORTED, "kge_topk: k=%lld above the supported maximum %d", (long long)k,
              TOPK_MAX_K);
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(out_scores && out_idx, KGE_ERR_INVALID, "kge_topk: null output pointer");
  KGE_REQUIRE(workspace && workspace_bytes >= kge_topk_workspace_bytes(B, N, k), KGE_ERR_WORKSPACE,
              "kge_topk: workspace of %zu bytes, need %zu", workspace_bytes, kge_topk_workspace_bytes(B, N, k));
  KGE_REQUIRE(((uintptr_t)workspace & 15) == 0, KGE_ERR_WORKSPACE, "kge_topk: workspace must be 16-byte aligned");
  return topk_impl("kge_topk", Q, bias, E, dtype, scale, B, d, N, k, out_scores, out_idx, apply_sigmoid, nullptr,
                   workspace, (hipStream_t)stream);
}

extern "C" int kge_topk_prepared(const float* Q, const float* bias, const void* E, int dtype, const float* scale, int64_t B,
                                 int64_t d, int64_t N, int64_t k, float* out_scores, int64_t* out_idx, int apply_sigmoid,
                                 const void* prepared, size_t prepared_bytes, void* workspace, size_t workspace_bytes,
                                 void* stream) {
  clear_error();
  int rc = check_contract("kge_topk_prepared", Q, E, dtype, scale, B, d, N);
  if (rc) return rc;
  KGE_REQUIRE(k >= 1 && k <= N, KGE_ERR_INVALID, "kge_topk_prepared: k=%lld outside [1, N=%lld]", (long long)k,
              (long long)N);
  KGE_REQUIRE(k <= TOPK_MAX_K, KGE_ERR_UNSUPPORTED, "kge_topk_prepared: k=%lld above the supported maximum %d",
              (long long)k, TOPK_MAX_K);
  KGE_REQUIRE(topk_has_prepared_form(dtype, d), KGE_ERR_UNSUPPORTED,
              "kge_topk_prepared: tables of dtype %d with d=%lld have no prepared form; call kge_topk", dtype, (long long)d);
  KGE_REQUIRE(prepared && prepared_bytes >= kge_topk_prepared_bytes(dtype, d, N), KGE_ERR_WORKSPACE,
              "kge_topk_prepared: prepared table of %zu bytes, need %zu", prepared_bytes,
              kge_topk_prepared_bytes(dtype, d, N));
  KGE_REQUIRE(((uintptr_t)prepared & 15) == 0, KGE_ERR_INVALID, "kge_topk_prepared: prepared must be 16-byte aligned");
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(out_scores && out_idx, KGE_ERR_INVALID, "kge_topk_prepared: null output pointer");
  KGE_REQUIRE(workspace && workspace_bytes >= kge_topk_prepared_workspace_bytes(B, N, k), KGE_ERR_WORKSPACE,
              "kge_topk_prepared: workspace of %zu bytes, need %zu", workspace_bytes,
              kge_topk_prepared_workspace_bytes(B, N, k));
  KGE_REQUIRE(((uintptr_t)workspace & 15) == 0, KGE_ERR_WORKSPACE, "kge_topk_prepared: workspace must be 16-byte aligned");
  return topk_impl("kge_topk_prepared", Q, bias, E, dtype, scale, B, d, N, k, out_scores, out_idx, apply_sigmoid, prepared,
                   workspace, (hipStream_t)stream);
}

namespace {
int topk_impl(const char* who, const float* Q, const float* bias, const void* E, int dtype, const float* scale, int64_t B,
              int64_t d, int64_t N, int64_t k, float* out_scores, int64_t* out_idx, int apply_sigmoid,
              const void* prepared, void* workspace, hipStream_t st) {
  int rc = KGE_OK;
  TopkWs ws;
  topk_ws_layout(B, N, k, workspace, &ws, prepared, prepared == nullptr);
  const int64_t first_rows = (N < TOPK_FIRST_ROWS) ? N : TOPK_FIRST_ROWS;
  hipLaunchKernelGGL(topk_init_kernel, dim3((unsigned)((B + 255) / 256)), dim3(256), 0, st, ws, B, (int32_t)first_rows);
  KGE_LAUNCH_CHECK("topk_init_kernel");

  // An int8 table with d == 128 is scanned by the integer filter (after the first round, which takes every row
  // anyway): its candidates are entity ids that passed a bound, scored exactly before they are ranked.  Every other
  // scan is the contraction's own top-k epilogue, whose candidates are exact keys.  The filter reads the table in
  // its prepared form (the caller's, or made here in the workspace) and the queries as int8 (made here).
  const bool id_filter = (topk_has_prepared_form(dtype, d) && N > TOPK_FIRST_ROWS);
  if (id_filter) {
    if (prepared == nullptr) {
      rc = topk_prepare_launch(E, scale, N, ws.rowmeta, ws.requant, st);
      if (rc) return rc;
    }
    hipLaunchKernelGGL(topk_i8_qprep_kernel, dim3((unsigned)((B + 3) / 4)), dim3(256), 0, st, Q, B, ws.qh, ws.qc);
    KGE_LAUNCH_CHECK("topk_i8_qprep_kernel");
  }
  // One scan of entity rows [e0, e1) with the thresholds `tau`, for all queries or those flagged in `active`.
  bool scan_was_filter = false;  // the last scan went through the int8 filter: its candidate buffers hold zeros
  auto launch_scan = [&](int64_t e0, int64_t e1, const float* tau, const int32_t* active, int rescan,
                         const char* name) -> int {
    scan_was_filter = false;
    ContractArgs a = make_args(Q, E, dtype, scale, B, d, N, e0, e1);
    if (e0 == 0 && !rescan) {
      // the first round: every row a candidate, written as dense keys (the candidate counts were set to match)
      TopkFirstArgs ef{ws.cand, (int64_t)TOPK_CAP, e0};
      return launch_contract<TopkFirstEpi>(dtype, a, ef, st, name);
    }
    // (the repair scan is exact as well: a query the bound cannot separate from most of the table, its threshold
    // tiny against the scales around it, would overflow its buffer again)
    // (short rounds are exact as well: the filter's extra launch to score its candidates, and the candidates its
    // bound lets through needlessly, cost more there than the exact epilogue does)
    if (!id_filter || rescan || e0 % host::TOPK_ROWMETA_ROWS != 0 || e1 - e0 <= host::TOPK_FILTER_MIN_ROWS) {
      if (rescan) {
        // a repair scan admits what ranks above the query's k-th best by KEY, so that ties with it at lower entity
        // ids, which an overflowing buffer may have dropped, are found again
        TopkKeyArgs ek;
        ek.tau = tau; ek.active = active; ek.cnt = ws.cnt; ek.cand = ws.cand; ek.cap = TOPK_CAP; ek.kth = ws.kth;
        return launch_contract<TopkKeyEpi>(dtype, a, ek, st, name);
      }
      TopkArgs ea{tau, active, ws.cnt, ws.cand, TOPK_CAP};
      return launch_contract<TopkEpi>(dtype, a, ea, st, name);
    }
    if (e1 <= e0) return KGE_OK;
    scan_was_filter = true;
    // the filter's workgroups cover TF_WG_QUERIES queries, one workgroup per CU: the same walk, its own shape
    a.n_qgroups = (int)((B + TF_WG_QUERIES - 1) / TF_WG_QUERIES);
    a.n_lanes = 32 / a.n_qgroups;
    if (a.n_lanes < 1) a.n_lanes = 1;
    int64_t chunk = (e1 - e0) / (8 * (int64_t)a.n_lanes * 4);
    chunk = (chunk + TF_STAGE_ROWS - 1) / TF_STAGE_ROWS * TF_STAGE_ROWS;
    if (chunk < TF_STAGE_ROWS) chunk = TF_STAGE_ROWS;
    if (chunk > 1024) chunk = 1024;
    a.chunk_rows = (int)chunk;
    a.n_chunks = (e1 - e0 + chunk - 1) / chunk;
    const int64_t nwg = 8 * (int64_t)a.n_qgroups * a.n_lanes;
    KGE_REQUIRE(nwg <= 0x7fffffffLL, KGE_ERR_INVALID, "%s: grid of %lld workgroups too large", name, (long long)nwg);
    I8FilterArgs ea{tau, active, ws.cnt, ws.cand_id, TOPK_CAP, ws.requant, ws.rowmeta, ws.qh, ws.qc};
    LaunchTimer timer;
    if (int trc = timer.begin(st)) return trc;
    hipLaunchKernelGGL(topk_i8_filter_kernel, dim3((unsigned)nwg), dim3(64 * TF_W), 0, st, a, ea);
    KGE_LAUNCH_CHECK(name);
    if (int trc = timer.end("topk_i8_filter_kernel")) return trc;
    hipLaunchKernelGGL(topk_rescore_kernel, dim3((unsigned)B, 4), dim3(256), 0, st, ws, a);
    KGE_LAUNCH_CHECK("topk_rescore_kernel");
    return KGE_OK;
  };
  // ranks the list (<= k entries) and this round's candidates (<= min(TOPK_CAP, rows scanned) entries) of every
  // query; j_spec: the rank whose score the next scan may use as its threshold (k: the k-th best itself)
  auto launch_select = [&](int64_t rows, int rescan, int64_t j_spec) {
    hipLaunchKernelGGL(topk_select_wave_kernel, dim3((unsigned)B), dim3(64), 0, st, ws, (int)k, rescan, (int)j_spec,
                       scan_was_filter ? 1 : 0);
    if (k + (rows < TOPK_CAP ? rows : TOPK_CAP) > SELECT_SMALL)  // kpad (<= 1024) + TOPK_CAP, padded to a power of two
      hipLaunchKernelGGL(topk_select_kernel, dim3((unsigned)B), dim3(256), 8192 * sizeof(unsigned long long), st, ws,
                         (int)k, rescan, (int)j_spec);
  };
  // round r scans (growth - 1) x what is already ranked
  const int64_t growth = host::topk_growth(k);
  int64_t e0 = 0, e1 = first_rows;
  while (e0 < N) {
    rc = launch_scan(e0, e1, ws.tau_scan, nullptr, 0, "kge_topk scan");
    if (rc) return rc;
    int64_t next = e1 * growth;
    next = (next < N) ? next : N;
    launch_select(e1 - e0, 0, host::topk_speculative_rank(k, e1, next - e1));
    KGE_LAUNCH_CHECK("topk_select_kernel");
    e0 = e1;
    e1 = next;
  }
  // queries whose candidate buffer overflowed in some round, or whose guessed threshold turned out too high, lost
  // entries: scan again with their final k-th best (a valid, tight threshold) until nothing overflows.
  int32_t n_dirty = 0;
  KGE_HIP_CHECK(hipMemcpyAsync(&n_dirty, ws.n_dirty, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  KGE_HIP_CHECK(hipStreamSynchronize(st));
  for (int iter = 0; n_dirty > 0 && iter < 16; ++iter) {
    rc = launch_scan(0, N, ws.tau, ws.dirty, 1, "kge_topk rescan");
    if (rc) return rc;
    launch_select(N, 1, k);
    KGE_LAUNCH_CHECK("topk_select_kernel");
    KGE_HIP_CHECK(hipMemcpyAsync(&n_dirty, ws.n_dirty, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    KGE_HIP_CHECK(hipStreamSynchronize(st));
  }
  KGE_REQUIRE(n_dirty == 0, KGE_ERR_OVERFLOW, "%s: %d queries still overflow their candidate buffers", who, n_dirty);
  const int64_t total = B * k;
  hipLaunchKernelGGL(topk_output_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, ws, B, (int)k, bias,
                     apply_sigmoid, out_scores, out_idx);
  KGE_LAUNCH_CHECK("topk_output_kernel");
  return KGE_OK;
}
}  // namespace

extern "C" int kge_row_minmax(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                              int64_t B, int64_t d, int64_t N, float* out_min, float* out_max, void* stream) {
  clear_error();
  int rc = check_contract("kge_row_minmax", Q, E, dtype, scale, B, d, N);
  if (rc) return rc;
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(out_min && out_max && out_min != out_max, KGE_ERR_INVALID, "kge_row_minmax: null or aliased output pointers");
  hipStream_t st = (hipStream_t)stream;
  uint32_t* kmin = (uint32_t*)out_min;  // the outputs hold order-preserving keys until the last kernel
  uint32_t* kmax = (uint32_t*)out_max;
  const dim3 g1((unsigned)((B + 255) / 256)), b1(256);
  hipLaunchKernelGGL(minmax_init_kernel, g1, b1, 0, st, kmin, kmax, B);
  KGE_LAUNCH_CHECK("minmax_init_kernel");
  ContractArgs a = make_args(Q, E, dtype, scale, B, d, N, 0, N);
  MinMaxArgs ea{kmin, kmax};
  rc = launch_contract<MinMaxEpi>(dtype, a, ea, st, "kge_row_minmax");
  if (rc) return rc;
  hipLaunchKernelGGL(minmax_final_kernel, g1, b1, 0, st, kmin, kmax, bias, B);
  KGE_LAUNCH_CHECK("minmax_final_kernel");
  return KGE_OK;
}

extern "C" size_t kge_bce_workspace_bytes(void) { return host::bce_ws_bytes(); }

extern "C" int kge_bce_multihot(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                                int64_t B, int64_t d, int64_t N, const int64_t* csr_row, const int64_t* row_ptr,
                                const int32_t* col, int64_t n_rows, float label_smoothing, float* loss,
                                void* workspace, size_t workspace_bytes, void* stream) {
  clear_error();
  int rc = check_contract("kge_bce_multihot", Q, E, dtype, scale, B, d, N);
  if (rc) return rc;
  KGE_REQUIRE(B >= 1, KGE_ERR_INVALID, "kge_bce_multihot: empty batch");
  KGE_REQUIRE(loss, KGE_ERR_INVALID, "kge_bce_multihot: null loss pointer");
  KGE_REQUIRE(!csr_row || (row_ptr && col), KGE_ERR_INVALID, "kge_bce_multihot: csr_row given without row_ptr / col");
  KGE_REQUIRE(workspace && workspace_bytes >= kge_bce_workspace_bytes(), KGE_ERR_WORKSPACE,
              "kge_bce_multihot: workspace of %zu bytes, need %zu", workspace_bytes, kge_bce_workspace_bytes());
  KGE_REQUIRE(((uintptr_t)workspace & 7) == 0, KGE_ERR_WORKSPACE, "kge_bce_multihot: workspace must be 8-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  double* sums = (double*)workspace;
  hipLaunchKernelGGL(bce_init_kernel, dim3(1), dim3(256), 0, st, sums);
  KGE_LAUNCH_CHECK("bce_init_kernel");
  ContractArgs a = make_args(Q, E, dtype, scale, B, d, N, 0, N);
  BceArgs ea{bias, sums, label_smoothing != 0.f ? 1 : 0};
  rc = launch_contract<BceEpi>(dtype, a, ea, st, "kge_bce_multihot");
  if (rc) return rc;
  if (csr_row && n_rows > 0) {
    dim3 grid((unsigned)B, BCE_POS_SPLIT), block(256);
    KGE_DISPATCH_DTYPE(dtype, bce_pos_kernel, grid, block, 0, st, a, bias, csr_row, row_ptr, col, n_rows, sums);
    KGE_LAUNCH_CHECK("bce_pos_kernel");
  }
  hipLaunchKernelGGL(bce_final_kernel, dim3(1), dim3(64), 0, st, sums, (double)B, (double)N, label_smoothing, loss);
  KGE_LAUNCH_CHECK("bce_final_kernel");
  return KGE_OK;
}

// ---- backward of the BCE step ------------------------------------------------------------------------
using host::BwdPlan;
using host::bwd_plan;

extern "C" size_t kge_bce_backward_workspace_bytes(int64_t B, int64_t d, int64_t N) {
  if (B < 1 || d < 1 || N < 1) return 0;
  return bwd_plan(B, d, N).total;
}

extern "C" int kge_bce_multihot_backward(const float* Q, const float* bias, const void* E, int dtype, int64_t B,
                                         int64_t d, int64_t N, const int64_t* csr_row, const int64_t* row_ptr,
                                         const int32_t* col, int64_t n_rows, float label_smoothing, float grad_out,
                                         float* loss, float* dQ, float* dbias, float* dE, void* workspace,
                                         size_t workspace_bytes, void* stream) {
  clear_error();
  KGE_REQUIRE(dtype == KGE_F32, KGE_ERR_UNSUPPORTED, "kge_bce_multihot_backward: fp32 tables only (got dtype %d)", dtype);
  int rc = check_contract("kge_bce_multihot_backward", Q, E, dtype, nullptr, B, d, N);
  if (rc) return rc;
  KGE_REQUIRE(B >= 1, KGE_ERR_INVALID, "kge_bce_multihot_backward: empty batch");
  KGE_REQUIRE(N <= (1 << 24), KGE_ERR_UNSUPPORTED, "kge_bce_multihot_backward: N=%lld exceeds 2^24", (long long)N);
  KGE_REQUIRE(dQ && dE, KGE_ERR_INVALID, "kge_bce_multihot_backward: null dQ or dE");
  KGE_REQUIRE((((uintptr_t)dQ | (uintptr_t)dE) & 15) == 0, KGE_ERR_INVALID,
              "kge_bce_multihot_backward: dQ and dE must be 16-byte aligned");
  KGE_REQUIRE(!csr_row || (row_ptr && col), KGE_ERR_INVALID,
              "kge_bce_multihot_backward: csr_row given without row_ptr / col");
  const BwdPlan p = bwd_plan(B, d, N);
  KGE_REQUIRE(workspace && workspace_bytes >= p.total, KGE_ERR_WORKSPACE,
              "kge_bce_multihot_backward: workspace of %zu bytes, need %zu", workspace_bytes, p.total);
  KGE_REQUIRE(((uintptr_t)workspace & 255) == 0, KGE_ERR_WORKSPACE,
              "kge_bce_multihot_backward: workspace must be 256-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  double* sums = (double*)ws;
  float* G = (float*)(ws + p.off_G);
  // K-major form (d a multiple of 4): both gradient contractions read G, E and Q where they lie; otherwise G is
  // also written transposed and E, Q are transposed into the workspace
  const bool kmajor = p.kmajor;  // (Q and E are 16-byte aligned: check_contract)
  float* GT = kmajor ? nullptr : (float*)(ws + p.off_GT);
  float* ET = (float*)(ws + p.off_ET);
  float* QT = (float*)(ws + p.off_QT);
  float* part = (float*)(ws + p.off_part);
  const float inv_bn = grad_out / ((float)B * (float)N);

  hipLaunchKernelGGL(bce_init_kernel, dim3(1), dim3(256), 0, st, sums);
  KGE_LAUNCH_CHECK("bce_init_kernel");
  if (dbias) {
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((B + 255) / 256)), dim3(256), 0, st, dbias, B);
    KGE_LAUNCH_CHECK("fill_zero_kernel");
  }
  // (1) scores -> g = (sigmoid(s) - dense part of y') * inv_bn, both layouts, and the loss sums
  ContractArgs a = make_args(Q, E, KGE_F32, nullptr, B, d, N, 0, N);
  GradArgs ga{bias, sums, G, GT, dbias, p.ldG, p.ldT, inv_bn, label_smoothing != 0.f ? inv_bn / (float)N : 0.f,
              label_smoothing != 0.f ? 1 : 0};
  rc = launch_ksplit<GradEpi>(a, ga, 1, st, "kge_bce_multihot_backward: scores");
  if (rc) return rc;
  if (csr_row && n_rows > 0) {
    dim3 grid((unsigned)(B < 512 ? B : 512)), block(256);
    if (loss) {
      hipLaunchKernelGGL((bce_pos_kernel<KGE_F32>), dim3((unsigned)B, BCE_POS_SPLIT), block, 0, st, a, bias, csr_row,
                         row_ptr, col, n_rows, sums);
      KGE_LAUNCH_CHECK("bce_pos_kernel");
    }
    const float pos = (label_smoothing != 0.f ? 1.0f - label_smoothing : 1.0f) * inv_bn;
    hipLaunchKernelGGL(grad_pos_kernel, grid, block, 0, st, csr_row, row_ptr, col, n_rows, B, N, G, p.ldG, GT, p.ldT,
                       dbias, pos);
    KGE_LAUNCH_CHECK("grad_pos_kernel");
  }
  if (loss) {
    hipLaunchKernelGGL(bce_final_kernel, dim3(1), dim3(64), 0, st, sums, (double)B, (double)N, label_smoothing, loss);
    KGE_LAUNCH_CHECK("bce_final_kernel");
  }
  // (2) the other operands with the summed index contiguous: ET [d, ldG], QT [d, ldT]
  if (!kmajor) {
    hipLaunchKernelGGL(transpose_kernel, dim3((unsigned)((d + 31) / 32), (unsigned)((N + 31) / 32)), dim3(256), 0, st,
                       (const float*)E, N, d, d, ET, p.ldG);
    KGE_LAUNCH_CHECK("transpose_kernel");
    hipLaunchKernelGGL(transpose_kernel, dim3((unsigned)((d + 31) / 32), (unsigned)((B + 31) / 32)), dim3(256), 0, st, Q,
                       B, d, d, QT, p.ldT);
    KGE_LAUNCH_CHECK("transpose_kernel");
  }
  // (3) dQ [B, d] = G . E: rows of G against rows of ET (or E itself, K-major), K = N split over grid.y, partial sums
  // reduced in order
  {
    ContractArgs b = make_args(G, kmajor ? (const float*)E : ET, KGE_F32, nullptr, B, N, d, 0, d);
    b.ldq = (int)p.ldG;
    b.lde = kmajor ? (int)d : (int)p.ldG;
    b.k_split_len = p.k_split_len;
    StoreArgs sa{p.k_splits > 1 ? part : dQ, nullptr, d, (int64_t)B * d};
    rc = launch_ksplit<StoreEpi>(b, sa, (unsigned)p.k_splits, st, "kge_bce_multihot_backward: dQ", kmajor ? 1 : 0);
    if (rc) return rc;
    if (p.k_splits > 1) {
      const int64_t n = B * d;
      hipLaunchKernelGGL(reduce_splits_kernel, dim3((unsigned)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048)),
                         dim3(256), 0, st, part, p.k_splits, n, dQ);
      KGE_LAUNCH_CHECK("reduce_splits_kernel");
    }
  }
  // (4) dE [N, d] = G^T . Q: rows of GT against rows of QT, K = B (or G and Q themselves, both K-major)
  {
    if (kmajor) {
      // the rows of Q as the "queries", the rows of G (N of them, read up to the padded pitch) as the "entities": a
      // workgroup's share of G is 256 neighbouring columns (1 KB of every row), and the result is stored transposed
      ContractArgs b = make_args(Q, G, KGE_F32, nullptr, d, B, p.ldG, 0, p.ldG);
      b.ldq = (int)d;
      b.lde = (int)p.ldG;
      StoreArgs sa{dE, nullptr, d, 0, N};
      rc = launch_ksplit<StoreTEpi>(b, sa, 1, st, "kge_bce_multihot_backward: dE", 3);
    } else {
      ContractArgs b = make_args(GT, QT, KGE_F32, nullptr, N, B, d, 0, d);
      b.ldq = (int)p.ldT;
      b.lde = (int)p.ldT;
      StoreArgs sa{dE, nullptr, d, 0};
      rc = launch_ksplit<StoreEpi>(b, sa, 1, st, "kge_bce_multihot_backward: dE");
    }
    if (rc) return rc;
  }
  return KGE_OK;
}

