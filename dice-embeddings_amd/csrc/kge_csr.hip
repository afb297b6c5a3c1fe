// Known-answer vocabulary -> CSR on the GPU (gfx950).
//
// dicee builds its filter vocabularies with Python dict-of-list loops over every triple
// (dicee/read_preprocess_save_load_kg/util.py:355-363 get_er_vocab, :366-374 get_re_vocab,
// :377-385 get_ee_vocab).  Here the same mapping is one radix sort of packed 64-bit keys
// (rocPRIM's device sort: a plain library sort) and three streaming kernels:
//   pack    (a, b, v) of every triple -> key = ((a * range_b + b) << vbits) | v
//   sort    ascending; equal (a, b) become adjacent with their values ascending
//   mark    first occurrence of every key (drops duplicate triples) and of every (a, b) pair
//   scan    exclusive prefix sums of both marks in one pass (two 32-bit counters in one 64-bit word)
//   scatter col[pos] = v; for the first entry of a pair: keys[row] = a * range_b + b, row_ptr[row] = pos
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

#include "kge_internal.h"

namespace kge {
namespace {

struct CsrWs {
  unsigned long long* key_in;
  unsigned long long* key_sorted;
  unsigned long long* marks;  // low 32 bits: unique-entry mark / count; high 32 bits: row-start mark / count
  void* sort_tmp;
  size_t sort_tmp_bytes;
  void* scan_tmp;
  size_t scan_tmp_bytes;
};

using host::align_up;

// Returns the total size, or 0 when rocPRIM cannot size its temporaries (no device).
size_t csr_ws_layout(int64_t n, void* base, CsrWs* ws, hipStream_t st) {
  size_t sort_bytes = 0, scan_bytes = 0;
  const size_t cnt = (size_t)(n < 1 ? 1 : n);
  unsigned long long* null_keys = nullptr;
  if (rocprim::radix_sort_keys(nullptr, sort_bytes, null_keys, null_keys, cnt, 0, 64, st) != hipSuccess) return 0;
  if (rocprim::exclusive_scan(nullptr, scan_bytes, null_keys, null_keys, 0ull, cnt, rocprim::plus<unsigned long long>(),
                              st) != hipSuccess)
    return 0;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    size_t o = off;
    off = align_up(off + bytes, 256);
    return o;
  };
  const size_t o_in = take(cnt * 8), o_sorted = take(cnt * 8), o_marks = take(cnt * 8);
  const size_t o_sort = take(sort_bytes ? sort_bytes : 1), o_scan = take(scan_bytes ? scan_bytes : 1);
  if (ws) {
    char* p = (char*)base;
    ws->key_in = (unsigned long long*)(p + o_in);
    ws->key_sorted = (unsigned long long*)(p + o_sorted);
    ws->marks = (unsigned long long*)(p + o_marks);
    ws->sort_tmp = p + o_sort;
    ws->sort_tmp_bytes = sort_bytes;
    ws->scan_tmp = p + o_scan;
    ws->scan_tmp_bytes = scan_bytes;
  }
  return off;
}

__global__ void __launch_bounds__(256) csr_pack_kernel(const int64_t* __restrict__ triples, int64_t n, int col_a,
                                                       int col_b, int col_v, int64_t range_a, int64_t range_b,
                                                       int64_t range_v, int vbits, unsigned long long invalid,
                                                       unsigned long long* __restrict__ key) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int64_t a = triples[3 * i + col_a], b = triples[3 * i + col_b], v = triples[3 * i + col_v];
    const bool ok = a >= 0 && a < range_a && b >= 0 && b < range_b && v >= 0 && v < range_v;
    key[i] = ok ? host::csr_pack_key(a, b, v, range_b, vbits) : invalid;
  }
}

__global__ void __launch_bounds__(256) csr_mark_kernel(const unsigned long long* __restrict__ key, int64_t n,
                                                       int vbits, unsigned long long invalid,
                                                       unsigned long long* __restrict__ marks) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const unsigned long long k = key[i];
    unsigned long long m = 0;
    if (k != invalid) {
      const bool first = (i == 0);
      const unsigned long long prev = first ? 0 : key[i - 1];
      if (first || prev != k) m = 1;
      if (first || (prev >> vbits) != (k >> vbits)) m |= 1ull << 32;
    }
    marks[i] = m;
  }
}

__global__ void __launch_bounds__(256) csr_scatter_kernel(const unsigned long long* __restrict__ key,
                                                          const unsigned long long* __restrict__ marks,
                                                          const unsigned long long* __restrict__ pos, int64_t n,
                                                          int vbits, int64_t* __restrict__ keys_out,
                                                          int64_t* __restrict__ row_ptr, int32_t* __restrict__ col,
                                                          int64_t* __restrict__ counts) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const unsigned long long vmask = (1ull << vbits) - 1;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const unsigned long long k = key[i], m = marks[i], p = pos[i];
    const int64_t entry = (int64_t)(p & 0xffffffffull), row = (int64_t)(p >> 32);
    if (m & 1) col[entry] = (int32_t)(k & vmask);
    if (m >> 32) {
      keys_out[row] = (int64_t)(k >> vbits);
      row_ptr[row] = entry;
    }
    if (i == n - 1) {
      const int64_t nnz = entry + (int64_t)(m & 1), rows = row + (int64_t)(m >> 32);
      row_ptr[rows] = nnz;
      counts[0] = rows;
      counts[1] = nnz;
    }
  }
}

// Out-of-range triples carry the key `invalid` (one bit above every valid key), so the sort puts them last.
__global__ void csr_count_invalid_kernel(const unsigned long long* __restrict__ key, int64_t n,
                                         unsigned long long invalid, int64_t* __restrict__ counts) {
  // the sort puts invalid keys last: binary search for the first one
  if (blockIdx.x != 0 || threadIdx.x != 0) return;
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (key[mid] != invalid) lo = mid + 1; else hi = mid;
  }
  counts[2] = n - lo;
}

__global__ void csr_empty_kernel(int64_t* row_ptr, int64_t* counts) {
  row_ptr[0] = 0;
  counts[0] = counts[1] = counts[2] = 0;
}

}  // namespace
}  // namespace kge

using namespace kge;

extern "C" size_t kge_csr_build_workspace_bytes(int64_t n) {
  clear_error();
  if (n < 0 || n >= (1LL << 31)) {
    set_error(KGE_ERR_INVALID, "kge_csr_build_workspace_bytes: n=%lld outside [0, 2^31)", (long long)n);
    return 0;
  }
  const size_t bytes = csr_ws_layout(n, nullptr, nullptr, nullptr);
  if (bytes == 0) set_error(KGE_ERR_HIP, "kge_csr_build_workspace_bytes: no HIP device to size the sort for");
  return bytes;
}

extern "C" int kge_csr_build(const int64_t* triples, int64_t n, int col_a, int col_b, int col_v, int64_t range_a,
                             int64_t range_b, int64_t range_v, int64_t* keys, int64_t* row_ptr, int32_t* col,
                             int64_t* counts, void* workspace, size_t workspace_bytes, void* stream) {
  clear_error();
  const host::Status rules = host::csr_build_rules(n, col_a, col_b, col_v, range_a, range_b, range_v);
  if (!rules.ok()) return set_error(rules.code, "%s", rules.msg);
  const host::CsrKeyLayout layout = host::csr_key_layout(range_a, range_b, range_v);
  const int vbits = layout.vbits, key_bits = layout.key_bits;
  KGE_REQUIRE(row_ptr && counts, KGE_ERR_INVALID, "kge_csr_build: null row_ptr or counts");
  hipStream_t st = (hipStream_t)stream;
  if (n == 0) {
    hipLaunchKernelGGL(csr_empty_kernel, dim3(1), dim3(1), 0, st, row_ptr, counts);
    KGE_LAUNCH_CHECK("csr_empty_kernel");
    return KGE_OK;
  }
  KGE_REQUIRE(triples && keys && col, KGE_ERR_INVALID, "kge_csr_build: null triples, keys or col");
  CsrWs ws;
  const size_t need = csr_ws_layout(n, workspace, &ws, st);
  KGE_REQUIRE(need != 0, KGE_ERR_HIP, "kge_csr_build: no HIP device to size the sort for");
  KGE_REQUIRE(workspace && workspace_bytes >= need, KGE_ERR_WORKSPACE, "kge_csr_build: workspace of %zu bytes, need %zu",
              workspace_bytes, need);
  KGE_REQUIRE(((uintptr_t)workspace & 7) == 0, KGE_ERR_WORKSPACE, "kge_csr_build: workspace must be 8-byte aligned");
  const unsigned grid = (unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  const unsigned long long invalid = layout.invalid;
  hipLaunchKernelGGL(csr_pack_kernel, dim3(grid), dim3(256), 0, st, triples, n, col_a, col_b, col_v, range_a, range_b,
                     range_v, vbits, invalid, ws.key_in);
  KGE_LAUNCH_CHECK("csr_pack_kernel");
  KGE_HIP_CHECK(rocprim::radix_sort_keys(ws.sort_tmp, ws.sort_tmp_bytes, ws.key_in, ws.key_sorted, (size_t)n, 0,
                                         (unsigned)(key_bits + 1), st));
  hipLaunchKernelGGL(csr_mark_kernel, dim3(grid), dim3(256), 0, st, ws.key_sorted, n, vbits, invalid, ws.marks);
  KGE_LAUNCH_CHECK("csr_mark_kernel");
  KGE_HIP_CHECK(rocprim::exclusive_scan(ws.scan_tmp, ws.scan_tmp_bytes, ws.marks, ws.key_in, 0ull, (size_t)n,
                                        rocprim::plus<unsigned long long>(), st));
  hipLaunchKernelGGL(csr_scatter_kernel, dim3(grid), dim3(256), 0, st, ws.key_sorted, ws.marks, ws.key_in, n, vbits,
                     keys, row_ptr, col, counts);
  KGE_LAUNCH_CHECK("csr_scatter_kernel");
  hipLaunchKernelGGL(csr_count_invalid_kernel, dim3(1), dim3(64), 0, st, ws.key_sorted, n, invalid, counts);
  KGE_LAUNCH_CHECK("csr_count_invalid_kernel");
  return KGE_OK;
}
