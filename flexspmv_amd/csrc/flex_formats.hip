// Edge-list preparation in front of a FlexSpmv launch: COO row ids -> CSR row pointer, stable sort of
// an edge list by row, and the permutation of per-edge tensors.  Interface: flexspmv_formats.h.
//
// Stands in for _coo_rows_to_csr_ptr of the reference (python_wrapper/dynamic_replace_submodule.py:20-41),
// which calls torch's COO -> CSR conversion or bincount + cumsum; the sort has no counterpart there (the
// reference assumes ascending row ids).
//
// All of this is HBM-bound integer work:
//   rows_to_ptr_kernel   reads every row id once (4 or 8 B / edge, eight ids per thread in 16-byte loads) and
//                        writes every pointer entry once (4 B / row): boundary i between edges i-1 and i
//                        gives row_ptr[r] = i for the rows r in (row[i-1], row[i]].  Almost all boundaries
//                        close zero or one row; longer runs of empty rows are filled by the whole wavefront,
//                        and a run longer than LONG_GAP rows switches the call to rows_search_kernel.
//   rows_search_kernel   the fallback for edge lists with huge runs of empty rows: one binary search per
//                        row.  It is always launched and returns at once unless the first kernel asked for it,
//                        so the host never has to look at device memory.
//   sort                 rocPRIM's radix sort on (row id, position) pairs over the bits num_rows needs.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <rocprim/rocprim.hpp>

#include "flexspmv_formats.h"

namespace {

constexpr int WAVE = 64;
constexpr int BLOCK = 256;
constexpr int LONG_GAP = 4096;  // empty-row runs longer than this go to the per-row search

thread_local char g_error[512] = "";
int fail(int code, const char* msg) {
  snprintf(g_error, sizeof(g_error), "%s", msg);
  return code;
}
int fail_hip(hipError_t e, const char* where) {
  snprintf(g_error, sizeof(g_error), "%s: %s", where, hipGetErrorString(e));
  return (int)e;
}

// findings[0]: FLEXSPMV_FINDING_* bits; findings[1]: non-zero when rows_search_kernel has to run
__global__ void clear_findings_kernel(int32_t* findings) {
  if (threadIdx.x < 4) findings[threadIdx.x] = 0;
}

// ids a thread looks at: two or four 16-byte loads
constexpr int PER_THREAD = 8;
constexpr int NOT_AN_ID = -2;  // a row id outside [0, num_rows): no boundary next to it is written

template <typename I>
__device__ inline int checked_id(const I v, const int num_rows, int& found) {
  if (v < 0 || (long long)v >= (long long)num_rows) {
    found |= FLEXSPMV_FINDING_OUT_OF_RANGE;
    return NOT_AN_ID;
  }
  return (int)v;
}

// Thread t owns the boundaries i = 8t .. 8t+7 (boundary i lies between edges i-1 and i; the list is
// extended by id[-1] = -1 and id[ne] = num_rows, so boundaries 0 and ne close the leading and trailing
// empty rows).  Every lane runs the same number of ballots: nothing returns early.
template <typename I, bool ALIGNED>
__global__ void __launch_bounds__(BLOCK)
rows_to_ptr_kernel(const I* __restrict__ rows, const int ne, const int num_rows, int32_t* __restrict__ row_ptr,
                   int32_t* __restrict__ findings) {
  constexpr int K = PER_THREAD;
  const long long base = ((long long)blockIdx.x * BLOCK + threadIdx.x) * K;
  const int lane = threadIdx.x & (WAVE - 1);
  int found = 0;
  int cur[K];
  if (ALIGNED && base + K <= ne) {
    constexpr int PER_LOAD = 16 / (int)sizeof(I);
    struct alignas(16) Chunk { I v[PER_LOAD]; };
    const Chunk* src = reinterpret_cast<const Chunk*>(rows + base);
#pragma unroll
    for (int c = 0; c < K / PER_LOAD; ++c) {
      const Chunk chunk = src[c];
#pragma unroll
      for (int q = 0; q < PER_LOAD; ++q) cur[c * PER_LOAD + q] = checked_id<I>(chunk.v[q], num_rows, found);
    }
  } else {
#pragma unroll
    for (int j = 0; j < K; ++j)
      cur[j] = (base + j < ne) ? checked_id<I>(rows[base + j], num_rows, found) : num_rows;
  }
  // the id before this thread's first one: the neighbouring lane's last, or a load for lane 0
  int prev = __shfl_up(cur[K - 1], 1);
  if (lane == 0) {
    if (base == 0) prev = -1;
    else if (base - 1 < ne) prev = checked_id<I>(rows[base - 1], num_rows, found);
    else prev = NOT_AN_ID;
  }

#pragma unroll
  for (int j = 0; j < K; ++j) {
    const long long i = base + j;
    const int hi = cur[j];
    int gap = 0;  // rows prev+1 .. hi receive i (hi == num_rows at i == ne: row_ptr[num_rows] = ne)
    if (i <= ne && prev != NOT_AN_ID && hi != NOT_AN_ID) {
      if (prev > hi) found |= FLEXSPMV_FINDING_UNSORTED; else gap = hi - prev;
    }
    if (gap >= 1 && gap <= 2) {
      row_ptr[prev + 1] = (int32_t)i;
      if (gap == 2) row_ptr[prev + 2] = (int32_t)i;
    }
    unsigned long long wide = __builtin_amdgcn_ballot_w64(gap > 2);
    while (wide != 0ull) {
      const int src = __builtin_ctzll(wide);
      wide &= wide - 1ull;
      const int s_lo = __builtin_amdgcn_readlane(prev, src);
      const int s_hi = __builtin_amdgcn_readlane(hi, src);
      const int s_i = __builtin_amdgcn_readlane((int)i, src);
      if (s_hi - s_lo > LONG_GAP) {
        if (lane == 0) atomicOr(&findings[1], 1);
        continue;
      }
      for (int r = s_lo + 1 + lane; r <= s_hi; r += WAVE) row_ptr[r] = s_i;
    }
    prev = hi;
  }
  if (found != 0) atomicOr(&findings[0], found);
}

constexpr int SEARCH_BLOCKS = 2048;

template <typename I>
__global__ void __launch_bounds__(BLOCK)
rows_search_kernel(const I* __restrict__ rows, const int ne, const int num_rows, int32_t* __restrict__ row_ptr,
                   const int32_t* __restrict__ findings) {
  if (findings[1] == 0 || findings[0] != 0) return;
  for (long long r = (long long)blockIdx.x * BLOCK + threadIdx.x; r <= num_rows; r += (long long)gridDim.x * BLOCK) {
    int lo = 0, hi = ne;  // first position whose row id is >= r
    while (lo < hi) {
      const int mid = lo + ((hi - lo) >> 1);
      if ((long long)rows[mid] < r) lo = mid + 1; else hi = mid;
    }
    row_ptr[r] = lo;
  }
}

// key of a row id for the sort: ids that do not fit a non-negative int32 become 0xffffffff, which reads
// back as -1 in sorted_rows and is reported as out of range by the pointer kernel
template <typename I>
struct RowKey {
  __host__ __device__ unsigned operator()(const I v) const {
    return (v < 0 || (long long)v > 0x7fffffffll) ? 0xffffffffu : (unsigned)v;
  }
};

int bits_for(int64_t num_rows) {
  int b = 1;
  while (b < 32 && ((int64_t)1 << b) < num_rows) ++b;
  return b;
}

template <typename I>
hipError_t sort_pairs(void* temp, size_t& temp_bytes, const I* rows, int32_t* sorted_rows, int32_t* permutation,
                      int64_t ne, int64_t num_rows, hipStream_t stream) {
  auto keys_in = rocprim::make_transform_iterator(rows, RowKey<I>());
  rocprim::counting_iterator<int32_t> positions(0);
  // ids past num_rows keep their high bits out of the sort; they are reported, not ordered
  return rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, reinterpret_cast<unsigned*>(sorted_rows), positions,
                                   permutation, (size_t)ne, 0u, (unsigned)bits_for(num_rows), stream);
}

// dst[k] = src[perm[k]] (gather) or dst[perm[k]] = src[k] (scatter) for rows of `vecs` vectors of type T.
// One thread moves one vector; T is the widest of 16, 8 and 4 bytes that divides the row and both base
// addresses, so an 8-byte value per edge is one load and one store (the side that follows the permutation
// touches a cache line per row whatever the width: that line, not the instruction count, is the cost).
template <bool SCATTER, typename T>
__global__ void __launch_bounds__(BLOCK)
permute_rows_kernel(const T* __restrict__ src, T* __restrict__ dst, const int32_t* __restrict__ perm,
                    const long long n, const int vecs) {
  const long long idx = (long long)blockIdx.x * BLOCK + threadIdx.x;
  if (idx >= n * vecs) return;
  const long long k = idx / vecs;
  const int w = (int)(idx - k * vecs);
  const long long other = perm[k];
  if (SCATTER) dst[other * vecs + w] = src[idx]; else dst[idx] = src[other * vecs + w];
}

template <bool SCATTER>
int permute_rows(const void* src, void* dst, const int32_t* perm, int64_t n, int64_t row_bytes, void* stream) {
  if (n < 0 || row_bytes <= 0 || (row_bytes & 3) != 0)
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "n must be >= 0 and row_bytes a positive multiple of 4");
  if (n == 0) return FLEXSPMV_FORMATS_OK;
  if (src == nullptr || dst == nullptr || perm == nullptr)
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "a pointer is NULL");
  const uintptr_t bits = (uintptr_t)src | (uintptr_t)dst | (uintptr_t)row_bytes;
  const int vec_bytes = (bits & 15u) == 0 ? 16 : ((bits & 7u) == 0 ? 8 : 4);
  const int64_t vecs = row_bytes / vec_bytes;
  const int64_t total = n * vecs;
  if (n >= ((int64_t)1 << 31) || vecs >= ((int64_t)1 << 20) || (total + BLOCK - 1) / BLOCK >= ((int64_t)1 << 31))
    return fail(FLEXSPMV_FORMATS_ERR_TOO_LARGE, "tensor too large for one launch");
  const dim3 grid((unsigned)((total + BLOCK - 1) / BLOCK));
  if (vec_bytes == 16)
    hipLaunchKernelGGL((permute_rows_kernel<SCATTER, uint4>), grid, dim3(BLOCK), 0, (hipStream_t)stream,
                       (const uint4*)src, (uint4*)dst, perm, (long long)n, (int)vecs);
  else if (vec_bytes == 8)
    hipLaunchKernelGGL((permute_rows_kernel<SCATTER, uint2>), grid, dim3(BLOCK), 0, (hipStream_t)stream,
                       (const uint2*)src, (uint2*)dst, perm, (long long)n, (int)vecs);
  else
    hipLaunchKernelGGL((permute_rows_kernel<SCATTER, uint32_t>), grid, dim3(BLOCK), 0, (hipStream_t)stream,
                       (const uint32_t*)src, (uint32_t*)dst, perm, (long long)n, (int)vecs);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "kernel launch failed");
  return FLEXSPMV_FORMATS_OK;
}

}  // namespace

extern "C" {

int flexspmv_coo_rows_to_csr(const void* row_ids, int index_bytes, int64_t ne, int64_t num_rows, int32_t* row_ptr,
                             int32_t* findings, void* stream) {
  if (index_bytes != 4 && index_bytes != 8)
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "index_bytes must be 4 or 8");
  if (ne < 0 || num_rows < 0) return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "ne and num_rows must be >= 0");
  if (row_ptr == nullptr || findings == nullptr || (ne > 0 && row_ids == nullptr))
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "a pointer is NULL");
  if (ne >= ((int64_t)1 << 31) - BLOCK || num_rows >= ((int64_t)1 << 31) - BLOCK)
    return fail(FLEXSPMV_FORMATS_ERR_TOO_LARGE, "ne and num_rows must stay below 2^31 (32-bit offsets)");
  hipStream_t s = (hipStream_t)stream;
  const long long threads = (ne + 1 + PER_THREAD - 1) / PER_THREAD;
  const unsigned edge_blocks = (unsigned)((threads + BLOCK - 1) / BLOCK);
  const long long all_row_blocks = (num_rows + 1 + BLOCK - 1) / BLOCK;
  const unsigned row_blocks = (unsigned)(all_row_blocks < SEARCH_BLOCKS ? all_row_blocks : SEARCH_BLOCKS);
  const bool aligned = ((uintptr_t)row_ids & 15u) == 0;
  hipLaunchKernelGGL(clear_findings_kernel, dim3(1), dim3(WAVE), 0, s, findings);
  auto run = [&](auto tag) {
    using I = decltype(tag);
    const I* ids = (const I*)row_ids;
    if (aligned)
      hipLaunchKernelGGL((rows_to_ptr_kernel<I, true>), dim3(edge_blocks), dim3(BLOCK), 0, s, ids, (int)ne,
                         (int)num_rows, row_ptr, findings);
    else
      hipLaunchKernelGGL((rows_to_ptr_kernel<I, false>), dim3(edge_blocks), dim3(BLOCK), 0, s, ids, (int)ne,
                         (int)num_rows, row_ptr, findings);
    hipLaunchKernelGGL(rows_search_kernel<I>, dim3(row_blocks), dim3(BLOCK), 0, s, ids, (int)ne, (int)num_rows,
                       row_ptr, (const int32_t*)findings);
  };
  if (index_bytes == 4) run(int32_t{}); else run(int64_t{});
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "kernel launch failed");
  return FLEXSPMV_FORMATS_OK;
}

size_t flexspmv_sort_workspace_bytes(int64_t ne, int64_t num_rows) {
  if (ne <= 0 || ne >= ((int64_t)1 << 31) || num_rows <= 0) return 0;
  size_t bytes = 0;
  // the key iterator's type does not change the scratch layout; the wider index type is queried
  if (sort_pairs<int64_t>(nullptr, bytes, (const int64_t*)nullptr, nullptr, nullptr, ne, num_rows, nullptr) != hipSuccess)
    return 0;
  size_t bytes32 = 0;
  if (sort_pairs<int32_t>(nullptr, bytes32, (const int32_t*)nullptr, nullptr, nullptr, ne, num_rows, nullptr) != hipSuccess)
    return 0;
  return bytes > bytes32 ? bytes : bytes32;
}

int flexspmv_sort_edges_by_row(const void* row_ids, int index_bytes, int64_t ne, int64_t num_rows,
                               int32_t* sorted_rows, int32_t* permutation, void* workspace, size_t workspace_bytes,
                               void* stream) {
  if (index_bytes != 4 && index_bytes != 8)
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "index_bytes must be 4 or 8");
  if (ne < 0 || num_rows <= 0) return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "ne must be >= 0 and num_rows > 0");
  if (ne == 0) return FLEXSPMV_FORMATS_OK;
  if (row_ids == nullptr || sorted_rows == nullptr || permutation == nullptr)
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "a pointer is NULL");
  if (ne >= ((int64_t)1 << 31) || num_rows >= ((int64_t)1 << 31))
    return fail(FLEXSPMV_FORMATS_ERR_TOO_LARGE, "ne and num_rows must stay below 2^31 (32-bit offsets)");
  const size_t need = flexspmv_sort_workspace_bytes(ne, num_rows);
  if (need > 0 && (workspace == nullptr || workspace_bytes < need))
    return fail(FLEXSPMV_FORMATS_ERR_WORKSPACE, "workspace is missing or smaller than flexspmv_sort_workspace_bytes()");
  size_t bytes = workspace_bytes;
  const hipError_t e =
      index_bytes == 4
          ? sort_pairs<int32_t>(workspace, bytes, (const int32_t*)row_ids, sorted_rows, permutation, ne, num_rows,
                                (hipStream_t)stream)
          : sort_pairs<int64_t>(workspace, bytes, (const int64_t*)row_ids, sorted_rows, permutation, ne, num_rows,
                                (hipStream_t)stream);
  if (e != hipSuccess) return fail_hip(e, "radix sort failed");
  return FLEXSPMV_FORMATS_OK;
}

int flexspmv_gather_rows(const void* src, void* dst, const int32_t* permutation, int64_t n, int64_t row_bytes,
                         void* stream) {
  return permute_rows<false>(src, dst, permutation, n, row_bytes, stream);
}

int flexspmv_scatter_rows(const void* src, void* dst, const int32_t* permutation, int64_t n, int64_t row_bytes,
                          void* stream) {
  return permute_rows<true>(src, dst, permutation, n, row_bytes, stream);
}

const char* flexspmv_formats_last_error(void) { return g_error; }

int flexspmv_formats_abi_version(void) { return FLEXSPMV_FORMATS_ABI_VERSION; }

}  // extern "C"
