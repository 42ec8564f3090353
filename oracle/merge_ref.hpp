// TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's merge-path partitioning and carry
// fix-ups.  Never included by the shipped package.
//
// Follows cpu_template/merged_spmv_template_reducer.h (the aggregator template repeats the same
// helpers): MergePathSearch :27-51, the reducer fix-up :56-70, the aggregator fix-up :75-87, and the
// per-thread split of OmpMergeSystem :101-121 (reducer) / cpu_template/merged_spmv_template_aggregator.h
// :99-111 (aggregator and map-only).
//
// Parity pin: oracle/merge_kat.cpp runs the same cases through these functions and through the
// functions of the reference's checked-in generated header merged_spmv.h (fixture
// tests/golden/merge_kat.json); tests additionally check merge_path_search against a brute-force merge.
#pragma once
#include <algorithm>

#include "tensor_ref.hpp"

namespace oracle {

struct Coord {
  int x;  // rows consumed
  int y;  // non-zeros consumed
};

// List B of the merge is the counting sequence 0, 1, 2, ... (merged_spmv_template_reducer.h:13-17).
struct Counting {
  int start;
  explicit Counting(int s) : start(s) {}
  int operator[](int i) const { return start + i; }
};

// Where diagonal `diagonal` crosses the merge path of A (row end offsets, length a_len) and
// B (length b_len): binary search for the first x with A[x] > B[diagonal - x - 1].   (:27-51)
template <typename AList, typename BList>
inline Coord merge_path_search(int diagonal, const AList& a, const BList& b, int a_len, int b_len) {
  int lo = std::max(diagonal - b_len, 0);
  int hi = std::min(diagonal, a_len);
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (a[mid] <= b[diagonal - mid - 1]) lo = mid + 1;
    else hi = mid;
  }
  Coord c;
  c.x = std::min(lo, a_len);
  c.y = diagonal - lo;
  return c;
}

struct Span {
  Coord begin, end;
};

// The slice of the merge path thread `tid` of `num_threads` consumes.                    (:101-121)
// `row_end` is the CSR row pointer already advanced by one (:97).
inline Span reducer_thread_span(int tid, int num_threads, const int* row_end, int num_rows, int nnz) {
  const int total = num_rows + nnz;
  const int per_thread = (total + num_threads - 1) / num_threads;
  const int d0 = std::min(per_thread * tid, total);
  const int d1 = std::min(d0 + per_thread, total);
  Counting nz(0);
  Span s;
  s.begin = merge_path_search(d0, row_end, nz, num_rows, nnz);
  s.end = merge_path_search(d1, row_end, nz, num_rows, nnz);
  return s;
}

// The flat edge range of thread `tid` in the aggregator / map-only variant: the split still counts
// num_rows + nnz items although only nnz exist          (merged_spmv_template_aggregator.h:99-111).
inline void flat_thread_range(int tid, int num_threads, int num_rows, int nnz, int& first, int& last) {
  const int total = num_rows + nnz;
  const int per_thread = (total + num_threads - 1) / num_threads;
  first = tid * per_thread;
  last = std::min(tid * per_thread + per_thread, nnz);
}

// Rows that span threads: add each thread's open-row partial, in thread order, skipping the last
// thread and rows past the end.                                                            (:56-70)
template <typename V, int D>
inline void reducer_carry_fixup(int num_threads, int num_rows, const int* carry_row,
                                const Tensor<V, D>* carry_val, V* y) {
  for (int tid = 0; tid < num_threads - 1; ++tid) {
    if (carry_row[tid] < num_rows) {
      for (int i = 0; i < D; ++i) y[carry_row[tid] * D + i] += carry_val[tid].values[i];
    }
  }
}

// Aggregator: per-thread partials are added in thread order and ASSIGNED to the output.   (:75-87)
template <typename V, int D>
inline void aggregator_fixup(int num_threads, const Tensor<V, D>* partial, V* out) {
  Tensor<V, D> total;
  for (int tid = 0; tid < num_threads; ++tid) total += partial[tid];
  for (int i = 0; i < D; ++i) out[i] = total.values[i];
}

}  // namespace oracle
