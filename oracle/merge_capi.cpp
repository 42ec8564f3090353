// TEST INFRASTRUCTURE ONLY -- C entry points over oracle/merge_ref.hpp so that tests can compare the
// restated merge-path search and thread partition with brute-force merges written in Python.
#include "merge_ref.hpp"

extern "C" {

// (x, y) where diagonal `diagonal` crosses the merge path; row_end has the leading 0 already removed.
void oracle_merge_path_search(int diagonal, const int* row_end, int num_rows, int nnz, int* out_xy) {
  oracle::Counting nz(0);
  const oracle::Coord c = oracle::merge_path_search(diagonal, row_end, nz, num_rows, nnz);
  out_xy[0] = c.x;
  out_xy[1] = c.y;
}

// the same for n diagonals: out_xy[2*i], out_xy[2*i+1] for diagonals[i]
void oracle_merge_path_search_many(const int* diagonals, int n, const int* row_end, int num_rows, int nnz, int* out_xy) {
  oracle::Counting nz(0);
  for (int i = 0; i < n; ++i) {
    const oracle::Coord c = oracle::merge_path_search(diagonals[i], row_end, nz, num_rows, nnz);
    out_xy[2 * i] = c.x;
    out_xy[2 * i + 1] = c.y;
  }
}

// begin/end coordinates of thread tid: out = {begin.x, begin.y, end.x, end.y}
void oracle_reducer_thread_span(int tid, int num_threads, const int* row_end, int num_rows, int nnz, int* out) {
  const oracle::Span s = oracle::reducer_thread_span(tid, num_threads, row_end, num_rows, nnz);
  out[0] = s.begin.x; out[1] = s.begin.y; out[2] = s.end.x; out[3] = s.end.y;
}

void oracle_flat_thread_range(int tid, int num_threads, int num_rows, int nnz, int* out) {
  oracle::flat_thread_range(tid, num_threads, num_rows, nnz, out[0], out[1]);
}

}  // extern "C"
