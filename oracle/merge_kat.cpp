// TEST INFRASTRUCTURE ONLY -- known-answer driver for merge-path search and the carry fix-ups.
//
// Compiled twice by oracle/build_oracle.py:
//   * with -DKAT_REFERENCE and -I<reference root>: calls MergePathSearch, both ApplyCarryOutFixup
//     overloads and the map-only OmpMergeSystem of the reference's checked-in generated header
//     merged_spmv.h (:27-51, :56-70, :75-87, :92-151); the output is the committed fixture
//     tests/golden/merge_kat.json
//   * without the macro: calls oracle/merge_ref.hpp; tests require identical lines (the OmpMergeSystem
//     lines exist only in the reference build and are compared with the generated oracle of the same
//     sub-graph by tests/test_oracle_pins.py).
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#ifdef KAT_REFERENCE
#include "merged_spmv.h"
static void search(int diag, const int* row_end, int rows, int nnz, int& x, int& y) {
  CountingInputIterator<int> nz(0);
  int2 c;
  MergePathSearch(diag, row_end, nz, rows, nnz, c);
  x = c.x; y = c.y;
}
template <typename V, int D> using T_ = Tensor<V, D>;
template <typename V, int D>
static void red_fix(int T, int rows, int* cr, T_<V, D>* cv, V* y) { ApplyCarryOutFixup<V, int, D>(T, rows, cr, cv, y); }
template <typename V, int D>
static void agg_fix(int T, T_<V, D>* part, V* out) { ApplyCarryOutFixup<V, int, D>(T, part, out); }
#else
#include "merge_ref.hpp"
static void search(int diag, const int* row_end, int rows, int nnz, int& x, int& y) {
  oracle::Counting nz(0);
  oracle::Coord c = oracle::merge_path_search(diag, row_end, nz, rows, nnz);
  x = c.x; y = c.y;
}
template <typename V, int D> using T_ = oracle::Tensor<V, D>;
template <typename V, int D>
static void red_fix(int T, int rows, int* cr, T_<V, D>* cv, V* y) { oracle::reducer_carry_fixup<V, D>(T, rows, cr, cv, y); }
template <typename V, int D>
static void agg_fix(int T, T_<V, D>* part, V* out) { oracle::aggregator_fixup<V, D>(T, part, out); }
#endif

static unsigned long long bits(double v) { uint64_t u; std::memcpy(&u, &v, 8); return u; }
static unsigned long long bits(float v) { uint32_t u; std::memcpy(&u, &v, 4); return u; }

// CSR row pointers (leading 0) of the test structures: empty rows at both ends and in runs, one long
// row, single-entry rows.
static const std::vector<std::vector<int>> kRowPtr = {
    {0, 3, 3, 3, 7, 8, 8, 20, 20},
    {0, 0, 0, 5},
    {0, 1, 2, 3, 4, 5, 6},
    {0, 17},
    {0, 0, 0, 0},
    {0, 2, 2, 9, 9, 9, 9, 10, 31, 31, 32},
};

template <typename V>
static void fixups(const char* tname) {
  {  // reducer: 5 threads, 6 rows; thread 2 points past the end, the last thread is never applied
    int cr[5] = {1, 1, 6, 4, 0};
    T_<V, 2> cv[5];
    for (int t = 0; t < 5; ++t) { cv[t].values[0] = V(0.1) * V(t + 1); cv[t].values[1] = V(-1.5) + V(t); }
    V y[12];
    for (int i = 0; i < 12; ++i) y[i] = V(i) * V(0.25);
    red_fix<V, 2>(5, 6, cr, cv, y);
    std::printf("reducer_fixup %s", tname);
    for (int i = 0; i < 12; ++i) std::printf(" %llx", bits(y[i]));
    std::printf("\n");
  }
  {  // aggregator: ordered sum of 7 partials, assigned (previous content ignored)
    T_<V, 3> part[7];
    for (int t = 0; t < 7; ++t)
      for (int i = 0; i < 3; ++i) part[t].values[i] = V(1) / V(3 + t * 3 + i);
    V out[3] = {V(99), V(99), V(99)};
    agg_fix<V, 3>(7, part, out);
    std::printf("aggregator_fixup %s %llx %llx %llx\n", tname, bits(out[0]), bits(out[1]), bits(out[2]));
  }
}

int main() {
  for (size_t s = 0; s < kRowPtr.size(); ++s) {
    const std::vector<int>& ptr = kRowPtr[s];
    const int rows = (int)ptr.size() - 1;
    const int nnz = ptr.back();
    const int* row_end = ptr.data() + 1;
    std::printf("search %zu", s);
    for (int d = 0; d <= rows + nnz; ++d) {
      int x, y;
      search(d, row_end, rows, nnz, x, y);
      std::printf(" %d,%d", x, y);
    }
    std::printf("\n");
  }
  fixups<float>("f32");
  fixups<double>("f64");
#ifdef KAT_REFERENCE
  // the generated map-only instance: bp_1[e] = bpoints[e][1] on int64 data, fake num_rows = ne
  const int ne = 37;
  for (int T : {1, 3, 8}) {
    std::vector<long> bpoints(2 * ne), bp_1(ne, -7);
    for (int e = 0; e < ne; ++e) { bpoints[2 * e] = 1000 + e; bpoints[2 * e + 1] = 5 * e - 11; }
    OmpMergeSystem<long, int>(T, bpoints.data(), bp_1.data(), ne, ne);
    std::printf("map_only_T%d i64", T);
    for (int e = 0; e < ne; ++e) std::printf(" %ld", bp_1[e]);
    std::printf("\n");
  }
#endif
  return 0;
}
