// TEST INFRASTRUCTURE ONLY -- known-answer driver for the per-item value type.
//
// Compiled twice by oracle/build_oracle.py:
//   * with -DKAT_REFERENCE and -I<reference root>: exercises the reference's own data_struct_shared.cuh
//     (plain C++ when no CUDA compiler is defined, data_struct_shared.cuh:12-36); its output is the
//     committed fixture tests/golden/tensor_kat.json
//   * without the macro: exercises oracle/tensor_ref.hpp; tests require identical output bits.
// Every line is "<case> <type> <hex bits of each result element>".
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <limits>

#ifdef KAT_REFERENCE
#include "data_struct_shared.cuh"
#else
#include "tensor_ref.hpp"
using namespace oracle;
#endif

template <typename V> struct Bits;
template <> struct Bits<float> { static unsigned long long of(float v) { uint32_t u; std::memcpy(&u, &v, 4); return u; } static const char* name() { return "f32"; } };
template <> struct Bits<long> { static unsigned long long of(long v) { return (unsigned long long)v; } static const char* name() { return "i64"; } };
template <> struct Bits<double> { static unsigned long long of(double v) { uint64_t u; std::memcpy(&u, &v, 8); return u; } static const char* name() { return "f64"; } };

#define KAT_EMIT(label, t) emit(label, t)
#define KAT_EMIT_SCALAR(label, v) emit_scalar(label, v)

template <typename V, int N>
static void emit(const char* label, const Tensor<V, N>& t) {
  std::printf("%s %s", label, Bits<V>::name());
  for (int i = 0; i < N; ++i) std::printf(" %llx", Bits<V>::of(t.values[i]));
  std::printf("\n");
}
template <typename V>
static void emit_scalar(const char* label, V v) {
  std::printf("%s %s %llx\n", label, Bits<V>::name(), Bits<V>::of(v));
}

template <typename V>
static void run() {
#include "tensor_kat_cases.inc"
}

template <typename V>
static void run_integer() {
#include "tensor_kat_cases_i64.inc"
}

int main() {
  run<float>();
  run<double>();
  run_integer<long>();
  return 0;
}
