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
template <> struct Bits<double> { static unsigned long long of(double v) { uint64_t u; std::memcpy(&u, &v, 8); return u; } static const char* name() { return "f64"; } };

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
  const V nan = std::numeric_limits<V>::quiet_NaN();
  const V a6[6] = {V(1.5), V(-2.25), V(0), V(3.125), V(-0.5), V(7)};
  const V b6[6] = {V(0.75), V(0), V(-4), V(2), V(0), V(-1.5)};
  const V c3[3] = {V(2), V(0), V(-3)};
  const V d2[2] = {V(0), V(4)};
  const V p3[3] = {V(0.3), V(2.5), V(1.75)};
  const V s3[3] = {nan, V(-0.0), V(1e-30)};
  Tensor<V, 6> A(a6), B(b6);
  Tensor<V, 3> C(c3), P(p3), S(s3);
  Tensor<V, 2> D(d2);
  Tensor<V, 1> one(V(2.5)), zero1(V(0));
  Tensor<V, 6> Z;

  emit("default_zero", Z);
  emit("neg", -A);
  emit("add_same", A + B);
  emit("sub_same", A - B);
  emit("mul_same", A * B);
  emit("div_same_guarded", A / B);
  emit("pow_same", P ^ C);
  emit("add_scalar", A + V(1.25));
  emit("sub_scalar", A - V(1.25));
  emit("mul_scalar", A * V(-3));
  emit("div_scalar_unguarded", C / V(0));
  emit("div_scalar", A / V(4));
  emit("pow_scalar", P ^ V(2));
  emit("scalar_add", V(2) + A);
  emit("scalar_sub", V(2) - A);
  emit("scalar_mul", V(2) * A);
  emit("scalar_div_guarded", V(3) / B);
  emit("scalar_pow", V(2) ^ C);
  emit("mixed_int_left_sub", 1 - A);
  emit("mixed_double_left_mul", 0.5 * A);
  emit("mixed_int_right_pow", P ^ 2);
  emit("mixed_double_right_div", A / 2.0);
  emit("mixed_int_left_div_guarded", 1 / B);
  emit("bcast_add_6_3", A + C);
  emit("bcast_sub_3_6", C - A);
  emit("bcast_mul_6_2", A * D);
  emit("bcast_div_6_3_unguarded", A / C);
  emit("bcast_div_6_1", A / one);
  emit("bcast_div_6_1_zero", A / zero1);
  emit("bcast_mul_1_6", one * A);
  emit("bcast_pow_6_3", B ^ C);
  emit("bcast_lt_6_3", A < C);
  emit("bcast_gt_6_2", A > D);
  emit("lt_same", A < B);
  emit("gt_same", A > B);
  emit("lt_scalar", A < V(1));
  emit("gt_scalar", A > V(1));
  emit("lt_fn", A.lt(V(0)));
  emit("gt_fn", A.gt(V(0)));
  emit("exp", C.exp());
  emit("abs", A.abs());
  emit("sign", A.sign());
  emit("sign_nan_negzero", S.sign());
  emit_scalar("l2norm_6", A.l2Norm());
  emit_scalar("l2norm_3", C.l2Norm());
  emit("where_ttt_same", _where(B, A, Z));
  emit("where_ttt_bcast", _where(D, A, C));
  emit("where_tss", _where(B, V(1), V(-1)));
  emit("where_tts", _where(C, A, V(9)));
  emit("where_tst", _where(C, V(9), A));
  emit("where_tts_literal", _where(B, A, 0.0));
  emit("where_tst_literal", _where(B, 0, A));
  emit("where_tss_literal", _where(B, 1, 0.5));
  emit("where_nan_cond", _where(S, P, C));
  Tensor<V, 1> g(A.values[3]);
  emit("getitem", g);
  Tensor<V, 6> cl(A);
  emit("clone", cl);
  Tensor<V, 3> acc;
  acc += C; acc += P;
  emit("accumulate", acc);
  Tensor<V, 3> fill; fill = V(4.5);
  emit("fill", fill);
  emit("chain_spring", (V(1.5) * (C.l2Norm() - V(3))) * C / C.l2Norm());
}

int main() {
  run<float>();
  run<double>();
  return 0;
}
