// TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's per-item value type.
//
// Nothing in the shipped package may include this file: it exists so that tests, the smoke check and
// the CPU-baseline leg of the benchmark have an independent statement of the arithmetic the HIP path
// must reproduce.
//
// Restates `Tensor<ValueT, Dim>` and its free operators from the reference's data_struct_shared.cuh
// (lines quoted per function below).  Semantics that differ from torch and are kept on purpose:
//   * default construction zero-fills                                   (data_struct_shared.cuh:93-98)
//   * same-width tensor/tensor division yields 0 where the divisor is 0 (:194-200); scalar/tensor
//     division is guarded the same way (:402-408); tensor/scalar is NOT guarded (:238-244); a division
//     between tensors of different width is NOT guarded either (the modulo-broadcast macro, :611-627)
//   * operator^ is pow                                                   (:202-208, :246-252, :410-417)
//   * tensors of different width combine by flat index modulo a[i%N] op b[i%M] (:611-659)
//   * lt / gt produce 0/1 in the value type                              (:325-344, :639-659)
//   * where(c, x, y) selects on c != 0 with modulo broadcast and scalar mixes (:498-609)
//   * sign(NaN) == 0                                                     (:70-75)
//   * l2 norm returns a bare scalar sqrt(sum v^2)                        (:346-353)
//   * arithmetic scalars of another type are cast to the value type first (:425-449)
//
// Parity pin: tests/golden/tensor_kat.json holds the output of oracle/tensor_kat.cpp compiled against
// the reference header itself; the same driver compiled against this file must print identical bits.
#pragma once
#include <cmath>
#include <cstdlib>
#include <type_traits>

namespace oracle {

template <typename V> inline V ref_pow(V b, V e) { return static_cast<V>(std::pow(b, e)); }   // :41-48
template <typename V> inline V ref_exp(V x) { return static_cast<V>(std::exp(x)); }          // :50-57
template <typename V> inline V ref_abs(V x) { using std::abs; return abs(x); }               // :59-67
template <typename V> inline V ref_sign(V x) {                                               // :69-75
  return x > V(0) ? V(1) : (x < V(0) ? V(-1) : V(0));
}

template <typename V, int N>
struct Tensor {
  V values[N];

  Tensor() { for (int i = 0; i < N; ++i) values[i] = V(0); }                                  // :93-98
  Tensor(V one) { static_assert(N == 1, "single-value construction needs width 1"); values[0] = one; } // :100-104
  Tensor(const V* src) { for (int i = 0; i < N; ++i) values[i] = src[i]; }                    // :106-111
  Tensor(V* src) { for (int i = 0; i < N; ++i) values[i] = src[i]; }

  V& operator[](int i) { return values[i]; }
  const V& operator[](int i) const { return values[i]; }

  Tensor& operator=(V fill) { for (int i = 0; i < N; ++i) values[i] = fill; return *this; }  // :140-146

  Tensor operator-() const { Tensor r; for (int i = 0; i < N; ++i) r.values[i] = -values[i]; return r; } // :159-166

  // same-width tensor (+)= tensor                                                              :172-209
  Tensor& operator+=(const Tensor& o) { for (int i = 0; i < N; ++i) values[i] += o.values[i]; return *this; }
  Tensor& operator-=(const Tensor& o) { for (int i = 0; i < N; ++i) values[i] -= o.values[i]; return *this; }
  Tensor& operator*=(const Tensor& o) { for (int i = 0; i < N; ++i) values[i] *= o.values[i]; return *this; }
  Tensor& operator/=(const Tensor& o) {
    for (int i = 0; i < N; ++i) values[i] = (o.values[i] != V(0)) ? V(values[i] / o.values[i]) : V(0);
    return *this;
  }
  Tensor& operator^=(const Tensor& o) { for (int i = 0; i < N; ++i) values[i] = ref_pow(values[i], o.values[i]); return *this; }

  // tensor (+)= scalar                                                                          :214-252
  Tensor& operator+=(V s) { for (int i = 0; i < N; ++i) values[i] += s; return *this; }
  Tensor& operator-=(V s) { for (int i = 0; i < N; ++i) values[i] -= s; return *this; }
  Tensor& operator*=(V s) { for (int i = 0; i < N; ++i) values[i] *= s; return *this; }
  Tensor& operator/=(V s) { for (int i = 0; i < N; ++i) values[i] /= s; return *this; }
  Tensor& operator^=(V s) { for (int i = 0; i < N; ++i) values[i] = ref_pow(values[i], s); return *this; }

  // binary forms built from the compound ones                                                   :258-271
  Tensor operator+(const Tensor& o) const { Tensor r = *this; r += o; return r; }
  Tensor operator-(const Tensor& o) const { Tensor r = *this; r -= o; return r; }
  Tensor operator*(const Tensor& o) const { Tensor r = *this; r *= o; return r; }
  Tensor operator/(const Tensor& o) const { Tensor r = *this; r /= o; return r; }
  Tensor operator^(const Tensor& o) const { Tensor r = *this; r ^= o; return r; }
  Tensor operator+(V s) const { Tensor r = *this; r += s; return r; }
  Tensor operator-(V s) const { Tensor r = *this; r -= s; return r; }
  Tensor operator*(V s) const { Tensor r = *this; r *= s; return r; }
  Tensor operator/(V s) const { Tensor r = *this; r /= s; return r; }
  Tensor operator^(V s) const { Tensor r = *this; r ^= s; return r; }

  Tensor exp() const { Tensor r; for (int i = 0; i < N; ++i) r.values[i] = ref_exp(values[i]); return r; }    // :294-301
  Tensor abs() const { Tensor r; for (int i = 0; i < N; ++i) r.values[i] = ref_abs(values[i]); return r; }    // :303-310
  Tensor sign() const { Tensor r; for (int i = 0; i < N; ++i) r.values[i] = ref_sign(values[i]); return r; }  // :312-319
  Tensor lt(V s) const { Tensor r; for (int i = 0; i < N; ++i) r.values[i] = values[i] < s ? V(1) : V(0); return r; } // :325-332
  Tensor gt(V s) const { Tensor r; for (int i = 0; i < N; ++i) r.values[i] = values[i] > s ? V(1) : V(0); return r; } // :334-341
  Tensor operator<(V s) const { return lt(s); }                                                 // :343
  Tensor operator>(V s) const { return gt(s); }                                                 // :344

  V l2Norm() const {                                                                            // :346-353
    V acc = V(0);
    for (int i = 0; i < N; ++i) acc += values[i] * values[i];
    return static_cast<V>(std::sqrt(acc));
  }
};

// scalar (op) tensor                                                                            :381-417
template <typename V, int N> inline Tensor<V, N> operator*(V s, const Tensor<V, N>& t) { return t * s; }
template <typename V, int N> inline Tensor<V, N> operator+(V s, const Tensor<V, N>& t) { return t + s; }
template <typename V, int N> inline Tensor<V, N> operator-(V s, const Tensor<V, N>& t) {
  Tensor<V, N> r; for (int i = 0; i < N; ++i) r.values[i] = s - t.values[i]; return r;
}
template <typename V, int N> inline Tensor<V, N> operator/(V s, const Tensor<V, N>& t) {
  Tensor<V, N> r; for (int i = 0; i < N; ++i) r.values[i] = (t.values[i] != V(0)) ? V(s / t.values[i]) : V(0); return r;
}
template <typename V, int N> inline Tensor<V, N> operator^(V s, const Tensor<V, N>& t) {
  Tensor<V, N> r; for (int i = 0; i < N; ++i) r.values[i] = ref_pow(s, t.values[i]); return r;
}

// arithmetic scalars of a different type are converted to V and re-dispatched                   :425-449
#define ORACLE_MIXED(op)                                                                                   \
  template <typename S, typename V, int N,                                                                 \
            typename std::enable_if<std::is_arithmetic<S>::value && !std::is_same<S, V>::value, int>::type = 0> \
  inline Tensor<V, N> operator op(S s, const Tensor<V, N>& t) { return static_cast<V>(s) op t; }           \
  template <typename S, typename V, int N,                                                                 \
            typename std::enable_if<std::is_arithmetic<S>::value && !std::is_same<S, V>::value, int>::type = 0> \
  inline Tensor<V, N> operator op(const Tensor<V, N>& t, S s) { return t op static_cast<V>(s); }
ORACLE_MIXED(+)
ORACLE_MIXED(-)
ORACLE_MIXED(*)
ORACLE_MIXED(/)
ORACLE_MIXED(^)
#undef ORACLE_MIXED

// tensors of different width: flat-index modulo broadcast, raw operator (no zero guard)         :611-659
// (for N == M overload resolution prefers the non-template members above, as in the reference)
#define ORACLE_BCAST(op)                                                                  \
  template <typename V, int N, int M>                                                     \
  inline Tensor<V, (N > M ? N : M)> operator op(const Tensor<V, N>& a, const Tensor<V, M>& b) { \
    Tensor<V, (N > M ? N : M)> r;                                                         \
    for (int i = 0; i < (N > M ? N : M); ++i) r[i] = a[i % N] op b[i % M];                \
    return r;                                                                             \
  }
ORACLE_BCAST(+)
ORACLE_BCAST(-)
ORACLE_BCAST(*)
ORACLE_BCAST(/)
#undef ORACLE_BCAST
template <typename V, int N, int M>
inline Tensor<V, (N > M ? N : M)> operator^(const Tensor<V, N>& a, const Tensor<V, M>& b) {
  Tensor<V, (N > M ? N : M)> r;
  for (int i = 0; i < (N > M ? N : M); ++i) r[i] = ref_pow(a[i % N], b[i % M]);
  return r;
}
template <typename V, int N, int M>
inline Tensor<V, (N > M ? N : M)> operator<(const Tensor<V, N>& a, const Tensor<V, M>& b) {
  Tensor<V, (N > M ? N : M)> r;
  for (int i = 0; i < (N > M ? N : M); ++i) r[i] = a[i % N] < b[i % M] ? V(1) : V(0);
  return r;
}
template <typename V, int N, int M>
inline Tensor<V, (N > M ? N : M)> operator>(const Tensor<V, N>& a, const Tensor<V, M>& b) {
  Tensor<V, (N > M ? N : M)> r;
  for (int i = 0; i < (N > M ? N : M); ++i) r[i] = a[i % N] > b[i % M] ? V(1) : V(0);
  return r;
}

// where(cond, x, y): cond != 0 selects x                                                        :498-609
namespace detail {
template <typename V, int N> inline V pick(const Tensor<V, N>& t, int i) { return t[i % N]; }
template <typename V, typename S, typename std::enable_if<std::is_arithmetic<S>::value, int>::type = 0>
inline V pick(S s, int) { return static_cast<V>(s); }
template <typename T> struct width { static constexpr int value = 1; };
template <typename V, int N> struct width<Tensor<V, N>> { static constexpr int value = N; };
constexpr int max3(int a, int b, int c) { return a > b ? (a > c ? a : c) : (b > c ? b : c); }
}  // namespace detail

template <typename V, int CN, typename X, typename Y>
inline Tensor<V, detail::max3(CN, detail::width<X>::value, detail::width<Y>::value)>
_where(const Tensor<V, CN>& cond, const X& x, const Y& y) {
  constexpr int OUT = detail::max3(CN, detail::width<X>::value, detail::width<Y>::value);
  Tensor<V, OUT> r;
  for (int i = 0; i < OUT; ++i) r[i] = (cond[i % CN] != V(0)) ? detail::pick<V>(x, i) : detail::pick<V>(y, i);
  return r;
}

}  // namespace oracle
