// Per-item value type used inside generated gfx950 kernels.
//
// A `Tensor<V, N>` is N values of one edge or vertex held in registers.  The operator set and its
// corner cases follow the reference's value type (data_struct_shared.cuh:80-661) because generated
// statements are written against it and results must agree with the reference's CPU path:
//   - default construction is all zeros                                     (:93-98)
//   - same-width tensor / tensor and scalar / tensor give 0 where the divisor is 0 (:194-200, :402-408)
//   - tensor / scalar and different-width tensor / tensor are plain divisions    (:238-244, :611-627)
//   - operator^ is pow                                                       (:202-208)
//   - different widths broadcast by flat index modulo                        (:611-659)
//   - comparisons yield 0/1 in V, where() selects on != 0                    (:325-344, :498-609)
//   - sign(NaN) is 0, l2Norm() is a scalar                                   (:70-75, :346-353)
//   - numbers of another arithmetic type are converted to V first            (:425-449)
// Everything is force-inlined; loops have constant trip counts and unroll into straight-line code.
#pragma once
#include <hip/hip_runtime.h>
#include <type_traits>

#define FLEX_DEV __device__ __forceinline__

namespace flex {

template <typename V> FLEX_DEV V v_pow(V b, V e) { return static_cast<V>(pow(b, e)); }
template <> FLEX_DEV float v_pow<float>(float b, float e) { return powf(b, e); }
template <> FLEX_DEV long v_pow<long>(long b, long e) { return static_cast<long>(pow(static_cast<double>(b), static_cast<double>(e))); }
template <typename V> FLEX_DEV V v_exp(V x) { return static_cast<V>(exp(x)); }
template <> FLEX_DEV float v_exp<float>(float x) { return expf(x); }
template <> FLEX_DEV long v_exp<long>(long x) { return static_cast<long>(exp(static_cast<double>(x))); }
template <typename V> FLEX_DEV V v_abs(V x) { return x < V(0) ? -x : x; }
template <> FLEX_DEV float v_abs<float>(float x) { return fabsf(x); }
template <> FLEX_DEV double v_abs<double>(double x) { return fabs(x); }
template <typename V> FLEX_DEV V v_sqrt(V x) { return static_cast<V>(sqrt(static_cast<double>(x))); }
template <> FLEX_DEV float v_sqrt<float>(float x) { return sqrtf(x); }
// sqrt to within one unit in the last place: the hardware instruction alone for float (with the scaling that
// keeps denormal arguments in its range) instead of the correctly rounded sequence, which is three times as
// long.  Used where the generator knows the value is a length (norm): 17 -> 6 instructions per edge.
template <typename V> FLEX_DEV V v_sqrt_1ulp(V x) { return v_sqrt(x); }
template <> FLEX_DEV float v_sqrt_1ulp<float>(float x) {
  const bool tiny = x < 0x1p-96f;
  const float r = __builtin_amdgcn_sqrtf(tiny ? x * 0x1p+32f : x);
  return tiny ? r * 0x1p-16f : r;
}
template <int E, typename V> FLEX_DEV V v_ipow(V x) {
  V y = x;
#pragma unroll
  for (int k = 1; k < E; ++k) y *= x;
  return y;
}
template <typename V> FLEX_DEV V v_sign(V x) { return x > V(0) ? V(1) : (x < V(0) ? V(-1) : V(0)); }

template <typename V, int N>
struct Tensor {
  V values[N];

  FLEX_DEV Tensor() {
#pragma unroll
    for (int i = 0; i < N; ++i) values[i] = V(0);
  }
  FLEX_DEV Tensor(V one) {
    static_assert(N == 1, "single-value construction needs width 1");
    values[0] = one;
  }
  FLEX_DEV explicit Tensor(const V* src) {
#pragma unroll
    for (int i = 0; i < N; ++i) values[i] = src[i];
  }
  // Vertex data addressed through an index (second memory level).
  static FLEX_DEV Tensor gathered(const V* src) {
#ifdef FLEX_TUNE_GATHER_POLICY
    Tensor t;
#pragma unroll
    for (int i = 0; i < N; ++i) {
#if FLEX_TUNE_GATHER_POLICY == 1
      t.values[i] = __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#elif FLEX_TUNE_GATHER_POLICY == 2
      t.values[i] = __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
#else
      t.values[i] = __builtin_nontemporal_load(src + i);
#endif
    }
    return t;
#else
    return Tensor(src);
#endif
  }
  FLEX_DEV V& operator[](int i) { return values[i]; }
  FLEX_DEV const V& operator[](int i) const { return values[i]; }
  FLEX_DEV Tensor& operator=(V fill) {
#pragma unroll
    for (int i = 0; i < N; ++i) values[i] = fill;
    return *this;
  }
  FLEX_DEV Tensor operator-() const {
    Tensor r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.values[i] = -values[i];
    return r;
  }
  FLEX_DEV Tensor& operator+=(const Tensor& o) {
#pragma unroll
    for (int i = 0; i < N; ++i) values[i] += o.values[i];
    return *this;
  }
  FLEX_DEV Tensor exp() const {
    Tensor r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.values[i] = v_exp(values[i]);
    return r;
  }
  FLEX_DEV Tensor abs() const {
    Tensor r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.values[i] = v_abs(values[i]);
    return r;
  }
  FLEX_DEV Tensor sign() const {
    Tensor r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.values[i] = v_sign(values[i]);
    return r;
  }
  // Powers with a literal exponent.  The reference spells every power pow(x, e) (operator^); for the
  // exponents below the direct form is the same value to within an ulp and an order of magnitude
  // cheaper than a general pow on the GPU.
  FLEX_DEV Tensor sqrt() const {
    Tensor r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.values[i] = v_sqrt(values[i]);
    return r;
  }
  template <int E>
  FLEX_DEV Tensor ipow() const {
    static_assert(E >= 1 && E <= 4, "small positive integer powers only");
    Tensor r;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const V x = values[i];
      V y = x;
#pragma unroll
      for (int k = 1; k < E; ++k) y *= x;
      r.values[i] = y;
    }
    return r;
  }
  FLEX_DEV V l2Norm() const {
    V acc = V(0);
#pragma unroll
    for (int i = 0; i < N; ++i) acc += values[i] * values[i];
    return v_sqrt_1ulp(acc);
  }
};

namespace detail {
template <typename T> struct is_tensor : std::false_type {};
template <typename V, int N> struct is_tensor<Tensor<V, N>> : std::true_type {};
constexpr int imax(int a, int b) { return a > b ? a : b; }

// One arithmetic step on two scalars; GUARD selects the divide-by-zero-gives-zero rule.
template <char OP, bool GUARD, typename V> FLEX_DEV V apply(V a, V b) {
  if constexpr (OP == '+') return a + b;
  else if constexpr (OP == '-') return a - b;
  else if constexpr (OP == '*') return a * b;
  else if constexpr (OP == '/') {
    if constexpr (GUARD) return (b != V(0)) ? V(a / b) : V(0);
    else return a / b;
  } else if constexpr (OP == '^') return v_pow(a, b);
  else if constexpr (OP == '<') return a < b ? V(1) : V(0);
  else return a > b ? V(1) : V(0);
}

// tensor (op) tensor: equal widths are element-wise (guarded division), unequal widths broadcast by
// flat index modulo with the plain operator.
template <char OP, typename V, int N, int M>
FLEX_DEV Tensor<V, imax(N, M)> tt(const Tensor<V, N>& a, const Tensor<V, M>& b) {
  Tensor<V, imax(N, M)> r;
#pragma unroll
  for (int i = 0; i < imax(N, M); ++i) r.values[i] = apply<OP, (N == M), V>(a.values[i % N], b.values[i % M]);
  return r;
}
// tensor (op) scalar: plain operator (division unguarded).
template <char OP, typename V, int N> FLEX_DEV Tensor<V, N> ts(const Tensor<V, N>& a, V s) {
  Tensor<V, N> r;
#pragma unroll
  for (int i = 0; i < N; ++i) r.values[i] = apply<OP, false, V>(a.values[i], s);
  return r;
}
// scalar (op) tensor: division guarded.
template <char OP, typename V, int N> FLEX_DEV Tensor<V, N> st(V s, const Tensor<V, N>& b) {
  Tensor<V, N> r;
#pragma unroll
  for (int i = 0; i < N; ++i) r.values[i] = apply<OP, true, V>(s, b.values[i]);
  return r;
}
}  // namespace detail

#define FLEX_BINARY(sym, ch)                                                                        \
  template <typename V, int N, int M>                                                               \
  FLEX_DEV Tensor<V, detail::imax(N, M)> operator sym(const Tensor<V, N>& a, const Tensor<V, M>& b) { \
    return detail::tt<ch>(a, b);                                                                    \
  }                                                                                                 \
  template <typename V, int N, typename S, typename std::enable_if<std::is_arithmetic<S>::value, int>::type = 0> \
  FLEX_DEV Tensor<V, N> operator sym(const Tensor<V, N>& a, S s) {                                  \
    return detail::ts<ch>(a, static_cast<V>(s));                                                    \
  }                                                                                                 \
  template <typename V, int N, typename S, typename std::enable_if<std::is_arithmetic<S>::value, int>::type = 0> \
  FLEX_DEV Tensor<V, N> operator sym(S s, const Tensor<V, N>& b) {                                  \
    return detail::st<ch>(static_cast<V>(s), b);                                                    \
  }
FLEX_BINARY(+, '+')
FLEX_BINARY(-, '-')
FLEX_BINARY(*, '*')
FLEX_BINARY(/, '/')
FLEX_BINARY(^, '^')
#undef FLEX_BINARY

// tensor / scalar for a tensor of several values: one division (the reciprocal) and a multiplication per
// value instead of a division per value; each quotient is within 1.5 units in the last place of the divided
// one (an IEEE float division is ten instructions, a multiplication one).  Integers keep the division, and so
// does a divisor so small that its reciprocal would overflow.
template <typename V, int N> FLEX_DEV Tensor<V, N> times_reciprocal(const Tensor<V, N>& a, V s) {
  if constexpr (std::is_floating_point<V>::value && N > 1) {
    const V r = V(1) / s;
    Tensor<V, N> q;
    // one branch per wavefront: the divisions run only if some lane's reciprocal is not finite
    if (__builtin_amdgcn_ballot_w64(!(r - r == V(0))) == 0ull) {
#pragma unroll
      for (int i = 0; i < N; ++i) q.values[i] = a.values[i] * r;
    } else {
#pragma unroll
      for (int i = 0; i < N; ++i) q.values[i] = a.values[i] / s;
    }
    return q;
  } else {
    return detail::ts<'/'>(a, s);
  }
}

// Comparisons exist as tensor-tensor (any widths) and tensor-scalar.
#define FLEX_COMPARE(sym, ch)                                                                       \
  template <typename V, int N, int M>                                                               \
  FLEX_DEV Tensor<V, detail::imax(N, M)> operator sym(const Tensor<V, N>& a, const Tensor<V, M>& b) { \
    return detail::tt<ch>(a, b);                                                                    \
  }                                                                                                 \
  template <typename V, int N, typename S, typename std::enable_if<std::is_arithmetic<S>::value, int>::type = 0> \
  FLEX_DEV Tensor<V, N> operator sym(const Tensor<V, N>& a, S s) {                                  \
    return detail::ts<ch>(a, static_cast<V>(s));                                                    \
  }
FLEX_COMPARE(<, '<')
FLEX_COMPARE(>, '>')
#undef FLEX_COMPARE

namespace detail {
template <typename V, typename X> FLEX_DEV V pick(const X& x, int i) {
  if constexpr (is_tensor<X>::value) return x.values[i % (int)(sizeof(x.values) / sizeof(V))];
  else return static_cast<V>(x);
}
template <typename V, typename X> constexpr int width_of() {
  if constexpr (is_tensor<X>::value) return (int)(sizeof(X) / sizeof(V));
  else return 1;
}
}  // namespace detail

// where(cond, x, y): x where cond != 0, else y; x and y may be tensors of any width or numbers.
template <typename V, int CN, typename X, typename Y>
FLEX_DEV Tensor<V, detail::imax(CN, detail::imax(detail::width_of<V, X>(), detail::width_of<V, Y>()))>
_where(const Tensor<V, CN>& cond, const X& x, const Y& y) {
  constexpr int OUT = detail::imax(CN, detail::imax(detail::width_of<V, X>(), detail::width_of<V, Y>()));
  Tensor<V, OUT> r;
#pragma unroll
  for (int i = 0; i < OUT; ++i)
    r.values[i] = (cond.values[i % CN] != V(0)) ? detail::pick<V>(x, i) : detail::pick<V>(y, i);
  return r;
}

}  // namespace flex
