// TEST INFRASTRUCTURE ONLY -- runs the known-answer cases of the per-item value type on the GPU
// against the header generated kernels are compiled with (flexspmv_amd/csrc/flex_tensor.hpp) and
// prints them in the format of oracle/tensor_kat.cpp ("<case> <type> <hex bits of each element>"),
// so that a test can set the lines beside tests/golden/tensor_kat.json (made from the reference's own
// data_struct_shared.cuh).  One thread evaluates every case; results leave through a word buffer
// (per case: element count, then the bits of each element).
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <limits>
#include <string>
#include <vector>

#include "flex_tensor.hpp"

using flex::_where;
using flex::Tensor;

#define KAT_NO_MEMBER_COMPARE 1

template <typename V> struct Bits;
template <> struct Bits<float> {
  static __host__ __device__ unsigned long long of(float v) { return (unsigned long long)__builtin_bit_cast(uint32_t, v); }
  static const char* name() { return "f32"; }
};
template <> struct Bits<double> {
  static __host__ __device__ unsigned long long of(double v) { return __builtin_bit_cast(uint64_t, v); }
  static const char* name() { return "f64"; }
};
template <> struct Bits<long> {
  static __host__ __device__ unsigned long long of(long v) { return (unsigned long long)v; }
  static const char* name() { return "i64"; }
};

struct Recorder {
  unsigned long long* out;
  int n;
  template <typename V, int N> __device__ void tensor(const Tensor<V, N>& t) {
    out[n++] = N;
    for (int i = 0; i < N; ++i) out[n++] = Bits<V>::of(t.values[i]);
  }
  template <typename V> __device__ void scalar(V v) {
    out[n++] = 1;
    out[n++] = Bits<V>::of(v);
  }
};

constexpr int MAX_WORDS = 4096;

// device pass: evaluate, record
#define KAT_EMIT(label, t) rec.tensor(t)
#define KAT_EMIT_SCALAR(label, v) rec.scalar(v)
template <typename V>
__global__ void float_cases(unsigned long long* out, int* words) {
  Recorder rec{out, 0};
#include "tensor_kat_cases.inc"
  *words = rec.n;
}
template <typename V>
__global__ void integer_cases(unsigned long long* out, int* words) {
  Recorder rec{out, 0};
#include "tensor_kat_cases_i64.inc"
  *words = rec.n;
}
#undef KAT_EMIT
#undef KAT_EMIT_SCALAR

#define CHECK(call)                                                                 \
  do {                                                                              \
    hipError_t e_ = (call);                                                         \
    if (e_ != hipSuccess) {                                                         \
      std::fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));               \
      return 2;                                                                     \
    }                                                                               \
  } while (0)

// Case labels in file order, read from the case lists' own text at build time: the build script passes
// them as KAT_FLOAT_LABELS / KAT_INT_LABELS (comma separated string literals).
static const char* const kFloatLabels[] = {KAT_FLOAT_LABELS};
static const char* const kIntLabels[] = {KAT_INT_LABELS};

template <typename V, typename Kernel>
static int run(Kernel kernel, const char* const* labels, int num_labels) {
  unsigned long long* d_out = nullptr;
  int* d_words = nullptr;
  CHECK(hipMalloc(&d_out, sizeof(unsigned long long) * MAX_WORDS));
  CHECK(hipMalloc(&d_words, sizeof(int)));
  CHECK(hipMemset(d_words, 0, sizeof(int)));
  hipLaunchKernelGGL(kernel, dim3(1), dim3(1), 0, 0, d_out, d_words);
  CHECK(hipGetLastError());
  CHECK(hipDeviceSynchronize());
  int words = 0;
  CHECK(hipMemcpy(&words, d_words, sizeof(int), hipMemcpyDeviceToHost));
  if (words <= 0 || words > MAX_WORDS) {
    std::fprintf(stderr, "unexpected word count %d\n", words);
    return 3;
  }
  std::vector<unsigned long long> out(words);
  CHECK(hipMemcpy(out.data(), d_out, sizeof(unsigned long long) * words, hipMemcpyDeviceToHost));
  int at = 0;
  for (int c = 0; c < num_labels; ++c) {
    if (at >= words) {
      std::fprintf(stderr, "fewer recorded cases than labels\n");
      return 4;
    }
    const int n = (int)out[at++];
    std::printf("%s %s", labels[c], Bits<V>::name());
    for (int i = 0; i < n; ++i) std::printf(" %llx", out[at++]);
    std::printf("\n");
  }
  if (at != words) {
    std::fprintf(stderr, "more recorded cases than labels\n");
    return 5;
  }
  CHECK(hipFree(d_out));
  CHECK(hipFree(d_words));
  return 0;
}

int main() {
  const int nf = (int)(sizeof(kFloatLabels) / sizeof(kFloatLabels[0]));
  const int ni = (int)(sizeof(kIntLabels) / sizeof(kIntLabels[0]));
  int rc = run<float>(float_cases<float>, kFloatLabels, nf);
  if (rc == 0) rc = run<double>(float_cases<double>, kFloatLabels, nf);
  if (rc == 0) rc = run<long>(integer_cases<long>, kIntLabels, ni);
  return rc;
}
