// A caller of the two C interfaces that knows nothing of Python or torch: device memory from hipMalloc,
// libraries opened with dlopen, symbols exactly as include/flexspmv.h and include/flexspmv_formats.h
// declare them.  It does what the reference's CPU test driver does for CSR SpMV (main.cpp:126-176: build a
// matrix, run the generated kernel, compare with a plain loop) on a 2-D 5-point Laplacian:
//
//   COO row ids --flexspmv_coo_rows_to_csr--> row pointer --flexspmv_launch--> y,   y vs. a host loop
//
// in float32 and float64.  Usage: spmv_from_c <libcsr_spmv.so> <libflexspmv_formats.so> [grid edge]
// Prints one line per check and "OK" at the end; any failure exits non-zero.
#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "flexspmv.h"
#include "flexspmv_formats.h"

#define HIP_OK(call)                                                                       \
  do {                                                                                     \
    hipError_t e_ = (call);                                                                \
    if (e_ != hipSuccess) {                                                                \
      fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
      return 2;                                                                            \
    }                                                                                      \
  } while (0)

template <typename F>
static F symbol(void* lib, const char* name) {
  void* p = dlsym(lib, name);
  if (p == nullptr) {
    fprintf(stderr, "missing symbol %s\n", name);
    exit(3);
  }
  return reinterpret_cast<F>(p);
}

template <typename V>
static int run(int n, int dtype, double tolerance, decltype(&flexspmv_launch) launch,
               decltype(&flexspmv_workspace_bytes) workspace_bytes, decltype(&flexspmv_last_error) last_error,
               decltype(&flexspmv_coo_rows_to_csr) rows_to_csr) {
  // 5-point Laplacian on an n x n grid, Dirichlet boundary, COO sorted by row, columns ascending
  const int N = n * n;
  std::vector<int32_t> rows, cols;
  std::vector<V> vals, x(N);
  for (int i = 0; i < n; ++i)
    for (int j = 0; j < n; ++j) {
      const int r = i * n + j;
      auto add = [&](int c, V v) { rows.push_back(r); cols.push_back(c); vals.push_back(v); };
      if (i > 0) add(r - n, V(-1));
      if (j > 0) add(r - 1, V(-1));
      add(r, V(4));
      if (j < n - 1) add(r + 1, V(-1));
      if (i < n - 1) add(r + n, V(-1));
    }
  unsigned state = 12345u;
  for (int r = 0; r < N; ++r) {
    state = state * 1664525u + 1013904223u;
    x[r] = V((state >> 8) * (2.0 / 16777216.0) - 1.0);
  }
  const int64_t ne = (int64_t)rows.size();

  int32_t *d_rows, *d_cols, *d_ptr, *d_findings;
  V *d_vals, *d_x, *d_y;
  HIP_OK(hipMalloc(&d_rows, ne * 4));
  HIP_OK(hipMalloc(&d_cols, ne * 4));
  HIP_OK(hipMalloc(&d_ptr, (N + 1) * 4));
  HIP_OK(hipMalloc(&d_findings, 16));
  HIP_OK(hipMalloc(&d_vals, ne * sizeof(V)));
  HIP_OK(hipMalloc(&d_x, N * sizeof(V)));
  HIP_OK(hipMalloc(&d_y, N * sizeof(V)));
  HIP_OK(hipMemcpy(d_rows, rows.data(), ne * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_cols, cols.data(), ne * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_vals, vals.data(), ne * sizeof(V), hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_x, x.data(), N * sizeof(V), hipMemcpyHostToDevice));
  HIP_OK(hipMemset(d_y, 0xff, N * sizeof(V)));  // outputs need no zero fill: every element is written

  // row pointer from the COO row ids
  int rc = rows_to_csr(d_rows, 4, ne, N, d_ptr, d_findings, nullptr);
  if (rc != 0) { fprintf(stderr, "flexspmv_coo_rows_to_csr failed: %d\n", rc); return 4; }
  std::vector<int32_t> ptr(N + 1);
  int32_t findings[4];
  HIP_OK(hipMemcpy(ptr.data(), d_ptr, (N + 1) * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(findings, d_findings, 16, hipMemcpyDeviceToHost));
  if (findings[0] != 0) { fprintf(stderr, "row ids reported as bad: %d\n", findings[0]); return 4; }
  for (int r = 0, e = 0; r <= N; ++r) {
    while (e < ne && rows[e] < r) ++e;
    if (ptr[r] != e) { fprintf(stderr, "row_ptr[%d] = %d, expected %d\n", r, ptr[r], e); return 4; }
  }
  printf("dtype %d: row pointer of %lld COO ids exact\n", dtype, (long long)ne);

  // the launch
  const size_t ws_bytes = workspace_bytes(dtype, N, ne);
  void* d_ws = nullptr;
  if (ws_bytes > 0) HIP_OK(hipMalloc(&d_ws, ws_bytes));
  void* value_inputs[2] = {d_vals, d_x};
  const int32_t* index_inputs[1] = {d_cols};
  void* outputs[1] = {d_y};
  flexspmv_launch_args args;
  memset(&args, 0, sizeof(args));
  args.struct_size = sizeof(args);
  args.dtype = dtype;
  args.value_inputs = value_inputs;
  args.num_value_inputs = 2;
  args.index_inputs = index_inputs;
  args.num_index_inputs = 1;
  args.outputs = outputs;
  args.num_outputs = 1;
  args.row_end_offsets = d_ptr;
  args.num_rows = N;
  args.num_cols = N;
  args.ne = ne;
  args.workspace = d_ws;
  args.workspace_bytes = ws_bytes;
  args.stream = nullptr;
  args.flags = 0;
  rc = launch(&args);
  if (rc != 0) { fprintf(stderr, "flexspmv_launch failed: %d %s\n", rc, last_error()); return 5; }
  HIP_OK(hipDeviceSynchronize());
  std::vector<V> y(N);
  HIP_OK(hipMemcpy(y.data(), d_y, N * sizeof(V), hipMemcpyDeviceToHost));

  double worst = 0.0;
  for (int r = 0; r < N; ++r) {
    double ref = 0.0, scale = 0.0;
    for (int e = ptr[r]; e < ptr[r + 1]; ++e) {
      ref += (double)vals[e] * (double)x[cols[e]];
      scale += std::fabs((double)vals[e] * (double)x[cols[e]]);
    }
    const double err = std::fabs((double)y[r] - ref) / (scale > 0 ? scale : 1.0);
    if (!(err <= worst)) worst = err;  // also catches NaN
  }
  printf("dtype %d: y = A x on %d rows, max error relative to the row scale %.3e (tolerance %.0e)\n", dtype, N, worst,
         tolerance);
  if (!(worst <= tolerance)) return 6;

  // a workspace that is too small is refused, with a message
  args.workspace_bytes = ws_bytes > 0 ? ws_bytes - 1 : 0;
  if (ws_bytes > 0 && (launch(&args) != FLEXSPMV_ERR_WORKSPACE || strlen(last_error()) == 0)) {
    fprintf(stderr, "short workspace was not refused\n");
    return 7;
  }
  hipFree(d_rows); hipFree(d_cols); hipFree(d_ptr); hipFree(d_findings);
  hipFree(d_vals); hipFree(d_x); hipFree(d_y); hipFree(d_ws);
  return 0;
}

int main(int argc, char** argv) {
  if (argc < 3) {
    fprintf(stderr, "usage: %s <libcsr_spmv.so> <libflexspmv_formats.so> [grid edge]\n", argv[0]);
    return 1;
  }
  const int n = argc > 3 ? atoi(argv[3]) : 300;
  void* kernel_lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  void* formats_lib = dlopen(argv[2], RTLD_NOW | RTLD_LOCAL);
  if (kernel_lib == nullptr || formats_lib == nullptr) {
    fprintf(stderr, "dlopen failed: %s\n", dlerror());
    return 1;
  }
  auto abi = symbol<decltype(&flexspmv_abi_version)>(kernel_lib, "flexspmv_abi_version");
  auto fabi = symbol<decltype(&flexspmv_formats_abi_version)>(formats_lib, "flexspmv_formats_abi_version");
  if (abi() != FLEXSPMV_ABI_VERSION || fabi() != FLEXSPMV_FORMATS_ABI_VERSION) {
    fprintf(stderr, "interface versions %d / %d do not match the headers\n", abi(), fabi());
    return 1;
  }
  auto signature = symbol<decltype(&flexspmv_signature)>(kernel_lib, "flexspmv_signature");
  if (strstr(signature(), "\"graph\": \"csr_spmv\"") == nullptr) {
    fprintf(stderr, "not the csr_spmv library: %s\n", signature());
    return 1;
  }
  auto launch = symbol<decltype(&flexspmv_launch)>(kernel_lib, "flexspmv_launch");
  auto workspace_bytes = symbol<decltype(&flexspmv_workspace_bytes)>(kernel_lib, "flexspmv_workspace_bytes");
  auto last_error = symbol<decltype(&flexspmv_last_error)>(kernel_lib, "flexspmv_last_error");
  auto rows_to_csr = symbol<decltype(&flexspmv_coo_rows_to_csr)>(formats_lib, "flexspmv_coo_rows_to_csr");
  int rc = run<float>(n, FLEXSPMV_F32, 1e-5, launch, workspace_bytes, last_error, rows_to_csr);
  if (rc == 0) rc = run<double>(n, FLEXSPMV_F64, 1e-12, launch, workspace_bytes, last_error, rows_to_csr);
  if (rc == 0) printf("OK\n");
  return rc;
}
