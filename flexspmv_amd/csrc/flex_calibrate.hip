// Calibration kernel for bench.py: what this GPU's memory system delivers for a given mix of reads and
// writes, with no arithmetic in the way.  One block per tile, as in the reducer: it reads the tile's share
// of a read buffer with 16-byte loads and writes the tile's share of an output buffer with 8-byte stores,
// tiles dealt to the XCDs in runs like the reducer's.  The quotient (bytes of a launch) / (this kernel's
// time for the same bytes) says how much of a kernel's distance to the HBM peak is the machine's.
// Not part of the launch path: nothing but bench.py loads this library.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

constexpr int BLOCK = 256;
constexpr int NUM_XCD = 8;

__device__ __forceinline__ int tile_of_block(int block, int xcd_shift) {
  if (xcd_shift == 0) return block;
  const int xcd = block & (NUM_XCD - 1), seq = block / NUM_XCD;
  return ((((seq >> xcd_shift) * NUM_XCD) + xcd) << xcd_shift) + (seq & ((1 << xcd_shift) - 1));
}

// read_vec: 16-byte loads per thread and tile; write_words: 8-byte words per tile (at most BLOCK)
template <bool NONTEMPORAL>
__global__ void __launch_bounds__(BLOCK)
stream_mix_kernel(const uint4* __restrict__ in, double* __restrict__ out, int tiles, int read_vec, int write_words,
                  int xcd_shift) {
  const int tile = tile_of_block(blockIdx.x, xcd_shift);
  if (tile >= tiles) return;
  const uint4* src = in + (size_t)tile * read_vec * BLOCK + threadIdx.x;
  unsigned acc = 0;
  int k = 0;
  for (; k + 4 <= read_vec; k += 4) {  // four loads in flight per thread
    const uint4 a = src[(size_t)k * BLOCK], b = src[(size_t)(k + 1) * BLOCK], c = src[(size_t)(k + 2) * BLOCK],
                d = src[(size_t)(k + 3) * BLOCK];
    acc += (a.x ^ a.y ^ a.z ^ a.w) + (b.x ^ b.y ^ b.z ^ b.w) + (c.x ^ c.y ^ c.z ^ c.w) + (d.x ^ d.y ^ d.z ^ d.w);
  }
  for (; k < read_vec; ++k) {
    const uint4 a = src[(size_t)k * BLOCK];
    acc += a.x ^ a.y ^ a.z ^ a.w;
  }
  // every thread's loads feed something that may be stored: the compiler cannot drop them
  if ((int)threadIdx.x < write_words) {
    double* p = out + (size_t)tile * write_words + threadIdx.x;
    if (NONTEMPORAL) __builtin_nontemporal_store((double)acc, p);
    else *p = (double)acc;
  } else if (acc == 0x9e3779b9u) {
    out[(size_t)tile * write_words] = 1.0;
  }
}

}  // namespace

extern "C" {

// Launch the calibration kernel on `stream`.  `in` holds tiles * read_bytes_per_tile bytes (a multiple of
// 4096 per tile), `out` tiles * write_bytes_per_tile bytes (a multiple of 8, at most 2048 per tile).
// Returns 0, or -1 for sizes outside those limits, or a hipError_t.
int flexspmv_calibrate_stream_mix(const void* in, void* out, int32_t tiles, int32_t read_bytes_per_tile,
                                  int32_t write_bytes_per_tile, int32_t xcd_shift, int32_t nontemporal, void* stream) {
  if (tiles <= 0 || read_bytes_per_tile <= 0 || read_bytes_per_tile % (16 * BLOCK) != 0 || write_bytes_per_tile < 0 ||
      write_bytes_per_tile % 8 != 0 || write_bytes_per_tile > 8 * BLOCK || xcd_shift < 0 || xcd_shift > 12)
    return -1;
  const int window = NUM_XCD << xcd_shift;
  const int grid = xcd_shift == 0 ? tiles : (tiles + window - 1) / window * window;
  const int read_vec = read_bytes_per_tile / (16 * BLOCK), write_words = write_bytes_per_tile / 8;
  if (nontemporal)
    hipLaunchKernelGGL(stream_mix_kernel<true>, dim3(grid), dim3(BLOCK), 0, (hipStream_t)stream, (const uint4*)in,
                       (double*)out, tiles, read_vec, write_words, xcd_shift);
  else
    hipLaunchKernelGGL(stream_mix_kernel<false>, dim3(grid), dim3(BLOCK), 0, (hipStream_t)stream, (const uint4*)in,
                       (double*)out, tiles, read_vec, write_words, xcd_shift);
  return (int)hipGetLastError();
}

}  // extern "C"
