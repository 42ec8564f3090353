// Edge-list preparation in front of a FlexSpmv launch: COO row ids -> CSR row pointer, stable sort of
// an edge list by row, and the permutation of per-edge tensors.  Interface: flexspmv_formats.h.
//
// Stands in for _coo_rows_to_csr_ptr of the reference (python_wrapper/dynamic_replace_submodule.py:20-41),
// which calls torch's COO -> CSR conversion or bincount + cumsum; the sort has no counterpart there (the
// reference assumes ascending row ids).
//
// All of this is HBM-bound integer work:
//   rows_to_ptr_kernel   reads every row id once (4 or 8 B / edge, eight ids per thread in 16-byte loads) and
//                        writes every pointer entry once (4 B / row): boundary i between edges i-1 and i
//                        gives row_ptr[r] = i for the rows r in (row[i-1], row[i]].  Almost all boundaries
//                        close zero or one row; longer runs of empty rows are filled by the whole wavefront,
//                        and a run longer than LONG_GAP rows switches the call to rows_search_kernel.
//   rows_search_kernel   the fallback for edge lists with huge runs of empty rows: one binary search per
//                        row.  It is always launched and returns at once unless the first kernel asked for it,
//                        so the host never has to look at device memory.
//   sort_*_kernel        stable radix sort of (row id, position) pairs over the bits num_rows needs: per
//                        8-bit digit a histogram per block, a scan, and a scatter that ranks with wave64
//                        ballots and orders a tile in LDS so that every digit's run leaves as one piece.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <type_traits>

#include "flexspmv_formats.h"

namespace {

constexpr int WAVE = 64;
constexpr int BLOCK = 256;
constexpr int LONG_GAP = 4096;  // empty-row runs longer than this go to the per-row search

thread_local char g_error[512] = "";
int fail(int code, const char* msg) {
  snprintf(g_error, sizeof(g_error), "%s", msg);
  return code;
}
int fail_hip(hipError_t e, const char* where) {
  snprintf(g_error, sizeof(g_error), "%s: %s", where, hipGetErrorString(e));
  return (int)e;
}

// findings[0]: FLEXSPMV_FINDING_* bits; findings[1]: non-zero when rows_search_kernel has to run
__global__ void clear_findings_kernel(int32_t* findings) {
  if (threadIdx.x < 4) findings[threadIdx.x] = 0;
}

// ids a thread looks at: two or four 16-byte loads
constexpr int PER_THREAD = 8;
constexpr int NOT_AN_ID = -2;  // a row id outside [0, num_rows): no boundary next to it is written

template <typename I>
__device__ inline int checked_id(const I v, const int num_rows, int& found) {
  if (v < 0 || (long long)v >= (long long)num_rows) {
    found |= FLEXSPMV_FINDING_OUT_OF_RANGE;
    return NOT_AN_ID;
  }
  return (int)v;
}

// Thread t owns the boundaries i = 8t .. 8t+7 (boundary i lies between edges i-1 and i; the list is
// extended by id[-1] = -1 and id[ne] = num_rows, so boundaries 0 and ne close the leading and trailing
// empty rows).  Every lane runs the same number of ballots: nothing returns early.
template <typename I, bool ALIGNED>
__global__ void __launch_bounds__(BLOCK)
rows_to_ptr_kernel(const I* __restrict__ rows, const int ne, const int num_rows, int32_t* __restrict__ row_ptr,
                   int32_t* __restrict__ findings) {
  constexpr int K = PER_THREAD;
  const long long base = ((long long)blockIdx.x * BLOCK + threadIdx.x) * K;
  const int lane = threadIdx.x & (WAVE - 1);
  int found = 0;
  int cur[K];
  if (ALIGNED && base + K <= ne) {
    constexpr int PER_LOAD = 16 / (int)sizeof(I);
    struct alignas(16) Chunk { I v[PER_LOAD]; };
    const Chunk* src = reinterpret_cast<const Chunk*>(rows + base);
#pragma unroll
    for (int c = 0; c < K / PER_LOAD; ++c) {
      const Chunk chunk = src[c];
#pragma unroll
      for (int q = 0; q < PER_LOAD; ++q) cur[c * PER_LOAD + q] = checked_id<I>(chunk.v[q], num_rows, found);
    }
  } else {
#pragma unroll
    for (int j = 0; j < K; ++j)
      cur[j] = (base + j < ne) ? checked_id<I>(rows[base + j], num_rows, found) : num_rows;
  }
  // the id before this thread's first one: the neighbouring lane's last, or a load for lane 0
  int prev = __shfl_up(cur[K - 1], 1);
  if (lane == 0) {
    if (base == 0) prev = -1;
    else if (base - 1 < ne) prev = checked_id<I>(rows[base - 1], num_rows, found);
    else prev = NOT_AN_ID;
  }

#pragma unroll
  for (int j = 0; j < K; ++j) {
    const long long i = base + j;
    const int hi = cur[j];
    int gap = 0;  // rows prev+1 .. hi receive i (hi == num_rows at i == ne: row_ptr[num_rows] = ne)
    if (i <= ne && prev != NOT_AN_ID && hi != NOT_AN_ID) {
      if (prev > hi) found |= FLEXSPMV_FINDING_UNSORTED; else gap = hi - prev;
    }
    if (gap >= 1 && gap <= 2) {
      row_ptr[prev + 1] = (int32_t)i;
      if (gap == 2) row_ptr[prev + 2] = (int32_t)i;
    }
    unsigned long long wide = __builtin_amdgcn_ballot_w64(gap > 2);
    while (wide != 0ull) {
      const int src = __builtin_ctzll(wide);
      wide &= wide - 1ull;
      const int s_lo = __builtin_amdgcn_readlane(prev, src);
      const int s_hi = __builtin_amdgcn_readlane(hi, src);
      const int s_i = __builtin_amdgcn_readlane((int)i, src);
      if (s_hi - s_lo > LONG_GAP) {
        if (lane == 0) atomicOr(&findings[1], 1);
        continue;
      }
      for (int r = s_lo + 1 + lane; r <= s_hi; r += WAVE) row_ptr[r] = s_i;
    }
    prev = hi;
  }
  if (found != 0) atomicOr(&findings[0], found);
}

constexpr int SEARCH_BLOCKS = 2048;

template <typename I>
__global__ void __launch_bounds__(BLOCK)
rows_search_kernel(const I* __restrict__ rows, const int ne, const int num_rows, int32_t* __restrict__ row_ptr,
                   const int32_t* __restrict__ findings) {
  if (findings[1] == 0 || findings[0] != 0) return;
  for (long long r = (long long)blockIdx.x * BLOCK + threadIdx.x; r <= num_rows; r += (long long)gridDim.x * BLOCK) {
    int lo = 0, hi = ne;  // first position whose row id is >= r
    while (lo < hi) {
      const int mid = lo + ((hi - lo) >> 1);
      if ((long long)rows[mid] < r) lo = mid + 1; else hi = mid;
    }
    row_ptr[r] = lo;
  }
}

// ---------------------------------------------------------------------------------------------------
// Stable sort of (row id, position) pairs: least-significant-digit radix sort, 8-bit digits over the
// bits num_rows needs.  Three kernels per digit, no atomics on memory and nothing to clear beforehand:
//   sort_histogram_kernel   block b counts the digits of its chunk of tiles -> hist[digit][b]
//   sort_scan_kernel        block d turns row d of hist into exclusive prefixes and leaves the row's sum
//   sort_scatter_kernel     block b ranks its tiles' items (wave64 ballots give every item the lanes that
//                           hold the same digit; wavefront counters in LDS carry the order across the 16
//                           items of a lane and across the block's wavefronts), orders a tile by digit in LDS
//                           and writes each digit's run to its place: neighbouring lanes write
//                           neighbouring words.
// Position order inside a tile is wavefront-major: item k of lane l of wavefront w is element
// w * 1024 + k * 64 + l, so every load is a whole 256-byte piece per wavefront.
// Bytes per edge and digit: 4 read by the histogram, 8 read + 8 written by the scatter (the first digit
// reads the caller's ids instead, 4 or 8 bytes, and no positions: they are the element numbers).

// key of a row id: ids that do not fit a non-negative int32 become 0xffffffff, which reads back as -1 in
// sorted_rows and is reported as out of range by the pointer kernel
template <typename I>
struct RowKey {
  __host__ __device__ unsigned operator()(const I v) const {
    return (v < 0 || (long long)v > 0x7fffffffll) ? 0xffffffffu : (unsigned)v;
  }
};

constexpr int RADIX_BITS = 8;
constexpr int RADIX = 1 << RADIX_BITS;
constexpr int SORT_ITEMS = 16;                          // per thread and tile
constexpr int SORT_WAVES = BLOCK / WAVE;
constexpr int COUNT_TILE = BLOCK * SORT_ITEMS;          // the histogram's blocks: 256 threads, 4096 ids at a time
// The scatter's blocks: 1024 threads and tiles of 16384 pairs for long lists (a digit's run of a tile is then
// 64 pairs on average, two whole lines: 117 M pairs take 2.25 ms against 2.9 with tiles of 4096), 256 threads
// and tiles of 4096 pairs where such tiles would leave the CUs a handful each (6 M pairs: 0.13 against 0.17 ms).
constexpr int BIG_SCATTER_BLOCK = 1024;
constexpr long long BIG_SCATTER_FROM = 16ll << 20;   // pairs
constexpr int SORT_MAX_BLOCKS = 4096;                   // a block takes several tiles beyond that many
constexpr int SORT_SCAN_ITEMS = SORT_MAX_BLOCKS / BLOCK;
constexpr int SORT_MAX_PASSES = 4;
static_assert(RADIX == BLOCK && BIG_SCATTER_BLOCK % BLOCK == 0, "thread d < 256 of a block owns digit d");

// Ids outside [0, num_rows) sort as the last row, num_rows - 1 (a digit more for them would cost a whole
// pass where num_rows is a power of two): they end up among that row's edges, in their original order,
// and keep their value in sorted_rows, where the pointer kernel finds them.
__device__ inline unsigned sort_digit(const unsigned key, const unsigned last_row, const int shift, const unsigned mask) {
  return ((key < last_row ? key : last_row) >> shift) & mask;
}

template <typename I, bool FIRST>
__device__ inline unsigned load_sort_key(const void* src, const long long i) {
  if (FIRST) return RowKey<I>()(reinterpret_cast<const I*>(src)[i]);
  return reinterpret_cast<const unsigned*>(src)[i];
}

__device__ inline unsigned wave_inclusive_sum(unsigned v, const int lane) {
#pragma unroll
  for (int off = 1; off < WAVE; off <<= 1) {
    const unsigned other = __shfl_up(v, off);
    if (lane >= off) v += other;
  }
  return v;
}

// Exclusive prefix of v over the block's WAVES wavefronts and the block's sum.  Two barriers; s_tmp holds
// WAVES words and is free again on return.
template <int WAVES>
__device__ inline unsigned block_exclusive_sum(const unsigned v, unsigned* s_tmp, unsigned& total) {
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const unsigned inclusive = wave_inclusive_sum(v, lane);
  if (lane == WAVE - 1) s_tmp[wave] = inclusive;
  __syncthreads();
  unsigned before = 0;
  total = 0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    const unsigned s = s_tmp[w];
    if (w < wave) before += s;
    total += s;
  }
  __syncthreads();
  return before + inclusive - v;
}

template <typename I, bool FIRST>
__global__ void __launch_bounds__(BLOCK)
sort_histogram_kernel(const void* __restrict__ keys_in, const long long ne, const unsigned last_row, const int shift,
                      const unsigned mask, const int tiles_per_block, const int blocks, unsigned* __restrict__ hist) {
  __shared__ unsigned s_cnt[SORT_WAVES][RADIX];
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
#pragma unroll
  for (int j = 0; j < RADIX / WAVE; ++j) s_cnt[wave][lane + j * WAVE] = 0;   // the wavefront's own counters
  const long long first_tile = (long long)blockIdx.x * tiles_per_block;
  for (int tl = 0; tl < tiles_per_block; ++tl) {
    const long long base = (first_tile + tl) * COUNT_TILE + wave * (WAVE * SORT_ITEMS);
    if (base >= ne) break;
    unsigned key[SORT_ITEMS];
#pragma unroll
    for (int k = 0; k < SORT_ITEMS; ++k) {
      const long long i = base + k * WAVE + lane;
      key[k] = load_sort_key<I, FIRST>(keys_in, i < ne ? i : ne - 1);
    }
#pragma unroll
    for (int k = 0; k < SORT_ITEMS; ++k) {
      const bool valid = base + k * WAVE + lane < ne;
      const unsigned d = sort_digit(key[k], last_row, shift, mask);
      // a wavefront whose items all hold one digit (sorted input, a hot row, the high digit of small
      // ids) adds once instead of 64 times to one counter
      const unsigned d0 = __builtin_amdgcn_readfirstlane(d);
      const unsigned long long active = __builtin_amdgcn_ballot_w64(valid);
      const unsigned long long same = __builtin_amdgcn_ballot_w64(valid && d == d0);
      if (same == active) {
        if (lane == 0 && active != 0ull) atomicAdd(&s_cnt[wave][d0], (unsigned)__builtin_popcountll(active));
      } else if (valid) {
        atomicAdd(&s_cnt[wave][d], 1u);
      }
    }
  }
  __syncthreads();
  unsigned sum = 0;
#pragma unroll
  for (int w = 0; w < SORT_WAVES; ++w) sum += s_cnt[w][threadIdx.x];
  hist[(size_t)threadIdx.x * blocks + blockIdx.x] = sum;
}

__global__ void __launch_bounds__(BLOCK)
sort_scan_kernel(unsigned* __restrict__ hist, const int blocks, unsigned* __restrict__ totals) {
  __shared__ unsigned s_tmp[SORT_WAVES];
  unsigned* row = hist + (size_t)blockIdx.x * blocks;
  const int per = (blocks + BLOCK - 1) / BLOCK;   // <= SORT_SCAN_ITEMS
  const int lo = threadIdx.x * per;
  unsigned v[SORT_SCAN_ITEMS];
  unsigned sum = 0;
#pragma unroll
  for (int j = 0; j < SORT_SCAN_ITEMS; ++j) {
    v[j] = (j < per && lo + j < blocks) ? row[lo + j] : 0u;
    sum += v[j];
  }
  unsigned total;
  unsigned run = block_exclusive_sum<SORT_WAVES>(sum, s_tmp, total);
#pragma unroll
  for (int j = 0; j < SORT_SCAN_ITEMS; ++j) {
    if (j < per && lo + j < blocks) row[lo + j] = run;
    run += v[j];
  }
  if (threadIdx.x == 0) totals[blockIdx.x] = total;
}

// LDS of a scatter block of THREADS threads
template <int THREADS>
struct ScatterShared {
  static constexpr int TILE = THREADS * SORT_ITEMS, WAVES = THREADS / WAVE;
  unsigned keys[TILE];
  int32_t vals[TILE];
  unsigned cnt[WAVES][RADIX];
  unsigned place[RADIX];   // where digit d's run of this tile goes, minus the run's start inside the tile
  unsigned tmp[WAVES];
};

// One tile of `count` pairs starting at element tile_at.  FULL: count == THREADS * 16, no lane is idle.
// next_of_digit (thread t < 256: digit t) is where the block's next item of that digit goes; advanced here.
template <typename I, bool FIRST, bool FULL, int THREADS>
__device__ inline void scatter_tile(ScatterShared<THREADS>& sh, const void* __restrict__ keys_in,
                                    const int32_t* __restrict__ vals_in, unsigned* __restrict__ keys_out,
                                    int32_t* __restrict__ vals_out, const long long tile_at, const int count,
                                    const unsigned last_row, const int shift, const unsigned mask,
                                    unsigned& next_of_digit) {
  const int t = threadIdx.x, lane = t & (WAVE - 1), wave = t / WAVE;
  const int first_pos = wave * (WAVE * SORT_ITEMS) + lane;   // item k of this lane is element first_pos + 64 k
  unsigned key[SORT_ITEMS];
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; ++k) {
    const int pos = first_pos + k * WAVE;
    key[k] = load_sort_key<I, FIRST>(keys_in, tile_at + ((FULL || pos < count) ? pos : 0));
  }
#pragma unroll
  for (int j = 0; j < RADIX / WAVE; ++j) sh.cnt[wave][lane + j * WAVE] = 0;
  // Per item, among the wavefront's 64 items of step k: its digit (bits 0-7), how many of them hold the same
  // digit (8-14), how many of those sit in lower lanes (16-21) and the lowest lane that holds it (24-29).
  // Arithmetic only: per bit of the digit, keep the lanes whose bit equals this lane's.
  unsigned info[SORT_ITEMS];
  const unsigned below_lo = lane < 32 ? (1u << lane) - 1u : 0xffffffffu;
  const unsigned below_hi = lane < 32 ? 0u : (1u << (lane - 32)) - 1u;
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; ++k) {
    const bool valid = FULL || first_pos + k * WAVE < count;
    const unsigned d = sort_digit(key[k], last_row, shift, mask);
    const unsigned long long active = FULL ? ~0ull : __builtin_amdgcn_ballot_w64(valid);
    unsigned peers_lo = (unsigned)active, peers_hi = (unsigned)(active >> 32);
#pragma unroll
    for (int b = 0; b < RADIX_BITS; ++b) {
      const int all_if_set = (int)(d << (31 - b)) >> 31;   // -1 where bit b of the digit is set, else 0
      const unsigned long long with_bit = __builtin_amdgcn_ballot_w64(all_if_set != 0);
      peers_lo &= ~((unsigned)with_bit ^ (unsigned)all_if_set);
      peers_hi &= ~((unsigned)(with_bit >> 32) ^ (unsigned)all_if_set);
    }
    const unsigned same = (unsigned)(__builtin_popcount(peers_lo) + __builtin_popcount(peers_hi));
    const unsigned below = (unsigned)(__builtin_popcount(peers_lo & below_lo) + __builtin_popcount(peers_hi & below_hi));
    const unsigned lowest = peers_lo != 0u ? (unsigned)__builtin_ctz(peers_lo) : 32u + (unsigned)__builtin_ctz(peers_hi);
    info[k] = valid ? (d | (same << 8) | (below << 16) | (lowest << 24)) : (d | ((unsigned)lane << 24));
    // finished here, one item at a time: left alone the compiler moves this arithmetic down to where info
    // is used and keeps the 128 lane masks of the ballots until then
    asm volatile("" : "+v"(info[k]));
  }
  // the positions travel with the keys; loaded here, they arrive while the counters are walked
  int32_t val[SORT_ITEMS];
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; ++k) {
    const int pos = first_pos + k * WAVE;
    const long long i = tile_at + ((FULL || pos < count) ? pos : 0);
    val[k] = FIRST ? (int32_t)i : vals_in[i];
  }
  // The lowest lane of every group moves the group's counter, step after step; every lane of the group
  // reads the value from before: its rank among the wavefront's items of that digit, in position order.
  unsigned digit_rank[SORT_ITEMS];
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; ++k) {
    const unsigned d = info[k] & 0xffu, same = (info[k] >> 8) & 0xffu, below = (info[k] >> 16) & 0xffu;
    const int lowest = (int)(info[k] >> 24);
    unsigned old = 0;
    if (lane == lowest && same != 0u) {
      old = sh.cnt[wave][d];
      sh.cnt[wave][d] = old + same;
    }
    old = __shfl(old, lowest);
    digit_rank[k] = d | ((old + below) << RADIX_BITS);
  }
  __syncthreads();
  {
    // thread t < 256: digit t's items per wavefront -> start of every wavefront's share inside the tile
    unsigned sum = 0;
    if (t < RADIX) {
#pragma unroll
      for (int w = 0; w < THREADS / WAVE; ++w) sum += sh.cnt[w][t];
    }
    unsigned unused;
    unsigned start = block_exclusive_sum<THREADS / WAVE>(sum, sh.tmp, unused);
    if (t < RADIX) {
      sh.place[t] = next_of_digit - start;   // modulo 2^32: the item at tile position i goes to place[d] + i
      next_of_digit += sum;
#pragma unroll
      for (int w = 0; w < THREADS / WAVE; ++w) {
        const unsigned c = sh.cnt[w][t];
        sh.cnt[w][t] = start;
        start += c;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; ++k) {
    if (FULL || first_pos + k * WAVE < count) {
      const unsigned at = sh.cnt[wave][digit_rank[k] & (RADIX - 1)] + (digit_rank[k] >> RADIX_BITS);
      sh.keys[at] = key[k];
      sh.vals[at] = val[k];
    }
  }
  __syncthreads();
#pragma unroll
  for (int m = 0; m < SORT_ITEMS; ++m) {
    const int i = t + m * THREADS;
    if (FULL || i < count) {
      const unsigned key_i = sh.keys[i];
      const unsigned to = sh.place[sort_digit(key_i, last_row, shift, mask)] + (unsigned)i;
      keys_out[to] = key_i;
      vals_out[to] = sh.vals[i];
    }
  }
  __syncthreads();
}

template <typename I, bool FIRST, int THREADS>
__global__ void __launch_bounds__(THREADS)
sort_scatter_kernel(const void* __restrict__ keys_in, const int32_t* __restrict__ vals_in,
                    unsigned* __restrict__ keys_out, int32_t* __restrict__ vals_out, const long long ne,
                    const unsigned last_row, const int shift, const unsigned mask, const int tiles_per_block,
                    const int blocks, const unsigned* __restrict__ hist, const unsigned* __restrict__ totals) {
  constexpr int TILE = THREADS * SORT_ITEMS;
  __shared__ ScatterShared<THREADS> sh;
  const int t = threadIdx.x;
  // thread t follows digit t: the digit's place in the output, then this block's place among the blocks
  unsigned unused;
  unsigned next_of_digit = block_exclusive_sum<THREADS / WAVE>(t < RADIX ? totals[t] : 0u, sh.tmp, unused);
  if (t < RADIX) next_of_digit += hist[(size_t)t * blocks + blockIdx.x];
  const long long first_tile = (long long)blockIdx.x * tiles_per_block;
  for (int tl = 0; tl < tiles_per_block; ++tl) {
    const long long tile_at = (first_tile + tl) * TILE;
    if (tile_at >= ne) break;   // the whole block leaves together
    if (ne - tile_at >= TILE)
      scatter_tile<I, FIRST, true, THREADS>(sh, keys_in, vals_in, keys_out, vals_out, tile_at, TILE, last_row, shift,
                                            mask, next_of_digit);
    else
      scatter_tile<I, FIRST, false, THREADS>(sh, keys_in, vals_in, keys_out, vals_out, tile_at, (int)(ne - tile_at),
                                             last_row, shift, mask, next_of_digit);
  }
}

// What a sort of ne pairs with ids below num_rows runs: digits, chunks and the scratch layout.
struct SortPlan {
  int passes;
  int shift[SORT_MAX_PASSES], bits[SORT_MAX_PASSES];
  int scatter_threads;            // BIG_SCATTER_BLOCK or BLOCK
  int tiles_per_block, blocks;    // scatter tiles (scatter_threads * 16 pairs) per block; blocks of both kernels
  size_t off_keys, off_vals, off_hist, off_totals, bytes;
};

SortPlan plan_sort(int64_t ne, int64_t num_rows) {
  SortPlan p{};
  int key_bits = 1;   // enough for num_rows - 1
  while (key_bits < 31 && ((int64_t)1 << key_bits) < num_rows) ++key_bits;
  p.passes = (key_bits + RADIX_BITS - 1) / RADIX_BITS;
  int shift = 0;
  for (int i = 0; i < p.passes; ++i) {
    p.bits[i] = key_bits / p.passes + (i < key_bits % p.passes ? 1 : 0);
    p.shift[i] = shift;
    shift += p.bits[i];
  }
  p.scatter_threads = ne >= BIG_SCATTER_FROM ? BIG_SCATTER_BLOCK : BLOCK;
  const int64_t tile = (int64_t)p.scatter_threads * SORT_ITEMS;
  const int64_t tiles = (ne + tile - 1) / tile;
  p.tiles_per_block = (int)((tiles + SORT_MAX_BLOCKS - 1) / SORT_MAX_BLOCKS);
  if (p.tiles_per_block < 1) p.tiles_per_block = 1;
  p.blocks = (int)((tiles + p.tiles_per_block - 1) / p.tiles_per_block);
  auto aligned = [](size_t n) { return (n + 255) & ~(size_t)255; };
  size_t at = 0;
  p.off_keys = at;   at += p.passes > 1 ? aligned((size_t)ne * 4) : 0;   // the second pair of buffers
  p.off_vals = at;   at += p.passes > 1 ? aligned((size_t)ne * 4) : 0;
  p.off_hist = at;   at += aligned((size_t)RADIX * p.blocks * 4);
  p.off_totals = at; at += aligned((size_t)RADIX * 4);
  p.bytes = at;
  return p;
}

template <typename I>
hipError_t sort_pairs(const SortPlan& p, void* workspace, const I* rows, int32_t* sorted_rows, int32_t* permutation,
                      int64_t ne, int64_t num_rows, hipStream_t stream) {
  char* ws = static_cast<char*>(workspace);
  unsigned* alt_keys = reinterpret_cast<unsigned*>(ws + p.off_keys);
  int32_t* alt_vals = reinterpret_cast<int32_t*>(ws + p.off_vals);
  unsigned* hist = reinterpret_cast<unsigned*>(ws + p.off_hist);
  unsigned* totals = reinterpret_cast<unsigned*>(ws + p.off_totals);
  const void* keys_in = rows;
  const int32_t* vals_in = nullptr;
  for (int i = 0; i < p.passes; ++i) {
    // the last digit writes the caller's arrays, the ones before it alternate so that it can
    const bool to_caller = ((p.passes - 1 - i) & 1) == 0;
    unsigned* keys_out = to_caller ? reinterpret_cast<unsigned*>(sorted_rows) : alt_keys;
    int32_t* vals_out = to_caller ? permutation : alt_vals;
    const unsigned mask = (1u << p.bits[i]) - 1u;
    const dim3 grid((unsigned)p.blocks), block(BLOCK);
    const unsigned last_row = (unsigned)(num_rows - 1);
    // a block of the histogram counts the pairs the scatter's block of the same number moves
    const int count_tiles = p.tiles_per_block * (p.scatter_threads * SORT_ITEMS / COUNT_TILE);
    if (i == 0) {
      hipLaunchKernelGGL((sort_histogram_kernel<I, true>), grid, block, 0, stream, keys_in, (long long)ne, last_row,
                         p.shift[i], mask, count_tiles, p.blocks, hist);
    } else {
      hipLaunchKernelGGL((sort_histogram_kernel<int32_t, false>), grid, block, 0, stream, keys_in, (long long)ne,
                         last_row, p.shift[i], mask, count_tiles, p.blocks, hist);
    }
    hipLaunchKernelGGL(sort_scan_kernel, dim3(RADIX), block, 0, stream, hist, p.blocks, totals);
    auto scatter = [&](auto first, auto threads) {
      constexpr bool FIRST = decltype(first)::value;
      constexpr int THREADS = decltype(threads)::value;
      using Id = typename std::conditional<FIRST, I, int32_t>::type;
      hipLaunchKernelGGL((sort_scatter_kernel<Id, FIRST, THREADS>), grid, dim3(THREADS), 0, stream, keys_in, vals_in,
                         keys_out, vals_out, (long long)ne, last_row, p.shift[i], mask, p.tiles_per_block, p.blocks,
                         (const unsigned*)hist, (const unsigned*)totals);
    };
    using Big = std::integral_constant<int, BIG_SCATTER_BLOCK>;
    using Small = std::integral_constant<int, BLOCK>;
    if (p.scatter_threads == BIG_SCATTER_BLOCK) {
      if (i == 0) scatter(std::true_type{}, Big{}); else scatter(std::false_type{}, Big{});
    } else {
      if (i == 0) scatter(std::true_type{}, Small{}); else scatter(std::false_type{}, Small{});
    }
    keys_in = keys_out;
    vals_in = vals_out;
  }
  return hipGetLastError();
}

// dst[k] = src[perm[k]] (gather) or dst[perm[k]] = src[k] (scatter) for rows of `vecs` vectors of type T.
// One thread moves one vector; T is the widest of 16, 8 and 4 bytes that divides the row and both base
// addresses, so an 8-byte value per edge is one load and one store (the side that follows the permutation
// touches a cache line per row whatever the width: that line, not the instruction count, is the cost).
template <bool SCATTER, typename T>
__global__ void __launch_bounds__(BLOCK)
permute_rows_kernel(const T* __restrict__ src, T* __restrict__ dst, const int32_t* __restrict__ perm,
                    const long long n, const int vecs) {
  const long long idx = (long long)blockIdx.x * BLOCK + threadIdx.x;
  if (idx >= n * vecs) return;
  const long long k = idx / vecs;
  const int w = (int)(idx - k * vecs);
  const long long other = perm[k];
  if (SCATTER) dst[other * vecs + w] = src[idx]; else dst[idx] = src[other * vecs + w];
}

template <bool SCATTER>
int permute_rows(const void* src, void* dst, const int32_t* perm, int64_t n, int64_t row_bytes, void* stream) {
  if (n < 0 || row_bytes <= 0 || (row_bytes & 3) != 0)
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "n must be >= 0 and row_bytes a positive multiple of 4");
  if (n == 0) return FLEXSPMV_FORMATS_OK;
  if (src == nullptr || dst == nullptr || perm == nullptr)
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "a pointer is NULL");
  const uintptr_t bits = (uintptr_t)src | (uintptr_t)dst | (uintptr_t)row_bytes;
  const int vec_bytes = (bits & 15u) == 0 ? 16 : ((bits & 7u) == 0 ? 8 : 4);
  const int64_t vecs = row_bytes / vec_bytes;
  const int64_t total = n * vecs;
  if (n >= ((int64_t)1 << 31) || vecs >= ((int64_t)1 << 20) || (total + BLOCK - 1) / BLOCK >= ((int64_t)1 << 31))
    return fail(FLEXSPMV_FORMATS_ERR_TOO_LARGE, "tensor too large for one launch");
  const dim3 grid((unsigned)((total + BLOCK - 1) / BLOCK));
  if (vec_bytes == 16)
    hipLaunchKernelGGL((permute_rows_kernel<SCATTER, uint4>), grid, dim3(BLOCK), 0, (hipStream_t)stream,
                       (const uint4*)src, (uint4*)dst, perm, (long long)n, (int)vecs);
  else if (vec_bytes == 8)
    hipLaunchKernelGGL((permute_rows_kernel<SCATTER, uint2>), grid, dim3(BLOCK), 0, (hipStream_t)stream,
                       (const uint2*)src, (uint2*)dst, perm, (long long)n, (int)vecs);
  else
    hipLaunchKernelGGL((permute_rows_kernel<SCATTER, uint32_t>), grid, dim3(BLOCK), 0, (hipStream_t)stream,
                       (const uint32_t*)src, (uint32_t*)dst, perm, (long long)n, (int)vecs);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "kernel launch failed");
  return FLEXSPMV_FORMATS_OK;
}

}  // namespace

extern "C" {

int flexspmv_coo_rows_to_csr(const void* row_ids, int index_bytes, int64_t ne, int64_t num_rows, int32_t* row_ptr,
                             int32_t* findings, void* stream) {
  if (index_bytes != 4 && index_bytes != 8)
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "index_bytes must be 4 or 8");
  if (ne < 0 || num_rows < 0) return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "ne and num_rows must be >= 0");
  if (row_ptr == nullptr || findings == nullptr || (ne > 0 && row_ids == nullptr))
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "a pointer is NULL");
  if (ne >= ((int64_t)1 << 31) - BLOCK || num_rows >= ((int64_t)1 << 31) - BLOCK)
    return fail(FLEXSPMV_FORMATS_ERR_TOO_LARGE, "ne and num_rows must stay below 2^31 (32-bit offsets)");
  hipStream_t s = (hipStream_t)stream;
  const long long threads = (ne + 1 + PER_THREAD - 1) / PER_THREAD;
  const unsigned edge_blocks = (unsigned)((threads + BLOCK - 1) / BLOCK);
  const long long all_row_blocks = (num_rows + 1 + BLOCK - 1) / BLOCK;
  const unsigned row_blocks = (unsigned)(all_row_blocks < SEARCH_BLOCKS ? all_row_blocks : SEARCH_BLOCKS);
  const bool aligned = ((uintptr_t)row_ids & 15u) == 0;
  hipLaunchKernelGGL(clear_findings_kernel, dim3(1), dim3(WAVE), 0, s, findings);
  auto run = [&](auto tag) {
    using I = decltype(tag);
    const I* ids = (const I*)row_ids;
    if (aligned)
      hipLaunchKernelGGL((rows_to_ptr_kernel<I, true>), dim3(edge_blocks), dim3(BLOCK), 0, s, ids, (int)ne,
                         (int)num_rows, row_ptr, findings);
    else
      hipLaunchKernelGGL((rows_to_ptr_kernel<I, false>), dim3(edge_blocks), dim3(BLOCK), 0, s, ids, (int)ne,
                         (int)num_rows, row_ptr, findings);
    hipLaunchKernelGGL(rows_search_kernel<I>, dim3(row_blocks), dim3(BLOCK), 0, s, ids, (int)ne, (int)num_rows,
                       row_ptr, (const int32_t*)findings);
  };
  if (index_bytes == 4) run(int32_t{}); else run(int64_t{});
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "kernel launch failed");
  return FLEXSPMV_FORMATS_OK;
}

size_t flexspmv_sort_workspace_bytes(int64_t ne, int64_t num_rows) {
  if (ne <= 0 || ne >= ((int64_t)1 << 31) || num_rows <= 0 || num_rows >= ((int64_t)1 << 31)) return 0;
  return plan_sort(ne, num_rows).bytes;
}

int flexspmv_sort_edges_by_row(const void* row_ids, int index_bytes, int64_t ne, int64_t num_rows,
                               int32_t* sorted_rows, int32_t* permutation, void* workspace, size_t workspace_bytes,
                               void* stream) {
  if (index_bytes != 4 && index_bytes != 8)
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "index_bytes must be 4 or 8");
  if (ne < 0 || num_rows <= 0) return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "ne must be >= 0 and num_rows > 0");
  if (ne == 0) return FLEXSPMV_FORMATS_OK;
  if (row_ids == nullptr || sorted_rows == nullptr || permutation == nullptr)
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "a pointer is NULL");
  if (ne >= ((int64_t)1 << 31) || num_rows >= ((int64_t)1 << 31))
    return fail(FLEXSPMV_FORMATS_ERR_TOO_LARGE, "ne and num_rows must stay below 2^31 (32-bit offsets)");
  const SortPlan plan = plan_sort(ne, num_rows);
  if (workspace == nullptr || workspace_bytes < plan.bytes)
    return fail(FLEXSPMV_FORMATS_ERR_WORKSPACE, "workspace is missing or smaller than flexspmv_sort_workspace_bytes()");
  if (((uintptr_t)workspace & 3u) != 0)
    return fail(FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT, "workspace must be aligned to 4 bytes");
  const hipError_t e =
      index_bytes == 4
          ? sort_pairs<int32_t>(plan, workspace, (const int32_t*)row_ids, sorted_rows, permutation, ne, num_rows,
                                (hipStream_t)stream)
          : sort_pairs<int64_t>(plan, workspace, (const int64_t*)row_ids, sorted_rows, permutation, ne, num_rows,
                                (hipStream_t)stream);
  if (e != hipSuccess) return fail_hip(e, "kernel launch failed");
  return FLEXSPMV_FORMATS_OK;
}

int flexspmv_gather_rows(const void* src, void* dst, const int32_t* permutation, int64_t n, int64_t row_bytes,
                         void* stream) {
  return permute_rows<false>(src, dst, permutation, n, row_bytes, stream);
}

int flexspmv_scatter_rows(const void* src, void* dst, const int32_t* permutation, int64_t n, int64_t row_bytes,
                          void* stream) {
  return permute_rows<true>(src, dst, permutation, n, row_bytes, stream);
}

const char* flexspmv_formats_last_error(void) { return g_error; }

int flexspmv_formats_abi_version(void) { return FLEXSPMV_FORMATS_ABI_VERSION; }

}  // extern "C"
