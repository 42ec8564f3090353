// Hand-written gfx950 kernels for one fused "select -> map -> reduce / aggregate" sub-graph.
//
// A generated translation unit defines a graph type G (see codegen/merged_gen_gpu.py) and instantiates
// the kernels below with it.  G supplies, for value type V:
//   G::Params                      pointer bundle (kernel argument)
//   FETCH_VALUES / FETCH_INDICES   V words and index words streamed per edge (handed through LDS)
//   RED / AGG / ROW widths         number of V values per-row reduced, globally summed, and read per row
//   fetch / gather                 first-level (streamed) and second-level (gathered) loads of edge e
//   put / get                      a Fetch to / from its LDS slot
//   edge(p, e, f, g, rv, tot, agg) the map for edge e; assigns its contributions tot / agg
//   load_row / store_row / add_row / store_agg   row-aligned sources and outputs
//
// What the kernels replace in the reference (CUDA + CUB):
//   tile_search_kernel   <- SpmvSearchKernel            include/merged_spmv_kernels.cuh:60-99
//   reduce_kernel        <- AgentFlexSpmv::ConsumeTile  cuda_template/reducer/merged_agent_spmv_template.cuh:350-445
//                           and ::reduce<>              :218-345 (segmented scan + atomics)
//   flat_kernel          <- the aggregator / map-only agent  cuda_template/aggregator/merged_agent_spmv_template.cuh:348-409
//   fixup_kernel         <- the per-row and per-tile atomicAdd sites (:315-325, :331-343;
//                           codegen/merged_gen_gpu.py:329-330), made deterministic
//
// Differences in design, all on purpose:
//   * every output row is written exactly once by the thread that consumes its row-end merge item, so
//     outputs need no zero fill and no atomics; tiles hand their open last row to a carry record that
//     fixup_kernel folds in tile order (same result on every run);
//   * aggregators are block partials + one ordered final sum instead of floating-point atomics;
//   * a reducer and an aggregator can share one pass over the edges;
//   * one small independent block per tile; block b takes tile b, so the 8 XCDs (one L2 each, workgroups
//     are dealt to them round-robin) work side by side on neighbouring tiles, in runs of 1 or 16 tiles
//     per XCD (tile_of_block).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "flex_tuning.hpp"
#include "flex_tensor.hpp"
#include "flex_wave.hpp"

namespace flex {

constexpr int NUM_XCD = 8;
constexpr int NUM_CUS = 256;  // MI355X: 8 XCDs of 32 CUs

// Aggregator partials a reducer block leaves per tile: one (its wavefronts' partials are added in the block,
// in wavefront order).  One per wavefront - no barrier at the end of the block, four times the words for
// the fix-up to read - measured 2 - 3 us slower per launch on Poisson 256^3 (step 319.2 us against 316.9).
#ifdef FLEX_TUNE_PARTIAL_PER_WAVE
template <int BLOCK> constexpr int partials_per_tile() { return BLOCK / 64; }
#else
template <int BLOCK> constexpr int partials_per_tile() { return 1; }
#endif


template <typename V, int N> struct Pack { V v[N > 0 ? N : 1]; };

template <typename V, int N> __device__ __forceinline__ void zero(Pack<V, N>& a) {
#pragma unroll
  for (int i = 0; i < N; ++i) a.v[i] = V(0);
}

// Loads of the read-once edge streams and stores of the write-once outputs.  The stores are
// non-temporal: neutral on the SpMV workloads (one output value per row), 7 % on the shallow-water kernel
// (three output arrays, 17 % of its bytes: 44.6 us against 47.9).  Non-temporal loads of the edge streams
// measured slower (Poisson 256^3: 374 us against 310) and stay a tuning switch.
#ifdef FLEX_TUNE_NT_LOADS
template <typename T> __device__ __forceinline__ T stream_load(const T* p) { return __builtin_nontemporal_load(p); }
#else
template <typename T> __device__ __forceinline__ T stream_load(const T* p) { return *p; }
#endif
#if defined(FLEX_TUNE_ABLATE_STORES)  // ablation (wrong results): what the row outputs cost
template <typename T> __device__ __forceinline__ void stream_store(T* p, T v) {
  if (v == T(123456789)) *p = v;
}
#elif defined(FLEX_TUNE_PLAIN_STORES)  // tuning switch
template <typename T> __device__ __forceinline__ void stream_store(T* p, T v) { *p = v; }
#else
template <typename T> __device__ __forceinline__ void stream_store(T* p, T v) { __builtin_nontemporal_store(v, p); }
#endif

// Merge-path coordinate on diagonal `diag` of the merge of A = row_end[0..num_rows) (end offset of each
// row) with B = 0..nnz-1.  Same search as the reference (include/merged_spmv_kernels.cuh:19-50):
// the result x is the number of rows whose end offset is <= the number of non-zeros taken so far.
__device__ __forceinline__ int2 merge_path_search(int diag, const int* __restrict__ row_end, int num_rows, int nnz) {
  int lo = max(diag - nnz, 0);
  int hi = min(diag, num_rows);
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (row_end[mid] <= diag - mid - 1) lo = mid + 1;
    else hi = mid;
  }
  return make_int2(min(lo, num_rows), diag - lo);
}

// The same coordinate with fewer dependent loads.  g(i) = row_end[i] + i + 1 is strictly increasing and
// the answer is the first i with g(i) > diag, so any probe sequence that keeps the bracket valid gives
// the identical result.  A few Newton-like probes (step = residual / average slope of g) land within
// a handful of rows when row lengths are regular; the bisection that follows bounds the cost when
// they are not.  The search is pure latency (about 25 dependent loads for 16 M rows), so fewer probes
// is what counts.
__device__ __forceinline__ int2 merge_path_search_interp(int diag, const int* __restrict__ row_end, int num_rows,
                                                         int nnz) {
  int lo = max(diag - nnz, 0);
  int hi = min(diag, num_rows);
  const float inv_slope = (float)num_rows / ((float)num_rows + (float)nnz);  // rows per merge item
  int p = (int)((float)diag * inv_slope);
#pragma unroll 1
  for (int it = 0; it < 4 && hi - lo > 4; ++it) {
    p = min(max(p, lo), hi - 1);
    const int gp = row_end[p] + p + 1;
    if (gp <= diag) lo = p + 1;
    else hi = p;
    p += (int)((float)(diag - gp) * inv_slope) + (gp <= diag ? 1 : 0);
  }
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (row_end[mid] <= diag - mid - 1) lo = mid + 1;
    else hi = mid;
  }
  return make_int2(min(lo, num_rows), diag - lo);
}

// How a launch cuts the merge path into tiles.  Tile boundary t lies on diagonal t * nominal; with
// snap_slack > 0 an interior boundary is moved back to the start of the nearest row whose index is a
// multiple of (snap_mask + 1) when that costs at most snap_slack merge items.  nominal + snap_slack is
// the tile capacity, so a tile never outgrows its block.  A tile that starts on such a row starts
// whole output lines (no row shared with the previous tile, no carry into it) - worth the smaller
// tiles where rows are short (meshes, stencils); the host turns it off where they are not.
struct Tiling {
  int num_tiles;
  int nominal;     // merge items between two diagonals
  int snap_slack;  // 0: boundaries stay on their diagonals
  int snap_mask;   // rows per output line - 1 (power of two - 1)
  int xcd_shift;   // runs of 2^xcd_shift consecutive tiles share an XCD (see tile_of_block)
  int row_group;   // row path: edges of a row staged at a time (<= the kernel's register budget; 0: that budget)
};

// split: the row the search stopped at, before the boundary was moved (boundary_from_split rebuilds the
// boundary from it).
__device__ __forceinline__ int2 tile_boundary(int t, const Tiling& tl, const int* __restrict__ row_end, int num_rows,
                                              int nnz, int& split) {
  const long long d = (long long)t * tl.nominal;
  const int diag = (int)min(d, (long long)num_rows + nnz);
#ifdef FLEX_TUNE_BISECTION_ONLY  // tuning switch: the reference's plain bisection
  int2 c = merge_path_search(diag, row_end, num_rows, nnz);
#else
  int2 c = merge_path_search_interp(diag, row_end, num_rows, nnz);
#endif
  split = c.x;
  if (tl.snap_slack > 0 && t > 0 && t < tl.num_tiles) {
    const int xs = c.x & ~tl.snap_mask;
    const int ys = xs > 0 ? row_end[xs - 1] : 0;  // first non-zero of row xs
    if ((c.x - xs) + (c.y - ys) <= tl.snap_slack) c = make_int2(xs, ys);
  }
  return c;
}

// The boundary a search on tile boundary t returns, rebuilt from a claimed split and three row ends: the one
// of the row before the split, the one of the row at it, and the one of the row before the row a snap would
// move the boundary to (values for rows outside the matrix are never looked at).  ok: the claim is what a
// search finds - g(i) = row_end[i] + i + 1 is strictly increasing and the split is the first i of its
// bracket with g(i) > diag, so its two neighbours decide.  A block that is handed the tile table of an
// earlier launch checks it this way against the row pointer of this launch: three loads that travel with
// the tile's own instead of a search in front of them.
__device__ __forceinline__ int2 boundary_from_split(int t, const Tiling& tl, int num_rows, int nnz, int split,
                                                    int end_before, int end_at, int end_before_snap_row, bool& ok) {
  const long long d = (long long)t * tl.nominal;
  const int diag = (int)min(d, (long long)num_rows + nnz);
  const int lo = max(diag - nnz, 0);
  const int hi = min(diag, num_rows);
  // every condition as the sign of a difference, so that a block's verdict is a handful of independent
  // scalar instructions and one OR instead of a chain of compares and branches
  const int in_bracket = (split - lo) | (hi - split);                                    // >= 0: lo <= split <= hi
  const int stops_here = split == hi ? 0 : (end_at + split - diag);                     // >= 0: g(split) > diag
  const int not_before = split == lo ? 0 : (diag - end_before - split);                 // >= 0: g(split - 1) <= diag
  ok = (in_bracket | stops_here | not_before) >= 0;
  int2 c = make_int2(split, diag - split);
  if (tl.snap_slack > 0 && t > 0 && t < tl.num_tiles) {
    const int xs = split & ~tl.snap_mask;
    const int ys = xs > 0 ? end_before_snap_row : 0;
    if ((c.x - xs) + (c.y - ys) <= tl.snap_slack) c = make_int2(xs, ys);
  }
  return c;
}

// The same boundary found by a group of W consecutive lanes (W = 8, 16, 32 or 64; all lanes of the group
// must call it; the result is the same in every lane of the group).  A search by one lane is a chain of
// dependent loads; here a link of the chain is one load per lane.  Dense rounds probe W consecutive rows
// around a guess: first the interpolated position, then that position corrected by the residual at the
// edge of the window just probed (a Newton step with a W-row window and the window's own slope).  Regular
// matrices end after two or three rounds (the 3-D stencil after four at most; with the global slope and three
// dense rounds one boundary in seventy needed seven to eleven, and the slowest group is the kernel's time).
// Where the corrections stop shrinking the bracket is cut W-fold per round instead.  The row-start load
// of a snapped boundary is served from loads of the round that found the answer.  Result: identical to
// tile_boundary (same monotone predicate, same rule).
template <int W>
__device__ __forceinline__ int2 group_tile_boundary(int t, const Tiling& tl, const int* __restrict__ row_end,
                                                    int num_rows, int nnz, int& split) {
  static_assert(W == 2 || W == 4 || W == 8 || W == 16 || W == 32 || W == 64, "group width");
  constexpr int LEAD = (W * 5) / 8;  // rows of the window below the guess (towards the row a snap moves back to)
  const int lane = lane_id();
  const int gbase = lane & ~(W - 1);  // first lane of my group
  const int glane = lane & (W - 1);
  constexpr unsigned long long GMASK = (W == 64) ? ~0ull : ((1ull << (W & 63)) - 1ull);
  auto group_ballot = [&](bool b) { return (__builtin_amdgcn_ballot_w64(b) >> gbase) & GMASK; };
  auto from_lane = [&](int v, int l) { return __builtin_amdgcn_ds_bpermute((gbase + l) << 2, v); };
  const long long d = (long long)t * tl.nominal;
  const int diag = (int)min(d, (long long)num_rows + nnz);
  int lo = max(diag - nnz, 0);
  int hi = min(diag, num_rows);
  // the answer: first i in [lo, hi) with row_end[i] + i + 1 > diag, else hi
  const float inv_slope = (float)num_rows / ((float)num_rows + (float)nnz);
  int guess = (int)((float)diag * inv_slope);
  int win_start = 0, win_end_value = 0;  // window of the round that found the answer, and this lane's probe
  int win_snap_value = 0;                // ... and what lanes 0 and 1 fetched for the snapping rule in that round
  bool win_valid = false;
  const bool snapping = tl.snap_slack > 0 && t > 0 && t < tl.num_tiles;
  // Dense rounds go on for as long as they converge: a round whose correction is not at least four times
  // smaller than the one before it (rows of very different lengths: no slope predicts them) ends them.
  // A whole wavefront per boundary (the search inside a reducer block, where every instruction is on the
  // block's critical path) keeps the plain form: its window is wide enough to hold the row the snapping
  // rule needs, and the refinements below bought it nothing (spring-mass 100^3: 33.5 us against 31.9).
  constexpr bool REFINED = W < 64;
  constexpr int MAX_DENSE_ROUNDS = REFINED ? 6 : 3;
  long long last_jump = 0;
#pragma unroll 1
  for (int round = 0; round < MAX_DENSE_ROUNDS && lo < hi; ++round) {
    const int guess_before = guess;
    const int w0 = min(max(guess - LEAD, lo), max(hi - W, lo));  // window [w0, w0 + W) inside [lo, hi)
    const int pos = w0 + glane;
    int end = 0;
    bool past = true;  // lanes at or beyond hi behave like "predicate true"
    if (pos < hi) {
      end = row_end[pos];
      past = end + pos + 1 > diag;
    }
    // A snapped boundary needs the end of the row before its snap row, which a narrow window rarely holds:
    // if the answer is in this window, the snap row is one of the first two multiples of the snap width at
    // or above (w0 rounded down), so lanes 0 and 1 fetch those two values in the same round instead of one
    // more dependent load afterwards.
    int snap_value = 0;
    if (REFINED && snapping && glane < 2) {
      const int row = (w0 & ~tl.snap_mask) + glane * (tl.snap_mask + 1) - 1;
      if (row >= 0 && row < num_rows) snap_value = row_end[row];
    }
    const unsigned long long m = group_ballot(past);
    // Rows per merge item around here, from the window's own ends, where all of it was probed and its rows
    // are about as long as the matrix's average: on a regular matrix the next guess then lands on the row
    // (the global ratio is off by the share of short boundary rows - thousands of rows on a 3-D stencil).
    float step_slope = inv_slope;
    if (REFINED && w0 + W <= hi) {
      const float local = (float)(W - 1) / (float)(from_lane(end, W - 1) - from_lane(end, 0) + (W - 1));
      if (local > 0.75f * inv_slope && local < 1.33f * inv_slope) step_slope = local;
    }
    if (m == 0ull) {  // every probed row ends before the diagonal: the answer lies beyond the window
      const int g_last = from_lane(end, W - 1) + (w0 + W - 1) + 1;
      lo = w0 + W;
      guess = (int)min((long long)lo + (long long)((float)(diag - g_last) * step_slope), (long long)hi);
    } else {
      const int j = __builtin_ctzll(m);
      if (j > 0 || w0 == lo) {  // rows before w0 + j end before the diagonal, row w0 + j (or hi) does not
        lo = hi = w0 + j;
        win_start = w0;
        win_end_value = end;
        win_snap_value = snap_value;
        win_valid = true;
      } else {  // the answer is at or before the window's first row
        const int g_first = from_lane(end, 0) + w0 + 1;
        hi = w0;
        guess = w0 - 1 - (int)((float)(g_first - diag) * step_slope);
      }
    }
    const long long jump = (long long)guess - guess_before;
    const long long jump_size = jump < 0 ? -jump : jump;
    if (REFINED && round > 0 && jump_size * 4 > last_jump) break;
    last_jump = jump_size;
  }
  const int probed_below = min(diag, num_rows);  // window lanes at or beyond this row hold no probe
#pragma unroll 1
  while (lo < hi) {  // W evenly spaced probes per round
    const int n = hi - lo;
    const int step = (n + W - 1) / W;
    const int pos = lo + (glane + 1) * step - 1;
    bool past = true;
    if (pos < hi) past = row_end[pos] + pos + 1 > diag;
    const unsigned long long m = group_ballot(past);
    const int j = (m == 0ull) ? W : __builtin_ctzll(m);
    // samples before j end before the diagonal, sample j (if any) does not
    const int new_lo = min(lo + j * step, hi);                               // one past sample j - 1
    const int new_hi = (j == W) ? hi : min(lo + (j + 1) * step - 1, hi);    // sample j itself (or hi)
    lo = new_lo;
    hi = new_hi;
  }
  int2 c = make_int2(min(lo, num_rows), diag - lo);
  split = c.x;
  if (snapping) {
    const int xs = c.x & ~tl.snap_mask;
    int ys = 0;
    if (xs > 0) {
      const int src = xs - 1 - win_start;                                       // lane that probed row xs - 1
      const int which = (xs - (win_start & ~tl.snap_mask)) / (tl.snap_mask + 1);  // lane that fetched it for the rule
      if (win_valid && src >= 0 && src < W && xs - 1 < probed_below) {
        ys = from_lane(win_end_value, src);
      } else if (REFINED && win_valid && xs >= (win_start & ~tl.snap_mask) && which < 2) {
        ys = from_lane(win_snap_value, which);
      } else {
        ys = row_end[xs - 1];
      }
    }
    if ((c.x - xs) + (c.y - ys) <= tl.snap_slack) c = make_int2(xs, ys);
  }
  return c;
}

// ... by a whole wavefront: the result is uniform, which the compiler is told
__device__ __forceinline__ int2 wave_tile_boundary(int t, const Tiling& tl, const int* __restrict__ row_end,
                                                   int num_rows, int nnz, int& split) {
  int2 c = group_tile_boundary<WAVE>(t, tl, row_end, num_rows, nnz, split);
  c.x = __builtin_amdgcn_readfirstlane(c.x);
  c.y = __builtin_amdgcn_readfirstlane(c.y);
  split = __builtin_amdgcn_readfirstlane(split);
  return c;
}

// One search per tile boundary: coords[t] is where tile t starts, coords[num_tiles] where the path ends.
// SEARCH_GROUP lanes per boundary: enough to cut the chain of dependent loads to a few links, few enough
// for all boundaries of a large launch to be searched at once.  The kernel's time follows the number of
// threads more than the number of rounds (Poisson 256^3 / R-MAT scale 22, us: 2 lanes 16.9 / 13.8, 4 lanes
// 9.2 / 11.9, 8 lanes 10.2 / 14.0, 16 lanes 12.1 / 17.5, 32 lanes 17.7 / 22.8; blocks of 64 threads, of 256
// within 1 us of that).
#ifndef FLEX_TUNE_SEARCH_BLOCK
#define FLEX_TUNE_SEARCH_BLOCK 64
#endif
constexpr int SEARCH_BLOCK = FLEX_TUNE_SEARCH_BLOCK;
#ifndef FLEX_TUNE_SEARCH_GROUP
#define FLEX_TUNE_SEARCH_GROUP 4
#endif
constexpr int SEARCH_GROUP = FLEX_TUNE_SEARCH_GROUP;
__global__ void __launch_bounds__(SEARCH_BLOCK)
tile_search_kernel(const Tiling tl, const int* __restrict__ row_end, int num_rows, int nnz, int2* __restrict__ coords,
                   int* __restrict__ splits) {
  const int t = (int)(blockIdx.x * (SEARCH_BLOCK / SEARCH_GROUP) + threadIdx.x / SEARCH_GROUP);
  if (t > tl.num_tiles) return;  // uniform per group
  int split;
#ifdef FLEX_TUNE_THREAD_SEARCH  // tuning switch: one lane searches
  if ((threadIdx.x & (SEARCH_GROUP - 1)) == 0) {
    coords[t] = tile_boundary(t, tl, row_end, num_rows, nnz, split);
    splits[t] = split;
  }
#else
  const int2 c = group_tile_boundary<SEARCH_GROUP>(t, tl, row_end, num_rows, nnz, split);
  if ((threadIdx.x & (SEARCH_GROUP - 1)) == 0) {
    coords[t] = c;
    splits[t] = split;
  }
#endif
}

// Which tile a block works on.  Blocks are dealt to the 8 XCDs round-robin (block % 8), each XCD with
// its own L2.  Runs of 2^xcd_shift consecutive tiles go to the same XCD, so that neighbouring tiles -
// which gather overlapping vertex data - share an L2, while all XCDs still work inside one window of
// 8 runs.  Runs of 16 cut the re-fetching of gathered data on meshes and stencils (Poisson 256^3: x is
// fetched 1.2 times instead of 3.6 times) and measured 1-4 % faster there; on power-law matrices they
// measured slower, so the host picks the run length per launch (Tiling::xcd_shift).
__device__ __forceinline__ int tile_of_block(int block, int xcd_shift) {
  if (xcd_shift == 0) return block;
  const int xcd = block & (NUM_XCD - 1), seq = block / NUM_XCD;
  return ((((seq >> xcd_shift) * NUM_XCD) + xcd) << xcd_shift) + (seq & ((1 << xcd_shift) - 1));
}
inline int grid_for_tiles(int num_tiles, int xcd_shift) {
  const int window = NUM_XCD << xcd_shift;
  return xcd_shift == 0 ? num_tiles : (num_tiles + window - 1) / window * window;
}

// Neighbouring edges a thread takes per first-level load on launches with short, regular rows: as many
// (a power of two, at most 4 and at most IPT) as keep what it fetches for them within 48 bytes.  Plain SpMV
// in float64 (12 bytes per edge): 4 - its 8- and 4-byte loads become 16-byte loads, 3 % on Poisson 256^3.
// The shallow-water map (28 bytes per edge, 16 of them one load already) stays at 1: 2 measured 2 % slower.
// Power-law launches always use 1: their map runs in coalesced edge order, where neighbouring lanes should
// hold neighbouring edges (R-MAT: 370 us with 2 or 4 against 344).
template <class G, int IPT>
constexpr int edges_per_load() {
  constexpr int bytes = G::FETCH_VALUES * (int)sizeof(typename G::Value) + G::FETCH_INDICES * 4;
  int epl = 1;
  while (epl * 2 <= 4 && epl * 2 <= IPT && IPT % (epl * 2) == 0 && epl * 2 * bytes <= 48) epl *= 2;
  return epl;
}

// LDS of a reducer block.  Fetched values and index words of the tile's edges, one finished total per row
// end for the merge path (TILE rows: a tile may consist of row ends only), one dump slot per lane for items
// that close no row.  Where everything fits a modest budget the totals are a region of their own; otherwise
// they lie over the fetched values and indices together - the walk has read its items from both by then -
// so that a block needs no more than the larger of the two.  The spring-mass map (two streamed values and an
// index per edge, three reduced values per row): 24.6 KB + the dump slots instead of 33.9 KB, 6 resident
// blocks per CU instead of 4.
#ifndef FLEX_TUNE_SEPARATE_OUT_BYTES
#define FLEX_TUNE_SEPARATE_OUT_BYTES (20 * 1024)
#endif
template <class G, int BLOCK, int IPT>
struct TileLds {
  using V = typename G::Value;
  static constexpr int TILE = BLOCK * IPT;
  static constexpr int REDN = G::RED_WIDTH > 0 ? G::RED_WIDTH : 1;
  static constexpr int FVN = G::FETCH_VALUES > 0 ? G::FETCH_VALUES : 1, FIN = G::FETCH_INDICES > 0 ? G::FETCH_INDICES : 1;
  static constexpr bool MAP_FIRST = G::ROW_WIDTH == 0;
  static constexpr int FV_ELEMS = (MAP_FIRST && REDN * TILE > FVN * TILE) ? REDN * TILE : FVN * TILE;  // fetched data / contributions
  static constexpr size_t FV_BYTES = (size_t)FV_ELEMS * sizeof(V), FI_BYTES = (size_t)FIN * TILE * 4;
  static constexpr size_t OUT_BYTES = (size_t)REDN * TILE * sizeof(V), DUMP_BYTES = (size_t)REDN * WAVE * sizeof(V);
  static constexpr bool SEPARATE_OUT = FV_BYTES + FI_BYTES + OUT_BYTES + DUMP_BYTES <= (size_t)FLEX_TUNE_SEPARATE_OUT_BYTES;
  static constexpr size_t FETCH_BYTES = FV_BYTES + FI_BYTES;
  static constexpr size_t MAIN_BYTES = SEPARATE_OUT ? FETCH_BYTES + OUT_BYTES : (FETCH_BYTES > OUT_BYTES ? FETCH_BYTES : OUT_BYTES);
  static constexpr size_t RAW_BYTES = MAIN_BYTES + DUMP_BYTES;
  // blocks of this kernel a CU holds at a time as far as LDS decides it (160 KB per CU; the small arrays
  // beside the raw buffer and the allocation granularity are worth another half KB per block)
  static constexpr int RESIDENT_PER_CU = (int)((160 * 1024) / (RAW_BYTES + 512)) < 8 ? (int)((160 * 1024) / (RAW_BYTES + 512)) : 8;
};

// ----------------------------------------------------------------------------------------------
// Reducer kernel.  One block per merge tile of at most BLOCK*IPT merge items (R row ends + Z non-zeros),
// found by the tile search.  Blocks are small and independent; overlap of one block's memory waits
// with another block's arithmetic is left to the hardware scheduler (6-8 resident blocks per CU), which
// measured far better than a persistent, software-pipelined loop.
//
//   1  first-level loads: IPT edges per thread in coalesced order (edge tensors, index arrays), the
//      end offset of tile row tid (first wavefront: also of row BLOCK + tid) and row-aligned sources
//   2  what was fetched goes to LDS; a block-wide vote (which doubles as the barrier that publishes
//      the LDS data) picks the reduction:
//      ROW path (every row of the tile is short and about as long as its neighbours - meshes,
//        stencils): thread r owns tile row r.  It takes the row's edges from LDS, gathers their vertex
//        data, runs the map and sums.  Neighbouring lanes are neighbouring rows, so their k-th edges
//        point at neighbouring vertices: a wavefront's gather touches a few cache lines instead of 64
//        (with one gather per lane in edge order the vector L1 is the limit: it looks up one line per
//        cycle, and the 7-point stencil kept it busy 86 % of the time).  Consecutive threads store
//        consecutive rows.
//      MERGE path (skewed rows): each thread owns IPT consecutive merge items as in the reference
//        (cuda_template/reducer/merged_agent_spmv_template.cuh:196-345).  Row ends become a bitmap
//        over merge positions in LDS (row i ends at position (row_end[i] - y0) + i); a popcount
//        replaces the per-thread diagonal search, so all LDS reads are independent and the walk is
//        branch-free register work; finished rows go through an LDS buffer to coalesced stores; open
//        totals are combined by a wave64 DPP segmented scan and a fold across waves.
// Loads are never placed under a branch (that would serialise them behind a wait each): out-of-range
// lanes read a clamped address, and per-item work is predicated.  Every row is written exactly once;
// the tile's open last row becomes a carry record for fixup_kernel.
// ----------------------------------------------------------------------------------------------
//
// check (uniform): c0 and c1 come from the tile table of an earlier launch, together with the splits they
// were derived from.  Six lanes then fetch the row ends that decide whether a search on this launch's row
// pointer would return the same two boundaries (boundary_from_split); the loads travel with the tile's own,
// the verdict is part of the vote, and a tile whose boundaries are not confirmed returns true before
// anything has been written: its block searches and comes back.
template <class G, int BLOCK, int IPT, int EPL>
__device__ __forceinline__ bool
reduce_tile(const int tile, const int2 c0, const int2 c1, const Tiling& tl, const bool check, const int split0,
            const int split1, const int num_rows, const int* __restrict__ row_end, const int nnz,
            const typename G::Params& p, int* __restrict__ carry_row, typename G::Value* __restrict__ carry_val,
            typename G::Value* __restrict__ agg_partials) {
  const int row_group_hint = tl.row_group;
  using V = typename G::Value;
  using Fetch = typename G::Fetch;
  using Gather = typename G::Gather;
  constexpr int TILE = BLOCK * IPT;
  constexpr int NW = BLOCK / WAVE;
  constexpr int NWORDS = TILE / 32;
  constexpr int FV = G::FETCH_VALUES, FI = G::FETCH_INDICES;
  constexpr int RED = G::RED_WIDTH, AGG = G::AGG_WIDTH, ROW = G::ROW_WIDTH;
  constexpr int REDN = RED > 0 ? RED : 1;
  constexpr int FVN = FV > 0 ? FV : 1, FIN = FI > 0 ? FI : 1;
  constexpr bool MAP_FIRST = (ROW == 0);  // merge path: the map runs before the walk (see below)
#ifndef FLEX_TUNE_ROW_PATH_MAX_LEN
#define FLEX_TUNE_ROW_PATH_MAX_LEN 32
#endif
  constexpr int ROW_PATH_MAX_LEN = FLEX_TUNE_ROW_PATH_MAX_LEN;  // longest row the row path accepts (0: never)
  // Edges whose fetched and gathered data a thread keeps in registers at a time: as many as fit a budget
  // of 32-bit registers (the shallow-water map in float64 needs 13 per edge, plain SpMV 3 to 5), so that
  // wide graphs keep their occupancy.
#ifndef FLEX_TUNE_STAGE_WORDS
#define FLEX_TUNE_STAGE_WORDS 40
#endif
  constexpr int STAGE_FIT = FLEX_TUNE_STAGE_WORDS / (G::EDGE_WORDS > 0 ? G::EDGE_WORDS : 1);
  constexpr int ROW_PATH_UNROLL = STAGE_FIT < 2 ? 2 : (STAGE_FIT > 8 ? 8 : STAGE_FIT);
  constexpr int MERGE_CHUNK = ROW_PATH_UNROLL < IPT ? ROW_PATH_UNROLL : IPT;  // likewise in the merge walk
  constexpr int ROW_PATH_MAX_ROWS = BLOCK + WAVE;  // rows (incl. the open one) whose ends are prefetched
  static_assert((IPT & (IPT - 1)) == 0 && IPT <= 32, "a thread's items must sit inside one bitmap word");
#ifndef FLEX_TUNE_UNSAFE_BIG_TILE  // experiment switch: row path only (the merge path would be wrong)
  static_assert(NWORDS <= WAVE, "one wavefront scans the bitmap words");
#endif

  // LDS (layout: TileLds)
  using Lds = TileLds<G, BLOCK, IPT>;
  constexpr size_t FV_BYTES = Lds::FV_BYTES, FETCH_BYTES = Lds::FETCH_BYTES, MAIN_BYTES = Lds::MAIN_BYTES,
                   DUMP_BYTES = Lds::DUMP_BYTES;
  constexpr bool SEPARATE_OUT = Lds::SEPARATE_OUT;
  static_assert(FV_BYTES % 16 == 0 && FETCH_BYTES % 16 == 0 && MAIN_BYTES % 16 == 0, "LDS regions stay 16-byte aligned");
  __shared__ __attribute__((aligned(16))) unsigned char s_raw[MAIN_BYTES + DUMP_BYTES];
  V* const s_fv = reinterpret_cast<V*>(s_raw);
  int* const s_fi = reinterpret_cast<int*>(s_raw + FV_BYTES);
  V* const s_out = reinterpret_cast<V*>(s_raw + (SEPARATE_OUT ? FETCH_BYTES : 0));
  // value c of row r at s_out[c * TILE + r]; value c of lane l's dump slot at s_out[DUMP_AT + c * WAVE + l]
  constexpr int DUMP_AT = (int)((MAIN_BYTES - (SEPARATE_OUT ? FETCH_BYTES : 0)) / sizeof(V));
  __shared__ unsigned s_bits[NWORDS];
  __shared__ int s_vote[NW];
  __shared__ int s_wave_key[NW];
  __shared__ V s_wave_val[NW][REDN];

  // The thread id is taken afresh on every call: a kernel holds this function twice (a tile taken from the
  // table, and the same tile again after a search when the table was refused), and the compiler would
  // otherwise share everything that only depends on the thread id between the two and keep it in
  // registers through the whole first tile.
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;

  const int x0 = c0.x, y0 = c0.y;
  const int R = c1.x - c0.x;  // row ends inside this tile
  const int Z = c1.y - c0.y;  // non-zeros inside this tile
  const int last_edge = nnz - 1;
  const int last_row = num_rows - 1;

  // Which edge of the tile a thread's k-th first-level load takes: EPL neighbouring edges per thread (its
  // loads of them merge into wider ones: 16 bytes per lane instead of 4 or 8), threads side by side.
  static_assert(EPL >= 1 && IPT % EPL == 0, "edges per load must divide the items per thread");
  auto slot_of = [&](const int k) { return (k / EPL) * (EPL * BLOCK) + tid * EPL + (k % EPL); };

  // 0: for a tile table that has to be confirmed, the three row ends that decide a boundary (the rows before
  // and at the split, and the row before the one a snap moves the boundary to).  The first wavefront fetches
  // them for the tile's start, the second for its end (a block of one wavefront: both), through the scalar
  // cache - the row pointer does not change during a launch -, so that they are counted apart from the
  // tile's vector loads: the verdict waits for these three words only and is worked out while the tile's
  // data are on the way.
  constexpr int CHECKERS = NW >= 2 ? 2 : 1;  // wavefronts that check a boundary
  const int wave_uniform = __builtin_amdgcn_readfirstlane(wave);  // the same number, known to be one per wavefront
  const bool checker = check && wave_uniform < CHECKERS;
  // (Like every load here they are not under a branch - the compiler would wait for them where the branch
  // ends, in front of the tile's loads: a launch that does not check reads the first row end three times.)
  int ends_a[3], ends_b[3] = {0, 0, 0};  // of this wavefront's boundary (a block of one wavefront: ends_b the tile's end)
  {
    typedef const __attribute__((address_space(4))) int* RowEnds;
    const RowEnds ends = (RowEnds)row_end;
    auto fetch = [&](const int split, int (&out)[3]) {
      out[0] = ends[min(max(split - 1, 0), num_rows - 1)];
      out[1] = ends[min(max(split, 0), num_rows - 1)];
      out[2] = ends[min(max((split & ~tl.snap_mask) - 1, 0), num_rows - 1)];
    };
    if constexpr (CHECKERS == 2) {
      fetch(wave_uniform == 0 ? split0 : split1, ends_a);
    } else {
      fetch(split0, ends_a);
      fetch(split1, ends_b);
    }
  }

  // 1: first-level loads.  A tile holds Z <= TILE non-zeros; lanes past Z re-read the tile's last
  // edge (one cache line, no extra traffic) instead of running into the next tile's edges.
  Fetch f[IPT];
  const int e_last = min(y0 + max(Z - 1, 0), last_edge);
  // Where every streamed word is an array of its own (edge tensors of width 1, index arrays), the LDS image of
  // a tile is its slice of those arrays as they lie in memory, and the launches with short regular rows
  // (EPL > 1) let the loads write it themselves (global_load_lds_dwordx4: 16 bytes per lane, a wavefront's
  // 1 KB lands contiguously): no landing registers, no LDS stores.  Poisson 256^3: 305.5 us against 307.7.
  // A tile that reaches past the end of the edge list takes the loads below instead.
#if defined(FLEX_TUNE_LDS_DIRECT_ALL)  // tuning switch: also on launches with long or irregular rows
  constexpr bool CAN_DIRECT = G::FETCH_CONTIGUOUS && TILE % (NW * WAVE * 4) == 0;
#elif !defined(FLEX_TUNE_NO_LDS_DIRECT)
  constexpr bool CAN_DIRECT = EPL > 1 && G::FETCH_CONTIGUOUS && TILE % (NW * WAVE * 4) == 0;
#else
  constexpr bool CAN_DIRECT = false;
#endif
  const bool direct = CAN_DIRECT && (long long)y0 + TILE <= (long long)nnz;  // uniform: every slot is an edge of the list
  if constexpr (CAN_DIRECT) {
   if (direct) {
    constexpr int VPL = 16 / (int)sizeof(V), VPIECE = WAVE * VPL;
#pragma unroll
    for (int w = 0; w < FV; ++w) {
      const V* src = G::value_stream(p, w) + y0;
#pragma unroll
      for (int i = 0; i < TILE / VPIECE / NW; ++i) {
        const int piece = i * NW + wave;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + piece * VPIECE + lane * VPL),
                                         (__attribute__((address_space(3))) void*)(s_fv + w * TILE + piece * VPIECE), 16, 0, 0);
      }
    }
    constexpr int IPIECE = WAVE * 4;
#pragma unroll
    for (int w = 0; w < FI; ++w) {
      const int* src = G::index_stream(p, w) + y0;
#pragma unroll
      for (int i = 0; i < TILE / IPIECE / NW; ++i) {
        const int piece = i * NW + wave;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + piece * IPIECE + lane * 4),
                                         (__attribute__((address_space(3))) void*)(s_fi + w * TILE + piece * IPIECE), 16, 0, 0);
      }
    }
   }
  }
  if (!direct) {
#pragma unroll
  for (int k = 0; k < IPT; k += EPL) {
    if constexpr (EPL == 1) {
      G::fetch(p, min(y0 + slot_of(k), e_last), f[k]);
    } else {
      // EPL neighbouring edges from one base address, so that the loads merge.  A group that would run past
      // the end of the edge list (last tile only; the host launches this variant only when there are at
      // least EPL edges) is read from the last EPL edges instead and shifted into place, so that slot j
      // still holds edge min(y0 + j, last edge).  A group past the tile's own edges simply reads the next
      // tile's: those slots are never used.
      const int want = y0 + slot_of(k);
      const int e0 = min(want, last_edge - (EPL - 1));
      const int shift = want - e0;  // 0 except at the very end of the edge list
      Fetch g[EPL];
#pragma unroll
      for (int q = 0; q < EPL; ++q) G::fetch(p, e0 + q, g[q]);
#pragma unroll
      for (int q = 0; q < EPL; ++q) {
        f[k + q] = g[EPL - 1];
#pragma unroll
        for (int r = q; r < EPL - 1; ++r)
          if (q + shift == r) f[k + q] = g[r];
      }
    }
  }
  }
  // ... and of the rows: thread tid holds the end of tile row tid, the first wavefront also the end
  // of row BLOCK + tid; lane 0 of each wavefront fetches the end of the row before its first one,
  // the other lanes get it from their neighbour, so every thread knows where its row starts.
  int re, re2 = 0, prev_lane0 = 0, prev2_lane0 = 0;
  Pack<V, ROW> rowv, rowv2;
  {
    const int r1 = min(x0 + tid, last_row);
    re = row_end[r1];
    if constexpr (ROW > 0) G::load_row(p, r1, rowv);
    if (lane == 0 && tid > 0) prev_lane0 = row_end[min(x0 + tid - 1, last_row)];
    if (wave == 0 && R + 1 > BLOCK) {  // uniform: only tiles with more rows than threads need a second pass
      const int r2 = min(x0 + BLOCK + tid, min(x0 + R, last_row));
      re2 = row_end[r2];
      if constexpr (ROW > 0) G::load_row(p, r2, rowv2);
      if (lane == 0) prev2_lane0 = row_end[min(x0 + BLOCK - 1, last_row)];
    }
  }

  int stale_bit = 0;
  if (checker) {  // are the boundaries this tile is being loaded with the ones a search would find?
    bool confirmed;
    if constexpr (CHECKERS == 2) {
      bool ok;
      const int2 n = boundary_from_split(tile + wave_uniform, tl, num_rows, nnz, wave_uniform == 0 ? split0 : split1,
                                         ends_a[0], ends_a[1], ends_a[2], ok);
      const int2 c = wave_uniform == 0 ? c0 : c1;
      confirmed = ok && n.x == c.x && n.y == c.y;
    } else {
      bool ok0, ok1;
      const int2 n0 = boundary_from_split(tile, tl, num_rows, nnz, split0, ends_a[0], ends_a[1], ends_a[2], ok0);
      const int2 n1 = boundary_from_split(tile + 1, tl, num_rows, nnz, split1, ends_b[0], ends_b[1], ends_b[2], ok1);
      confirmed = ok0 && ok1 && n0.x == c0.x && n0.y == c0.y && n1.x == c1.x && n1.y == c1.y;
    }
    stale_bit = confirmed ? 0 : 2;
  }

  if (tid < NWORDS) s_bits[tid] = 0u;

  // 2: hand-over through LDS, in coalesced order.  Every slot of the tile is written (slots past Z hold
  // copies of the tile's last edge), so a clamped read always finds a real edge.
  if (!direct) {
#pragma unroll
    for (int k = 0; k < IPT; ++k) G::template put<TILE>(f[k], s_fv, s_fi, slot_of(k));
  } else {
    __builtin_amdgcn_s_waitcnt(0);  // this wavefront's pieces have landed in LDS (the barrier below publishes them)
  }

  // vote - can every row of this tile be summed by one thread?  Row i of the tile spans the
  // tile-relative non-zeros [end(i-1), end(i)), with end(-1) = 0 and, for the row still open at the
  // end of the tile (i == R), end = Z.
  const bool few_rows = (R + 1 <= ROW_PATH_MAX_ROWS);
  int start1 = 0, len1 = 0, start2 = 0, len2 = 0;
  {
    const int end1 = (tid < R) ? re - y0 : Z;
    int prev = wave_shift_up1<int>(end1, 0);
    if (lane == 0) prev = (tid > 0) ? prev_lane0 - y0 : 0;
    if (tid <= R) {
      start1 = prev;
      len1 = end1 - prev;
    }
    if (wave == 0) {
      const int end2 = (BLOCK + tid < R) ? re2 - y0 : Z;
      int prev2 = wave_shift_up1<int>(end2, 0);
      if (lane == 0) prev2 = prev2_lane0 - y0;
      if (BLOCK + tid <= R) {
        start2 = prev2;
        len2 = end2 - prev2;
      }
    }
  }
  // ... and are the rows regular?  A thread per row pays for the longest row of its wavefront, so the row
  // path only wins when no row is much longer than the tile's average (meshes, stencils); on skewed
  // tiles with short rows the merge path measured about 10 % faster.
  const int longest = max(len1, len2);
#ifdef FLEX_TUNE_ROW_PATH_ANY_SHAPE  // tuning switch: length limit only
  const bool uneven = false;
#else
  const bool uneven = 4 * (longest - 1) * (R + 1) > 5 * Z;  // longer than 1.25 x average + 1
#endif
  const bool my_vote = (longest > ROW_PATH_MAX_LEN) | !few_rows | uneven;
  // the ballot is taken by the whole wavefront (inside a branch it would only see the branch's lanes)
  const unsigned long long wave_votes = __builtin_amdgcn_ballot_w64(my_vote);
  const int vote_bits = ((wave_votes != 0ull) ? 1 : 0) | stale_bit;
  if (lane == 0) s_vote[wave] = vote_bits;
  __syncthreads();
  int any_vote = 0;
#pragma unroll
  for (int w = 0; w < NW; ++w) any_vote |= s_vote[w];
  if ((any_vote & 2) != 0) return true;  // uniform: nothing has left the block yet
#ifdef FLEX_TUNE_FORCE_MERGE  // tuning switch: always the merge path, decided at run time (same code)
  const bool irregular = (any_vote & 1) != 0 || nnz > 0;
#else
  const bool irregular = (any_vote & 1) != 0;
#endif

  Pack<V, AGG> agg;
  zero(agg);

  if (!irregular) {
    // ---------------- ROW path ----------------
    // A row's edges are handled a group at a time: LDS reads, then all their gathers, then the arithmetic.
    // The group is as large as the register budget allows, cut down to the launch's average row length
    // (a slot no row uses still costs every lane a gather).  The first group is unconditional (lanes of
    // shorter rows read clamped slots and discard the result).  The group size is a compile-time constant
    // of the code that runs: one copy of the row path per size between the budget and half of it.
    auto row_path = [&](auto group_tag) {
      constexpr int GROUP = decltype(group_tag)::value;
      auto sum_row = [&](const int r, const int start, const int len, const Pack<V, ROW>& rv) {
        Pack<V, RED> tot;
        zero(tot);
        auto add_edge = [&](const int yi, const Fetch& fe, const Gather& ge) {
          Pack<V, RED> dt;
          Pack<V, AGG> da;
          G::edge(p, y0 + yi, fe, ge, rv, dt, da);
#pragma unroll
          for (int c = 0; c < RED; ++c) tot.v[c] += dt.v[c];
#pragma unroll
          for (int c = 0; c < AGG; ++c) agg.v[c] += da.v[c];
        };
        for (int base = 0; base == 0 || base < len; base += GROUP) {
          Fetch fe[GROUP];
          Gather ge[GROUP];
#pragma unroll
          for (int it = 0; it < GROUP; ++it) G::template get<TILE>(s_fv, s_fi, min(start + base + it, TILE - 1), fe[it]);
#pragma unroll
          for (int it = 0; it < GROUP; ++it) G::gather(p, fe[it], ge[it]);
#pragma unroll
          for (int it = 0; it < GROUP; ++it) {
            if (base + it < len) {
#ifdef FLEX_TUNE_ROW_BRANCH  // tuning switch: keep the predicate as a branch on the exec mask instead of selects
              asm volatile("" ::: "memory");
#endif
              add_edge(start + base + it, fe[it], ge[it]);
            }
          }
        }
        if (r < R) {
          G::store_row(p, x0 + r, tot);
        } else {  // r == R: the row still open at the end of the tile becomes the tile's carry
          const int row = x0 + r;
          carry_row[tile] = (row < num_rows && len > 0) ? row : -1;
#pragma unroll
          for (int c = 0; c < RED; ++c) carry_val[(size_t)tile * RED + c] = tot.v[c];
        }
      };
      if (tid <= R) sum_row(tid, start1, len1, rowv);
      if (wave == 0 && BLOCK + tid <= R) sum_row(BLOCK + tid, start2, len2, rowv2);
    };
    constexpr int U = ROW_PATH_UNROLL;
    const int group = (row_group_hint > 0 && row_group_hint < U) ? row_group_hint : U;  // uniform over the launch
    if (group >= U) row_path(std::integral_constant<int, U>{});
    else if (U - 1 >= 2 && group == U - 1) row_path(std::integral_constant<int, (U - 1 >= 2 ? U - 1 : 2)>{});
    else if (U - 2 >= 2 && group == U - 2) row_path(std::integral_constant<int, (U - 2 >= 2 ? U - 2 : 2)>{});
    else if (U - 3 >= 2 && group == U - 3) row_path(std::integral_constant<int, (U - 3 >= 2 ? U - 3 : 2)>{});
    else row_path(std::integral_constant<int, (U - 4 >= 2 ? U - 4 : 2)>{});
  } else {
    // ---------------- MERGE path ----------------
    // Graphs without row-aligned sources run the map here, in coalesced edge order, from the registers of
    // the first-level loads (neighbouring lanes hold neighbouring edges of a row, whose columns ascend: the
    // gathers of a power-law matrix hit the same lines far more often than in per-thread item order) and
    // hand the contributions to the walk through LDS.  Graphs with row-aligned sources need the row of
    // every edge first: their walk takes the fetched data from LDS and gathers per item.
    constexpr bool OUT_OVERLAPS = !SEPARATE_OUT;  // s_out lies over data the walk reads
    V* const s_x = s_fv;  // MAP_FIRST: contributions [c * TILE + j]; nobody reads s_fv after the vote
    if constexpr (MAP_FIRST) {
      const Pack<V, ROW> no_row{};
      if constexpr (CAN_DIRECT) {
        if (direct) {  // the edges went to LDS without passing through registers: take them from there
#pragma unroll       // (a thread reads its own slots only, and s_x below overwrites just those)
          for (int k = 0; k < IPT; ++k) G::template get<TILE>(s_fv, s_fi, slot_of(k), f[k]);
        }
      }
#pragma unroll
      for (int k0 = 0; k0 < IPT; k0 += MERGE_CHUNK) {
        Gather g[MERGE_CHUNK];
#pragma unroll
        for (int k = 0; k < MERGE_CHUNK; ++k) G::gather(p, f[k0 + k], g[k]);
#pragma unroll
        for (int k = 0; k < MERGE_CHUNK; ++k) {
          const int j = slot_of(k0 + k);
          if (G::EDGE_PURE || j < Z) {
            Pack<V, RED> dt;
            Pack<V, AGG> da;
            G::edge(p, y0 + j, f[k0 + k], g[k], no_row, dt, da);
#pragma unroll
            for (int c = 0; c < RED; ++c) s_x[c * TILE + j] = dt.v[c];
#pragma unroll
            for (int c = 0; c < AGG; ++c) agg.v[c] += (j < Z) ? da.v[c] : V(0);
          }
        }
      }
    }
    // row ends -> bitmap over merge positions (rows beyond the prefetched ones are read here)
    if (tid < R) {
      const int pos = (re - y0) + tid;
      atomicOr(&s_bits[pos >> 5], 1u << (pos & 31));
    }
    for (int i = tid + BLOCK; i < R; i += BLOCK) {
      const int pos = (row_end[x0 + i] - y0) + i;
      atomicOr(&s_bits[pos >> 5], 1u << (pos & 31));
    }
    __syncthreads();
    // Every wavefront scans the bitmap for itself (lane l takes word l): the number of row ends before
    // each word, then each thread picks up its own word and that word's count from the lane that holds
    // them.  No second barrier, no LDS round trip.
    unsigned word;
    int word_prefix;
    {
      const unsigned my_word = s_bits[lane < NWORDS ? lane : 0];
      int cnt[1] = {lane < NWORDS ? (int)__popc(my_word) : 0};
      const int own = cnt[0];
      wave_segmented_inclusive_sum<int, 1>(0, cnt);
      const int src_lane = (tid * IPT) >> 5;  // < NWORDS <= WAVE
      word = (unsigned)__builtin_amdgcn_ds_bpermute(src_lane << 2, (int)my_word);
      word_prefix = __builtin_amdgcn_ds_bpermute(src_lane << 2, cnt[0] - own);
    }

    // this thread's IPT merge items
    const int tile_items = R + Z;
    const int d0 = tid * IPT;
    const int n_items = max(0, min(IPT, tile_items - d0));
    const int sh = d0 & 31;
    constexpr unsigned FULL = (IPT == 32) ? 0xffffffffu : ((1u << IPT) - 1u);
    const unsigned ends = (word >> sh) & FULL;                                        // items that are row ends
    const unsigned nzs = ~ends & (n_items >= IPT ? FULL : ((1u << n_items) - 1u));  // ... that are non-zeros
    const int xs = word_prefix + __popc(word & ((1u << sh) - 1u));                    // rows before my items
    const int ys = d0 - xs;                                                            // non-zeros before them

    // what the walk needs for my items, from LDS (a row-end item reads the edge after it: harmless):
    // the contributions (MAP_FIRST) or the fetched data
    Pack<V, RED> xv[MAP_FIRST ? IPT : 1];
    Fetch fe[MAP_FIRST ? 1 : IPT];
    int xrel[IPT];
#pragma unroll
    for (int it = 0; it < IPT; ++it) {
      const int before = __popc(ends & ((1u << it) - 1u));
      xrel[it] = xs + before;
      const int yi = ys + it - before;  // < TILE by construction
      if constexpr (MAP_FIRST) {
#pragma unroll
        for (int c = 0; c < RED; ++c) xv[it].v[c] = s_x[c * TILE + yi];
      } else {
        G::template get<TILE>(s_fv, s_fi, yi, fe[it]);
      }
    }

    if constexpr (OUT_OVERLAPS) __syncthreads();  // every thread has read its items: the buffer now serves as s_out

    Pack<V, RED> tot;
    zero(tot);
#pragma unroll
    for (int it0 = 0; it0 < IPT; it0 += MERGE_CHUNK) {
      Gather ge[MERGE_CHUNK];
      if constexpr (!MAP_FIRST) {
#pragma unroll
        for (int k = 0; k < MERGE_CHUNK; ++k) G::gather(p, fe[it0 + k], ge[k]);
      }
#pragma unroll
      for (int k = 0; k < MERGE_CHUNK; ++k) {
        const int it = it0 + k;
        const bool nz = (nzs >> it) & 1u;
        const bool end = (ends >> it) & 1u;
        if constexpr (MAP_FIRST) {
#pragma unroll
          for (int c = 0; c < RED; ++c) tot.v[c] += nz ? xv[it].v[c] : V(0);
        } else {
          if (nz) {
            // row-aligned sources are read from memory here: graphs that use them are mesh-like and
            // take the row path, so this is the uncommon case
            Pack<V, RED> dt;
            Pack<V, AGG> da;
            Pack<V, ROW> rv;
            G::load_row(p, x0 + xrel[it], rv);
            G::edge(p, y0 + ys + it - (xrel[it] - xs), fe[it], ge[k], rv, dt, da);
#pragma unroll
            for (int c = 0; c < RED; ++c) tot.v[c] += dt.v[c];
#pragma unroll
            for (int c = 0; c < AGG; ++c) agg.v[c] += da.v[c];
          }
        }
        // a row end parks the finished total in the output buffer (other items write a dump slot)
        {
#pragma unroll
          for (int c = 0; c < RED; ++c) s_out[end ? c * TILE + xrel[it] : DUMP_AT + c * WAVE + lane] = tot.v[c];
        }
#pragma unroll
        for (int c = 0; c < RED; ++c) tot.v[c] = end ? V(0) : tot.v[c];
      }
    }

    // block-wide segmented scan of the open totals, keyed by the row each thread ended in
    const int key = xs + __popc(ends);
    V run[REDN];
#pragma unroll
    for (int c = 0; c < RED; ++c) run[c] = tot.v[c];
    wave_segmented_inclusive_sum<V, REDN>(key, run);
    int in_key = wave_shift_up1<int>(key, -1);
    V in_val[REDN];
#pragma unroll
    for (int c = 0; c < RED; ++c) in_val[c] = wave_shift_up1<V>(run[c], V(0));
    if (lane == WAVE - 1) {
      s_wave_key[wave] = key;
#pragma unroll
      for (int c = 0; c < RED; ++c) s_wave_val[wave][c] = run[c];
    }
    __syncthreads();

    int pk = -1;
    V pv[REDN];
#pragma unroll
    for (int c = 0; c < RED; ++c) pv[c] = V(0);
#pragma unroll
    for (int w = 0; w < NW - 1; ++w) {
      if (w < wave) {
        const int k = s_wave_key[w];
#pragma unroll
        for (int c = 0; c < RED; ++c) pv[c] = (k == pk) ? static_cast<V>(pv[c] + s_wave_val[w][c]) : s_wave_val[w][c];
        pk = k;
      }
    }
    if (wave > 0) {
      if (lane == 0) {
        in_key = pk;
#pragma unroll
        for (int c = 0; c < RED; ++c) in_val[c] = pv[c];
      } else if (in_key == pk) {
#pragma unroll
        for (int c = 0; c < RED; ++c) in_val[c] += pv[c];
      }
    }
    // the first row a thread closed may have started in earlier threads: add what they carried in
    // (only this thread ever touches that row's slot, so a plain read-modify-write is safe)
    if (ends != 0u && in_key == xs) {
#pragma unroll
      for (int c = 0; c < RED; ++c) s_out[c * TILE + xs] += in_val[c];
    }
    // tile carry-out: what the tile accumulated for the row still open at its end
    if (tid == BLOCK - 1) {
      if (key == pk) {
#pragma unroll
        for (int c = 0; c < RED; ++c) run[c] += pv[c];
      }
      // the open row has non-zeros in this tile unless the tile's last merge item is a row end
      const int last_item = tile_items - 1;
      const bool open_empty = Z == 0 || (R > 0 && ((s_bits[last_item >> 5] >> (last_item & 31)) & 1u) != 0u);
      const int row = x0 + key;
      carry_row[tile] = (row < num_rows && !open_empty) ? row : -1;
#pragma unroll
      for (int c = 0; c < RED; ++c) carry_val[(size_t)tile * RED + c] = run[c];
    }
    __syncthreads();

    // the tile's finished rows leave LDS as coalesced stores
    for (int i = tid; i < R; i += BLOCK) {
      Pack<V, RED> t;
#pragma unroll
      for (int c = 0; c < RED; ++c) t.v[c] = s_out[c * TILE + i];
      G::store_row(p, x0 + i, t);
    }
  }

  // one aggregator partial per tile: the wavefronts' partials added in wavefront order (fixup_kernel adds the
  // tiles' partials in a fixed order)
  if constexpr (AGG > 0) {
    wave_sum_to_last_lane<V, AGG>(agg.v);
#ifndef FLEX_TUNE_PARTIAL_PER_WAVE
    __shared__ V s_tile_agg[NW][AGG];
    if (lane == WAVE - 1) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) s_tile_agg[wave][c] = agg.v[c];
    }
    __syncthreads();
    if (tid == 0) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) {
        V t = s_tile_agg[0][c];
        for (int w = 1; w < NW; ++w) t += s_tile_agg[w][c];
        agg_partials[(size_t)tile * AGG + c] = t;
      }
    }
#else  // tuning switch: one partial per wavefront, no barrier
    if (lane == WAVE - 1) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) agg_partials[((size_t)tile * NW + wave) * AGG + c] = agg.v[c];
    }
#endif
  }
  return false;
}

// Where a reducer block takes its tile's two boundaries from.
enum TileSource : int {
  TILES_FROM_TABLE = 0,   // the table holds this launch's boundaries (tile_search_kernel ran, or the caller
                          // vouches for the table of an earlier launch): taken as they are
  TILES_CONFIRMED = 1,    // the table may hold an earlier launch's boundaries, or anything else: taken if
                          // this launch's row pointer confirms them (reduce_tile), searched otherwise
  TILES_SEARCHED = 2      // the block searches
};

// One block per tile.  A block that searches does so with its first two wavefronts, one boundary each, on
// the two diagonals that bound the tile (the reference lets two threads do it when its grid is smaller than
// the device, cuda_template/reducer/merged_spmv_template.cuh:97-119, merged_agent_spmv_template.cuh:412-435)
// and leaves boundary and split in the table, where the next launch on the same scratch finds them.
// The default, TILES_CONFIRMED, makes the search a once-per-matrix cost without a promise from the caller:
// a solver loop or a time stepper launches on one row structure again and again, its blocks read the
// boundaries of the launch before, load their tiles, and the three row ends per boundary that prove the
// boundaries right arrive with the tile's data (Poisson 256^3: no 9 us search kernel in front of the
// reducer; spring-mass 100^3: no 3 us of search in front of every block's loads).  Table entries are only
// ever used after this proof or after a search, whatever the scratch held: garbage, the table of another
// matrix, or entries another block of this launch is replacing at the same moment.
// With FLEX_TUNE_PERSISTENT (tuning switch) a launch has at most that many blocks per CU; each walks
// tiles blockIdx.x, blockIdx.x + gridDim.x, ... and reads the coordinates of its next tile while it
// works on the current one.
template <class G, int BLOCK, int IPT, int EPL>
__global__ void __launch_bounds__(BLOCK)
reduce_kernel(int2* coords, int* splits, const int source, const Tiling tl, const int num_rows,
              const int* __restrict__ row_end, const int nnz, const typename G::Params p, int* __restrict__ carry_row,
              typename G::Value* __restrict__ carry_val, typename G::Value* __restrict__ agg_partials,
              unsigned* __restrict__ ticket) {
  const int num_tiles = tl.num_tiles;
#ifdef FLEX_TUNE_TICKET_SUM
  if (blockIdx.x == 0 && threadIdx.x == 0) *ticket = 0u;  // arms the last-block detection of fixup_kernel
#endif
#ifdef FLEX_TUNE_PERSISTENT
  int tile = blockIdx.x;
  if (tile >= num_tiles) return;
  int2 c0 = coords[tile], c1 = coords[tile + 1];
  while (true) {
    const int next = tile + (int)gridDim.x;
    const bool more = next < num_tiles;
    int2 n0 = c0, n1 = c1;
    if (more) {
      n0 = coords[next];
      n1 = coords[next + 1];
    }
    reduce_tile<G, BLOCK, IPT, EPL>(tile, c0, c1, tl, false, 0, 0, num_rows, row_end, nnz, p, carry_row, carry_val, agg_partials);
    if (!more) break;
    __syncthreads();  // the tile's LDS is free again
    tile = next;
    c0 = n0;
    c1 = n1;
  }
#else
  const int tile = tile_of_block(blockIdx.x, tl.xcd_shift);
  if (tile >= num_tiles) return;
  __shared__ int2 s_coord[2];
  __shared__ int s_split[2];
  int2 c0 = make_int2(0, 0), c1 = make_int2(0, 0);
  int split0 = 0, split1 = 0;
  bool have = false, check = false;
  if (source != TILES_SEARCHED) {
    // Read through the scalar cache, as a kernel argument would be: one request per block, no vector
    // registers.  An entry another block of this launch replaces at the same moment may come back old:
    // it is then refused like any other stale entry.
    typedef const __attribute__((address_space(4))) int* TableWords;
    const TableWords entries = (TableWords)coords + 2 * tile;
    c0 = make_int2(entries[0], entries[1]);
    c1 = make_int2(entries[2], entries[3]);
    have = true;
    if (source == TILES_CONFIRMED) {
      split0 = ((TableWords)splits)[tile];
      split1 = ((TableWords)splits)[tile + 1];
      // whatever the table held, a tile is only loaded from inside the matrix and never outgrows the block
      // (signs of differences, OR-ed: no chain of compares in front of the block's first loads; a difference of
      // two entries only counts where both are in range, and for each entry one of the range terms is exact)
      const int signs = c0.x | (num_rows - c0.x) | c0.y | (nnz - c0.y) | c1.x | (num_rows - c1.x) | c1.y | (nnz - c1.y) |
                        split0 | (num_rows - split0) | split1 | (num_rows - split1);
      const int order = (c1.x - c0.x) | (c1.y - c0.y) | (BLOCK * IPT - (c1.x - c0.x) - (c1.y - c0.y));
      const bool sane = signs >= 0 && order >= 0;
      have = check = sane;
    }
  }
  // Straight-line: the tile as the table has it; behind it, for a block without usable entries, the search
  // and the tile code a second time (a loop around one copy keeps every kernel argument and everything
  // derived from the thread id in registers through the whole tile: 12 scalar spills and up to 17 more
  // vector registers, 3 % of the kernel on the 3-D stencil).
  if (have) {
    const bool refused = reduce_tile<G, BLOCK, IPT, EPL>(tile, c0, c1, tl, check, split0, split1, num_rows, row_end, nnz,
                                                         p, carry_row, carry_val, agg_partials);
    if (!refused) return;
    __syncthreads();  // every thread has read the verdict; the tile's LDS is free again
  }
  {
    const int w = (int)threadIdx.x / WAVE;
    if (BLOCK >= 2 * WAVE) {  // the first two wavefronts search one boundary each
      if (w < 2) {
        int split;
        const int2 c = wave_tile_boundary(tile + w, tl, row_end, num_rows, nnz, split);
        if ((threadIdx.x & (WAVE - 1)) == 0) {
          s_coord[w] = c;
          s_split[w] = split;
        }
      }
    } else {
      int sa, sb;
      const int2 a = wave_tile_boundary(tile, tl, row_end, num_rows, nnz, sa);
      const int2 b = wave_tile_boundary(tile + 1, tl, row_end, num_rows, nnz, sb);
      if (threadIdx.x == 0) {
        s_coord[0] = a;
        s_coord[1] = b;
        s_split[0] = sa;
        s_split[1] = sb;
      }
    }
    __syncthreads();
    c0 = s_coord[0];
    c1 = s_coord[1];
    c0.x = __builtin_amdgcn_readfirstlane(c0.x);
    c0.y = __builtin_amdgcn_readfirstlane(c0.y);
    c1.x = __builtin_amdgcn_readfirstlane(c1.x);
    c1.y = __builtin_amdgcn_readfirstlane(c1.y);
    if (threadIdx.x == 0) {
      coords[tile] = c0;
      splits[tile] = s_split[0];
      if (tile == num_tiles - 1) {
        coords[num_tiles] = c1;
        splits[num_tiles] = s_split[1];
      }
    }
    reduce_tile<G, BLOCK, IPT, EPL>(tile, c0, c1, tl, false, 0, 0, num_rows, row_end, nnz, p, carry_row, carry_val,
                                    agg_partials);
  }
#endif
}

// ----------------------------------------------------------------------------------------------
// Flat kernel (aggregator and map-only graphs): tiles are plain edge ranges, no row structure.
// ----------------------------------------------------------------------------------------------
template <class G, int BLOCK, int IPT>
__global__ void __launch_bounds__(BLOCK)
flat_kernel(const typename G::Params p, const int nnz, const int num_tiles,
            typename G::Value* __restrict__ agg_partials) {
  using V = typename G::Value;
  constexpr int TILE = BLOCK * IPT;
  constexpr int NW = BLOCK / WAVE;
  constexpr int AGG = G::AGG_WIDTH;
  __shared__ V s_wave_agg[NW][AGG > 0 ? AGG : 1];

  const int tid = threadIdx.x;
  Pack<V, AGG> agg;
  zero(agg);
  const int last_edge = nnz - 1;
  for (int tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
    const long long base = (long long)tile * TILE;
    // loads are unconditional (out-of-range lanes re-read the last edge) so that they overlap
    typename G::Fetch f[IPT];
    typename G::Gather g[IPT];
#pragma unroll
    for (int k = 0; k < IPT; ++k) G::fetch(p, (int)min(base + k * BLOCK + tid, (long long)last_edge), f[k]);
#pragma unroll
    for (int k = 0; k < IPT; ++k) G::gather(p, f[k], g[k]);
#pragma unroll
    for (int k = 0; k < IPT; ++k) {
      const long long e = base + k * BLOCK + tid;
      if (e < nnz) {
        Pack<V, 0> no_row, no_total;
        Pack<V, AGG> da;
        G::edge(p, (int)e, f[k], g[k], no_row, no_total, da);
#pragma unroll
        for (int c = 0; c < AGG; ++c) agg.v[c] += da.v[c];
      }
    }
  }
  if constexpr (AGG > 0) {
    wave_sum_to_last_lane<V, AGG>(agg.v);
    if ((tid & (WAVE - 1)) == WAVE - 1) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) s_wave_agg[tid / WAVE][c] = agg.v[c];
    }
    __syncthreads();
    if (tid == 0) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) {
        V s = s_wave_agg[0][c];
        for (int w = 1; w < NW; ++w) s += s_wave_agg[w][c];
        agg_partials[(size_t)blockIdx.x * AGG + c] = s;
      }
    }
  }
}

// ----------------------------------------------------------------------------------------------
// Fix-up: fold tile carries into their rows (tile order) and reduce the aggregator partials.
// Tiles are handled in chunks of BLOCK, a thread per tile.  A run of tiles that carry into the same row is
// summed by a block-wide segmented scan (wave64 DPP scan, then a fold across the wavefronts in order); the
// thread of the run's last tile adds the total to the row.  A run that starts in the chunk and goes on
// beyond it - a row of millions of non-zeros - is finished by the whole block: it walks the following
// tiles BLOCK at a time for as long as they carry into that row and adds them up in a fixed order; the
// chunks those tiles belong to see that their leading tiles continue an earlier run and leave them alone.
// Nothing here depends on timing: the same sums in the same order on every run, no atomics.
// The aggregator partials (PARTS_PER_TILE per tile: one, or one per wavefront of the reducer block) are summed in a
// fixed order.
//   SINGLE = false: block b handles tiles [b*BLOCK, (b+1)*BLOCK) and leaves its aggregator sum in
//                   block_partials[b]; aggregate_kernel adds those, again in a fixed order.
//   SINGLE = true:  one block walks all chunks (launches of a few thousand tiles) and assigns the
//                   aggregator outputs itself: one kernel less.
// (Finishing the sum in the last fix-up block to finish, found with a ticket counter - FLEX_TUNE_TICKET_SUM -,
// was measured twice and is slower, also with the row outputs stored non-temporally: Poisson 256^3 step
// 323.0 us against 319.0; each block's release at device scope costs more than the 4.6 us kernel it saves.)
// ----------------------------------------------------------------------------------------------
template <class G, int BLOCK, int PARTS_PER_TILE, bool SINGLE>
__global__ void __launch_bounds__(BLOCK)
fixup_kernel(const typename G::Params p, const int num_tiles, const int* __restrict__ carry_row,
             const typename G::Value* __restrict__ carry_val, const typename G::Value* __restrict__ agg_partials,
             typename G::Value* __restrict__ block_partials, unsigned* __restrict__ ticket) {
  using V = typename G::Value;
  constexpr int RED = G::RED_WIDTH, AGG = G::AGG_WIDTH;
  constexpr int REDN = RED > 0 ? RED : 1;
  constexpr int NW = BLOCK / WAVE;
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  __shared__ int s_key[NW];
  __shared__ V s_val[NW][REDN];
  __shared__ int s_trail_row;
  __shared__ V s_trail_val[REDN];
  Pack<V, AGG> acc;
  zero(acc);
  const int first_chunk = SINGLE ? 0 : (int)blockIdx.x * BLOCK;
  const int chunk_step = SINGLE ? BLOCK : num_tiles;  // not SINGLE: one chunk per block
  // One block for all chunks: one pass with all loads in flight together sums the aggregator partials and
  // looks whether any run is longer than a tile.  If none is (always on row-snapped launches, where no
  // tile carries at all), every carry goes to its row as it is and the chunk loop below is skipped.
  bool may_have_runs = true;
  bool partials_done = false;
  if constexpr (SINGLE) {
    constexpr int KEPT = 4;  // carries a thread keeps in registers between the two phases
    int kept_row[KEPT];
    bool multi = false;
    for (int i = 0, t = tid; t < num_tiles; ++i, t += BLOCK) {
      if constexpr (RED > 0) {
        const int row = carry_row[t];
        const int next_row = (t + 1 < num_tiles) ? carry_row[t + 1] : -2;
        multi |= (row >= 0 && next_row == row);
        if (i < KEPT) kept_row[i] = row;
      }
      if constexpr (AGG > 0) {
#pragma unroll
        for (int w = 0; w < PARTS_PER_TILE; ++w) {
#pragma unroll
          for (int c = 0; c < AGG; ++c) acc.v[c] += agg_partials[((size_t)t * PARTS_PER_TILE + w) * AGG + c];
        }
      }
    }
    partials_done = true;
    if constexpr (RED > 0) {
      may_have_runs = __syncthreads_or(multi ? 1 : 0) != 0;
      if (!may_have_runs) {
        for (int i = 0, t = tid; t < num_tiles; ++i, t += BLOCK) {
          const int row = (i < KEPT) ? kept_row[i] : carry_row[t];
          if (row >= 0 && !(t > 0 && carry_row[t - 1] == row)) {
            Pack<V, RED> sum;
#pragma unroll
            for (int c = 0; c < RED; ++c) sum.v[c] = carry_val[(size_t)t * RED + c];
            G::add_row(p, row, sum);
          }
        }
      }
    } else {
      may_have_runs = false;
    }
  }
  for (int chunk = first_chunk; chunk < num_tiles && (!SINGLE || may_have_runs); chunk += chunk_step) {
    const int t = chunk + tid;
    const bool valid = t < num_tiles;
    if constexpr (RED > 0) {
      const int row = valid ? carry_row[t] : -1;
      const int next_row = (valid && t + 1 < num_tiles) ? carry_row[t + 1] : -2;
      V run[REDN];
#pragma unroll
      for (int c = 0; c < RED; ++c) run[c] = (row >= 0) ? carry_val[(size_t)t * RED + c] : V(0);
      // Most chunks have no run of more than one tile (none at all on row-snapped launches): then a tile's
      // carry goes to its row as it is, unless the tile continues a run that an earlier chunk owns.
      if (!may_have_runs || !__syncthreads_or((row >= 0 && next_row == row) ? 1 : 0)) {
        if (row >= 0 && !(t > 0 && carry_row[t - 1] == row)) {
          Pack<V, RED> sum;
#pragma unroll
          for (int c = 0; c < RED; ++c) sum.v[c] = run[c];
          G::add_row(p, row, sum);
        }
      } else {
        // does the chunk start inside a run that an earlier chunk owns?
        const int chunk_first_row = carry_row[chunk];
        const bool leading_continues = chunk > 0 && chunk_first_row >= 0 && carry_row[chunk - 1] == chunk_first_row;
        // segmented inclusive sums over the chunk, keyed by row (equal rows are contiguous)
        wave_segmented_inclusive_sum<V, REDN>(row, run);
        if (tid == 0) s_trail_row = -1;
        if (lane == WAVE - 1) {
          s_key[wave] = row;
#pragma unroll
          for (int c = 0; c < RED; ++c) s_val[wave][c] = run[c];
        }
        __syncthreads();
        {
          int pk = -3;
          V pv[REDN];
#pragma unroll
          for (int c = 0; c < RED; ++c) pv[c] = V(0);
          for (int w = 0; w < NW - 1; ++w) {
            if (w < wave) {
              const int k = s_key[w];
#pragma unroll
              for (int c = 0; c < RED; ++c) pv[c] = (k == pk) ? static_cast<V>(pv[c] + s_val[w][c]) : s_val[w][c];
              pk = k;
            }
          }
          if (wave > 0 && row >= 0 && row == pk) {  // my run began in an earlier wavefront of this chunk
#pragma unroll
            for (int c = 0; c < RED; ++c) run[c] += pv[c];
          }
        }
        const bool mine = row >= 0 && !(leading_continues && row == chunk_first_row);
        const bool part_end = next_row != row || tid == BLOCK - 1;  // last tile of the run inside this chunk
        if (mine && part_end) {
          if (next_row != row) {  // the run ends here
            Pack<V, RED> sum;
#pragma unroll
            for (int c = 0; c < RED; ++c) sum.v[c] = run[c];
            G::add_row(p, row, sum);
          } else {  // it goes on in the following chunks: the block finishes it together
            s_trail_row = row;
#pragma unroll
            for (int c = 0; c < RED; ++c) s_trail_val[c] = run[c];
          }
        }
        __syncthreads();
        const int trail_row = s_trail_row;
        if (trail_row >= 0) {  // uniform
          V ext[REDN];
#pragma unroll
          for (int c = 0; c < RED; ++c) ext[c] = V(0);
          // EXT_STEP chunks per vote, all their loads in flight together (the values are fetched whether or
          // not the tile belongs to the run: a load under the test would wait for the row first)
          constexpr int EXT_STEP = 4;
          const int last_tile = num_tiles - 1;
          for (int base = chunk + BLOCK; base < num_tiles; base += EXT_STEP * BLOCK) {
            int urow[EXT_STEP];
            V uval[EXT_STEP][REDN];
#pragma unroll
            for (int k = 0; k < EXT_STEP; ++k) {
              const int u = min(base + k * BLOCK + tid, last_tile);
              urow[k] = carry_row[u];
#pragma unroll
              for (int c = 0; c < RED; ++c) uval[k][c] = carry_val[(size_t)u * RED + c];
            }
            bool all_same = true;
#pragma unroll
            for (int k = 0; k < EXT_STEP; ++k) {
              const bool same = base + k * BLOCK + tid < num_tiles && urow[k] == trail_row;
              all_same &= same;
              if (same) {
#pragma unroll
                for (int c = 0; c < RED; ++c) ext[c] += uval[k][c];
              }
            }
            if (!__syncthreads_and(all_same ? 1 : 0)) break;  // the run is contiguous: a mismatch ends it
          }
          wave_sum_to_last_lane<V, REDN>(ext);
          __syncthreads();  // s_val is free again
          if (lane == WAVE - 1) {
#pragma unroll
            for (int c = 0; c < RED; ++c) s_val[wave][c] = ext[c];
          }
          __syncthreads();
          if (tid == 0) {
            Pack<V, RED> sum;
#pragma unroll
            for (int c = 0; c < RED; ++c) {
              V x = s_trail_val[c];
              for (int w = 0; w < NW; ++w) x += s_val[w][c];
              sum.v[c] = x;
            }
            G::add_row(p, trail_row, sum);
          }
        }
        __syncthreads();  // before the next chunk reuses the shared arrays
      }
    }
    if constexpr (AGG > 0) {
      if (valid && !partials_done) {
#pragma unroll
        for (int w = 0; w < PARTS_PER_TILE; ++w) {
#pragma unroll
          for (int c = 0; c < AGG; ++c) acc.v[c] += agg_partials[((size_t)t * PARTS_PER_TILE + w) * AGG + c];
        }
      }
    }
  }
  if constexpr (AGG > 0) {
    __shared__ V s_wave_agg[NW][AGG];
    __shared__ int s_is_last;
    (void)s_is_last;
    wave_sum_to_last_lane<V, AGG>(acc.v);
    if (lane == WAVE - 1) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) s_wave_agg[wave][c] = acc.v[c];
    }
    __syncthreads();
    if (tid == 0) {
      Pack<V, AGG> total;
#pragma unroll
      for (int c = 0; c < AGG; ++c) {
        V s = s_wave_agg[0][c];
        for (int w = 1; w < NW; ++w) s += s_wave_agg[w][c];
        total.v[c] = s;
      }
      if constexpr (SINGLE) {
        G::store_agg(p, total);
      } else {
#ifdef FLEX_TUNE_TICKET_SUM
        // tuning switch (measured slower, see fixup_kernel's header): the block that draws the last ticket adds the
        // blocks' partials itself.  Each block publishes its partial before it takes a ticket (release at device
        // scope), the last one acquires after taking its own.  The reducer kernel zeroes the ticket.
#pragma unroll
        for (int c = 0; c < AGG; ++c)
          __hip_atomic_store(&block_partials[(size_t)blockIdx.x * AGG + c], total.v[c], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
        __atomic_thread_fence(__ATOMIC_RELEASE);
        const unsigned drawn = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        s_is_last = (drawn == gridDim.x - 1) ? 1 : 0;
#else
#pragma unroll
        for (int c = 0; c < AGG; ++c) block_partials[(size_t)blockIdx.x * AGG + c] = total.v[c];
#endif
      }
    }
#ifdef FLEX_TUNE_TICKET_SUM
    if constexpr (!SINGLE) {
      __syncthreads();
      if (s_is_last) {
        __atomic_thread_fence(__ATOMIC_ACQUIRE);
        Pack<V, AGG> fin;
        zero(fin);
        for (int j = tid; j < (int)gridDim.x; j += BLOCK) {
#pragma unroll
          for (int c = 0; c < AGG; ++c)
            fin.v[c] += __hip_atomic_load(&block_partials[(size_t)j * AGG + c], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        wave_sum_to_last_lane<V, AGG>(fin.v);
        __syncthreads();
        if (lane == WAVE - 1) {
#pragma unroll
          for (int c = 0; c < AGG; ++c) s_wave_agg[wave][c] = fin.v[c];
        }
        __syncthreads();
        if (tid == 0) {
          Pack<V, AGG> total;
#pragma unroll
          for (int c = 0; c < AGG; ++c) {
            V t = s_wave_agg[0][c];
            for (int w = 1; w < NW; ++w) t += s_wave_agg[w][c];
            total.v[c] = t;
          }
          G::store_agg(p, total);
        }
      }
    }
#endif
  }
}

// Final aggregator sum: one block adds `count` partial vectors in a fixed order and assigns the
// outputs (the reference assigns too: cpu_template/merged_spmv_template_aggregator.h:75-87).
template <class G, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
aggregate_kernel(const typename G::Params p, const typename G::Value* __restrict__ partials, const int count) {
  using V = typename G::Value;
  constexpr int AGG = G::AGG_WIDTH;
  constexpr int NW = BLOCK / WAVE;
  if constexpr (AGG > 0) {
    __shared__ V s_wave_agg[NW][AGG];
    Pack<V, AGG> acc;
    zero(acc);
    for (int j = threadIdx.x; j < count; j += BLOCK) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) acc.v[c] += partials[(size_t)j * AGG + c];
    }
    wave_sum_to_last_lane<V, AGG>(acc.v);
    if ((threadIdx.x & (WAVE - 1)) == WAVE - 1) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) s_wave_agg[threadIdx.x / WAVE][c] = acc.v[c];
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      Pack<V, AGG> total;
#pragma unroll
      for (int c = 0; c < AGG; ++c) {
        V s = s_wave_agg[0][c];
        for (int w = 1; w < NW; ++w) s += s_wave_agg[w][c];
        total.v[c] = s;
      }
      G::store_agg(p, total);
    }
  }
}

}  // namespace flex
