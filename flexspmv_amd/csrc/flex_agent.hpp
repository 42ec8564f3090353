// Hand-written gfx950 kernels for one fused "select -> map -> reduce / aggregate" sub-graph.
//
// A generated translation unit defines a graph type G (see codegen/merged_gen_gpu.py) and instantiates
// the kernels below with it.  G supplies, for value type V:
//   G::Params                      pointer bundle (kernel argument)
//   XCH / RED / AGG / ROW widths   number of V values per edge passed through LDS, per-row reduced,
//                                  globally summed, and staged per tile row
//   stage1(p, e, xch, agg)         selector + map for edge e in coalesced order; fills xch, adds to agg
//   stage2(p, e, row, xch, rv, tot, agg)   the part of the map that needs the row; adds to tot / agg
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
//   * blocks are mapped to tiles so that each XCD (one L2 each, workgroups are dealt round-robin to the
//     8 XCDs) walks a contiguous range of tiles and gathered vertex data stays in that XCD's L2.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flex_tensor.hpp"
#include "flex_wave.hpp"

namespace flex {

constexpr int NUM_XCD = 8;

// Optional phase timing for tuning builds: with -DFLEX_PHASE_CLOCKS thread 0 of every block adds the
// clock ticks it spent in each phase of reduce_kernel to g_phase_ticks.  Compiled out otherwise.
#ifdef FLEX_PHASE_CLOCKS
__device__ unsigned long long g_phase_ticks[16];
#define FLEX_TICK_INIT                      \
  unsigned long long tick_ = wall_clock64(); \
  unsigned long long ticks_[12] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}
#define FLEX_TICK(slot)                                \
  do {                                                 \
    const unsigned long long now_ = wall_clock64();    \
    ticks_[slot] += now_ - tick_;                      \
    tick_ = now_;                                      \
  } while (0)
#define FLEX_TICK_FLUSH                                                          \
  do {                                                                           \
    if (threadIdx.x == 0)                                                        \
      for (int i_ = 0; i_ < 12; ++i_) atomicAdd(&g_phase_ticks[i_], ticks_[i_]); \
  } while (0)
#else
#define FLEX_TICK(slot) do {} while (0)
#define FLEX_TICK_INIT do {} while (0)
#define FLEX_TICK_FLUSH do {} while (0)
#endif

template <typename V, int N> struct Pack { V v[N > 0 ? N : 1]; };

template <typename V, int N> __device__ __forceinline__ void zero(Pack<V, N>& a) {
#pragma unroll
  for (int i = 0; i < N; ++i) a.v[i] = V(0);
}

// Streaming (read-once) loads and write-once stores bypass temporal caching so that gathered vertex
// data, not the edge stream, occupies L2.
#ifdef FLEX_TUNE_PLAIN_STREAMS  // tuning switch: ordinary (temporal) loads and stores for the streams
template <typename T> __device__ __forceinline__ T stream_load(const T* p) { return *p; }
template <typename T> __device__ __forceinline__ void stream_store(T* p, T v) { *p = v; }
#else
template <typename T> __device__ __forceinline__ T stream_load(const T* p) { return __builtin_nontemporal_load(p); }
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

// One search per tile boundary: coords[t] is where tile t starts, coords[num_tiles] where the path ends.
__global__ void __launch_bounds__(256)
tile_search_kernel(int num_tiles, int tile_items, const int* __restrict__ row_end, int num_rows, int nnz,
                   int2* __restrict__ coords) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t > num_tiles) return;
  const long long d = (long long)t * tile_items;
  const int diag = (int)min(d, (long long)num_rows + nnz);
  coords[t] = merge_path_search(diag, row_end, num_rows, nnz);
}

// How persistent blocks share the tiles: block b runs on XCD b % 8 (workgroups are dealt to the XCDs
// round-robin), XCD k owns the contiguous tile range [k*per, (k+1)*per), and the blocks of one XCD
// interleave over that range so that at any time an XCD works on neighbouring tiles.
struct TileWalk {
  int tile, end, step;
};
__device__ __forceinline__ TileWalk tiles_of_block(int block, int grid, int num_tiles) {
  const int per = (num_tiles + NUM_XCD - 1) / NUM_XCD;
  const int xcd = block % NUM_XCD;
  const int slots = grid / NUM_XCD;  // grid is a multiple of NUM_XCD
  TileWalk w;
#ifdef FLEX_TUNE_ROUND_ROBIN_TILES  // tuning switch: plain grid-stride assignment, no XCD locality
  w.tile = block;
  w.end = num_tiles;
  w.step = grid;
  (void)per; (void)xcd; (void)slots;
#else
  w.tile = xcd * per + block / NUM_XCD;
  w.end = min((xcd + 1) * per, num_tiles);
  w.step = slots;
#endif
  return w;
}

// ----------------------------------------------------------------------------------------------
// Reducer kernel.  Persistent blocks; each iteration consumes one merge tile of BLOCK*IPT merge
// items (row ends + non-zeros):
//   A  row-end offsets of the tile's rows become a bitmap over merge positions in LDS
//      (row i ends at merge position (row_end[i] - y0) + i); row-aligned vertex data is staged in LDS
//   B  second-level loads (gathers) of the block's NEXT tile are issued from its first-level data
//   C  first-level loads (edge tensors, index arrays, row ends) of the tile AFTER NEXT are issued;
//      both stay in flight during everything below (about 100 KB per CU must be in flight to
//      saturate HBM, and registers are the only store large enough for it)
//   D  the map runs in coalesced edge order; values needed per row go to LDS
//   E  one wavefront turns the bitmap into per-word prefix counts
//   F  each thread owns IPT consecutive merge items: its bitmap bits say which are row ends and a
//      popcount gives its merge coordinate (the result of the per-thread diagonal search of the
//      reference, cuda_template/reducer/merged_agent_spmv_template.cuh:196-215, without a search),
//      so its LDS reads are independent and the walk is branch-free register work; finished rows go
//      to an LDS output buffer
//   G  wave64 DPP segmented scan of the threads' open totals and a fold across waves; each thread
//      adds its carry-in to the first row it closed
//   H  the tile's rows leave LDS as coalesced stores
// The kernel is bound by instruction issue as much as by memory, so loads are never placed under a
// branch (out-of-range lanes read a clamped address) and per-item work is predicated, not branched.
// ----------------------------------------------------------------------------------------------
template <class G, int BLOCK, int IPT>
__global__ void __launch_bounds__(BLOCK)
reduce_kernel(const typename G::Params p, const int* __restrict__ row_end, const int num_rows, const int nnz,
              const int2* __restrict__ coords, const int num_tiles, int* __restrict__ carry_row,
              typename G::Value* __restrict__ carry_val, typename G::Value* __restrict__ agg_partials) {
  using V = typename G::Value;
  constexpr int TILE = BLOCK * IPT;
  constexpr int NW = BLOCK / WAVE;
  constexpr int NWORDS = TILE / 32;
  constexpr int XCH = G::XCH_WIDTH, RED = G::RED_WIDTH, AGG = G::AGG_WIDTH, ROW = G::ROW_WIDTH;
  constexpr int REDN = RED > 0 ? RED : 1;
  constexpr int OUT_CAP = 2 * BLOCK;        // finished rows of a tile buffered in LDS
  constexpr int OUT_STRIDE = OUT_CAP + WAVE;  // + one dump slot per lane for items that close no row
  static_assert((IPT & (IPT - 1)) == 0 && IPT <= 32, "a thread's items must sit inside one bitmap word");
  static_assert(NWORDS <= WAVE, "one wavefront scans the bitmap words");

  __shared__ V s_xch[(XCH > 0 ? XCH : 1) * TILE];
  __shared__ V s_row[(ROW > 0 ? ROW * (TILE + 1) : 1)];
  __shared__ V s_out[REDN * OUT_STRIDE];
  __shared__ unsigned s_bits[2][NWORDS];
  __shared__ int s_word_prefix[NWORDS];
  __shared__ int s_wave_key[NW];
  __shared__ V s_wave_val[NW][REDN];
  __shared__ V s_wave_agg[NW][AGG > 0 ? AGG : 1];

  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;

  TileWalk tw = tiles_of_block(blockIdx.x, gridDim.x, num_tiles);
  Pack<V, AGG> agg;
  zero(agg);
  if (tid < NWORDS) {
    s_bits[0][tid] = 0u;
    s_bits[1][tid] = 0u;
  }
  __syncthreads();
  if (tw.tile >= tw.end) {
    // a block without tiles still owns an aggregator partial slot
    if constexpr (AGG > 0) {
      if (tid == 0) {
#pragma unroll
        for (int c = 0; c < AGG; ++c) agg_partials[(size_t)blockIdx.x * AGG + c] = V(0);
      }
    }
    return;
  }

  const int last_edge = nnz - 1;
  const int last_row = num_rows - 1;

  // First-level loads of a tile starting at merge coordinate c: IPT edges per thread in coalesced
  // order plus one row per thread.  When the whole window is in range (every tile but the last few)
  // addresses are linear in the thread id; otherwise they are clamped to the last valid element.
  auto prefetch = [&](const int2 c, typename G::Fetch (&f)[IPT], int& re, Pack<V, ROW>& rowv) {
    if (c.y + TILE <= nnz && c.x + BLOCK <= num_rows) {
#pragma unroll
      for (int k = 0; k < IPT; ++k) G::fetch(p, c.y + tid + k * BLOCK, f[k]);
      re = row_end[c.x + tid];
      if constexpr (ROW > 0) G::load_row(p, c.x + tid, rowv);
    } else {
#pragma unroll
      for (int k = 0; k < IPT; ++k) G::fetch(p, min(c.y + tid + k * BLOCK, last_edge), f[k]);
      re = row_end[min(c.x + tid, last_row)];
      if constexpr (ROW > 0) G::load_row(p, min(c.x + tid, last_row), rowv);
    }
  };

  // Software pipeline over this block's tiles t(i) = first + i*step, all state in registers:
  //   fetch(i+2) and gather(i+1) are issued at the top of iteration i and stay in flight while
  //   tile i is processed from data that was issued one iteration earlier.
  // Tile ids past the block's range map to the empty tile at the end of the merge path.
  auto coord_of = [&](int t, int2& lo, int2& hi) {
    const int u = (t < tw.end) ? t : num_tiles;
    lo = coords[u];
    hi = coords[min(u + 1, num_tiles)];
  };
  int2 c0, c1, b0, b1, d0c, d1c, e0, e1;
  coord_of(tw.tile, c0, c1);
  coord_of(tw.tile + tw.step, b0, b1);
  coord_of(tw.tile + 2 * tw.step, d0c, d1c);

  typename G::Fetch fa[IPT], fb[IPT];
  typename G::Gather ga[IPT];
  int re_a, re_b;
  Pack<V, ROW> rowv_a, rowv_b;
  prefetch(c0, fa, re_a, rowv_a);
  prefetch(b0, fb, re_b, rowv_b);
#pragma unroll
  for (int k = 0; k < IPT; ++k) G::gather(p, fa[k], ga[k]);

  int buf = 0;
  FLEX_TICK_INIT;
  for (int tile = tw.tile; tile < tw.end; tile += tw.step, buf ^= 1) {
    const int x0 = c0.x, y0 = c0.y;
    const int R = c1.x - c0.x;  // row ends inside this tile
    const int Z = c1.y - c0.y;  // non-zeros inside this tile
    coord_of(tile + 3 * tw.step, e0, e1);

    // B: gathers of the next tile (its first-level data was issued one iteration ago)
    typename G::Gather gb[IPT];
#pragma unroll
    for (int k = 0; k < IPT; ++k) G::gather(p, fb[k], gb[k]);

    // C: first-level loads of the tile after next
    typename G::Fetch fc[IPT];
    int re_c;
    Pack<V, ROW> rowv_c;
    prefetch(d0c, fc, re_c, rowv_c);
    FLEX_TICK(0);

    // A: row ends -> bitmap; row-aligned sources -> LDS (both prefetched for the first BLOCK rows)
    if (tid < R) {
      const int pos = (re_a - y0) + tid;
      atomicOr(&s_bits[buf][pos >> 5], 1u << (pos & 31));
    }
    for (int i = tid + BLOCK; i < R; i += BLOCK) {
      const int pos = (row_end[x0 + i] - y0) + i;
      atomicOr(&s_bits[buf][pos >> 5], 1u << (pos & 31));
    }
    if constexpr (ROW > 0) {
      if (tid <= R) {
#pragma unroll
        for (int c = 0; c < ROW; ++c) s_row[c * (TILE + 1) + tid] = rowv_a.v[c];
      }
      for (int i = tid + BLOCK; i <= R; i += BLOCK) {
        Pack<V, ROW> rv;
        G::load_row(p, min(x0 + i, last_row), rv);
#pragma unroll
        for (int c = 0; c < ROW; ++c) s_row[c * (TILE + 1) + i] = rv.v[c];
      }
    }
    FLEX_TICK(1);

    // D: map in coalesced order.  Without side effects it runs for every lane (slots past Z are
    // never read back as non-zeros); with stores or stage-1 aggregators it is predicated.
#pragma unroll
    for (int k = 0; k < IPT; ++k) {
      const int j = k * BLOCK + tid;
      if (G::STAGE1_PURE || j < Z) {
        Pack<V, XCH> xv;
        G::stage1(p, y0 + j, fa[k], ga[k], xv, agg);
#pragma unroll
        for (int c = 0; c < XCH; ++c) s_xch[c * TILE + j] = xv.v[c];
      }
    }
    FLEX_TICK(2);
#ifndef FLEX_ABLATE_NO_WALK  // tuning switch: stop after the map (measures the memory side alone)
    __syncthreads();
    FLEX_TICK(3);

    // E: exclusive prefix of the bitmap's per-word popcounts; clear the other bitmap for the next tile
    if (wave == 0) {
      int cnt[1] = {lane < NWORDS ? (int)__popc(s_bits[buf][lane < NWORDS ? lane : 0]) : 0};
      const int own = cnt[0];
      wave_segmented_inclusive_sum<int, 1>(0, cnt);
      if (lane < NWORDS) {
        s_word_prefix[lane] = cnt[0] - own;
        s_bits[buf ^ 1][lane] = 0u;
      }
    }
    __syncthreads();
    FLEX_TICK(4);

    // F: this thread's IPT merge items
    const int tile_items = R + Z;
    const int d0 = tid * IPT;
    const int n_items = max(0, min(IPT, tile_items - d0));
    const unsigned word = s_bits[buf][d0 >> 5];
    const int sh = d0 & 31;
    constexpr unsigned FULL = (IPT == 32) ? 0xffffffffu : ((1u << IPT) - 1u);
    const unsigned ends = (word >> sh) & FULL;                                        // items that are row ends
    const unsigned nzs = ~ends & (n_items >= IPT ? FULL : ((1u << n_items) - 1u));  // ... that are non-zeros
    const int xs = s_word_prefix[d0 >> 5] + __popc(word & ((1u << sh) - 1u));        // rows before my items
    const int ys = d0 - xs;                                                            // non-zeros before them
    const bool direct = R > OUT_CAP;  // (rare) more rows than the LDS output buffer holds: store directly

    Pack<V, XCH> xv[IPT];
    Pack<V, ROW> rvs[IPT];
    int xrel[IPT];
#pragma unroll
    for (int it = 0; it < IPT; ++it) {
      const int before = __popc(ends & ((1u << it) - 1u));
      xrel[it] = xs + before;
      const int yi = ys + it - before;  // < TILE by construction
#pragma unroll
      for (int c = 0; c < XCH; ++c) xv[it].v[c] = s_xch[c * TILE + yi];
      if constexpr (ROW > 0) {
#pragma unroll
        for (int c = 0; c < ROW; ++c) rvs[it].v[c] = s_row[c * (TILE + 1) + xrel[it]];
      }
    }

    Pack<V, RED> tot;
    zero(tot);
    const int dump = OUT_CAP + lane;
#pragma unroll
    for (int it = 0; it < IPT; ++it) {
      const bool nz = (nzs >> it) & 1u;
      const bool end = (ends >> it) & 1u;
      Pack<V, RED> dt;
      Pack<V, AGG> da;
      if constexpr (G::STAGE2_PURE) {
        // the contribution of a non-zero is computed for every item and masked in
        G::contrib(p, y0 + ys + it - (xrel[it] - xs), x0 + xrel[it], xv[it], rvs[it], dt, da);
#pragma unroll
        for (int c = 0; c < RED; ++c) tot.v[c] += nz ? dt.v[c] : V(0);
#pragma unroll
        for (int c = 0; c < AGG; ++c)
          if ((G::AGG2_MASK >> c) & 1u) agg.v[c] += nz ? da.v[c] : V(0);
      } else {
        if (nz) {
          G::contrib(p, y0 + ys + it - (xrel[it] - xs), x0 + xrel[it], xv[it], rvs[it], dt, da);
#pragma unroll
          for (int c = 0; c < RED; ++c) tot.v[c] += dt.v[c];
#pragma unroll
          for (int c = 0; c < AGG; ++c)
            if ((G::AGG2_MASK >> c) & 1u) agg.v[c] += da.v[c];
        }
      }
      // a row end parks the finished total in the output buffer (other items write a dump slot)
      if (!direct) {
        const int slot = end ? xrel[it] : dump;
#pragma unroll
        for (int c = 0; c < RED; ++c) s_out[c * OUT_STRIDE + slot] = tot.v[c];
      } else if (end) {
        G::store_row(p, x0 + xrel[it], tot);
      }
#pragma unroll
      for (int c = 0; c < RED; ++c) tot.v[c] = end ? V(0) : tot.v[c];
    }

    FLEX_TICK(5);
    // G: block-wide segmented scan of the open totals, keyed by the row each thread ended in
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
    FLEX_TICK(6);
    __syncthreads();
    FLEX_TICK(7);

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
      if (!direct) {
#pragma unroll
        for (int c = 0; c < RED; ++c) s_out[c * OUT_STRIDE + xs] += in_val[c];
      } else {
        Pack<V, RED> cin;
#pragma unroll
        for (int c = 0; c < RED; ++c) cin.v[c] = in_val[c];
        G::add_row(p, x0 + xs, cin);
      }
    }
    // tile carry-out: what the tile accumulated for the row still open at its end
    if (tid == BLOCK - 1) {
      if (key == pk) {
#pragma unroll
        for (int c = 0; c < RED; ++c) run[c] += pv[c];
      }
      const int row = x0 + key;
      carry_row[tile] = (row < num_rows) ? row : -1;
#pragma unroll
      for (int c = 0; c < RED; ++c) carry_val[(size_t)tile * RED + c] = run[c];
    }
    FLEX_TICK(8);
    __syncthreads();
    FLEX_TICK(9);

    // H: the tile's finished rows leave LDS as coalesced stores
    if (!direct) {
      for (int i = tid; i < R; i += BLOCK) {
        Pack<V, RED> t;
#pragma unroll
        for (int c = 0; c < RED; ++c) t.v[c] = s_out[c * OUT_STRIDE + i];
        G::store_row(p, x0 + i, t);
      }
    }

    FLEX_TICK(10);
#endif
    // rotate the pipeline
    c0 = b0; c1 = b1;
    b0 = d0c; b1 = d1c;
    d0c = e0; d1c = e1;
#pragma unroll
    for (int k = 0; k < IPT; ++k) {
      fa[k] = fb[k];
      ga[k] = gb[k];
      fb[k] = fc[k];
    }
    re_a = re_b;
    rowv_a = rowv_b;
    re_b = re_c;
    rowv_b = rowv_c;
  }

  FLEX_TICK_FLUSH;
  // one aggregator partial per block
  if constexpr (AGG > 0) {
    wave_sum_to_last_lane<V, AGG>(agg.v);
    if (lane == WAVE - 1) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) s_wave_agg[wave][c] = agg.v[c];
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
        Pack<V, G::XCH_WIDTH> unused;
        G::stage1(p, (int)e, f[k], g[k], unused, agg);
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
// Fix-up: fold tile carries into their rows (tile order) and finish the aggregators (fixed order).
// Blocks [0, carry_blocks) handle carries, the last block sums the aggregator partials.
// ----------------------------------------------------------------------------------------------
template <class G, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
fixup_kernel(const typename G::Params p, const int num_tiles, const int carry_blocks,
             const int* __restrict__ carry_row, const typename G::Value* __restrict__ carry_val,
             const typename G::Value* __restrict__ agg_partials, const int num_partials) {
  using V = typename G::Value;
  constexpr int RED = G::RED_WIDTH, AGG = G::AGG_WIDTH;
  constexpr int NW = BLOCK / WAVE;
  if ((int)blockIdx.x < carry_blocks) {
    if constexpr (RED > 0) {
      const int t = blockIdx.x * BLOCK + threadIdx.x;
      if (t >= num_tiles) return;
      const int row = carry_row[t];
      if (row < 0) return;
      if (t > 0 && carry_row[t - 1] == row) return;  // not the first tile of this row's run
      Pack<V, RED> sum;
#pragma unroll
      for (int c = 0; c < RED; ++c) sum.v[c] = carry_val[(size_t)t * RED + c];
      for (int u = t + 1; u < num_tiles && carry_row[u] == row; ++u) {
#pragma unroll
        for (int c = 0; c < RED; ++c) sum.v[c] += carry_val[(size_t)u * RED + c];
      }
      G::add_row(p, row, sum);
    }
    return;
  }
  if constexpr (AGG > 0) {
    __shared__ V s_wave_agg[NW][AGG];
    Pack<V, AGG> acc;
    zero(acc);
    for (int j = threadIdx.x; j < num_partials; j += BLOCK) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) acc.v[c] += agg_partials[(size_t)j * AGG + c];
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
