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

template <typename V, int N> struct Pack { V v[N > 0 ? N : 1]; };

template <typename V, int N> __device__ __forceinline__ void zero(Pack<V, N>& a) {
#pragma unroll
  for (int i = 0; i < N; ++i) a.v[i] = V(0);
}

// Streaming (read-once) loads and write-once stores bypass temporal caching so that gathered vertex
// data, not the edge stream, occupies L2.
template <typename T> __device__ __forceinline__ T stream_load(const T* p) { return __builtin_nontemporal_load(p); }
template <typename T> __device__ __forceinline__ void stream_store(T* p, T v) { __builtin_nontemporal_store(v, p); }

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
  w.tile = xcd * per + block / NUM_XCD;
  w.end = min((xcd + 1) * per, num_tiles);
  w.step = slots;
  return w;
}

// ----------------------------------------------------------------------------------------------
// Reducer kernel.  Persistent blocks; each iteration consumes one merge tile of BLOCK*IPT merge
// items (row ends + non-zeros):
//   A  row-end offsets of the tile's rows become a bitmap over merge positions in LDS
//      (row i ends at merge position (row_end[i] - y0) + i); row-aligned vertex data is staged in LDS
//   B  second-level loads (gathers) of the current tile are issued from the prefetched first level
//   C  first-level loads (edge tensors, index arrays) of the block's NEXT tile are issued, so they are
//      in flight during everything below
//   D  the map runs in coalesced edge order; values needed per row go to LDS
//   E  one wavefront turns the bitmap into per-word prefix counts
//   F  each thread owns IPT consecutive merge items: its bitmap bits say which are row ends, a
//      popcount gives its merge coordinate (the result of the per-thread diagonal search of the
//      reference, cuda_template/reducer/merged_agent_spmv_template.cuh:196-215, without a search),
//      so all its LDS reads are independent; it walks them in registers
//   G  wave64 DPP segmented scan of the threads' open totals, then a fold across waves
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
  static_assert((IPT & (IPT - 1)) == 0 && IPT <= 32, "a thread's items must sit inside one bitmap word");
  static_assert(NWORDS <= WAVE, "one wavefront scans the bitmap words");

  __shared__ V s_xch[(XCH > 0 ? XCH : 1) * TILE];
  __shared__ V s_row[(ROW > 0 ? ROW * (TILE + 1) : 1)];
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

  // prologue: first-level loads of the first tile.  Loads are never put under a branch (that would
  // serialise them behind a wait each): out-of-range lanes re-read the last valid edge instead.
  typename G::Fetch cur[IPT];
  int2 c0 = coords[tw.tile];
  int2 c1 = coords[tw.tile + 1];
  const int last_edge = nnz - 1;
#pragma unroll
  for (int k = 0; k < IPT; ++k) G::fetch(p, min(c0.y + k * BLOCK + tid, last_edge), cur[k]);
  // ... and of its rows: thread i holds row c0.x + i (tiles with more than BLOCK rows finish in a loop)
  const int last_row = num_rows - 1;
  int re_cur = row_end[min(c0.x + tid, last_row)];
  Pack<V, ROW> rowv_cur;
  if constexpr (ROW > 0) G::load_row(p, min(c0.x + tid, last_row), rowv_cur);

  int buf = 0;
  for (int tile = tw.tile; tile < tw.end; tile += tw.step, buf ^= 1) {
    const int x0 = c0.x, y0 = c0.y;
    const int R = c1.x - c0.x;  // row ends inside this tile
    const int Z = c1.y - c0.y;  // non-zeros inside this tile
    const int next = tile + tw.step;
    const int2 n0 = coords[min(next, num_tiles)];
    const int2 n1 = coords[min(next + 1, num_tiles)];

    // A: row ends -> bitmap; row-aligned sources -> LDS (both prefetched for the first BLOCK rows)
    if (tid < R) {
      const int pos = (re_cur - y0) + tid;
      atomicOr(&s_bits[buf][pos >> 5], 1u << (pos & 31));
    }
    for (int i = tid + BLOCK; i < R; i += BLOCK) {
      const int pos = (row_end[x0 + i] - y0) + i;
      atomicOr(&s_bits[buf][pos >> 5], 1u << (pos & 31));
    }
    if constexpr (ROW > 0) {
      if (tid <= R) {
#pragma unroll
        for (int c = 0; c < ROW; ++c) s_row[c * (TILE + 1) + tid] = rowv_cur.v[c];
      }
      for (int i = tid + BLOCK; i <= R; i += BLOCK) {
        Pack<V, ROW> rv;
        G::load_row(p, min(x0 + i, last_row), rv);
#pragma unroll
        for (int c = 0; c < ROW; ++c) s_row[c * (TILE + 1) + i] = rv.v[c];
      }
    }

    // B: gathers of this tile
    typename G::Gather gat[IPT];
#pragma unroll
    for (int k = 0; k < IPT; ++k) G::gather(p, cur[k], gat[k]);

    // C: first-level loads of the next tile (of the path's end when there is none)
    typename G::Fetch nxt[IPT];
#pragma unroll
    for (int k = 0; k < IPT; ++k) G::fetch(p, min(n0.y + k * BLOCK + tid, last_edge), nxt[k]);
    const int re_nxt = row_end[min(n0.x + tid, last_row)];
    Pack<V, ROW> rowv_nxt;
    if constexpr (ROW > 0) G::load_row(p, min(n0.x + tid, last_row), rowv_nxt);

    // D: map in coalesced order
#pragma unroll
    for (int k = 0; k < IPT; ++k) {
      const int j = k * BLOCK + tid;
      if (j < Z) {
        Pack<V, XCH> xv;
        G::stage1(p, y0 + j, cur[k], gat[k], xv, agg);
#pragma unroll
        for (int c = 0; c < XCH; ++c) s_xch[c * TILE + j] = xv.v[c];
      }
    }
    __syncthreads();

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

    // F: this thread's IPT merge items
    const int tile_items = R + Z;
    const int d0 = tid * IPT;
    const int n_items = max(0, min(IPT, tile_items - d0));
    const unsigned word = s_bits[buf][d0 >> 5];
    const int sh = d0 & 31;
    const unsigned mine = (word >> sh) & ((IPT == 32) ? 0xffffffffu : ((1u << IPT) - 1u));
    const int xs = s_word_prefix[d0 >> 5] + __popc(word & ((1u << sh) - 1u));  // rows before my items
    const int ys = d0 - xs;                                                      // non-zeros before them

    Pack<V, XCH> xv[IPT];
    Pack<V, ROW> rvs[IPT];
#pragma unroll
    for (int it = 0; it < IPT; ++it) {
      const int before = __popc(mine & ((1u << it) - 1u));
      const int yi = min(ys + it - before, TILE - 1);
#pragma unroll
      for (int c = 0; c < XCH; ++c) xv[it].v[c] = s_xch[c * TILE + yi];
      if constexpr (ROW > 0) {
        const int xi = min(xs + before, TILE);
#pragma unroll
        for (int c = 0; c < ROW; ++c) rvs[it].v[c] = s_row[c * (TILE + 1) + xi];
      }
    }

    Pack<V, RED> tot, head;
    zero(tot);
    zero(head);
    bool have_head = false;
    int head_row = 0;
    int x = xs, y = ys;
#pragma unroll
    for (int it = 0; it < IPT; ++it) {
      if (it < n_items) {
        if (!((mine >> it) & 1u)) {
          G::stage2(p, y0 + y, x0 + x, xv[it], rvs[it], tot, agg);
          ++y;
        } else {
          if (!have_head) {
            have_head = true;
            head_row = x0 + x;
            head = tot;
          } else {
            G::store_row(p, x0 + x, tot);
          }
          zero(tot);
          ++x;
        }
      }
    }

    // G: block-wide segmented scan of the open totals, keyed by the row each thread ended in
    const int key = x;
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
    for (int w = 0; w < wave; ++w) {
      const int k = s_wave_key[w];
#pragma unroll
      for (int c = 0; c < RED; ++c) pv[c] = (k == pk) ? static_cast<V>(pv[c] + s_wave_val[w][c]) : s_wave_val[w][c];
      pk = k;
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
    // the first row a thread closes may have started in earlier threads: add what they carried in
    if (have_head) {
      if (in_key + x0 == head_row) {
#pragma unroll
        for (int c = 0; c < RED; ++c) head.v[c] += in_val[c];
      }
      G::store_row(p, head_row, head);
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

    // rotate the pipeline
    c0 = n0;
    c1 = n1;
#pragma unroll
    for (int k = 0; k < IPT; ++k) cur[k] = nxt[k];
    re_cur = re_nxt;
    rowv_cur = rowv_nxt;
  }

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
