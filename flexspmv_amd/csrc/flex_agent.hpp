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

// Which tile a block works on: block b runs on XCD b % 8, and XCD k owns tiles [k*per, (k+1)*per).
__device__ __forceinline__ int tile_of_block(int block, int num_tiles) {
  const int per = (num_tiles + NUM_XCD - 1) / NUM_XCD;
  return (block % NUM_XCD) * per + block / NUM_XCD;
}
inline int grid_for_tiles(int num_tiles) {
  const int per = (num_tiles + NUM_XCD - 1) / NUM_XCD;
  return per * NUM_XCD;
}

// ----------------------------------------------------------------------------------------------
// Reducer kernel: one block per merge tile of BLOCK*IPT merge items (row ends + non-zeros).
// ----------------------------------------------------------------------------------------------
template <class G, int BLOCK, int IPT>
__global__ void __launch_bounds__(BLOCK)
reduce_kernel(const typename G::Params p, const int* __restrict__ row_end, const int num_rows, const int nnz,
              const int2* __restrict__ coords, const int num_tiles, int* __restrict__ carry_row,
              typename G::Value* __restrict__ carry_val, typename G::Value* __restrict__ agg_partials) {
  using V = typename G::Value;
  constexpr int TILE = BLOCK * IPT;
  constexpr int NW = BLOCK / WAVE;
  constexpr int XCH = G::XCH_WIDTH, RED = G::RED_WIDTH, AGG = G::AGG_WIDTH, ROW = G::ROW_WIDTH;

  __shared__ int s_row_end[TILE + 1];
  __shared__ V s_xch[(XCH > 0 ? XCH : 1) * TILE];
  __shared__ V s_row[(ROW > 0 ? ROW * (TILE + 1) : 1)];
  __shared__ int s_wave_key[NW];
  __shared__ V s_wave_val[NW][RED > 0 ? RED : 1];
  __shared__ V s_wave_agg[NW][AGG > 0 ? AGG : 1];

  const int tile = tile_of_block(blockIdx.x, num_tiles);
  if (tile >= num_tiles) return;
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;

  const int2 c0 = coords[tile];
  const int2 c1 = coords[tile + 1];
  const int x0 = c0.x, y0 = c0.y;
  const int R = c1.x - c0.x;  // row ends inside this tile
  const int Z = c1.y - c0.y;  // non-zeros inside this tile

  // Row-end offsets of the tile's rows (plus the open row that follows) into LDS.
  for (int i = tid; i <= R; i += BLOCK) {
    const int r = min(x0 + i, num_rows - 1);
    s_row_end[i] = row_end[r];
    if constexpr (ROW > 0) {
      Pack<V, ROW> rv;
      G::load_row(p, r, rv);
#pragma unroll
      for (int c = 0; c < ROW; ++c) s_row[c * (TILE + 1) + i] = rv.v[c];
    }
  }

  // Stage 1: selector + map in coalesced edge order; values the walk needs go through LDS.
  Pack<V, AGG> agg;
  zero(agg);
#pragma unroll
  for (int k = 0; k < IPT; ++k) {
    const int j = k * BLOCK + tid;
    if (j < Z) {
      Pack<V, XCH> xv;
      G::stage1(p, y0 + j, xv, agg);
#pragma unroll
      for (int c = 0; c < XCH; ++c) s_xch[c * TILE + j] = xv.v[c];
    }
  }
  __syncthreads();

  // Each thread owns IPT consecutive merge items; find where they start (diagonal search in LDS).
  const int tile_items = R + Z;
  const int d0 = min(tid * IPT, tile_items);
  const int n_items = min(IPT, tile_items - d0);
  int x, y;
  {
    int lo = max(d0 - Z, 0), hi = min(d0, R);
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (s_row_end[mid] <= y0 + d0 - mid - 1) lo = mid + 1;
      else hi = mid;
    }
    x = lo;
    y = d0 - lo;
  }

  // Walk the merge path: a non-zero adds to the running total, a row end emits the total.
  Pack<V, RED> tot, head;
  zero(tot);
  zero(head);
  bool have_head = false;
  int head_row = 0;
  int cur_end = s_row_end[x];
  Pack<V, ROW> rv;
  if constexpr (ROW > 0) {
#pragma unroll
    for (int c = 0; c < ROW; ++c) rv.v[c] = s_row[c * (TILE + 1) + x];
  }
#pragma unroll
  for (int it = 0; it < IPT; ++it) {
    if (it < n_items) {
      if (y0 + y < cur_end) {
        Pack<V, XCH> xv;
#pragma unroll
        for (int c = 0; c < XCH; ++c) xv.v[c] = s_xch[c * TILE + y];
        G::stage2(p, y0 + y, x0 + x, xv, rv, tot, agg);
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
        cur_end = s_row_end[x];
        if constexpr (ROW > 0) {
#pragma unroll
          for (int c = 0; c < ROW; ++c) rv.v[c] = s_row[c * (TILE + 1) + x];
        }
      }
    }
  }

  // Block-wide segmented scan of the open totals, keyed by the row each thread ended in.
  const int key = x;
  V run[RED > 0 ? RED : 1];
#pragma unroll
  for (int c = 0; c < RED; ++c) run[c] = tot.v[c];
  wave_segmented_inclusive_sum<V, (RED > 0 ? RED : 1)>(key, run);
  int in_key = wave_shift_up1<int>(key, -1);
  V in_val[RED > 0 ? RED : 1];
#pragma unroll
  for (int c = 0; c < RED; ++c) in_val[c] = wave_shift_up1<V>(run[c], V(0));

  if constexpr (AGG > 0) wave_sum_to_last_lane<V, AGG>(agg.v);
  if (lane == WAVE - 1) {
    s_wave_key[wave] = key;
#pragma unroll
    for (int c = 0; c < RED; ++c) s_wave_val[wave][c] = run[c];
#pragma unroll
    for (int c = 0; c < AGG; ++c) s_wave_agg[wave][c] = agg.v[c];
  }
  __syncthreads();

  // Fold the totals of the waves in front of this one.
  int pk = -1;
  V pv[RED > 0 ? RED : 1];
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

  // The first row a thread closes may have started in earlier threads: add what they carried in.
  if (have_head) {
    if (in_key + x0 == head_row) {
#pragma unroll
      for (int c = 0; c < RED; ++c) head.v[c] += in_val[c];
    }
    G::store_row(p, head_row, head);
  }

  // Tile carry-out: what the tile accumulated for the row that is still open at its end.
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
  if constexpr (AGG > 0) {
    if (tid == 0) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) {
        V s = s_wave_agg[0][c];
        for (int w = 1; w < NW; ++w) s += s_wave_agg[w][c];
        agg_partials[(size_t)tile * AGG + c] = s;
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
  for (int tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
    const long long base = (long long)tile * TILE;
#pragma unroll
    for (int k = 0; k < IPT; ++k) {
      const long long e = base + k * BLOCK + tid;
      if (e < nnz) {
        Pack<V, G::XCH_WIDTH> unused;
        G::stage1(p, (int)e, unused, agg);
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
