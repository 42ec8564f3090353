// Reducer kernel for launches that keep the most-gathered rows of the gather source in LDS.
//
// A power-law matrix gathers from a few thousand columns most of the time (R-MAT scale 22: 30 720 of 4.2 M
// columns hold 52 % of the non-zeros) and from everywhere else the rest of the time.  A 4-byte gather that
// misses the vector L1 is one request to the L2 whatever it brings back, and the L2s serve about 0.2 T
// requests per second: the reducer of flex_agent.hpp spends two thirds of its time there.  Here the caller
// names the hot rows once (index arrays re-encoded by flexspmv_encode_hot_rows: entry ~i stands for hot row
// i), a small kernel copies them into a table per launch, and every block keeps that table in LDS, where a
// gather costs an LDS read instead of an L2 request.
//
// The table only pays for itself when a block lives long enough to amortise loading it, so this kernel is
// persistent: one block of WAVES wavefronts per CU, and - because a block that owns a whole CU cannot hide
// its barriers behind other blocks - no barriers after the table is loaded: every wavefront walks its own
// merge tiles of 64 x IPT items (wave tile t, t + number of wavefronts, ...) with the machinery of the
// block-wide merge path (row-end bitmap, popcount instead of a diagonal search, register walk, DPP segmented
// scan) cut down to one wavefront, whose LDS traffic needs no barrier.  Every wave tile leaves a carry
// record; fixup_kernel folds them as it folds the block tiles' records.
//
// Graphs: the map must not depend on row-aligned sources (it runs in coalesced edge order before the walk)
// and must gather one source through one selector (G::HOT_DIM > 0).
#pragma once
#include "flex_agent.hpp"

namespace flex {

constexpr int CU_LDS_BYTES = 160 * 1024;  // gfx950

// table[i] = source row hot_rows[i]
template <class G>
__global__ void __launch_bounds__(256)
hot_fill_kernel(const typename G::Params p, const int* __restrict__ hot_rows, const int num_hot,
                typename G::Value* __restrict__ table) {
  constexpr int D = G::HOT_DIM > 0 ? G::HOT_DIM : 1;
  const int i = (int)(blockIdx.x * 256 + threadIdx.x);
  if (i >= num_hot) return;
  const typename G::Value* src = G::hot_source(p) + (size_t)hot_rows[i] * D;
#pragma unroll
  for (int d = 0; d < D; ++d) table[(size_t)i * D + d] = src[d];
}

template <class G, int WAVES, int IPT>
struct WaveTile {
  using V = typename G::Value;
  static constexpr int WTILE = WAVE * IPT;
  static constexpr int NWORDS = WTILE / 32;
  static constexpr int REDN = G::RED_WIDTH > 0 ? G::RED_WIDTH : 1;
  static constexpr int D = G::HOT_DIM > 0 ? G::HOT_DIM : 1;
  static constexpr int SLAB_ELEMS = REDN * (WTILE + WAVE);  // contributions, then finished rows + a dump slot per lane
  static constexpr size_t FIXED_BYTES = (size_t)WAVES * (SLAB_ELEMS * sizeof(V) + NWORDS * 4) + 256;
  // rows of the gather source a block can keep in LDS beside its wavefronts' buffers
  static constexpr int HOT_CAPACITY =
      (G::HOT_DIM > 0 && G::ROW_WIDTH == 0 && FIXED_BYTES < (size_t)CU_LDS_BYTES)
          ? (int)(((size_t)CU_LDS_BYTES - FIXED_BYTES) / (D * sizeof(V))) : 0;
  static_assert((IPT & (IPT - 1)) == 0 && IPT <= 32 && NWORDS <= WAVE, "a lane's items sit inside one bitmap word");
};

// The LDS unit performs the accesses of one wavefront in the order they were issued, so a lane reads what
// another lane of its wavefront wrote earlier in program order without any wait; this only keeps the compiler
// from moving memory operations across the point where that happens.  (A fence, even at wavefront scope, would
// also wait for every global load and store in flight - the prefetched edges of the next tile among them.)
__device__ __forceinline__ void wave_lds_sync() { __builtin_amdgcn_wave_barrier(); }

// Makes the compiler treat a value as used (and possibly changed) here: every 32-bit word goes through an
// empty asm statement.
template <typename T> __device__ __forceinline__ void keep_in_registers(T& t) {
  static_assert(sizeof(T) % 4 == 0, "whole registers");
  uint32_t w[sizeof(T) / 4];
  __builtin_memcpy(w, &t, sizeof(T));
#pragma unroll
  for (size_t i = 0; i < sizeof(T) / 4; ++i) asm volatile("" : "+v"(w[i]));
  __builtin_memcpy(&t, w, sizeof(T));
}

template <class G, int WAVES, int IPT>
__global__ void __launch_bounds__(WAVES * WAVE)
wave_reduce_kernel(const int2* __restrict__ coords, const int num_tiles, const int num_rows, const int* __restrict__ row_end,
                   const int nnz, const typename G::Params p, int* __restrict__ carry_row,
                   typename G::Value* __restrict__ carry_val, typename G::Value* __restrict__ wave_partials,
                   const typename G::Value* __restrict__ hot_table, const int num_hot) {
  using V = typename G::Value;
  using Fetch = typename G::Fetch;
  using Gather = typename G::Gather;
  using WT = WaveTile<G, WAVES, IPT>;
  constexpr int WTILE = WT::WTILE, NWORDS = WT::NWORDS, D = WT::D;
  constexpr int RED = G::RED_WIDTH, AGG = G::AGG_WIDTH, REDN = WT::REDN;
  constexpr int HOT_ELEMS = WT::HOT_CAPACITY > 0 ? WT::HOT_CAPACITY * D : 1;
  constexpr int DUMP_AT = REDN * WTILE;
  static_assert(G::ROW_WIDTH == 0, "the map runs before the rows of the edges are known");

  __shared__ __attribute__((aligned(16))) V s_hot[HOT_ELEMS];
  __shared__ __attribute__((aligned(16))) V s_slab[WAVES][WT::SLAB_ELEMS];
  __shared__ unsigned s_bits[WAVES][NWORDS];

  const int lane = (int)threadIdx.x & (WAVE - 1);
  const int wave = (int)threadIdx.x / WAVE;
  const int num_lds = min(num_hot, WT::HOT_CAPACITY);  // table rows kept in LDS; the others are read from the table
  // the table, 16 bytes per lane and eight loads in flight per thread (the scratch it comes from is 256-byte
  // aligned and sized for the full capacity: whole vectors may be read beyond num_hot rows)
  {
    constexpr int VEC = 16 / (int)sizeof(V), UNROLL = 8;
    using Vec = __attribute__((ext_vector_type(4))) unsigned;
    const Vec* src = reinterpret_cast<const Vec*>(hot_table);
    Vec* dst = reinterpret_cast<Vec*>(s_hot);
    const int vecs = min((num_lds * D + VEC - 1) / VEC, HOT_ELEMS / VEC);
    for (int base = 0; base < vecs; base += UNROLL * WAVES * WAVE) {
      Vec v[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int i = base + u * WAVES * WAVE + (int)threadIdx.x;
        v[u] = src[min(i, vecs - 1)];
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int i = base + u * WAVES * WAVE + (int)threadIdx.x;
        if (i < vecs) dst[i] = v[u];
      }
    }
  }
  __syncthreads();  // the only barrier: from here on every wavefront is on its own

  V* const slab = s_slab[wave];
  unsigned* const bits = s_bits[wave];
  const int first = (int)blockIdx.x * WAVES + wave;
  const int stride = (int)gridDim.x * WAVES;
  const int last_edge = nnz - 1;
  Pack<V, AGG> agg;
  zero(agg);
  const Pack<V, 0> no_row{};

  // Software pipeline: the edges of a wavefront's next tile are on their way while it works on the current
  // one (a wavefront that owns a sixteenth of a CU has no neighbours to hide its round trips behind).
  // The coordinates of a wavefront's tiles are fetched 64 tiles at a time, one tile per lane, and handed out
  // by lane: no round trip for them inside the loop.
  int2 batch_c0 = make_int2(0, 0), batch_c1 = make_int2(0, 0);
  auto load_batch = [&](const int batch) {
    const long long t = (long long)first + ((long long)batch * WAVE + lane) * stride;
    const int tc = (int)min(t, (long long)num_tiles - 1);
    batch_c0 = coords[tc];
    batch_c1 = coords[tc + 1];
  };
  struct TileAt {
    int x0, y0, R, Z;  // uniform
    int re0;           // end of tile row `lane`
  };
  auto tile_coords = [&](const int iter, TileAt& t) {
    const int k = iter & (WAVE - 1);
    t.x0 = __builtin_amdgcn_readlane(batch_c0.x, k);
    t.y0 = __builtin_amdgcn_readlane(batch_c0.y, k);
    t.R = __builtin_amdgcn_readlane(batch_c1.x, k) - t.x0;  // row ends inside the tile
    t.Z = __builtin_amdgcn_readlane(batch_c1.y, k) - t.y0;  // non-zeros inside the tile
  };
  // first-level loads in coalesced order; lanes past Z re-read the tile's last edge
  auto tile_loads = [&](TileAt& t, Fetch (&f)[IPT]) {
    const int e_last = min(t.y0 + max(t.Z - 1, 0), last_edge);
#pragma unroll
    for (int k = 0; k < IPT; ++k) G::fetch(p, min(t.y0 + k * WAVE + lane, e_last), f[k]);
    t.re0 = row_end[min(t.x0 + lane, num_rows - 1)];
  };
  const int my_tiles = first < num_tiles ? (num_tiles - first + stride - 1) / stride : 0;
  auto clamp_iter = [&](const int i) { return i < my_tiles ? i : my_tiles - 1; };  // past the end: the last tile again

  // One step reduces a tile.  Three tiles are under way per wavefront meanwhile: this one (its edges and its
  // gathers from memory have arrived), the next one (edges arrived; its gathers are issued first thing and have
  // the whole step to come back) and the one after (its edges are requested as soon as the map has used up this
  // tile's, and have the walk to come back).  Two sets of registers take turns (the loop below calls the step
  // with the sets swapped): nothing is copied from one set to another, which would have to wait for the data.
  auto step = [&](const int iter, TileAt& tX, Fetch (&fX)[IPT], Gather (&cX)[IPT], TileAt& tY, Fetch (&fY)[IPT],
                  Gather (&cY)[IPT]) {
    const int tile = first + iter * stride;
#pragma unroll
    for (int k = 0; k < IPT; ++k) G::gather_cold(p, fY[k], hot_table, num_lds, cY[k]);

    // the map, in coalesced edge order; contributions go to the slab
    const int x0 = tX.x0, y0 = tX.y0, R = tX.R, Z = tX.Z, re0 = tX.re0;
    if (lane < NWORDS) bits[lane] = 0u;
    {
      Gather g[IPT], g_table[IPT];
#pragma unroll
      for (int k = 0; k < IPT; ++k) G::gather_table(fX[k], (typename G::HotTablePtr)s_hot, num_lds, g_table[k]);
      // what the loads brought back is used from here on (and the compiler may not turn the selection below
      // into a branch around either load)
#pragma unroll
      for (int k = 0; k < IPT; ++k) {
        keep_in_registers(cX[k]);
        keep_in_registers(g_table[k]);
      }
#pragma unroll
      for (int k = 0; k < IPT; ++k) G::pick_hot(fX[k], num_lds, cX[k], g_table[k], g[k]);
#pragma unroll
      for (int k = 0; k < IPT; ++k) {
        const int j = k * WAVE + lane;
        if (G::EDGE_PURE || j < Z) {
          Pack<V, RED> dt;
          Pack<V, AGG> da;
          G::edge(p, y0 + j, fX[k], g[k], no_row, dt, da);
#pragma unroll
          for (int c = 0; c < RED; ++c) slab[c * WTILE + j] = dt.v[c];
#pragma unroll
          for (int c = 0; c < AGG; ++c) agg.v[c] += (j < Z) ? da.v[c] : V(0);
        }
      }
    }
    // this tile's edges are used up: their registers take the edges of the tile after next
    {
      const int i2 = clamp_iter(iter + 2);
      if ((i2 & (WAVE - 1)) == 0 && i2 == iter + 2) load_batch(i2 / WAVE);  // (lanes of earlier tiles are not needed again)
      tile_coords(i2, tX);
      tile_loads(tX, fX);
    }

    // row ends -> bitmap over merge positions
    if (lane < R) {
      const int pos = (re0 - y0) + lane;
      atomicOr(&bits[pos >> 5], 1u << (pos & 31));
    }
    // tiles of mostly empty rows have hundreds of row ends: four loads in flight per lane
    for (int base = WAVE; base < R; base += 4 * WAVE) {
      int ends4[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) ends4[u] = row_end[x0 + min(base + u * WAVE + lane, R - 1)];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = base + u * WAVE + lane;
        if (i < R) {
          const int pos = (ends4[u] - y0) + i;
          atomicOr(&bits[pos >> 5], 1u << (pos & 31));
        }
      }
    }
    wave_lds_sync();

    unsigned word;
    int word_prefix;
    {
      const unsigned my_word = bits[lane < NWORDS ? lane : 0];
      int cnt[1] = {lane < NWORDS ? (int)__popc(my_word) : 0};
      const int own = cnt[0];
      wave_segmented_inclusive_sum<int, 1>(0, cnt);
      const int src_lane = (lane * IPT) >> 5;
      word = (unsigned)__builtin_amdgcn_ds_bpermute(src_lane << 2, (int)my_word);
      word_prefix = __builtin_amdgcn_ds_bpermute(src_lane << 2, cnt[0] - own);
    }
    const int tile_items = R + Z;
    const int d0 = lane * IPT;
    const int n_items = max(0, min(IPT, tile_items - d0));
    const int sh = d0 & 31;
    constexpr unsigned FULL = (IPT == 32) ? 0xffffffffu : ((1u << IPT) - 1u);
    const unsigned ends = (word >> sh) & FULL;
    const unsigned nzs = ~ends & (n_items >= IPT ? FULL : ((1u << n_items) - 1u));
    const int xs = word_prefix + __popc(word & ((1u << sh) - 1u));  // rows before my items
    const int ys = d0 - xs;                                          // non-zeros before them

    Pack<V, RED> xv[IPT];
    int xrel[IPT];
#pragma unroll
    for (int it = 0; it < IPT; ++it) {
      const int before = __popc(ends & ((1u << it) - 1u));
      xrel[it] = xs + before;
      const int yi = min(ys + it - before, WTILE - 1);
#pragma unroll
      for (int c = 0; c < RED; ++c) xv[it].v[c] = slab[c * WTILE + yi];
    }
    wave_lds_sync();  // every lane has its items: the slab now takes the finished rows

    Pack<V, RED> tot;
    zero(tot);
#pragma unroll
    for (int it = 0; it < IPT; ++it) {
      const bool nz = (nzs >> it) & 1u;
      const bool end = (ends >> it) & 1u;
#pragma unroll
      for (int c = 0; c < RED; ++c) tot.v[c] += nz ? xv[it].v[c] : V(0);
#pragma unroll
      for (int c = 0; c < RED; ++c) slab[end ? c * WTILE + xrel[it] : DUMP_AT + c * WAVE + lane] = tot.v[c];
#pragma unroll
      for (int c = 0; c < RED; ++c) tot.v[c] = end ? V(0) : tot.v[c];
    }

    // segmented scan of the open totals, keyed by the row each lane ended in
    const int key = xs + __popc(ends);
    V run[REDN];
#pragma unroll
    for (int c = 0; c < RED; ++c) run[c] = tot.v[c];
    wave_segmented_inclusive_sum<V, REDN>(key, run);
    const int in_key = wave_shift_up1<int>(key, -1);
    V in_val[REDN];
#pragma unroll
    for (int c = 0; c < RED; ++c) in_val[c] = wave_shift_up1<V>(run[c], V(0));
    // the first row a lane closed may have started in earlier lanes (only this lane touches that row's slot)
    if (ends != 0u && in_key == xs) {
#pragma unroll
      for (int c = 0; c < RED; ++c) slab[c * WTILE + xs] += in_val[c];
    }
    // carry-out: what the tile accumulated for the row still open at its end
    if (lane == WAVE - 1) {
      const int last_item = tile_items - 1;
      const bool open_empty = Z == 0 || (R > 0 && ((bits[last_item >> 5] >> (last_item & 31)) & 1u) != 0u);
      const int row = x0 + key;
      carry_row[tile] = (row < num_rows && !open_empty) ? row : -1;
#pragma unroll
      for (int c = 0; c < RED; ++c) carry_val[(size_t)tile * RED + c] = run[c];
    }
    wave_lds_sync();

    // the tile's finished rows leave LDS as coalesced stores
    for (int i = lane; i < R; i += WAVE) {
      Pack<V, RED> t;
#pragma unroll
      for (int c = 0; c < RED; ++c) t.v[c] = slab[c * WTILE + i];
      G::store_row(p, x0 + i, t);
    }
    wave_lds_sync();  // before the next tile reuses slab and bitmap
  };

  if (my_tiles > 0) {
    TileAt tA{0, 0, 0, 0, 0}, tB{0, 0, 0, 0, 0};
    Fetch fA[IPT], fB[IPT];
    Gather cA[IPT], cB[IPT];
    load_batch(0);
    tile_coords(0, tA);
    tile_loads(tA, fA);
#pragma unroll
    for (int k = 0; k < IPT; ++k) G::gather_cold(p, fA[k], hot_table, num_lds, cA[k]);
    tile_coords(clamp_iter(1), tB);
    tile_loads(tB, fB);
#pragma unroll 1
    for (int iter = 0; iter < my_tiles; iter += 2) {
      step(iter, tA, fA, cA, tB, fB, cB);
      if (iter + 1 < my_tiles) step(iter + 1, tB, fB, cB, tA, fA, cA);
    }
  }

  // one aggregator partial per wavefront of the grid (also from wavefronts that had no tile)
  if constexpr (AGG > 0) {
    wave_sum_to_last_lane<V, AGG>(agg.v);
    if (lane == WAVE - 1) {
#pragma unroll
      for (int c = 0; c < AGG; ++c) wave_partials[(size_t)first * AGG + c] = agg.v[c];
    }
  }
}

}  // namespace flex
