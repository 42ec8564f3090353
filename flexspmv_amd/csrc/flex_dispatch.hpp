// Host-side dispatch shared by every generated library: sizes the tiling, carves the workspace and
// launches the kernels of flex_agent.hpp on the caller's stream.
//
// Replaces the reference's merged_spmv_dispatch / merged_spmv_launch pair
// (cuda_template/reducer/merged_spmv_template.cuh:22-182): same responsibilities (tile count from
// num_rows + num_nonzeros, temp-storage carving, optional search kernel, the +1 shift that turns the
// CSR row pointer into row END offsets at :169), but one call instead of the size-query-then-run
// protocol, and the caller owns the scratch so nothing is allocated per launch.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <mutex>

#include "flex_agent.hpp"
#include "flexspmv.h"

// Scratch of flexspmv_launch_static: device memory that belongs to the library itself, so that entry point
// never allocates.  One copy exists on every GPU the library is loaded on, at its own address; host code
// reaches it only through the per-device pointer that static_scratch() resolves (the array's name is
// a host-side stand-in, not a device address).  File scope, internal linkage, and a name no generated
// identifier can take (those start with q_ or carry a graph's tensor names inside Graph<>).
static __device__ __align__(256) unsigned char flexspmv_static_scratch_bytes[FLEXSPMV_STATIC_SCRATCH_BYTES];

namespace flex {

inline thread_local char g_last_error[512] = "";
inline int fail(int code, const char* msg) {
  snprintf(g_last_error, sizeof(g_last_error), "%s", msg);
  return code;
}
inline int fail_hip(hipError_t e, const char* where) {
  snprintf(g_last_error, sizeof(g_last_error), "%s: %s", where, hipGetErrorString(e));
  return (int)e;
}

// HIP events of the dominant kernel of a launch made with FLEXSPMV_FLAG_TIME_KERNEL.  They are attached to the
// kernel's own dispatch (hipExtLaunchKernelGGL), so their difference is the kernel's execution time on
// the launch stream - events recorded before and after the launch also count the dispatch of the kernel
// and of the two event markers, 5 - 8 us on a 300 us kernel.
struct KernelTimer {
  hipEvent_t start = nullptr, stop = nullptr;
  bool armed = false;
  bool ready() {
    if (start == nullptr && (hipEventCreate(&start) != hipSuccess || hipEventCreate(&stop) != hipSuccess)) return false;
    return true;
  }
};
inline thread_local KernelTimer g_timer;
inline int last_kernel_ms(float* ms) {
  if (ms == nullptr || !g_timer.armed) return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "no timed launch on this thread");
  hipError_t e = hipEventSynchronize(g_timer.stop);
  if (e == hipSuccess) e = hipEventElapsedTime(ms, g_timer.start, g_timer.stop);
  if (e != hipSuccess) return fail_hip(e, "reading kernel timer");
  return FLEXSPMV_OK;
}

// Address of flexspmv_static_scratch_bytes on the current device, resolved once per device (the first call on a device asks
// the runtime; later calls read the table).  NULL with g_last_error set when the runtime refuses.
constexpr int MAX_DEVICES = 64;
inline char* static_scratch() {
  static std::mutex lock;
  static void* table[MAX_DEVICES] = {};
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) {
    fail_hip(e, "hipGetDevice");
    return nullptr;
  }
  if (device < 0 || device >= MAX_DEVICES) {
    fail(FLEXSPMV_ERR_BAD_ARGUMENT, "device ordinal beyond the static scratch table");
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(lock);
  if (table[device] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(flexspmv_static_scratch_bytes));
    if (e != hipSuccess || ptr == nullptr) {
      fail_hip(e, "hipGetSymbolAddress(flexspmv_static_scratch_bytes)");
      return nullptr;
    }
    table[device] = ptr;
  }
  return (char*)table[device];
}

// Launch-shape printing, the reference's debug_synchronous (cuda_template/reducer/merged_spmv_template.cuh:106-124,
// :131-137): with FLEXSPMV_FLAG_DEBUG_SYNC in args->flags, or FLEXSPMV_DEBUG_LAUNCH=1 in the environment, every
// kernel of a launch is reported on stderr - grid, block, static LDS bytes, registers - and the stream is
// synchronized after it so that an error names its kernel (no synchronization while the stream is being captured).
inline bool debug_launch_env() {
  static const bool on = [] {
    const char* v = getenv("FLEXSPMV_DEBUG_LAUNCH");
    return v != nullptr && v[0] != 0 && v[0] != '0';
  }();
  return on;
}
template <typename KernelT>
inline int debug_report(const char* name, KernelT kernel, unsigned grid, unsigned block, hipStream_t stream) {
  hipFuncAttributes attr{};
  const bool known = hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(kernel)) == hipSuccess;
  fprintf(stderr, "[flexspmv] %s<<<%u, %u, 0, %p>>>  static LDS %zu B, %d registers per thread\n", name, grid, block,
          (void*)stream, known ? attr.sharedSizeBytes : (size_t)0, known ? attr.numRegs : 0);
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return FLEXSPMV_OK;
  }
  const hipError_t e = hipStreamSynchronize(stream);
  if (e != hipSuccess) return fail_hip(e, name);
  return FLEXSPMV_OK;
}

constexpr size_t align_up(size_t n, size_t a = 256) { return (n + a - 1) / a * a; }
constexpr int FIXUP_BLOCK = 256;
constexpr int MAX_PERSISTENT_BLOCKS = 8192;  // upper bound used to size the aggregator partials

// Number of blocks that are resident at once on the current device for a kernel (all CUs filled),
// rounded down to a multiple of the XCD count; queried once per kernel and device.
struct GridCache {
  int device = -1;
  int grid = 0;
};
template <typename KernelT>
inline int resident_grid(KernelT kernel, int block_threads, GridCache& cache) {
  int& cached_device = cache.device;
  int& cached_grid = cache.grid;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return NUM_XCD;
  if (device == cached_device && cached_grid > 0) return cached_grid;
  int cus = 0, per_cu = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) cus = 256;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, block_threads, 0) != hipSuccess || per_cu <= 0)
    per_cu = 1;
  int grid = cus * per_cu;
  grid = grid / NUM_XCD * NUM_XCD;
  if (grid < NUM_XCD) grid = NUM_XCD;
  if (grid > MAX_PERSISTENT_BLOCKS) grid = MAX_PERSISTENT_BLOCKS;
  cached_device = device;
  cached_grid = grid;
  return grid;
}

// Launch-shape policy (tuning switches in capitals; the defaults are what measured best on MI355X).
#ifndef FLEX_TUNE_SNAP_BYTES
#define FLEX_TUNE_SNAP_BYTES 128  // tiles start on rows whose outputs start a line of this many bytes (0: never)
#endif
#ifndef FLEX_TUNE_XCD_RUN_SHIFT
#define FLEX_TUNE_XCD_RUN_SHIFT 4  // launches with row-snapped tiles hand runs of 2^4 tiles to one XCD
#endif
#ifndef FLEX_TUNE_INBLOCK_MAX_TILES
#define FLEX_TUNE_INBLOCK_MAX_TILES 4096  // launches of at most this many tiles search inside the reducer blocks
#endif
#ifndef FLEX_TUNE_SINGLE_FIXUP_MAX_TILES
#define FLEX_TUNE_SINGLE_FIXUP_MAX_TILES 4096  // launches of at most this many tiles fold carries and aggregators in one block
#endif
constexpr int SINGLE_FIXUP_BLOCK = 1024;

template <class G, int BLOCK, int IPT, bool REDUCER>
struct Dispatch {
  using V = typename G::Value;
  static constexpr int TILE = BLOCK * IPT;

  struct Layout {
    Tiling tiling;
    int num_tiles;
    int flat_blocks;
    int carry_blocks;
    bool search_in_blocks;
    bool single_fixup;
    size_t off_coords, off_splits, off_carry_row, off_carry_val, off_partials, off_block_partials, off_ticket, total;
  };

  // Row-snapped tiles pay with smaller tiles (capacity minus the slack a boundary may be moved by), so
  // they are used where a line's worth of rows is a small part of a tile: the slack is the merge items
  // of that many average rows, and snapping is off when it exceeds an eighth of the tile.
  static Tiling tiling_for(int64_t num_rows, int64_t ne) {
    Tiling t;
    t.nominal = TILE;
    t.snap_slack = 0;
    t.snap_mask = 0;
    t.xcd_shift = 0;
    t.row_group = 0;
    if (REDUCER && FLEX_TUNE_SNAP_BYTES > 0 && num_rows > 0) {
      const int snap_rows = FLEX_TUNE_SNAP_BYTES / (int)sizeof(V) > 1 ? FLEX_TUNE_SNAP_BYTES / (int)sizeof(V) : 1;
      const int64_t slack = (snap_rows * (num_rows + ne) + num_rows - 1) / num_rows;  // snap_rows average rows
      if (slack <= TILE / 8) {
        t.snap_slack = (int)slack;
        t.snap_mask = snap_rows - 1;
        t.nominal = TILE - (int)slack;
        t.xcd_shift = FLEX_TUNE_XCD_RUN_SHIFT;  // short rows: neighbouring tiles gather neighbouring data
#ifndef FLEX_TUNE_NO_ROW_GROUP
        t.row_group = (int)((ne + num_rows - 1) / num_rows);  // average row length, rounded up
#endif
#ifndef FLEX_TUNE_NO_ROW_CAP
        // a thread per row: a tile of more than BLOCK average rows sends its first wavefront through a
        // second pass (a whole gather - map - store chain for a handful of rows)
        const int64_t block_rows_items = (int64_t)BLOCK * (num_rows + ne) / num_rows;
        if (block_rows_items < t.nominal && block_rows_items >= TILE / 2) t.nominal = (int)block_rows_items;
#endif
      }
    }
    const int64_t items = REDUCER ? num_rows + ne : ne;
#ifndef FLEX_TUNE_NO_ROUND_BALANCE
    // A launch of a few rounds of blocks (all CUs filled with as many blocks as fit, then again): its last
    // round should be a full one.  2.35 rounds take the time of 3, so the tiles shrink until there are 3
    // rounds of them (spring-mass 100^3: 3 909 tiles of 1 776 items -> 4 606 of 1 507, kernel 24.7 -> 23.2 us);
    // not where that would cost more than a quarter of the tile, and not for launches of more than four
    // rounds, whose last round is a small part of the whole (the shallow-water launch, 6.5 rounds made 7:
    // 44.4 -> 46.2 us, the smaller tiles cost more than the round).
    if (REDUCER) {
      constexpr int64_t PER_ROUND = (int64_t)NUM_CUS * TileLds<G, BLOCK, IPT>::RESIDENT_PER_CU;
      const int64_t tiles = (items + t.nominal - 1) / t.nominal;
      if (tiles > PER_ROUND && tiles < 4 * PER_ROUND && tiles % PER_ROUND != 0) {
        const int64_t rounds = (tiles + PER_ROUND - 1) / PER_ROUND;
        const int64_t nominal = (items + rounds * PER_ROUND - 1) / (rounds * PER_ROUND);
        if (nominal * 4 >= (int64_t)t.nominal * 3) t.nominal = (int)nominal;
      }
    }
#endif
#ifdef FLEX_TUNE_NOMINAL  // tuning switch: merge items per tile
    if (FLEX_TUNE_NOMINAL <= TILE - t.snap_slack) t.nominal = FLEX_TUNE_NOMINAL;
#endif
    t.num_tiles = (int)((items + t.nominal - 1) / t.nominal);
    return t;
  }

  static bool layout(int64_t num_rows, int64_t ne, Layout& l) {
    const int64_t items = REDUCER ? num_rows + ne : ne;
    if (items <= 0 || num_rows + ne >= ((int64_t)1 << 31) - TILE) return false;
    l.tiling = tiling_for(num_rows, ne);
    l.num_tiles = l.tiling.num_tiles;
    l.flat_blocks = l.num_tiles < MAX_PERSISTENT_BLOCKS ? l.num_tiles : MAX_PERSISTENT_BLOCKS;
    l.search_in_blocks = REDUCER && l.num_tiles <= FLEX_TUNE_INBLOCK_MAX_TILES;
    // ... twice as many where tiles start on rows: hardly a tile carries then, and the block only walks the records
    // (spring-mass 100^3, 4 606 tiles: 2.6 us; with a carry per tile 8 192 tiles cost one block 20 us)
    l.single_fixup = REDUCER && l.num_tiles <= FLEX_TUNE_SINGLE_FIXUP_MAX_TILES * (l.tiling.snap_slack > 0 ? 2 : 1);
    size_t off = 0;
    l.off_coords = off;
    if (REDUCER) off += align_up(sizeof(int2) * ((size_t)l.num_tiles + 1));
    l.off_splits = off;
    if (REDUCER) off += align_up(sizeof(int) * ((size_t)l.num_tiles + 1));
    l.off_carry_row = off;
    if (REDUCER) off += align_up(sizeof(int) * (size_t)l.num_tiles);
    l.off_carry_val = off;
    if (REDUCER) off += align_up(sizeof(V) * (size_t)l.num_tiles * (G::RED_WIDTH > 0 ? G::RED_WIDTH : 1));
    l.carry_blocks = (l.num_tiles + FIXUP_BLOCK - 1) / FIXUP_BLOCK;
    l.off_partials = off;
    const size_t parts = REDUCER ? (size_t)l.num_tiles * partials_per_tile<BLOCK>() : (size_t)MAX_PERSISTENT_BLOCKS;
    if (G::AGG_WIDTH > 0) off += align_up(sizeof(V) * parts * G::AGG_WIDTH);
    l.off_block_partials = off;
    if (REDUCER && G::AGG_WIDTH > 0) off += align_up(sizeof(V) * (size_t)l.carry_blocks * G::AGG_WIDTH);
    l.off_ticket = off;
#ifdef FLEX_TUNE_TICKET_SUM
    off += align_up(sizeof(unsigned));
#endif
    l.total = off;
    return true;
  }

  static size_t workspace_bytes(int64_t num_rows, int64_t ne) {
    Layout l;
    if (!layout(num_rows, ne, l)) return 0;
    return l.total;
  }

  static int tiling(int64_t num_rows, int64_t ne, int32_t* out) {
    Layout l;
    if (out == nullptr) return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "out is NULL");
    if (!layout(num_rows, ne, l))
      return fail(FLEXSPMV_ERR_TOO_LARGE, "num_rows + ne must be positive and stay below 2^31 (32-bit offsets)");
    out[0] = l.tiling.num_tiles;
    out[1] = l.tiling.nominal;
    out[2] = l.tiling.snap_slack;
    out[3] = l.tiling.snap_mask + 1;
    out[4] = TILE;
    out[5] = l.search_in_blocks ? 1 : 0;
    return FLEXSPMV_OK;
  }

  // Checks shared by every entry point that launches: sizes, workspace, row pointer.
  static int check(const flexspmv_launch_args* a, Layout& l, size_t workspace_bytes_available) {
    if (a->ne <= 0) return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "selector index must be non-empty (ne > 0)");
    if (REDUCER && a->num_rows <= 0) return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "num_rows must be positive");
    if (!layout(a->num_rows, a->ne, l))
      return fail(FLEXSPMV_ERR_TOO_LARGE, "num_rows + ne must stay below 2^31 (32-bit offsets)");
    if (l.total > workspace_bytes_available)
      return fail(FLEXSPMV_ERR_WORKSPACE, "workspace is missing or smaller than flexspmv_workspace_bytes()");
    if (REDUCER && a->row_end_offsets == nullptr)
      return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "row_end_offsets is required by a reducer sub-graph");
    return FLEXSPMV_OK;
  }

  static int run(const typename G::Params& p, const flexspmv_launch_args* a) {
    Layout l;
    const int bad = check(a, l, a->workspace == nullptr ? 0 : a->workspace_bytes);
    if (bad != FLEXSPMV_OK) return bad;
    return launch(p, a, l, (char*)a->workspace);
  }

  // flexspmv_launch_static: the same launch with the library's own scratch; allocates nothing.
  static int run_static(const typename G::Params& p, const flexspmv_launch_args* a) {
    if ((a->flags & FLEXSPMV_FLAG_TIME_KERNEL) != 0)
      return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "FLEXSPMV_FLAG_TIME_KERNEL creates events; flexspmv_launch_static does not take it");
    Layout l;
    const int bad = check(a, l, l_unbounded());
    if (bad != FLEXSPMV_OK) return bad;
    if (l.total > (size_t)FLEXSPMV_STATIC_SCRATCH_BYTES) {
      snprintf(g_last_error, sizeof(g_last_error),
               "flexspmv_launch_static: these sizes need %zu bytes of scratch, the library's static buffer holds %zu "
               "(FLEXSPMV_STATIC_SCRATCH_BYTES); use flexspmv_launch with a caller-owned workspace",
               l.total, (size_t)FLEXSPMV_STATIC_SCRATCH_BYTES);
      return FLEXSPMV_ERR_WORKSPACE;
    }
    char* ws = static_scratch();
    if (ws == nullptr) return FLEXSPMV_ERR_WORKSPACE;
    return launch(p, a, l, ws);
  }
  static constexpr size_t l_unbounded() { return ~(size_t)0; }

  // The kernels of one launch, on a->stream, with scratch at ws (l.total bytes, 256-byte aligned).
  static int launch(const typename G::Params& p, const flexspmv_launch_args* a, const Layout& l, char* ws) {
    static thread_local GridCache grid_cache;  // one per kernel instantiation and host thread
    hipStream_t stream = (hipStream_t)a->stream;
    const bool timed = (a->flags & FLEXSPMV_FLAG_TIME_KERNEL) != 0 && g_timer.ready();
    if (timed) g_timer.armed = false;  // untimed launches leave the last timed kernel's events readable
    const bool debug = (a->flags & FLEXSPMV_FLAG_DEBUG_SYNC) != 0 || debug_launch_env();
    int debug_rc = FLEXSPMV_OK;
    auto report = [&](const char* name, auto kernel, int grid, int block) {
      if (debug && debug_rc == FLEXSPMV_OK) debug_rc = debug_report(name, kernel, (unsigned)grid, (unsigned)block, stream);
    };
    V* partials = (V*)(ws + l.off_partials);
    const int nnz = (int)a->ne;

    if constexpr (REDUCER) {
      const int num_rows = (int)a->num_rows;
      const int* row_end = a->row_end_offsets + 1;  // CSR pointer -> row END offsets
      int2* coords = (int2*)(ws + l.off_coords);
      int* splits = (int*)(ws + l.off_splits);
      int* carry_row = (int*)(ws + l.off_carry_row);
      V* carry_val = (V*)(ws + l.off_carry_val);
      unsigned* ticket = (unsigned*)(ws + l.off_ticket);
      if (debug)
        fprintf(stderr, "[flexspmv] reducer launch: %d rows, %d non-zeros, %d tiles of %d merge items (capacity %d, snap slack %d), "
                "%zu bytes of scratch\n", num_rows, nnz, l.num_tiles, l.tiling.nominal, TILE, l.tiling.snap_slack, l.total);

      // Where the blocks take their boundaries from.  By default from the table the launch before left in
      // this scratch, each block confirming its two entries against this launch's row pointer and searching
      // where they do not hold (first launch, another matrix): no search kernel, no search in front of the
      // loads.  Per step, against a search on every launch: Poisson 256^3 316.6 -> 311.9 us (the reducer pays
      // 0.8 us for the confirmation, the search kernel cost 9), R-MAT scale 22 356.9 -> 345.7, shallow water
      // 47.6 -> 46.0, spring-mass 100^3 30.6 -> 28.5 (no search in front of every block's loads).
      // FLEXSPMV_FLAG_SEARCH_TILES: the row structure changes from launch to launch, so nothing is tried: a
      // search kernel for large launches, the blocks' own search for small ones (where a kernel for it costs
      // more than the search).  FLEXSPMV_FLAG_REUSE_TILES: the caller vouches for the table.
      int source = TILES_CONFIRMED;
      if ((a->flags & FLEXSPMV_FLAG_REUSE_TILES) != 0) source = TILES_FROM_TABLE;
      else if ((a->flags & FLEXSPMV_FLAG_SEARCH_TILES) != 0) source = l.search_in_blocks ? TILES_SEARCHED : TILES_FROM_TABLE;
#ifdef FLEX_TUNE_PERSISTENT  // tuning switch: persistent blocks only read the table
      source = TILES_FROM_TABLE;
      const bool search_first = (a->flags & FLEXSPMV_FLAG_REUSE_TILES) == 0;
#else
      const bool search_first = source == TILES_FROM_TABLE && (a->flags & FLEXSPMV_FLAG_REUSE_TILES) == 0;
#endif
      if (search_first) {
        constexpr int per_block = SEARCH_BLOCK / SEARCH_GROUP;
        const int search_blocks = (l.num_tiles + 1 + per_block - 1) / per_block;
        hipLaunchKernelGGL(tile_search_kernel, dim3(search_blocks), dim3(SEARCH_BLOCK), 0, stream, l.tiling, row_end,
                           num_rows, nnz, coords, splits);
        report("tile_search_kernel", tile_search_kernel, search_blocks, SEARCH_BLOCK);
      }
#ifdef FLEX_TUNE_PERSISTENT
      const int reduce_grid = l.num_tiles < 256 * FLEX_TUNE_PERSISTENT ? l.num_tiles : 256 * FLEX_TUNE_PERSISTENT;
#else
      const int reduce_grid = grid_for_tiles(l.num_tiles, l.tiling.xcd_shift);
#endif
      // launches with short regular rows (row-snapped tiles) take several neighbouring edges per load
      constexpr int EPL = edges_per_load<G, IPT>();
      const bool wide_loads = EPL > 1 && l.tiling.snap_slack > 0 && nnz >= EPL;
      auto launch_reducer = [&](auto kernel, const char* name) {
        if (timed) {
          hipExtLaunchKernelGGL(kernel, dim3(reduce_grid), dim3(BLOCK), 0, stream, g_timer.start, g_timer.stop, 0, coords,
                                splits, source, l.tiling, num_rows, row_end, nnz, p, carry_row, carry_val, partials, ticket);
          g_timer.armed = true;
        } else {
          hipLaunchKernelGGL(kernel, dim3(reduce_grid), dim3(BLOCK), 0, stream, coords, splits, source, l.tiling, num_rows,
                             row_end, nnz, p, carry_row, carry_val, partials, ticket);
        }
        report(name, kernel, reduce_grid, BLOCK);
      };
      if (wide_loads) launch_reducer(reduce_kernel<G, BLOCK, IPT, EPL>, "reduce_kernel (several edges per load)");
      else launch_reducer(reduce_kernel<G, BLOCK, IPT, 1>, "reduce_kernel");
      V* block_partials = (V*)(ws + l.off_block_partials);
      constexpr int PARTS = partials_per_tile<BLOCK>();
      if (l.single_fixup) {
        hipLaunchKernelGGL((fixup_kernel<G, SINGLE_FIXUP_BLOCK, PARTS, true>), dim3(1), dim3(SINGLE_FIXUP_BLOCK), 0,
                           stream, p, l.num_tiles, (const int*)carry_row, (const V*)carry_val, (const V*)partials,
                           block_partials, ticket);
        report("fixup_kernel (one block)", fixup_kernel<G, SINGLE_FIXUP_BLOCK, PARTS, true>, 1, SINGLE_FIXUP_BLOCK);
      } else {
        hipLaunchKernelGGL((fixup_kernel<G, FIXUP_BLOCK, PARTS, false>), dim3(l.carry_blocks), dim3(FIXUP_BLOCK), 0,
                           stream, p, l.num_tiles, (const int*)carry_row, (const V*)carry_val, (const V*)partials,
                           block_partials, ticket);
        report("fixup_kernel", fixup_kernel<G, FIXUP_BLOCK, PARTS, false>, l.carry_blocks, FIXUP_BLOCK);
#ifndef FLEX_TUNE_TICKET_SUM
        if (G::AGG_WIDTH > 0) {
          hipLaunchKernelGGL((aggregate_kernel<G, FIXUP_BLOCK>), dim3(1), dim3(FIXUP_BLOCK), 0, stream, p,
                             (const V*)block_partials, l.carry_blocks);
          report("aggregate_kernel", aggregate_kernel<G, FIXUP_BLOCK>, 1, FIXUP_BLOCK);
        }
#endif
      }
    } else {
      int grid = resident_grid(flat_kernel<G, BLOCK, IPT>, BLOCK, grid_cache);
      if (grid > l.num_tiles) grid = l.num_tiles;
      if (debug)
        fprintf(stderr, "[flexspmv] flat launch: %d edges, %d tiles of %d edges, %zu bytes of scratch\n", nnz, l.num_tiles,
                TILE, l.total);
      if (timed) {
        hipExtLaunchKernelGGL((flat_kernel<G, BLOCK, IPT>), dim3(grid), dim3(BLOCK), 0, stream, g_timer.start,
                              g_timer.stop, 0, p, nnz, l.num_tiles, partials);
        g_timer.armed = true;
      } else {
        hipLaunchKernelGGL((flat_kernel<G, BLOCK, IPT>), dim3(grid), dim3(BLOCK), 0, stream, p, nnz, l.num_tiles,
                           partials);
      }
      report("flat_kernel", flat_kernel<G, BLOCK, IPT>, grid, BLOCK);
      if (G::AGG_WIDTH > 0) {
        hipLaunchKernelGGL((aggregate_kernel<G, FIXUP_BLOCK>), dim3(1), dim3(FIXUP_BLOCK), 0, stream, p,
                           (const V*)partials, grid);
        report("aggregate_kernel", aggregate_kernel<G, FIXUP_BLOCK>, 1, FIXUP_BLOCK);
      }
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail_hip(e, "kernel launch failed");
    return debug_rc;
  }
};

inline int check_counts(const flexspmv_launch_args* a, int nv, int ni, int no) {
  if (a == nullptr) return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "args is NULL");
  if (a->struct_size != sizeof(flexspmv_launch_args))
    return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "struct_size does not match this library's flexspmv_launch_args");
  if ((a->flags & ~(FLEXSPMV_FLAG_TIME_KERNEL | FLEXSPMV_FLAG_REUSE_TILES | FLEXSPMV_FLAG_KEEP_TILES |
                    FLEXSPMV_FLAG_DEBUG_SYNC | FLEXSPMV_FLAG_SEARCH_TILES)) != 0)
    return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "unknown bits in flags");
  if (a->num_value_inputs != nv || a->num_index_inputs != ni || a->num_outputs != no)
    return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "argument counts do not match flexspmv_signature()");
  if ((nv > 0 && a->value_inputs == nullptr) || (ni > 0 && a->index_inputs == nullptr) ||
      (no > 0 && a->outputs == nullptr))
    return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "a pointer array is NULL");
  for (int i = 0; i < nv; ++i)
    if (a->value_inputs[i] == nullptr) return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "a value input pointer is NULL");
  for (int i = 0; i < no; ++i)
    if (a->outputs[i] == nullptr) return fail(FLEXSPMV_ERR_BAD_ARGUMENT, "an output pointer is NULL");
  return FLEXSPMV_OK;
}

}  // namespace flex
