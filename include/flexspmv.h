/* C interface of a generated FlexSpmv library for MI355X (gfx950).
 *
 * One shared library is generated per fused sub-graph (select -> map -> reduce / aggregate).  Every
 * such library exports the same symbols below; nothing in the signatures is a torch type, so
 * any host (Python ctypes, a torch extension, C++) can bind them.
 *
 * What each entry point stands in for in the reference:
 *   flexspmv_launch           merged::merged_spmv_launch<ValueT, OffsetT>(FlexParams, d_temp, temp_bytes,
 *                             debug, stream)  (cuda_template/reducer/merged_spmv_template.cuh:146-182,
 *                             cuda_template/aggregator/merged_spmv_template.cuh) as driven by
 *                             merged_spmv_launch_typed (cuda_template/merged_binding_template.cu:10-53);
 *                             the pointer arrays replace the generated FlexParams fields
 *                             (cuda_template/merged_utils_template.cuh:243-262).
 *   flexspmv_workspace_bytes  the size-query call of the same function with d_temp_storage == NULL
 *                             (cuda_template/reducer/merged_spmv_template.cuh:83-87).
 *   flexspmv_signature        the argument list the reference bakes into the generated binding
 *                             (codegen/merged_gen_binding.py:27-78,112-134); here it is data.
 *   flexspmv_last_error       the strings TORCH_CHECK raises (cuda_template/merged_binding_template.cu:40-50).
 *   flexspmv_abi_version      no counterpart; lets a loader reject a stale library.
 *   flexspmv_tiling           the tile arithmetic of the reference's dispatch (num_merge_tiles from
 *                             num_rows + num_nonzeros and the policy's tile size,
 *                             cuda_template/reducer/merged_spmv_template.cuh:60-80), as data.
 *   flexspmv_last_kernel_ms   the GpuTimer bracket of the reference's CUDA harness
 *                             (src/flex_spmv_full_red.cu:298-330, utils.h:634-669), narrowed to the
 *                             dominant kernel of one launch so that a roofline can be measured live.
 */
#ifndef FLEXSPMV_H_
#define FLEXSPMV_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLEXSPMV_ABI_VERSION 5

/* Scratch a library keeps for flexspmv_launch_static (bytes, per library and per GPU it is used on). */
#define FLEXSPMV_STATIC_SCRATCH_BYTES (4u << 20)

/* flexspmv_launch_args.flags */
#define FLEXSPMV_FLAG_TIME_KERNEL 1u /* attach HIP events to the dominant kernel's dispatch on args->stream */
/* The tile table.  A launch of a library with a reducer cuts the merge path into tiles; the boundaries
 * are what the reference searches for on every call (include/merged_spmv_kernels.cuh:60-99).  Here every
 * launch leaves them in its workspace, and a later launch on that workspace tries them: each block takes
 * the two boundaries of its tile from the table, loads the tile, and checks with three row ends per
 * boundary - fetched together with the tile - that a search on this launch's row_end_offsets would return
 * exactly them.  Where that holds (a solver loop, a time stepper: the same matrix again) no search runs;
 * where it does not (first launch on a workspace, another matrix, a workspace that held anything else)
 * the block searches and nothing of the table is used.  Results never depend on what the workspace held.
 * For speed, give every matrix that is launched repeatedly a workspace of its own.
 *
 * FLEXSPMV_FLAG_REUSE_TILES: skip the check as well.  The caller guarantees that the previous launch of this
 * library with this workspace completed, used the same dtype, num_rows, ne and the same, unmodified
 * row_end_offsets, and that nothing else wrote to the workspace since. */
#define FLEXSPMV_FLAG_REUSE_TILES 2u
/* The table is int32 pairs (rows, non-zeros) for tile boundaries 0 .. num_tiles at the start of the
 * workspace.  It can be read back after a launch and compared with a CPU merge-path search (see
 * flexspmv_tiling for the diagonals).  This flag is accepted and changes nothing (it used to ask small
 * launches for the table). */
#define FLEXSPMV_FLAG_KEEP_TILES 4u
/* The reference's debug_synchronous argument (cuda_template/reducer/merged_spmv_template.cuh:106-124,131-137):
 * every kernel of the launch is reported on stderr (grid, block, static LDS bytes, registers) and the stream is
 * synchronized after it, so that an error is returned by the launch that caused it and names its kernel.  The
 * environment variable FLEXSPMV_DEBUG_LAUNCH=1 turns the same on for every launch of the process.  While the
 * stream is being captured the report is printed and the synchronization left out. */
#define FLEXSPMV_FLAG_DEBUG_SYNC 8u
/* Do not try the table of an earlier launch: for callers whose row structure changes from launch to launch,
 * where trying it would fail in every block.  Large launches then run a search kernel in front of the reducer
 * (one search per boundary instead of two per block), small ones search inside the blocks. */
#define FLEXSPMV_FLAG_SEARCH_TILES 16u

/* Value types a library may have been generated for (flexspmv_launch_args.dtype). */
enum flexspmv_dtype { FLEXSPMV_F32 = 0, FLEXSPMV_F64 = 1, FLEXSPMV_I64 = 2 };

/* Return codes.  Positive values are hipError_t codes passed through unchanged. */
enum flexspmv_status {
  FLEXSPMV_OK = 0,
  FLEXSPMV_ERR_BAD_ARGUMENT = -1,  /* NULL pointer, wrong count, size <= 0, struct_size mismatch */
  FLEXSPMV_ERR_BAD_DTYPE = -2,     /* dtype not compiled into this library */
  FLEXSPMV_ERR_TOO_LARGE = -3,     /* num_rows + ne does not fit 32-bit offsets */
  FLEXSPMV_ERR_WORKSPACE = -4      /* workspace missing or smaller than flexspmv_workspace_bytes() */
};

/* Arguments of one launch.  All pointers are device pointers valid on the current device.
 *   value_inputs   value tensors in binding order: non-gather inputs (placeholder order), then gather
 *                  sources (order of first use); row-major [n][Dim], contiguous.  In-place map ops
 *                  (setitem / copy_ / add_) write through these pointers.
 *   index_inputs   one int32 array of ne entries per unique selector module, binding order.  An array
 *                  listed under "row_aligned_index_inputs" in flexspmv_signature() is never dereferenced:
 *                  the caller guarantees that it equals the row id of every edge, and the value inputs
 *                  listed under "row_indexed_value_inputs" are then read at every row id 0 .. num_rows-1
 *                  (rows without edges included), so they must hold at least num_rows items.
 *   outputs        one buffer per output in binding order: reducer [num_rows][Dim], aggregator [Dim],
 *                  map output [ne][Dim].  Every element is overwritten; no zero fill is needed.
 *   row_end_offsets  int32[num_rows + 1] with a leading 0 (CSR row pointer); ignored (may be NULL) by
 *                  libraries without a reducer.
 *   ne             number of edges (non-zeros); must be > 0.
 *   workspace      scratch of at least flexspmv_workspace_bytes(...) bytes, 256-byte aligned, uninitialised
 *                  or in whatever state an earlier launch left it.  Its contents mean nothing to the caller;
 *                  they only have to be left alone between two launches when the second one carries
 *                  FLEXSPMV_FLAG_REUSE_TILES (and are worth leaving alone otherwise: see the tile table).
 *   stream         hipStream_t to launch on (NULL = default stream).  The call is asynchronous.
 */
typedef struct flexspmv_launch_args {
  uint32_t struct_size; /* sizeof(flexspmv_launch_args) */
  int32_t dtype;        /* enum flexspmv_dtype */
  void* const* value_inputs;
  int32_t num_value_inputs;
  const int32_t* const* index_inputs;
  int32_t num_index_inputs;
  void* const* outputs;
  int32_t num_outputs;
  const int32_t* row_end_offsets;
  int64_t num_rows;
  int64_t num_cols;
  int64_t ne;
  void* workspace;
  size_t workspace_bytes;
  void* stream;
  uint32_t flags; /* 0 or FLEXSPMV_FLAG_* */
} flexspmv_launch_args;

/* Run the fused sub-graph once.  Returns FLEXSPMV_OK, a negative flexspmv_status, or a hipError_t. */
int flexspmv_launch(const flexspmv_launch_args* args);

/* flexspmv_launch without any allocation.  No counterpart in the reference; it is for callers that cannot
 * allocate device memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Same arguments and results as flexspmv_launch, except that args->workspace / workspace_bytes are ignored:
 * tile table, carries and aggregator partials live in a buffer of FLEXSPMV_STATIC_SCRATCH_BYTES that is part
 * of the library's device image (one copy per GPU, held until the process ends).  The call makes no
 * hipMalloc / hipFree and creates no events, so FLEXSPMV_FLAG_TIME_KERNEL is refused (BAD_ARGUMENT).  Sizes
 * whose flexspmv_workspace_bytes() exceeds the buffer are refused with FLEXSPMV_ERR_WORKSPACE and a message
 * that names both figures.  The first call on each GPU looks the buffer's address up (make it outside a
 * capture); nothing in the buffer has to be cleared between calls - every word a launch reads it has
 * written first.  All calls of one library on one GPU share the buffer: calls that overlap in time
 * (two streams, two threads) race on it, and FLEXSPMV_FLAG_REUSE_TILES refers to the previous call of
 * either entry point that used this buffer. */
int flexspmv_launch_static(const flexspmv_launch_args* args);

/* Scratch bytes flexspmv_launch needs for these sizes (0 is a valid answer). */
size_t flexspmv_workspace_bytes(int32_t dtype, int64_t num_rows, int64_t ne);

/* JSON text describing the binding: argument names and kinds, value widths, outputs, compiled
 * dtypes and the tile policy.  The pointer stays valid for the life of the library. */
const char* flexspmv_signature(void);

/* Message of the last failed call on this thread ("" if none). */
const char* flexspmv_last_error(void);

/* Duration in milliseconds of the dominant kernel (the reducer kernel, or the flat kernel of an
 * aggregator / map-only library) of the calling thread's most recent flexspmv_launch that carried
 * FLEXSPMV_FLAG_TIME_KERNEL (launches without the flag made since do not disturb it).  Blocks until that kernel has finished.  Returns FLEXSPMV_OK, or
 * FLEXSPMV_ERR_BAD_ARGUMENT when no such launch was made. */
int flexspmv_last_kernel_ms(float* ms);

/* How a launch of these sizes cuts the merge path of (row end offsets, 0 .. ne-1) into tiles:
 *   out[0] num_tiles     tile t covers the path from boundary t to boundary t + 1
 *   out[1] nominal       boundary t lies on diagonal min(t * nominal, num_rows + ne) ...
 *   out[2] snap_slack    ... unless 0 < t < num_tiles and the start of row (x & ~(snap_rows - 1)), x the
 *   out[3] snap_rows     row coordinate on that diagonal, is at most snap_slack merge items back: then the
 *                        boundary is that row start.  snap_slack = 0: boundaries stay on their diagonals.
 *   out[4] tile_capacity merge items a block can hold (threads x items per thread of the policy); at least
 *                        nominal + snap_slack, and more where a cap on the rows per tile shortens nominal
 *   out[5] search_in_blocks  1 when a launch with FLEXSPMV_FLAG_SEARCH_TILES searches inside the reducer blocks,
 *                        0 when it runs a search kernel (launches without the flag never run one)
 * For libraries without a reducer the tiles are plain edge ranges of `nominal` edges.
 * Returns FLEXSPMV_OK, FLEXSPMV_ERR_BAD_DTYPE or FLEXSPMV_ERR_TOO_LARGE. */
int flexspmv_tiling(int32_t dtype, int64_t num_rows, int64_t ne, int32_t out[6]);

/* FLEXSPMV_ABI_VERSION the library was built against. */
int flexspmv_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FLEXSPMV_H_ */
