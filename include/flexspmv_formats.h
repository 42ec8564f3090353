/* C interface of the edge-list preparation step that sits in front of a FlexSpmv launch on MI355X
 * (gfx950): a reducer's COO row ids become the CSR row pointer the kernels consume, and an edge list
 * whose row ids are not ascending is brought into row order once.
 *
 * One library (libflexspmv_formats.so) exports every symbol below.  All data pointers are device
 * pointers valid on the current device, all calls are asynchronous on the given hipStream_t, and none
 * of them allocates: scratch comes in through the workspace arguments.
 *
 * What each entry point stands in for in the reference:
 *   flexspmv_coo_rows_to_csr      _coo_rows_to_csr_ptr (python_wrapper/dynamic_replace_submodule.py:20-41):
 *                                 torch's COO -> CSR conversion, or bincount + cumsum, of the reducer's
 *                                 row ids.  The reference silently assumes ascending ids; here unsorted
 *                                 and out-of-range ids are detected and reported.
 *   flexspmv_sort_edges_by_row    no counterpart: the reference's toy model draws unsorted row ids
 *                                 (easier_spmv.py:126-127) and its wrapper mis-describes them.  A stable
 *                                 sort by row keeps the order of the edges inside every row, hence the
 *                                 summation order of the original list.
 *   flexspmv_gather_rows /        the permutation applied to the per-edge tensors going into a launch and
 *   flexspmv_scatter_rows         to the per-edge results coming out of it.
 *   flexspmv_formats_last_error,  as flexspmv_last_error / flexspmv_abi_version of a generated library.
 *   flexspmv_formats_abi_version
 */
#ifndef FLEXSPMV_FORMATS_H_
#define FLEXSPMV_FORMATS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLEXSPMV_FORMATS_ABI_VERSION 1

/* Return codes (negative); positive values are hipError_t codes passed through unchanged. */
enum flexspmv_formats_status {
  FLEXSPMV_FORMATS_OK = 0,
  FLEXSPMV_FORMATS_ERR_BAD_ARGUMENT = -1, /* NULL pointer, negative size, index width not 4 or 8 */
  FLEXSPMV_FORMATS_ERR_TOO_LARGE = -3,    /* ne or num_rows does not fit 32-bit offsets */
  FLEXSPMV_FORMATS_ERR_WORKSPACE = -4     /* workspace missing or too small */
};

/* Bits the kernels OR into *findings (a device int32 the caller reads back when it wants to know). */
#define FLEXSPMV_FINDING_UNSORTED 1     /* some row id is smaller than its predecessor */
#define FLEXSPMV_FINDING_OUT_OF_RANGE 2 /* some row id is negative or >= num_rows */

/* CSR row pointer of ascending COO row ids: row_ptr[r] = number of ids smaller than r, r = 0..num_rows
 * (int32[num_rows + 1], row_ptr[0] = 0, row_ptr[num_rows] = ne).
 *   row_ids      int32 or int64 [ne] (index_bytes = 4 or 8); may be NULL when ne == 0
 *   findings     device int32[4]: word 0 receives FLEXSPMV_FINDING_* bits (cleared first by the call),
 *                the other words are scratch.  When a bit is set, row_ptr holds no meaningful result,
 *                but every write stayed inside row_ptr.
 */
int flexspmv_coo_rows_to_csr(const void* row_ids, int index_bytes, int64_t ne, int64_t num_rows,
                             int32_t* row_ptr, int32_t* findings, void* stream);

/* Scratch bytes flexspmv_sort_edges_by_row needs: per-block digit counters, and a second pair of
 * int32[ne] buffers when the ids need more than one 8-bit digit (num_rows > 256).  0 when ne == 0 or a
 * size is out of range. */
size_t flexspmv_sort_workspace_bytes(int64_t ne, int64_t num_rows);

/* Stable sort of the edges by row id (radix sort over the bits num_rows - 1 needs; kernels of this
 * library only: it clears nothing, allocates nothing and may be captured into a HIP graph).
 *   sorted_rows   int32[ne]: the row ids in ascending order
 *   permutation   int32[ne]: permutation[k] = position in the original list of the edge now at k
 *   workspace     flexspmv_sort_workspace_bytes(ne, num_rows) bytes, 4-byte aligned; must not overlap
 *                 row_ids, sorted_rows or permutation
 * Row ids must lie in [0, num_rows).  An id outside is ordered as if it were num_rows - 1 (it stays in
 * its original order among that row's edges), keeps its value in sorted_rows (-1 if it does not fit an
 * int32) and is reported by flexspmv_coo_rows_to_csr on sorted_rows.  row_ids may alias neither output.
 * ne == 0 is allowed. */
int flexspmv_sort_edges_by_row(const void* row_ids, int index_bytes, int64_t ne, int64_t num_rows,
                               int32_t* sorted_rows, int32_t* permutation, void* workspace,
                               size_t workspace_bytes, void* stream);

/* dst[k] = src[permutation[k]] for k < n; one entry is row_bytes bytes (a multiple of 4). src and dst
 * must not overlap. */
int flexspmv_gather_rows(const void* src, void* dst, const int32_t* permutation, int64_t n,
                         int64_t row_bytes, void* stream);

/* dst[permutation[k]] = src[k] for k < n (the inverse of flexspmv_gather_rows). */
int flexspmv_scatter_rows(const void* src, void* dst, const int32_t* permutation, int64_t n,
                          int64_t row_bytes, void* stream);

/* Message of the last failed call on this thread ("" if none). */
const char* flexspmv_formats_last_error(void);

/* FLEXSPMV_FORMATS_ABI_VERSION the library was built against. */
int flexspmv_formats_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FLEXSPMV_FORMATS_H_ */
