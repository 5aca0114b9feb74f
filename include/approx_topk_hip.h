/*
 * C ABI of libapprox_topk_hip.so: bucketed approximate top-k on AMD gfx950.
 *
 * This is the boundary a binding (ctypes, pybind11, cgo, ...) targets.  It takes
 * plain device pointers, sizes and a HIP stream; it never allocates device
 * memory, never synchronises and never throws.  All work is enqueued on the
 * stream that is passed in, so calls are asynchronous and can be captured into
 * a HIP graph.  Every function returns ATK_OK (0) or a negative atk_status.
 *
 * The entry points replace the native interface of the reference
 * (graphcore-research/pytorch-approx-topk):
 *   PriorityQueueTopK(self, k, j, dim, largest, interleaved, multithread_buckets,
 *                     values, indices)
 *       approx_topk/priority_queue_approx_topk.cu:378-387, bound with pybind11 at
 *       cu:523-525 and called from approx_topk/priority_queue.py:70-80;
 *   torch.topk(stage_1_values, k, sorted=False) + gather
 *       approx_topk/priority_queue.py:85-88 (stage 2);
 *   the Triton launches of approx_topk/experimental/bucketed_argmax.py:171-199.
 *
 * Conventions shared by all entry points
 *   - A "row" is one slice along the top-k dimension.  Elements of a row are
 *     adjacent in memory; consecutive rows are `row_stride` elements apart.
 *   - Outputs are dense: values[rows][k] in the input dtype, indices[rows][k]
 *     as int64 positions within the row.  `values` may be NULL in every entry
 *     point that writes results: then only the indices are written, the same
 *     ones.  (No counterpart in the reference, whose operator always returns
 *     both, priority_queue.py:63-88: for callers that gather other tensors by
 *     the indices and never read the selected elements; at fp32 [128, 2^20],
 *     k = 65536, j = 2 with int32 indices the call takes 96 instead of 106 us.)
 *   - Selection order: a beats b when value(a) > value(b), or the values are
 *     equal and index(a) < index(b).  -0.0 equals +0.0, NaN ranks above +inf.
 *   - `ws` is caller-owned scratch of at least the matching *_workspace_bytes();
 *     it may be NULL when that size is 0.  Its contents need no initialisation.
 *   - Alignment: the input, `values` and candidate values to the element size,
 *     indices to their width (8 bytes; 4 for the *_i32 entry points), `ws` to
 *     16 bytes (256 recommended); otherwise ATK_ERR_ALIGN.  Input, `values`
 *     and `indices` that are all 16-byte aligned, with `row_stride` a multiple
 *     of 16 bytes' worth of elements, additionally get the 16-byte-vector kernels.
 */
#ifndef APPROX_TOPK_HIP_H_
#define APPROX_TOPK_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types: the set cu:449-453 dispatches over (AT_DISPATCH_ALL_TYPES plus
 * Half and BFloat16). */
typedef enum atk_dtype {
  ATK_F32 = 0, ATK_F16 = 1, ATK_BF16 = 2, ATK_F64 = 3, ATK_U8 = 4,
  ATK_I8 = 5, ATK_I16 = 6, ATK_I32 = 7, ATK_I64 = 8
} atk_dtype;

/* How a row of n elements is cut into b buckets. */
typedef enum atk_layout {
  /* bucket c = { i : i mod b == c }; first n mod b buckets one longer
   * (CalculateBucket, cu:37-46) */
  ATK_INTERLEAVED = 0,
  /* contiguous runs; the first n mod b buckets one longer (cu:47-54) */
  ATK_BALANCED = 1,
  /* contiguous runs of ceil(n/b) over the row padded with the dtype minimum to
   * b*ceil(n/b) (bucketed_argmax.py:22-31,39-41); j must be 1 */
  ATK_CEIL_CHUNK = 2,
  /* interleaved over the same padded row (bucketed_argmax.py:35-37); j must be 1 */
  ATK_INTERLEAVED_PADDED = 3
} atk_layout;

typedef enum atk_status {
  ATK_OK = 0,
  ATK_ERR_DTYPE = -1,      /* unknown atk_dtype */
  ATK_ERR_J = -2,          /* j outside 1..4, or j does not divide k0 (cu:402,434) */
  ATK_ERR_K = -3,          /* k0 > n (cu:329-330), k > k0, or a negative size */
  ATK_ERR_LAYOUT = -4,     /* unknown layout, or a padded layout with j != 1 */
  ATK_ERR_WORKSPACE = -5,  /* ws is NULL or smaller than *_workspace_bytes() */
  ATK_ERR_LAUNCH = -6,     /* the HIP runtime rejected a launch */
  ATK_ERR_ARG = -7,        /* NULL data pointer, row_stride < n, misc. */
  ATK_ERR_TOO_LARGE = -8,  /* a size exceeds what the kernels index (cu:328,337,357) */
  ATK_ERR_ALIGN = -9,      /* a pointer is not aligned as the conventions above require */
  ATK_ERR_SCRATCH = -10    /* atk_topk_noalloc: the call needs more than ATK_NOALLOC_SCRATCH_BYTES */
} atk_status;

/* Opaque hipStream_t (NULL = the default stream). */
typedef void* atk_stream_t;

/* ABI version of the library; bumped when a signature changes. */
int atk_version(void);

/* Static, human-readable text for a status code. */
const char* atk_strerror(int status);

/*
 * Stage 1: per row, cut the n elements into b = k0 / j buckets and write the j
 * best of every bucket to values/indices[row][c*j + s], s ascending from the
 * weakest to the best of the bucket's j.  Replaces ThreadTopK/BlockTopK
 * (cu:149-289) and the Triton arg-max kernels (bucketed_argmax.py:70-142).
 * k0 == 0 or rows == 0 is a no-op.
 */
size_t atk_stage1_workspace_bytes(int64_t rows, int64_t n, int64_t k0, int j,
                                  int layout, int dtype);
int atk_stage1(const void* x, int64_t rows, int64_t n, int64_t row_stride,
               int64_t k0, int j, int layout, int dtype,
               void* values, int64_t* indices,
               void* ws, size_t ws_bytes, atk_stream_t stream);

/*
 * Stage 2: per row, the k best of k0 candidates (cand_values[row][p],
 * cand_indices[row][p]), written in increasing p.  Candidate indices within a
 * row must be distinct and lie in [0, index_bound).  Replaces torch.topk +
 * gather at priority_queue.py:85-88.
 */
size_t atk_select_workspace_bytes(int64_t rows, int64_t k0, int64_t k, int dtype);
int atk_select(const void* cand_values, const int64_t* cand_indices,
               int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype,
               void* values, int64_t* indices,
               void* ws, size_t ws_bytes, atk_stream_t stream);

/*
 * Both stages: stage 1 with k0 candidates per row into the workspace, then the
 * k best of them into values/indices[rows][k].  With k == k0 this is stage 1
 * writing straight to the outputs.  Replaces the whole body of
 * approx_topk.topk after argument checks (priority_queue.py:63-88).
 */
size_t atk_topk_workspace_bytes(int64_t rows, int64_t n, int64_t k0, int j,
                                int64_t k, int layout, int dtype);
/*
 * The same for one particular call: 0 when the input's address and row stride
 * let the one-kernel path take it, which parks no candidates (never more than
 * atk_topk_workspace_bytes).  Same call site as above: the workspace the
 * operator allocates before the native call (priority_queue.py:63-88).
 */
size_t atk_topk_workspace_bytes_at(const void* x, int64_t rows, int64_t n, int64_t row_stride,
                                   int64_t k0, int j, int64_t k, int layout, int dtype);
int atk_topk(const void* x, int64_t rows, int64_t n, int64_t row_stride,
             int64_t k0, int j, int64_t k, int layout, int dtype,
             void* values, int64_t* indices,
             void* ws, size_t ws_bytes, atk_stream_t stream);

/*
 * The same two entry points with int32 indices, for consumers that gather with
 * 32-bit offsets (the index write is two thirds of the output traffic of
 * atk_stage1 on 4-byte elements).  No counterpart in the reference, whose
 * outputs are int64 (priority_queue.py:67).  Workspace as for the int64
 * versions.  ATK_ERR_TOO_LARGE when a row (its padded length, for the padded
 * layouts) has positions beyond 2^31 - 1.
 */
int atk_stage1_i32(const void* x, int64_t rows, int64_t n, int64_t row_stride,
                   int64_t k0, int j, int layout, int dtype,
                   void* values, int32_t* indices,
                   void* ws, size_t ws_bytes, atk_stream_t stream);
int atk_topk_i32(const void* x, int64_t rows, int64_t n, int64_t row_stride,
                 int64_t k0, int j, int64_t k, int layout, int dtype,
                 void* values, int32_t* indices,
                 void* ws, size_t ws_bytes, atk_stream_t stream);

/*
 * Diagnostics: which kernels atk_topk (atk_stage1 when k == k0) would enqueue
 * for these arguments, as text ("name<parameters> grid=... block=...", several
 * kernels joined by " + "), truncated to text_bytes - 1 characters.  Enqueues
 * nothing.  No counterpart in the reference, whose dispatch is one templated
 * launch (cu:306-375); here the planner picks among several kernels, and a
 * benchmark record should say which one it timed.
 */
int atk_describe(const void* x, int64_t rows, int64_t n, int64_t row_stride,
                 int64_t k0, int j, int64_t k, int layout, int dtype,
                 const void* values, const void* indices, char* text, size_t text_bytes);

/*
 * atk_topk without a workspace argument and without any allocation.  No
 * counterpart in the reference: it is for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  The scratch memory atk_topk would take from the caller
 * (stage-1 candidates, partial queues of rows cut into slabs, stage 2's
 * histograms and counts) lives in an array of ATK_NOALLOC_SCRATCH_BYTES inside
 * the library's device code, one copy per GPU, held until the process ends.
 * A call that needs more (atk_topk_workspace_bytes_at() of the same arguments)
 * returns ATK_ERR_SCRATCH and enqueues nothing.  The device the stream belongs
 * to must be current.  All calls on one GPU share that GPU's array: calls that
 * may run concurrently on one GPU (different streams, different host threads)
 * race on it and must be serialised by the caller; calls on one stream are
 * ordered and safe.  Nothing in the array needs to survive between calls and
 * nothing needs clearing by the caller.  Results are those of atk_topk.
 */
#define ATK_NOALLOC_SCRATCH_BYTES ((size_t)8 << 20)
int atk_topk_noalloc(const void* x, int64_t rows, int64_t n, int64_t row_stride,
                     int64_t k0, int j, int64_t k, int layout, int dtype,
                     void* values, int64_t* indices, atk_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* APPROX_TOPK_HIP_H_ */
