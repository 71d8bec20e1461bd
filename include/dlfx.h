/*
 * dlfx -- C ABI of the MI355X (gfx950) axis primitives: reduce, arg_reduce,
 * scan, sort, argsort, top_k over strided N-d views.
 *
 * This is the boundary a dlf build binds in place of the gpgpu::dnn routines
 * for these operations (reference declarations: gpgpu/include/gdnn.h:108-182,
 * bodies gpgpu/src/gdnn.cpp:833-1347).  Each entry point below names the
 * reference function it replaces.
 *
 * Conventions shared by every call
 *   stream     a hipStream_t passed as void*; work is enqueued asynchronously on
 *              it and the call returns without synchronising.
 *   dtype      a dlfx_dtype -- the element type T of the reference template
 *              instantiation (gdnn.cpp:847-1347, 1851-1894).
 *   dims       extents of the (already axis-moved) view, `rank` entries.
 *   strides    element strides, signed: a reference stride that wrapped as
 *              size_t (negative step) is passed as the negative number it means.
 *   offset     element offset of the view's first element from the pointer.
 *   x, y, idx  device pointers to the start of the buffers (Buffer<T>::data()).
 *              Outputs may alias inputs where the reference allows it
 *              (in-place scan / sort / argsort).
 *   scratch    device memory owned by the caller, at least the number of bytes
 *              the matching *_scratch_bytes() query returns (256-byte aligned);
 *              may be NULL when that number is 0.  Its contents are undefined
 *              on entry and on return; two calls that overlap in time must not
 *              share it.
 *   return     DLFX_OK or a negative dlfx_status; nothing is enqueued when the
 *              status is an argument error.
 * Ranks above DLFX_MAX_RANK (after merging mergeable dimensions) are rejected.
 * No call allocates or frees device memory.
 */
#ifndef DLFX_H_
#define DLFX_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DLFX_MAX_RANK 8

typedef void* dlfx_stream_t; /* hipStream_t */

typedef enum dlfx_dtype {
    DLFX_F32 = 0,
    DLFX_F64 = 1,
    DLFX_I32 = 2,
    DLFX_I64 = 3,
    DLFX_F16 = 4,   /* IEEE half: every entry point (sums and scans accumulate in fp32, rounded once) */
    DLFX_I16 = 5,   /* arg_reduce, sort, argsort, top_k (the reference's int16 instantiations) and merge */
    DLFX_BOOL = 6,  /* one byte per element; input of scan_nonzero only */
    DLFX_C64 = 7,   /* complex of two floats (the reference's float2): reduce, count, scan */
    DLFX_C128 = 8   /* complex of two doubles (double2): reduce, count, scan */
} dlfx_dtype;

typedef enum dlfx_status {
    DLFX_OK = 0,
    DLFX_ERR_INVALID_ARGUMENT = -1,  /* null pointer, negative extent, m*n mismatch ... */
    DLFX_ERR_UNSUPPORTED_DTYPE = -2,
    DLFX_ERR_UNKNOWN_OP = -3,        /* `name` is not one this library implements */
    DLFX_ERR_SCRATCH_TOO_SMALL = -4,
    DLFX_ERR_RANK = -5,              /* view rank above DLFX_MAX_RANK */
    DLFX_ERR_LAUNCH = -6,            /* HIP reported an error; see dlfx_last_hip_error */
    DLFX_ERR_TOO_LARGE = -7,         /* an extent exceeds what the kernels index */
    DLFX_ERR_CAPTURING = -8          /* a first call on a device that may not be recorded into a graph */
} dlfx_status;

/* Library version: major*10000 + minor*100 + patch. */
int dlfx_version(void);
/* Static, human-readable text for a dlfx_status. */
const char* dlfx_status_string(int status);
/* hipError_t of the last DLFX_ERR_LAUNCH on the calling thread (0 if none). */
int dlfx_last_hip_error(void);

/* Process-wide tuning knobs (not thread-safe against running calls).  Keys:
 *   "scan_poll_limit"  how many times a scan tile polls a predecessor's published
 *                      state before it folds that predecessor's input itself
 *                      (default 2048; 0 makes every tile help itself at once).
 *   "sort_poll_limit"  the same bound for the per-digit tile chaining of a radix pass.
 *   "sort_wave_rows"   longest row (64, 128, 256 or 512; default 512) sorted by one wavefront
 *                      in registers; longer rows of up to 16384 elements (8-byte keys: 8192,
 *                      16-bit keys: 4096) take one workgroup.
 *   "sort_buckets"     1 (default): rows of 4-byte keys longer than 16384 elements and of 8-byte
 *                      keys longer than 8192 (up to about 2.6 million elements) are cut into
 *                      buckets of equal depth by value and each bucket is sorted on chip; 0: every
 *                      row takes the least-significant-digit-first passes.  Same results either
 *                      way, but not the same scratch: the bucket route needs one pair of
 *                      ping-pong buffers where the digit passes need two, so set this before
 *                      dlfx_sort_scratch_bytes / dlfx_argsort_scratch_bytes / dlfx_top_k_scratch_bytes
 *                      of the calls it is to hold for.
 *   "sort_compare_max" fullest counting bin (default 32) of a bucket whose entries are still ranked
 *                      by comparing them; fuller bins send the bucket through stable digit passes
 *                      (0: every bucket).  Same results for every value.
 *   "topk_thread_rows" longest row (default 256; half of it for 8-byte keys) for which top_k
 *                      with a limit of at most 8 over at least 16384 contiguous rows gives
 *                      each row to one thread.
 *   "topk_cols_waves"  wavefronts (1, 4 or 8; 0, the default: by the shape) that share a block of
 *                      64 neighbouring rows, each with a piece of the axis, when top_k with a
 *                      small limit runs along an axis that is not the innermost.
 *   "scan_cols_per_lane" the most neighbouring columns (1 or 2; 0, the default: 2 where the
 *                      layout allows) that a lane takes in one access when two-byte elements
 *                      are scanned along an axis that is not the innermost.
 * Returns DLFX_ERR_UNKNOWN_OP for an unknown key or out-of-range value.  No
 * counterpart in the reference (its database/ tuning tables play this role). */
int dlfx_set_tuning(const char* key, int64_t value);

/* ---------------------------------------------------------------- reduce
 * Replaces gpgpu::dnn::reduce<T> (gdnn.h:108-114; caller
 * dlf/include/tensor/reduce_detail.h:91-101).  x_dims lists the kept extents
 * followed by the reduced extents (the transposed view prepare_reduce builds);
 * m = product of kept, n = product of reduced; output element r (row-major
 * over y_dims) receives Final(fold(Map(x[r, 0..n)))).
 * name: reduce_sum, reduce_mean, reduce_max, reduce_min, reduce_log_sum_exp,
 *       reduce_sum_exp, reduce_log_sum, reduce_prod, reduce_asum,
 *       reduce_sum_square, reduce_nrm2, reduce_amax, reduce_amin
 *       (dlf/include/tensor/xfn.h:661-805).  The exp/log/sqrt reducers accept
 *       floating dtypes only.
 */
size_t dlfx_reduce_scratch_bytes(int dtype, int64_t m, int64_t n);
int dlfx_reduce(dlfx_stream_t stream, const char* name, int dtype, int64_t m, int64_t n,
                int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                const void* x, int64_t x_offset,
                int y_rank, const int64_t* y_dims, const int64_t* y_strides,
                void* y, int64_t y_offset,
                void* scratch, size_t scratch_bytes);

/* ---------------------------------------------------------------- reduce, allocation-free
 * No counterpart in the reference.  For callers that cannot allocate device memory or carry a
 * scratch buffer: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  Same arguments, results and status codes as dlfx_reduce, without the scratch
 * pair: the partial accumulators of long-row and strided-axis reductions live in an array of
 * DLFX_REDUCE_STATIC_SCRATCH_BYTES bytes that is part of the library's device code (every GPU
 * the library runs on holds one copy until the process ends).  The call allocates and frees
 * nothing.  The array covers every shape dlfx_reduce accepts (its scratch query never asks for
 * more); a shape whose partials would not fit is refused with DLFX_ERR_TOO_LARGE and nothing
 * is enqueued.  The first call on a device looks the array's address up (the device that is
 * current must be the one the stream belongs to), which may load the library's device code:
 * that call must come before any stream capture -- while `stream` is being captured it is
 * refused with DLFX_ERR_CAPTURING and nothing is enqueued; later calls on the device record
 * like any other launch.  All calls on one GPU share that GPU's
 * array: calls that overlap in time on one GPU -- different streams, or different host threads
 * -- race on it and must be serialised by the caller.
 */
#define DLFX_REDUCE_STATIC_SCRATCH_BYTES 3178496
int dlfx_reduce_static(dlfx_stream_t stream, const char* name, int dtype, int64_t m, int64_t n,
                       int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                       const void* x, int64_t x_offset,
                       int y_rank, const int64_t* y_dims, const int64_t* y_strides,
                       void* y, int64_t y_offset);

/* ---------------------------------------------------------------- logits head
 * No counterpart in the reference: the five calls its classification heads make on one
 * [m, n] matrix of logits -- reduce_sum, reduce_max, argmax, reduce_log_sum_exp and top_k
 * (largest, sorted) along the last axis -- in one launch and one read, for callers bound by
 * launch latency (m * n of a megabyte or so).  Every result equals what the separate call
 * writes (dlfx_reduce / dlfx_arg_reduce / dlfx_top_k on the same rows): the same fp64
 * accumulation rounded once, the first maximum, and among the k best larger values first,
 * -0.0 and +0.0 as one value, lower index first among equals.
 * x: m rows of n fp32 elements, row r at x + x_offset + r * row_stride (row_stride >= n).
 * Outputs are dense and any may be NULL: sum, max, log_sum_exp [m] fp32; argmax [m] int32;
 * best_values [m, k] fp32 and best_indices [m, k] int32 (k == 0: neither is written).
 * DLFX_F32 only; n <= DLFX_LOGITS_HEAD_MAX_N and k <= DLFX_LOGITS_HEAD_MAX_K (a row lives in
 * the registers of one wavefront), otherwise DLFX_ERR_TOO_LARGE: use the separate calls.
 */
#define DLFX_LOGITS_HEAD_MAX_N 2048
#define DLFX_LOGITS_HEAD_MAX_K 8
int dlfx_logits_head(dlfx_stream_t stream, int dtype, int64_t m, int64_t n,
                     const void* x, int64_t x_offset, int64_t row_stride,
                     void* sum, void* max, int32_t* argmax, void* log_sum_exp,
                     int64_t k, void* best_values, int32_t* best_indices);

/* ---------------------------------------------------------------- arg_reduce
 * Replaces gpgpu::dnn::arg_reduce<T> (gdnn.h:138-144; caller
 * reduce_detail.h:134-147).  The reduced axis is the last one of x_dims
 * (extent k, n_rows = size / k).  name: "argmax" | "argmin".  The first
 * occurrence wins ties (reduce_detail.h:120-128).  index_dtype DLFX_I32 is the
 * reference's Buffer<int>; DLFX_I64 writes 64-bit indices.
 */
size_t dlfx_arg_reduce_scratch_bytes(int dtype, int64_t n_rows, int64_t k);
int dlfx_arg_reduce(dlfx_stream_t stream, const char* name, int dtype, int index_dtype,
                    int64_t n_rows, int64_t k,
                    int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                    const void* x, int64_t x_offset,
                    int y_rank, const int64_t* y_dims, const int64_t* y_strides,
                    void* y, int64_t y_offset,
                    void* scratch, size_t scratch_bytes);

/* ---------------------------------------------------------------- scan
 * Replaces gpgpu::dnn::scan<T> (gdnn.h:124-129; caller
 * reduce_detail.h:244-253).  The scanned axis is the last one of dims (extent
 * n, m rows); x and y share dims and have independent strides; a reverse scan
 * arrives as flipped views (negative last strides).
 * name: "cumsum" | "cumprod" | "cummax" | "cummin".
 */
size_t dlfx_scan_scratch_bytes(int dtype, int64_t m, int64_t n);
int dlfx_scan(dlfx_stream_t stream, const char* name, int dtype, int64_t m, int64_t n,
              int exclusive, int rank, const int64_t* dims,
              const void* x, int64_t x_offset, const int64_t* x_strides,
              void* y, int64_t y_offset, const int64_t* y_strides,
              void* scratch, size_t scratch_bytes);

/* ---------------------------------------------------------------- sort
 * Replaces gpgpu::dnn::sort<T> (gdnn.h:157-161; caller
 * dlf/include/tensor/reorder_detail.h:617-627).  Sorts every row of the last
 * axis; dir 0 ascending, 1 descending.
 */
size_t dlfx_sort_scratch_bytes(int dtype, int64_t m, int64_t n);
int dlfx_sort(dlfx_stream_t stream, int dir, int dtype, int rank, const int64_t* dims,
              const void* x, int64_t x_offset, const int64_t* x_strides,
              void* y, int64_t y_offset, const int64_t* y_strides,
              void* scratch, size_t scratch_bytes);

/* ---------------------------------------------------------------- argsort
 * Replaces both gpgpu::dnn::argsort<T> overloads (gdnn.h:163-174; callers
 * reorder_detail.h:667-677, 951-963).  y == NULL is the index-only overload.
 * The order is stable: equal keys keep ascending source index, for both
 * directions.  index_dtype DLFX_I32 is the reference's Buffer<int32_t>.
 */
size_t dlfx_argsort_scratch_bytes(int dtype, int64_t m, int64_t n);
int dlfx_argsort(dlfx_stream_t stream, int dir, int dtype, int index_dtype,
                 int rank, const int64_t* dims,
                 const void* x, int64_t x_offset, const int64_t* x_strides,
                 void* y, int64_t y_offset, const int64_t* y_strides,
                 void* idx, int64_t i_offset, const int64_t* i_strides,
                 void* scratch, size_t scratch_bytes);

/* ---------------------------------------------------------------- top_k
 * Replaces gpgpu::dnn::top_k<T> (gdnn.h:176-182; caller
 * reorder_detail.h:1062-1073).  Selects `limit` elements per row of the last
 * axis of x (dir 1: largest, 0: smallest), written in sorted order; among equal
 * values the lowest source index is taken first.  y and idx share y_dims
 * (last extent == limit <= last extent of x_dims).
 */
size_t dlfx_top_k_scratch_bytes(int dtype, int64_t m, int64_t n, int64_t limit);
int dlfx_top_k(dlfx_stream_t stream, int64_t limit, int dir, int dtype, int index_dtype,
               int rank, const int64_t* x_dims, const int64_t* y_dims,
               const void* x, int64_t x_offset, const int64_t* x_strides,
               void* y, int64_t y_offset, const int64_t* y_strides,
               void* idx, int64_t i_offset, const int64_t* i_strides,
               void* scratch, size_t scratch_bytes);

/* ---------------------------------------------------------------- count
 * Replaces gpgpu::dnn::count<T> (gdnn.h:116-122; caller reduce.h:160-175): the number of
 * elements of each row that equal *value.  Views as for dlfx_reduce (kept dims then reduced
 * dims); y holds 32-bit counts.  `value` points to one element of `dtype` in host memory.
 */
size_t dlfx_count_scratch_bytes(int dtype, int64_t m, int64_t n);
int dlfx_count(dlfx_stream_t stream, int dtype, int64_t m, int64_t n, const void* value,
               int x_rank, const int64_t* x_dims, const int64_t* x_strides,
               const void* x, int64_t x_offset,
               int y_rank, const int64_t* y_dims, const int64_t* y_strides,
               int32_t* y, int64_t y_offset,
               void* scratch, size_t scratch_bytes);

/* ---------------------------------------------------------------- scan_nonzero
 * Replaces gpgpu::dnn::scan_nonzero<T> (gdnn.h:131-136; caller reduce.h:426-429): running
 * count of the elements that are not zero along the last axis, as 32-bit integers.  Views as
 * for dlfx_scan.
 */
size_t dlfx_scan_nonzero_scratch_bytes(int dtype, int64_t m, int64_t n);
int dlfx_scan_nonzero(dlfx_stream_t stream, int dtype, int64_t m, int64_t n,
                      int exclusive, int rank, const int64_t* dims,
                      const void* x, int64_t x_offset, const int64_t* x_strides,
                      int32_t* y, int64_t y_offset, const int64_t* y_strides,
                      void* scratch, size_t scratch_bytes);

/* ---------------------------------------------------------------- softmax family
 * Replaces gpgpu::dnn::softmax / logsoftmax / hardmax<T> (gdnn.h:253-264; callers
 * dnn_detail.h:292-295, 324-327, 352-355) on the rows of a contiguous [m, n] matrix.  The
 * reference works in place on x; here y may be x (in place) or another buffer.
 * name: "softmax" | "logsoftmax" | "hardmax".  Floating-point types (hardmax: int32, int64 too).
 * Scratch is optional: fewer than 256 rows that are too long for one workgroup's registers
 * (more than 32768 4-byte or 16384 8-byte elements) are cut into tiles that the whole device
 * works on when scratch of dlfx_softmax_scratch_bytes() bytes (16-byte aligned) is given, and
 * are walked by one workgroup per row when it is not (scratch NULL); every other shape needs none.
 */
size_t dlfx_softmax_scratch_bytes(int dtype, int64_t m, int64_t n);
int dlfx_softmax(dlfx_stream_t stream, const char* name, int dtype, int64_t m, int64_t n,
                 const void* x, int64_t x_offset, void* y, int64_t y_offset,
                 void* scratch, size_t scratch_bytes);

/* ---------------------------------------------------------------- merge
 * Replaces gpgpu::dnn::merge<T> (gdnn.h:147-155; caller reorder_detail.h:496-506).  x and y
 * are sorted along their last axis (dir 0 ascending, 1 descending) and share z's leading
 * extents; z's last extent is the sum of theirs.  Equal elements keep "x before y".
 * m = number of rows of z, n = its last extent.
 */
size_t dlfx_merge_scratch_bytes(int dtype, int64_t m, int64_t n);
int dlfx_merge(dlfx_stream_t stream, int dir, int dtype, int rank,
               const int64_t* x_dims, const int64_t* x_strides, const void* x, int64_t x_offset,
               const int64_t* y_dims, const int64_t* y_strides, const void* y, int64_t y_offset,
               const int64_t* z_dims, const int64_t* z_strides, void* z, int64_t z_offset,
               void* scratch, size_t scratch_bytes);

/* ---------------------------------------------------------------- gather_indices
 * Replaces gpgpu::dnn::gather_indices (gdnn.h:328-332; caller reduce.h:446-449): `indices`
 * holds the inclusive running count of non-zero elements over the m elements of a tensor of
 * extents `dims` in row-major order, n is the total.  For every element that raised the
 * count, its coordinates are written to column (count - 1) of a [rank, n] matrix
 * (row_major) or to row (count - 1) of an [n, rank] matrix.
 */
int dlfx_gather_indices(dlfx_stream_t stream, int64_t m, int64_t n, int row_major,
                        int rank, const int64_t* dims,
                        const int32_t* indices, int64_t indices_offset,
                        int32_t* output, int64_t output_offset);

/* ---------------------------------------------------------------- copy
 * Replaces the strided gpgpu::dnn::copy<T> (gdnn.h:14-17; routine xcopy.cpp:59-81): element
 * (i0, ..., ik) of the view (dims, x_strides) of x goes to the same element of the view
 * (dims, y_strides) of y.  A stride of 0 on the x side repeats elements.  The views must not
 * overlap unless they are the same dense view.  Every dtype (elements move as opaque words).
 * This is the device-side reorder(X, Y) the front-ends use before the in-place softmax family
 * and for sort / argsort along an axis of extent 1.
 */
int dlfx_copy(dlfx_stream_t stream, int dtype, int rank, const int64_t* dims,
              const void* x, int64_t x_offset, const int64_t* x_strides,
              void* y, int64_t y_offset, const int64_t* y_strides);

/* ---------------------------------------------------------------- fill
 * Replaces gpgpu::dnn::fill<T> (gdnn.h:20-26): every element of the view becomes *value (one
 * element of `dtype` in host memory, read before the call returns).
 */
int dlfx_fill(dlfx_stream_t stream, int dtype, int rank, const int64_t* dims, const int64_t* strides,
              void* x, int64_t x_offset, const void* value);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* DLFX_H_ */
