/*
 * minuet_hip.h — C ABI of libminuet_hip.so: the sparse-convolution hot path
 * (Map -> Gather -> grouped GEMM -> Scatter) as hand-written gfx950 HIP kernels.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void*; NULL = the null stream).  Inputs are borrowed and never
 * written; outputs are caller-allocated.  Temporaries come from the
 * library's own per-stream scratch arena (mnt_buffer_* below).  All work is
 * enqueued on the given stream; entry points that must read a scalar back
 * (documented per function) synchronise that stream before returning.
 *
 * Return convention: 0 on success, non-zero on failure; the message of the
 * last failure on the calling thread is returned by mnt_last_error().
 *
 * Each declaration cites the interface of the reference (paths relative to
 * the reference checkout) that a binding would route to it.
 */
#ifndef MINUET_HIP_H_
#define MINUET_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* integer element types of coordinate / index tensors */
#define MNT_INT32 0
#define MNT_INT64 1
/* feature element types */
#define MNT_FLOAT32 0
#define MNT_FLOAT16 1
#define MNT_BFLOAT16 2

/* activation applied by the fused forward's epilogue */
#define MNT_ACT_NONE 0
#define MNT_ACT_RELU 1
#define MNT_ACT_LEAKY_RELU 2
#define MNT_ACT_RELU6 3

#define MNT_MAX_NDIM 4

/* ---- library ----------------------------------------------------------- */

/* ABI version of this header (bumped on any signature change). */
int mnt_abi_version(void);

/* Message of the last failed call on this thread ("" if none).
 * Replaces MinuetException::what(), csrc/minuet/common/exception.h:9-21. */
const char *mnt_last_error(void);

/* ---- scratch arena (csrc/minuet/torch/cuda_memory_buffer.cu:6-47,
 *      csrc/minuet/cuda/buffer_pool.cu:100-216) ----------------------------- */
int mnt_buffer_preallocate(void *stream, size_t bytes);   /* cuda_preallocate_buffer */
int mnt_buffer_free(void *stream);                        /* cuda_free_buffers (synchronises) */
int mnt_buffer_set_growth(void *stream, float growth);    /* cuda_set_buffer_growth */
int mnt_buffer_set_page_size(void *stream, size_t bytes); /* cuda_set_buffer_page_size */
size_t mnt_buffer_total_size(void *stream);               /* cuda_buffer_total_size */
size_t mnt_buffer_used_size(void *stream);                /* cuda_buffer_used_size */
int mnt_reset_error(void);                                /* cuda_reset_error */
/* cuda_device_reset (csrc/minuet/torch/cuda_memory_buffer.cu:38,47).  The
 * reference calls cudaDeviceReset(), which also destroys the context PyTorch
 * allocates from; here the call waits for the device and gives back what the
 * LIBRARY holds on the current device (the arenas of every stream with their
 * pages, persistent blocks and pinned staging blocks) and clears the error
 * state, so that tensors of the process stay valid.  Pending two-phase calls
 * are forgotten. */
int mnt_device_reset(void);

/* Threading.  The library keeps state per (device, stream): the scratch arena,
 * what the two-phase entry points hand from their first call to their second,
 * a pinned staging block.  None of it is locked, so the contract is ONE CALLER
 * THREAD PER STREAM AT A TIME.  It is enforced: a call takes the state of every
 * stream it touches for the calling thread until it returns, and a thread
 * that enters on a stream another thread is inside of fails with a message
 * instead of racing.  Threads on different streams run side by side.
 * mnt_stream_acquire keeps a stream for the calling thread ACROSS calls (every
 * other thread's calls on it fail until mnt_stream_release); a caller that
 * hands a stream from thread to thread brackets its use with the pair.
 * The reference is called with the interpreter lock held for the whole of
 * every _C function (csrc/minuet/torch/common.h:17-21), which serialises
 * everything; a ctypes binding releases that lock, hence the rule here. */
int mnt_stream_acquire(void *stream);
int mnt_stream_release(void *stream);

/* How often, and for how long in total, library calls of this process have
 * made the host wait for a result of the device (every such wait is the poll
 * of one completion flag in pinned memory) since the last reset of the tally.
 * Either output may be null; reset != 0 clears the tally after reading it.
 * No counterpart in the reference, whose waits are stream synchronisations
 * inside its functions (e.g. csrc/minuet/cuda/functions/query_sorted_index.cu:
 * 13-119, three of them); bench.py reports the figure per Map step. */
int mnt_host_wait_stats(int64_t *waits_out, int64_t *nanoseconds_out, int reset);

/* ---- Map: coordinate sort ---------------------------------------------- */

/* Stable lexicographic arg-sort of coords[n, ndim] (dimension 0 most
 * significant); with batch_dims[num_batches+1] the result is batch-major.
 * indices_out[n] has element type index_dtype (= the type of batch_dims when
 * given).  sorted_coords_out (nullable) receives coords[indices_out] and
 * bounds_host_out (nullable, HOST, 8 x int64) the per-dimension minima [0..3]
 * and maxima [4..7] of the coordinates.
 * Synchronises once (coordinate bounds are read back to size the keys).
 * Replaces cuda_arg_sort_coordinates / cuda_multi_arg_sort_coordinates,
 * csrc/minuet/torch/cuda_arg_sort_coordinates.cu:8-70 and
 * csrc/minuet/cuda/functions/arg_sort_coodrinates.cu:273-469. */
int mnt_arg_sort_coordinates(const void *coords, int64_t n, int ndim, int coord_dtype,
                             const void *batch_dims, int64_t num_batches, int index_dtype,
                             void *indices_out, void *sorted_coords_out,
                             int64_t *bounds_host_out, void *stream);

/* ---- Map: unique ------------------------------------------------------- */

/* Run-end counting on SORTED coords: idx_out[0]=0, idx_out[i+1]=idx_out[i]+
 * [row i is the last of its run or of its batch]; *num_unique_out = idx_out[n].
 * Synchronises once.  Replaces the first half of cuda_unique_coordinates /
 * cuda_multi_unique_coordinates, csrc/minuet/torch/cuda_unique_coordinates.cu:8-85
 * (UniqueCoordinates::operator(), csrc/minuet/cuda/functions/unique_coordinates.cu:10-95). */
int mnt_unique_coordinates(const void *sorted_coords, int64_t n, int ndim, int coord_dtype,
                           const void *batch_dims, int64_t num_batches, int index_dtype,
                           void *idx_out, int64_t *num_unique_out, void *stream);

/* unique_out[idx[i]] = sorted_coords[i] wherever idx[i] != idx[i+1].
 * Replaces FillUniqueCoordinates, csrc/minuet/cuda/functions/unique_coordinates.cu:97-102. */
int mnt_fill_unique_coordinates(const void *sorted_coords, int64_t n, int ndim, int coord_dtype,
                                const void *idx, int index_dtype, void *unique_out, void *stream);

/* Target voxel set of a strided layer in one call: floor(c / stride) * stride,
 * sort, unique.  Phase 1 returns the count (synchronises once) and keeps the
 * sorted keys in the arena slot of this stream; phase 2 writes the coordinates
 * and target_batch_dims_out[num_batches+1] (nullable, element type
 * index_dtype).  Phase 2 must follow phase 1 on the same stream with no other
 * library call in between.  source_bounds_host (nullable, 8 x int64: minima
 * in [0..3], maxima in [4..7]) spares the reduction over the coordinates and
 * its wait when the caller knows them.  Replaces the torch expression in
 * KernelMapCache.get_target_coordinates, minuet/nn/convolutions.py:84-99. */
int mnt_target_coordinates_count(const void *source_coords, int64_t n, int ndim, int coord_dtype,
                                 const int64_t *target_stride, const void *batch_dims,
                                 int64_t num_batches, int index_dtype,
                                 const int64_t *source_bounds_host,
                                 int64_t *num_targets_out, void *stream);
int mnt_target_coordinates_fill(void *target_coords_out, void *target_batch_dims_out,
                                void *stream);

/* Both phases in one call for a caller that hands over room for the worst case:
 * target_coords_out holds capacity >= n rows, of which the first
 * *num_targets_out are written (there are never more targets than sources).
 * The coordinates are written while the host waits for the count, so nothing
 * is launched after the wait.  Needs n > 0.  Same reference expression
 * (minuet/nn/convolutions.py:84-99). */
int mnt_target_coordinates(const void *source_coords, int64_t n, int ndim, int coord_dtype,
                           const int64_t *target_stride, const void *batch_dims,
                           int64_t num_batches, int index_dtype,
                           const int64_t *source_bounds_host, void *target_coords_out,
                           int64_t capacity, void *target_batch_dims_out,
                           int64_t *num_targets_out, void *stream);

/* ---- Map: query -------------------------------------------------------- */

/* Dense kernel map: kernel_map_out[o*T + t] = j with sources[j] == targets[t] +
 * offsets[o] (same batch), else -1.  sources/targets sorted; offsets[O, ndim]
 * is a device array of coord_dtype.  batch dims (both or neither) have element
 * type batch_dtype and num_batches+1 entries; kernel_map_out has out_dtype.
 * Synchronises once (bounds).  Replaces cuda_query_sorted_index_with_offsets /
 * cuda_multi_query_sorted_index_with_offsets,
 * csrc/minuet/torch/cuda_sparse_convolution_mapping.cu:9-93. */
int mnt_query_sorted_index_with_offsets(const void *sources, int64_t num_sources,
                                        const void *targets, int64_t num_targets,
                                        const void *offsets, int64_t num_offsets,
                                        int ndim, int coord_dtype,
                                        const void *source_batch_dims,
                                        const void *target_batch_dims,
                                        int64_t num_batches, int batch_dtype,
                                        void *kernel_map_out, int out_dtype, void *stream);

/* sizes_out[o] = #{t : kernel_map[o,t] != -1} (device, index_dtype).
 * Replaces cuda_compute_kernel_map_sizes,
 * csrc/minuet/torch/cuda_sparse_convolution_mapping.cu:95-121. */
int mnt_compute_kernel_map_sizes(const void *kernel_map, int64_t num_offsets,
                                 int64_t num_targets, int index_dtype, void *sizes_out,
                                 void *stream);

/* mnt_compute_kernel_map_sizes for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): same arguments, same kernels, same result, but the per-(offset,
 * tile of 512 targets) hit counts live in a device array that is part of the
 * library image (MNT_STATIC_SCRATCH_WORDS 32-bit words, held by every GPU the
 * library runs on until the process ends) instead of the scratch arena.  The
 * call makes no hipMalloc / hipFree and touches no arena; a map that needs more
 * than num_offsets * (ceil(num_targets / 512) + 1) <= MNT_STATIC_SCRATCH_WORDS
 * words is refused with an error.  All calls on one GPU share the array:
 * calls that overlap on one GPU (two streams, two threads) race; calls on one
 * stream are ordered.  The first call on a device looks the array's address
 * up and should be made outside stream capture.  No counterpart in the
 * reference, which allocates from its buffer pool in every call. */
#define MNT_STATIC_SCRATCH_WORDS (1u << 20)
int mnt_compute_kernel_map_sizes_static(const void *kernel_map, int64_t num_offsets,
                                        int64_t num_targets, int index_dtype, void *sizes_out,
                                        void *stream);

/* Rank tables: target_masks[o,t] = rank of the hit among the hits of row o in
 * target order, source_masks[o, kernel_map[o,t]] = the same rank, -1 elsewhere.
 * Replaces cuda_compute_kernel_map_masks,
 * csrc/minuet/torch/cuda_sparse_convolution_mapping.cu:123-156. */
int mnt_compute_kernel_map_masks(const void *kernel_map, int64_t num_offsets,
                                 int64_t num_sources, int64_t num_targets, int index_dtype,
                                 void *source_masks_out, void *target_masks_out, void *stream);

/* Kernel-map build of KernelMapCache.get_kernel_map on a miss
 * (minuet/nn/convolutions.py:147-170) in two calls with no intermediate
 * tensors on the host side.
 *
 * mnt_kernel_map_query: dense map (kernel_map_out, int32 [O,T], rows in offset
 * order), per-offset sizes and the stable ascending size order (reorder != 0;
 * identity otherwise).  offsets_host[O*ndim] is a HOST array of int64.
 * order_host_out[j] is the offset of output row j and sizes_host_out[j] its
 * hit count.  source_bounds_host / target_bounds_host (nullable, 8 x int64:
 * per-dimension minima in [0..3], maxima in [4..7]) are the coordinate bounds
 * when the caller already knows them, e.g. from mnt_arg_sort_coordinates;
 * whatever is missing is reduced on the device.  bounds_host_out (nullable,
 * 16 x int64) receives the bounds used (sources then targets).  Synchronises
 * once for the sizes and once more only when bounds had to be computed.
 *
 * mnt_kernel_map_emit: must directly follow the query on the same stream, with
 * kernel_map_out still alive.  Writes any non-null output: the rank tables
 * source_masks_out [O,S] / target_masks_out [O,T] (row j <-> offset order[j]),
 * the pair lists in_idx_out / out_idx_out [nnz] (rows concatenated in output
 * row order, hits in target order) and device copies of sizes / order.
 * Does not synchronise.  Replaces the chain compute_kernel_map_sizes ->
 * torch.sort -> kernel_map[order] -> compute_kernel_map_masks. */
int mnt_kernel_map_query(const void *sources, int64_t num_sources,
                         const void *targets, int64_t num_targets,
                         const int64_t *offsets_host, int64_t num_offsets,
                         int ndim, int coord_dtype,
                         const void *source_batch_dims, const void *target_batch_dims,
                         int64_t num_batches, int batch_dtype, int reorder,
                         const int64_t *source_bounds_host, const int64_t *target_bounds_host,
                         int64_t *bounds_host_out, int32_t *kernel_map_out,
                         int64_t *sizes_host_out, int64_t *order_host_out, void *stream);
int mnt_kernel_map_emit(int32_t *source_masks_out, int32_t *target_masks_out,
                        int32_t *in_idx_out, int32_t *out_idx_out,
                        int32_t *sizes_dev_out, int32_t *order_dev_out, void *stream);

/* mnt_kernel_map_query and mnt_kernel_map_emit in one call, for callers that
 * can hand over the pair lists before their length is known: in_idx_out /
 * out_idx_out (nullable, together) have room for list_capacity >= O * T
 * entries each, of which the first nnz = sum(sizes) are written.  The tables
 * are written while the host waits for the sizes, so the call costs one wait
 * and no launch after it.  Needs S, T, O > 0.  Same reference code
 * (minuet/nn/convolutions.py:147-170). */
int mnt_kernel_map_build(const void *sources, int64_t num_sources,
                         const void *targets, int64_t num_targets,
                         const int64_t *offsets_host, int64_t num_offsets,
                         int ndim, int coord_dtype,
                         const void *source_batch_dims, const void *target_batch_dims,
                         int64_t num_batches, int batch_dtype, int reorder,
                         const int64_t *source_bounds_host, const int64_t *target_bounds_host,
                         int64_t *bounds_host_out, int32_t *kernel_map_out,
                         int32_t *source_masks_out, int32_t *target_masks_out,
                         int32_t *in_idx_out, int32_t *out_idx_out, int64_t list_capacity,
                         int32_t *sizes_dev_out, int32_t *order_dev_out,
                         int64_t *sizes_host_out, int64_t *order_host_out, void *stream);

/* The pair lists alone, for callers that need neither the dense map nor the rank
 * tables: arguments as mnt_kernel_map_build without kernel_map_out and the
 * two tables; in_idx_out / out_idx_out have room for list_capacity >= O * T
 * entries each, of which the first nnz = sum(sizes) are written.  The query
 * keeps each wavefront's hits compacted in scratch instead of writing the
 * dense map, and one more launch moves them to their list positions, so the
 * dense [O, T] map is neither written nor read back.  One wait (sizes and
 * order; the lists are being written meanwhile), one more only when bounds
 * are missing.  Needs S, T, O > 0.  Same reference code
 * (minuet/nn/convolutions.py:147-170, with the lists taking the place of the
 * rank tables of csrc/minuet/cuda/functions/scan.cu:292-365). */
int mnt_kernel_map_lists(const void *sources, int64_t num_sources,
                         const void *targets, int64_t num_targets,
                         const int64_t *offsets_host, int64_t num_offsets,
                         int ndim, int coord_dtype,
                         const void *source_batch_dims, const void *target_batch_dims,
                         int64_t num_batches, int batch_dtype, int reorder,
                         const int64_t *source_bounds_host, const int64_t *target_bounds_host,
                         int64_t *bounds_host_out,
                         int32_t *in_idx_out, int32_t *out_idx_out, int64_t list_capacity,
                         int32_t *sizes_dev_out, int32_t *order_dev_out,
                         int64_t *sizes_host_out, int64_t *order_host_out, void *stream);

/* The Map step of a stride-1 (submanifold) layer on raw input in ONE call:
 * arg-sort of coords[n, ndim] (one cloud, no batch_dims) as
 * mnt_arg_sort_coordinates does it (indices_out int32 [n], sorted_coords_out
 * [n, ndim]) followed by the pair lists of the kernel map of the sorted cloud
 * onto itself as mnt_kernel_map_lists builds them (offsets_host int64 [O, ndim],
 * lists with room for list_capacity >= O * n entries, sizes / order on the
 * device and on the host).  bounds_host_out (8 x int64) receives the
 * coordinate minima [0..3] and maxima [4..7].
 * For clouds of 2 048 .. 2 097 152 rows and up to 64 offsets the whole step is
 * a chain of six launches (bounds, dealing into a slab per bucket, listing the
 * ranking work, ranking, query, list placing) that never returns to the host
 * in between: key layouts, bucket totals and the query plan are worked out on
 * the device, and the host waits once, for the sizes.  Offsets that come in pairs d / -d are looked up once
 * per pair there: a cloud mapped onto itself has the pair list of -d equal to
 * the pair list of d with the two indices exchanged, in the same order.  A
 * cloud the chain declines (a bucket beyond 4 096 rows, keys that do not fit
 * a word, equal rows under paired offsets) and every other shape go through
 * the two separate entry points inside this call; the results are the same.
 * Replaces F.arg_sort_coordinates (minuet/nn/functional/indexing.py:14-56)
 * followed by the miss path of KernelMapCache.get_kernel_map
 * (minuet/nn/convolutions.py:147-170). */
int mnt_sorted_kernel_map_lists(const void *coords, int64_t n, int ndim, int coord_dtype,
                                const int64_t *offsets_host, int64_t num_offsets, int reorder,
                                int32_t *indices_out, void *sorted_coords_out,
                                int32_t *in_idx_out, int32_t *out_idx_out, int64_t list_capacity,
                                int32_t *sizes_dev_out, int32_t *order_dev_out,
                                int64_t *bounds_host_out, int64_t *sizes_host_out,
                                int64_t *order_host_out, void *stream);

/* Target-major row lists of a kernel map whose pair lists exist, from its dense
 * int32 map kernel_map[O, T] (original offset order): row_ptr_out[T + 1] and
 * out_pos_out[nnz] such that the product of list entry p (list row j in the
 * order order_host[j] -> offset, NULL = offset order, sizes_host[j] hits each,
 * hits in target order: the numbering of in_idx / out_idx) belongs at buffer
 * row out_pos_out[p] and target t owns the consecutive buffer rows
 * row_ptr_out[t] .. row_ptr_out[t + 1] - 1, in list-row order.  Feeds
 * mnt_sparse_convolution_forward_rows.  Does not wait for the device.  At most
 * 1024 offsets.  Takes the place of the rank table target_masks
 * (csrc/minuet/cuda/functions/scan.cu:292-365) as what Scatter is driven by. */
int mnt_kernel_map_row_lists(const int32_t *kernel_map, int64_t num_offsets, int64_t num_targets,
                             const int64_t *sizes_host, const int64_t *order_host,
                             int32_t *row_ptr_out, int32_t *out_pos_out, void *stream);

/* Per-offset (in_idx, out_idx) pair lists from a dense int32 kernel map: for row
 * o the hits in target order are written at list positions
 * cumsum_host[o] .. cumsum_host[o]+sizes[o]-1 (cumsum_host[O+1], HOST, exclusive
 * prefix of the row sizes, e.g. from mnt_compute_kernel_map_sizes).  This is
 * the inverse of the two rank tables of mnt_compute_kernel_map_masks. */
int mnt_kernel_map_pair_lists(const int32_t *kernel_map, int64_t num_offsets,
                              int64_t num_targets, const int64_t *cumsum_host,
                              int32_t *in_idx_out, int32_t *out_idx_out, void *stream);

/* The two halves of mnt_kernel_map_query for callers that may never need the
 * rank tables (the single-kernel forward reads the dense map only):
 * mnt_kernel_map_dense runs the query alone (same arguments and kernel_map_out
 * as mnt_kernel_map_query) and does not wait for anything when both bounds are
 * given; mnt_kernel_map_tables derives sizes and order from such a dense map
 * later, after which mnt_kernel_map_emit writes the tables as usual.  Same
 * reference code as mnt_kernel_map_query (minuet/nn/convolutions.py:147-170). */
int mnt_kernel_map_dense(const void *sources, int64_t num_sources,
                         const void *targets, int64_t num_targets,
                         const int64_t *offsets_host, int64_t num_offsets,
                         int ndim, int coord_dtype,
                         const void *source_batch_dims, const void *target_batch_dims,
                         int64_t num_batches, int batch_dtype,
                         const int64_t *source_bounds_host,
                         const int64_t *target_bounds_host,
                         int64_t *bounds_host_out,
                         int32_t *kernel_map_out, void *stream);
int mnt_kernel_map_tables(const int32_t *kernel_map, int64_t num_sources,
                          int64_t num_targets, int64_t num_offsets, int reorder,
                          int64_t *sizes_host_out, int64_t *order_host_out, void *stream);

/* ---- GMaS: padding plan (host only) -------------------------------------- */

/* Greedy contiguous grouping of size-ascending offsets: extend a bucket while
 * (max*count - sum)/sum <= threshold; has_threshold == 0 -> one bucket,
 * threshold < 0 -> singletons.  Writes boundaries (first 0, last O) and
 * returns their count through num_boundaries_out (buckets_out holds O+1).
 * Replaces GeneratePaddingBuckets,
 * csrc/minuet/cuda/functions/sparse_convolution.cu:16-43. */
int mnt_generate_padding_buckets(const int64_t *sizes_host, int64_t num_offsets,
                                 int has_threshold, double threshold,
                                 int64_t *buckets_out, int64_t *num_boundaries_out);

/* Each offset of a bucket owns max-size-in-bucket rows; cumsum_out[O+1].
 * Replaces ComputeCumsumKernelPaddedSizes, sparse_convolution.cu:272-292. */
int mnt_cumsum_kernel_padded_sizes(const int64_t *sizes_host, int64_t num_offsets,
                                   const int64_t *buckets, int64_t num_boundaries,
                                   int64_t *cumsum_out);

/* ---- GMaS: forward ------------------------------------------------------- */

/* out[T, Cout] = sum over offsets of gather(sources) x weights[order[o]],
 * scattered target-stationary in offset order with fp32 accumulation.
 * sources[S, Cin], weights[O, Cin, Cout], out: float_dtype; masks [O,S] / [O,T],
 * order (nullable) and sizes [O]: device arrays of index_dtype.
 * sizes_host (nullable, int64[O]) spares the read-back of sizes; without it
 * the call synchronises once.  gather_tile / scatter_tile are elements per
 * lane (0 = pick automatically).  parallel is accepted for signature
 * compatibility (all offsets run in one grouped launch).
 * gather_index (nullable, int32[nnz]): the in_idx list of mnt_kernel_map_emit
 * for the same kernel map, i.e. per offset, in the order of `order`, the
 * source row of each buffer row.  With it the Gather step is folded into the
 * GEMM's operand load (no gather buffer, source_masks unused); without it
 * the three steps run as separate kernels.  Both forms give identical output.
 * Replaces cuda_sparse_convolution_forward,
 * csrc/minuet/torch/cuda_sparse_convolution_forward.cu:136-213 and
 * SparseConvolutionForward::operator(),
 * csrc/minuet/cuda/functions/sparse_convolution.cu:504-661. */
int mnt_sparse_convolution_forward(int64_t gather_tile, int64_t scatter_tile,
                                   int allow_shortcut_matmul, int64_t parallel,
                                   int has_threshold, double threshold,
                                   const void *sources, const void *weights,
                                   const void *source_masks, const void *target_masks,
                                   const void *kernel_map_order, const void *kernel_map_sizes,
                                   const int64_t *sizes_host,
                                   int64_t num_sources, int64_t num_targets,
                                   int64_t num_offsets, int64_t num_source_features,
                                   int64_t num_target_features,
                                   int index_dtype, int float_dtype,
                                   const int32_t *gather_index,
                                   void *out, void *stream);

/* The same forward with an epilogue applied to every summed output row before
 * it is rounded to float_dtype:
 *   out[t][c] = act(sum[t][c] * channel_scale[c] + channel_shift[c] + residual[t][c])
 * channel_scale / channel_shift: fp32[Cout] device vectors, residual: [T, Cout]
 * of float_dtype (16-byte aligned); each is skipped when NULL.  activation is
 * one of MNT_ACT_*; negative_slope is used by MNT_ACT_LEAKY_RELU only.  This is
 * how the layers that follow a convolution in the reference's networks
 * (the bias add of minuet/nn/convolutions.py:496-497, an inference-mode
 * minuet/nn/normalizations.py BatchNorm, minuet/nn/activations.py ReLU /
 * LeakyReLU / ReLU6 and a residual sum) are absorbed into Scatter's single
 * write of the output row.
 * packed_weights (nullable): the output of mnt_pack_weights for `weights`,
 * kept by the caller for as long as the weights do not change; the pass then
 * skips its own packing.  Packed weights are in the layer's own offset order,
 * so with a kernel_map_order the call also needs order_host (int64[O], the
 * host copy of kernel_map_order; NULL otherwise). */
int mnt_sparse_convolution_forward_fused(int64_t gather_tile, int64_t scatter_tile,
                                         int allow_shortcut_matmul, int64_t parallel,
                                         int has_threshold, double threshold,
                                         const void *sources, const void *weights,
                                         const void *source_masks, const void *target_masks,
                                         const void *kernel_map_order,
                                         const void *kernel_map_sizes,
                                         const int64_t *sizes_host,
                                         int64_t num_sources, int64_t num_targets,
                                         int64_t num_offsets, int64_t num_source_features,
                                         int64_t num_target_features,
                                         int index_dtype, int float_dtype,
                                         const int32_t *gather_index,
                                         const float *channel_scale, const float *channel_shift,
                                         const void *residual, int activation,
                                         float negative_slope,
                                         const void *packed_weights,
                                         const int64_t *order_host,
                                         void *out, void *stream);

/* The same convolution driven by lists instead of rank tables: the grouped GEMM
 * reads the source row of list entry p through in_idx[p] (Gather folded into
 * its operand load) and writes the product to buffer row out_pos[p]; Scatter
 * then sums, for target t, the CONSECUTIVE buffer rows row_ptr[t] ..
 * row_ptr[t + 1] - 1 in fp32 and applies the epilogue: no rank table and no
 * row list is read, the buffer streams through once.  in_idx: the list of
 * mnt_kernel_map_emit / _lists; out_pos, row_ptr: mnt_kernel_map_row_lists;
 * sizes_host / order_host (int64[O], order_host NULL = offset order) as those
 * calls return them; weights [O, Cin, Cout] in the layer's own offset order,
 * packed_weights (nullable) their mnt_pack_weights form.  Rows are summed in
 * list-row order, the centre offset with the others (the reference adds it
 * last as well, sparse_convolution.cu:647-660), so results agree with
 * mnt_sparse_convolution_forward to rounding.  Epilogue arguments as in
 * mnt_sparse_convolution_forward_fused.  Same reference code
 * (csrc/minuet/cuda/functions/sparse_convolution.cu:504-661). */
int mnt_sparse_convolution_forward_rows(int64_t scatter_tile, const void *sources,
                                        const void *weights, const int64_t *sizes_host,
                                        const int64_t *order_host, const int32_t *in_idx,
                                        const int32_t *out_pos, const int32_t *row_ptr,
                                        int64_t num_sources, int64_t num_targets,
                                        int64_t num_offsets, int64_t num_source_features,
                                        int64_t num_target_features, int float_dtype,
                                        const float *channel_scale, const float *channel_shift,
                                        const void *residual, int activation, float negative_slope,
                                        const void *packed_weights, void *out, void *stream);

/* Offset groups of a 3 x 3 x 3 layer, from its dense int32 map
 * kernel_map[27, T] (original offset order).  Along each of the three axes the
 * 27 offsets fall into 9 groups of 3 that differ along that axis only;
 * group_offsets_host int32 [3][9][3] lists them (offset index of member m of
 * group j along axis a; every axis lists each of the 27 offsets once).  A
 * target belongs to a group when any of the group's offsets reaches a source.
 * The axis with the fewest (group, target) rows is chosen ON THE DEVICE and
 * written to head_out[0]; head_out[1 + j] = rows of group j (head_out: 16 x
 * int32); rank_out int32 [9, T] = rank of target t among the rows of group j
 * (-1: not in the group); src_out int32 [9 * T, 4] = the three source rows (-1:
 * none) of row i of group j at [j * T + i] (fourth word unused; 16-byte
 * aligned).  Three launches, nothing is read back.  Feeds
 * mnt_sparse_convolution_forward_groups.  No counterpart in the reference,
 * whose kernel map has one row per offset
 * (minuet/nn/convolutions.py:147-170). */
int mnt_kernel_map_offset_groups(const int32_t *kernel_map, int64_t num_targets,
                                 const int32_t *group_offsets_host, int32_t *rank_out,
                                 int32_t *src_out, int32_t *head_out, void *stream);

/* The convolution of mnt_sparse_convolution_forward over the offset groups of
 * mnt_kernel_map_offset_groups (rank, src, head, group_offsets_host as there):
 * the three offsets of a group are multiplied in one product whose K dimension
 * is their three weight matrices one after the other, the data row of a target
 * being its three source rows end to end (zeros where an offset has none), so
 * a group writes one buffer row per target it reaches instead of one per
 * (offset, target) pair; Scatter then sums at most 9 rows per target.  For
 * clouds that are dense along the chosen axis this halves the buffer traffic
 * that bounds wide layers, at 1.3 x the multiplications.  16-bit features
 * whose rows are whole 128-byte chunks, Cout a multiple of 8, 27 offsets;
 * packed_weights = mnt_pack_weights of the weights in the layer's own offset
 * order.  Sums differ from the other forms' in order only.  Epilogue arguments
 * as in mnt_sparse_convolution_forward_fused.  Same reference code
 * (csrc/minuet/cuda/functions/sparse_convolution.cu:504-661). */
int mnt_sparse_convolution_forward_groups(const void *sources, const void *packed_weights,
                                          const int32_t *rank, const int32_t *src,
                                          const int32_t *head, const int32_t *group_offsets_host,
                                          int64_t num_sources, int64_t num_targets,
                                          int64_t num_source_features, int64_t num_target_features,
                                          int float_dtype, const float *channel_scale,
                                          const float *channel_shift, const void *residual,
                                          int activation, float negative_slope, void *out,
                                          void *stream);

/* Weights [O, Cin, Cout] -> the layout the matrix kernels stage:
 * packed[O][Np][Kp] = W^T per offset, K-contiguous, zero-padded to
 * Np = ceil(Cout / 32) * 32 rows of Kp = ceil(Cin * e / 128) * 128 / e elements
 * (e = element size).  Offsets stay in the order given.  Takes the place of
 * PermuteWeights (csrc/minuet/cuda/kernels/permute_weights.cuh:8-36), which the
 * reference runs inside every forward. */
int mnt_pack_weights(const void *weights, int64_t num_offsets, int64_t num_source_features,
                     int64_t num_target_features, int float_dtype, void *packed_out,
                     void *stream);

/* Timers used by the autotuner: run the named stage once on scratch buffers and
 * return the elapsed milliseconds through ms_out (synchronise).
 * Replace cuda_time_gather / cuda_time_scatter / cuda_time_gemm,
 * csrc/minuet/torch/cuda_sparse_convolution_forward.cu:7-134 (TimeGather,
 * TimeScatter, TimeGEMM: csrc/minuet/cuda/functions/sparse_convolution.cu:294-502). */
int mnt_time_gather(int64_t tile, int allow_shortcut_matmul, int has_threshold, double threshold,
                    const void *source_masks, const void *kernel_map_sizes,
                    int64_t num_sources, int64_t num_targets, int64_t num_offsets,
                    int64_t num_source_features, int64_t num_target_features,
                    int index_dtype, int float_dtype, float *ms_out, void *stream);
int mnt_time_scatter(int64_t tile, int allow_shortcut_matmul, int has_threshold, double threshold,
                     const void *target_masks, const void *kernel_map_sizes,
                     int64_t num_sources, int64_t num_targets, int64_t num_offsets,
                     int64_t num_source_features, int64_t num_target_features,
                     int index_dtype, int float_dtype, float *ms_out, void *stream);
int mnt_time_gemm(int allow_shortcut_matmul, int64_t parallel, int has_threshold, double threshold,
                  const void *weights, const void *kernel_map_sizes,
                  int64_t num_sources, int64_t num_targets, int64_t num_offsets,
                  int64_t num_source_features, int64_t num_target_features,
                  int index_dtype, int float_dtype, float *ms_out, void *stream);

/* The same convolution computed output-stationary from the dense kernel map
 * instead of the rank tables: kernel_map[O, T] (int32, source row per
 * (offset, target) in the ORIGINAL offset order, -1 for none), i.e. the output
 * of mnt_query_sorted_index_with_offsets / mnt_kernel_map_query; weights
 * [O, Cin, Cout] in the same offset order.  No gather or GEMM-output buffer is
 * written: each wavefront keeps 32 output rows in its matrix accumulators and
 * walks the offsets.  Requires Cin * sizeof(element) to be a multiple of 16
 * and at most 2048, Cout % 4 == 0 and Cout <= 512.  16-bit rows of 4 or 8
 * bytes (2 or 4 input channels) are taken as well when `weights` is given,
 * Cout <= 128 and ceil(O * Cin / 16) * ceil(Cout / 32) KiB + 18 KiB of LDS
 * stay within 64 KiB: such layers, and 16-byte rows under the same
 * conditions, run a kernel that lays the offsets side by side along K and
 * reads `weights` as they are (packed_weights is not used).  Rows beyond 128 bytes are
 * walked in chunks and more than 128 output channels in groups of 128; the
 * form pays for rows of up to 128 bytes and up to 128 output channels, where
 * the three-kernel form is bound by its buffer traffic, and loses beyond
 * (its matrix work covers the empty (offset, target) pairs too).  The epilogue arguments are those of
 * mnt_sparse_convolution_forward_fused; packed_weights (nullable) is the
 * output of mnt_pack_weights for `weights`.  Results agree with the other forms to
 * rounding (sums are kept in fp32 over all offsets and rounded once).
 * Covers the same reference code as mnt_sparse_convolution_forward
 * (csrc/minuet/cuda/functions/sparse_convolution.cu:504-661); the reference
 * has no single-kernel counterpart. */
int mnt_sparse_convolution_forward_implicit(const void *sources, const void *weights,
                                            const int32_t *kernel_map,
                                            int64_t num_sources, int64_t num_targets,
                                            int64_t num_offsets, int64_t num_source_features,
                                            int64_t num_target_features, int float_dtype,
                                            const float *channel_scale,
                                            const float *channel_shift, const void *residual,
                                            int activation, float negative_slope,
                                            const void *packed_weights,
                                            void *out, void *stream);

/* The dense kernel map of the transposed layer that shares a forward layer's
 * map (minuet/nn/convolutions.py:119-133 reuses the forward map with the rank
 * tables swapped): inverse_out[O, S] with inverse_out[o][m] = t wherever
 * kernel_map[o][t] = m, -1 elsewhere.  Feeds
 * mnt_sparse_convolution_forward_implicit for transposed convolutions. */
int mnt_kernel_map_invert(const int32_t *kernel_map, int64_t num_offsets, int64_t num_targets,
                          int64_t num_sources, int32_t *inverse_out, void *stream);

/* ---- Map: building a pass's coordinates and kernel maps ahead ------------- */

/* A network that has seen one cloud asks for the same coordinate levels and
 * kernel maps, in the same order, for the next one.  With the list of those
 * requests (the items below) the library builds all of them for a new cloud on
 * a worker thread and a stream of its own while the caller goes on enqueueing
 * layers: mnt_lookahead_start returns at once, mnt_lookahead_wait(item) blocks
 * until that item is built, makes `stream` wait for the kernels that wrote it
 * and returns its size.  Every item is built by the entry point a caller would
 * use for it (mnt_target_coordinates, mnt_kernel_map_dense,
 * mnt_kernel_map_tables + mnt_kernel_map_emit, mnt_kernel_map_invert), so the
 * results are theirs; outputs go to buffers the caller allocated for the worst
 * case (no level has more rows than level 0).
 *
 * Levels: level 0 is the cloud given to mnt_lookahead_start; a COORDS item
 * makes level `target_level` from level `source_level`.
 *   MNT_AHEAD_COORDS  stride[ndim]; out0 = coordinates [capacity, ndim],
 *                     out1 = batch boundaries [num_batches + 1] (batched clouds);
 *                     size = number of rows.
 *   MNT_AHEAD_DENSE   source_level, target_level, offsets (host, int64
 *                     [num_offsets, ndim], alive until the session ends);
 *                     out0 = kernel map [num_offsets, T] int32 (capacity >=
 *                     num_offsets * T ints); size = T.
 *   MNT_AHEAD_TABLES  dense_item, reorder; out0 / out1 = rank tables [O, S] /
 *                     [O, T], out2 / out3 = pair lists (capacity entries each),
 *                     out4 / out5 = device sizes / order [O]; host0 / host1 =
 *                     host sizes / order int64 [O]; size = number of pairs.
 *   MNT_AHEAD_INVERT  dense_item; out0 = inverse map [O, S]; size = S.
 * bounds_out (nullable, 8 x int64 per level, -1 flags unknown in
 * bounds_known_out) receives the coordinate bounds of every level.
 * One session per process at a time; mnt_lookahead_finish waits for the worker
 * to go idle (items nobody waited for are still built, or skipped after an
 * error) and makes `stream` wait for everything it enqueued: call it before
 * the buffers are released.  An item that fails makes its wait return non-zero
 * with the message in mnt_last_error(); items that depend on it fail too.
 * No counterpart in the reference, whose KernelMapCache builds every map when
 * a layer first asks for it (minuet/nn/convolutions.py:58-173). */
enum { MNT_AHEAD_COORDS = 0, MNT_AHEAD_DENSE = 1, MNT_AHEAD_TABLES = 2, MNT_AHEAD_INVERT = 3 };
typedef struct mnt_lookahead_item {
  int32_t kind;
  int32_t source_level, target_level, dense_item, reorder;
  int32_t reserved;
  int64_t stride[4];
  const int64_t *offsets;
  int64_t num_offsets;
  int64_t capacity;
  void *out0, *out1, *out2, *out3, *out4, *out5;
  int64_t *host0, *host1;
} mnt_lookahead_item;
int mnt_lookahead_start(const void *coords, int64_t n, int ndim, int coord_dtype,
                        const void *batch_dims, int64_t num_batches, int index_dtype,
                        const int64_t *bounds_host, const mnt_lookahead_item *items,
                        int num_items, int num_levels, int64_t *bounds_out,
                        int32_t *bounds_known_out, void *stream);
int mnt_lookahead_wait(int item, void *stream, int64_t *size_out);
int mnt_lookahead_finish(void *stream);

/* ---- stage timing -------------------------------------------------------- */

/* Streams `bytes` of device memory through one plain kernel (kind 0: copy a -> b,
 * `bytes` read and `bytes` written; 1: read only; 2: write only), `repeats`
 * times back to back between two stream events, and returns the milliseconds
 * of ONE pass: the memory ceilings of the machine at hand, which a benchmark
 * quotes beside the vendor's peak.  The buffers come from the stream's scratch
 * arena.  No counterpart in the reference. */
int mnt_time_memory(int kind, size_t bytes, int repeats, float *ms_out, void *stream);

/* Facts of the current device for a benchmark's record, facts_out[0..5]:
 * compute units, engine clock (kHz), memory clock (kHz), memory bus width
 * (bits), L2 bytes, device memory bytes.  No counterpart in the reference. */
int mnt_device_facts(int64_t *facts_out, int capacity);

/* Launches per timing run of mnt_time_gather / _scatter / _gemm (default 1, the
 * reference's protocol: one launch between two events, which also times the
 * launch gap).  With more, the launches go back to back between the events and
 * the time of one is returned: the sustained rate of the kernel alone. */
int mnt_timer_repeats(int repeats);

/* mnt_profile_enable(1) makes the instrumented entry points (sort, query, emit,
 * forward) record a timestamp event on their stream after every stage; (0)
 * turns that off.  Either call discards what was recorded so far.
 * mnt_profile_read waits for the last event and returns up to `capacity`
 * intervals between consecutive marks, in recording order: ms_out[i] and the
 * NUL-terminated stage name at labels_out + i*label_stride.  Intervals named
 * "enter:*" are the gaps between two entry points (host time).  Reading clears
 * the record.  No counterpart in the reference; used by the benchmark for
 * per-kernel roofline figures. */
int mnt_profile_enable(int on);
int mnt_profile_read(int capacity, float *ms_out, char *labels_out, int label_stride,
                     int *count_out);

#ifdef __cplusplus
}
#endif
#endif /* MINUET_HIP_H_ */
