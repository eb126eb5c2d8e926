/*
 * gear_hip.h — C ABI of libgearhip.so: the MI355X (gfx950) replay-sampling hot path of GEAR.
 *
 * Everything here is plain C: raw pointers, 64-bit sizes, a `void* stream` that is a
 * hipStream_t (NULL = the default stream).  Unless a comment says otherwise a function
 *   - returns 0 on success, a positive hipError_t on a HIP failure, or a negative
 *     GEAR_HIP_E* code on an argument error (never throws, never exits),
 *   - only enqueues work on `stream` (no device or stream synchronisation),
 *   - allocates nothing: outputs and workspaces are owned by the caller,
 *   - takes DEVICE-ACCESSIBLE pointers (hipMalloc memory, or pinned+mapped host memory for the
 *     zero-copy table case) for every array argument.
 *
 * Each entry point cites the reference interface (bigrl-team/gear, path:line) that it replaces.
 */
#ifndef GEAR_HIP_H_
#define GEAR_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GEAR_HIP_ABI_VERSION 1

/* every entry point below is exported from libgearhip.so */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

/* negative error codes (argument / usage errors detected on the host) */
#define GEAR_HIP_EINVAL (-1)      /* null pointer, negative size, inconsistent arguments     */
#define GEAR_HIP_EWORKSPACE (-2)  /* workspace pointer null or smaller than the *_bytes query */
#define GEAR_HIP_ERANGE (-3)      /* a size exceeds what the kernels index (see each call)    */
#define GEAR_HIP_EALIGN (-4)      /* a pointer that must be naturally aligned is not          */
#define GEAR_HIP_ENOTREADY (-5)   /* one-time set-up is missing and cannot run now (see call)  */

/* ---- runtime ------------------------------------------------------------------------------ */

/* ABI version of the loaded library (== GEAR_HIP_ABI_VERSION it was built with). */
int gear_hip_abi_version(void);

/* Select the HIP device for the calling thread.
 * Replaces gear::cuda::init / libgear.core.init (src/cuda/init.cu:6-18). */
int gear_hip_set_device(int device_id);

/* Number of visible HIP devices, or a negative/positive error as above in *count's place.
 * Replaces the visible_device_count probe of src/env.cc:48-53. */
int gear_hip_device_count(int *count);

/* Human-readable text for a code returned by any function of this header (static storage). */
const char *gear_hip_error_string(int code);

/* Table memory.  Replace gear::memory::CudaUVMemory::alloc/free (src/memory/cuda_uvm.cc:10-54:
 * cudaHostAlloc mapped|portable) and gear::memory::CudaMemory (src/memory/cuda_memory.cc:6-28).
 * These four DO allocate / free and may synchronise; they are set-up calls, not hot-path calls.
 * gear_hip_host_alloc returns pinned host memory that the GPU reads in place (zero-copy);
 * *dev_ptr receives the device-side alias of the same bytes. */
int gear_hip_host_alloc(size_t bytes, void **host_ptr, void **dev_ptr);
int gear_hip_host_free(void *host_ptr);
int gear_hip_device_alloc(size_t bytes, void **dev_ptr);
int gear_hip_device_free(void *dev_ptr);

/* Blocking copy of `bytes` between any two of host / pinned / device memory (direction inferred
 * from the pointers).  A set-up call for filling and reading back device-resident tables
 * (stands where Span::copy uses memcpy on the host-resident table, include/common/span.h:73-79). */
int gear_hip_memcpy(void *dst, const void *src, size_t bytes);

/* Pin + map an existing host range (SysV shared memory segment of a TrajectoryTable).
 * Replaces the cudaHostRegister(Mapped|Portable) of gear::memory::SharedMemory::alloc
 * (src/memory/shared_memory.cc:59-61) and the cudaHostUnregister of ::free (:70).
 * Some ROCm installations refuse registration of existing memory; the error is returned and
 * the caller falls back to gear_hip_host_alloc. */
int gear_hip_host_register(void *host_ptr, size_t bytes, void **dev_ptr);
int gear_hip_host_unregister(void *host_ptr);

/* ---- trajectory-window gather ------------------------------------------------------------- */

/* Fused window arithmetic + byte gather of one column.
 * Replaces gear::cuda::launch_fused_subcopy_collect + fused_subcopy_collect
 * (src/cuda/copy.cu:91-134,217-242) as called by CpuTrajectoryStorageHandler::fused_subcopy
 * (src/storage/handler.cc:133-154) behind libgear.core handler.subcopy
 * (src/storage/pybind.cc:140-146).
 *
 * For window g in [0,num):
 *     lsub = max(tss[g] + ofst, 0);  rsub = min(lsub + span, lens[g]);
 *     n    = max(rsub - lsub, 0) * step_bytes;
 *     npad = pad_head ? dst_stride - n : 0;
 *     dst[g*dst_stride + npad .. +n) = src[idxs[g]*traj_stride + col_base + lsub*step_bytes .. +n)
 * src       table base (HBM, or pinned mapped host memory: the zero-copy path)
 * dst       contiguous [num, dst_stride] bytes, 16-byte aligned (any torch tensor is)
 * idxs/tss/lens  int64[num] on the device: trajectory index, timestep, trajectory length
 * traj_stride    bytes per trajectory (T * sum of per-step column bytes; src/storage/table.cc:14-16)
 * step_bytes     bytes per step of this column (ColumnSpec::size, src/storage/specs.cc:10-14)
 * col_base       accu_stride(column) * T (src/storage/handler.cc:143-145)
 * dst_stride     bytes per window in dst (pattern.length * step_bytes, handler.cc:146-147)
 * zero_fill      0: padding bytes of dst are left untouched, as in the reference (whose caller
 *                pre-zeroes the batch with torch.zeros, gear/loader/offline_loader.py:181-189);
 *                1: the kernel writes the padding zeros itself, so dst may be uninitialised.
 * mask_out       NULL, or uint8[num, span] on the device: 1 where the step holds copied data,
 *                0 where it is padding (no reference counterpart; benchmark config 3's mask).
 * All offsets are 64-bit (the reference's kernel truncates them to int, copy.cu:93-115).
 * Requires n <= dst_stride for every window (GEAR_HIP_EINVAL if span*step_bytes > dst_stride). */
int gear_hip_subcopy(const void *src, void *dst, int64_t num, const int64_t *idxs,
                     const int64_t *tss, const int64_t *lens, int pad_head, int64_t ofst,
                     int64_t span, int64_t traj_stride, int64_t step_bytes, int64_t col_base,
                     int64_t dst_stride, int zero_fill, uint8_t *mask_out, void *stream);

/* One launch for several columns of the same batch of windows (no reference counterpart as an
 * entry point: it is the per-column loop of OfflineLoader.fused_iterate,
 * gear/loader/offline_loader.py:178-203, folded into one grid).
 * cols points to `ncols` descriptors in HOST memory (copied into kernel arguments). */
typedef struct gear_hip_column_desc {
  void *dst;          /* [num, dst_stride] bytes on the device, 16-byte aligned */
  uint8_t *mask_out;  /* NULL or uint8[num, span] */
  int64_t ofst, span; /* SubscribePattern offset / length (include/storage/handler.h:17-31) */
  int64_t step_bytes, col_base, dst_stride;
  int32_t pad_head, zero_fill;
} gear_hip_column_desc;
#define GEAR_HIP_MAX_COLUMNS 16
int gear_hip_subcopy_multi(const void *src, int64_t num, const int64_t *idxs, const int64_t *tss,
                           const int64_t *lens, int64_t traj_stride,
                           const gear_hip_column_desc *cols, int ncols, void *stream);

/* The same launch with the batch checked against the table on the device: a window whose
 * trajectory index lies outside [0, capacity) reads nothing (its rows are all padding, its mask
 * all 0) and lens[g] is clamped to trajectory_length, so no index a caller passes can make the
 * kernel read outside the table.  The reference's kernel trusts its inputs
 * (src/cuda/copy.cu:110-123); capacity = 0 / trajectory_length = 0 switch the respective check
 * off, which is what gear_hip_subcopy_multi does. */
int gear_hip_subcopy_multi_checked(const void *src, int64_t num, const int64_t *idxs,
                                   const int64_t *tss, const int64_t *lens, int64_t traj_stride,
                                   int64_t capacity, int64_t trajectory_length,
                                   const gear_hip_column_desc *cols, int ncols, void *stream);

/* Generic slice gather: dst[dst_offsets[g] .. +strides[g]) = src[src_offsets[g] .. +strides[g]).
 * Replaces launch_vary_stride_copy_collect / vary_stride_copy_collect
 * (src/cuda/copy.cu:47-89,175-215; libgear.core.vcopy / copy_debug, copy.cu:247-258).
 * strides[g] <= max_stride must hold; slices with strides[g] <= 0 copy nothing.
 * Any byte alignment of src/dst offsets is accepted (the reference requires 16 B). */
int gear_hip_vcopy(const void *src, void *dst, int64_t num, const int64_t *src_offsets,
                   const int64_t *dst_offsets, const int64_t *strides, int64_t max_stride,
                   void *stream);

/* Same with one fixed slice length.  Replaces launch_fix_stride_copy_collect /
 * fix_stride_copy_collect (src/cuda/copy.cu:12-45,138-173; libgear.core.copy, copy.cu:246). */
int gear_hip_copy(const void *src, void *dst, int64_t num, const int64_t *src_offsets,
                  const int64_t *dst_offsets, int64_t stride, void *stream);

/* Device-side restatement of CpuTrajectoryStorageHandler::sub (src/storage/handler.cc:78-131):
 * fills src_offsets/dst_offsets/copy_lens (int64[num], device) from idxs/tss/lens without the
 * host loop and the three H2D copies of gear/loader/offline_loader.py:260-277. */
int gear_hip_sub(int64_t num, const int64_t *idxs, const int64_t *tss, const int64_t *lens,
                 int pad_head, int64_t ofst, int64_t span, int64_t traj_stride,
                 int64_t step_bytes, int64_t col_base, int64_t *src_offsets,
                 int64_t *dst_offsets, int64_t *copy_lens, void *stream);

/* Sampled flat step index -> window arguments of gear_hip_subcopy, for tables whose priorities
 * are kept per step (benchmark configs 4 and 5):  f = flat[j] (mod `modulo` when modulo > 0);
 *     idxs[j] = f / trajectory_length;  tss[j] = f % trajectory_length;  lens[j] = tss[j] + 1
 * (lens may be NULL).  lens = ts + 1 is the offline convention "timestep == length" of
 * gear/loader/offline_loader.py:200-201,263 applied to a step inside a trajectory: the window
 * never reaches past the sampled step.  Stands where the loader looks timesteps up on the host
 * (gear/loader/offline_loader.py:168-177). */
int gear_hip_split_step_index(const int64_t *flat, int64_t num, int64_t trajectory_length,
                              int64_t modulo, int64_t *idxs, int64_t *tss, int64_t *lens,
                              void *stream);

/* out[j] = table[idx[j]] + add for int64 tables on the device (0 where idx[j] is outside [0,n)).
 * Replaces the host-side look-ups of the sampled batch: iset.timesteps[indices.cpu()]
 * (gear/loader/offline_loader.py:168-177) and concat_indices[draws]
 * (gear/sampler/global_sampler.py:131,172,196). */
int gear_hip_take_i64(const int64_t *table, int64_t n, const int64_t *idx, int64_t num,
                      int64_t add, int64_t *out, void *stream);

/* ---- weighted sampler: prefix sum + search ------------------------------------------------ */

/* Inclusive prefix sum of fp32 priorities accumulated and written in fp64:
 *     out[i] = sum_{j<=i} (double) in[j]
 * One pass over the input for up to 4096 ranges (n <= 67.1 M): every workgroup publishes the sum
 * of its range and adds the sums of all earlier ranges, with a bounded wait (a workgroup that
 * waited too long sums the missing range itself and publishes it: same bits, no kernel can
 * hang).  Two launches (range sums, then the scan) beyond that, for a stream under graph capture,
 * and with GEAR_HIP_SCAN_SINGLE_PASS=0; three (a launch in between scans the range sums) beyond
 * 16384 ranges (n > 134 M).  The result is bit-identical in all cases and on every run.  Replaces
 * gear::cuda::launch_prefix_sum /
 * one_dimension_prefix_sum (src/cuda/one_dim_prefix_sum.cu:125-273; libgear.core.prefix_sum,
 * :276-278), which is fp32 and only correct for one block.
 * workspace: device memory of at least gear_hip_scan_workspace_bytes(n) bytes, 256-byte aligned;
 * its contents need not be initialised (the call initialises it on `stream`).
 * n may be 0 (nothing is written).  n <= 2^40.  `out` must be 16-byte aligned.
 * One workspace serves one call at a time.  Two one-pass calls that share a workspace while both
 * run cannot hang (the wait is bounded) but may find each other's words; a range that could not
 * be completed is marked: its prefixes are NaN (fp64 / fp32 results) or start from INT64_MIN
 * (gear_hip_scan_i64: negative results where the inputs are not).
 * Rounding: inside a range (2048, 4096 or 8192 elements, by n) the prefix is a running sum of a
 * fixed association; the offset of a range is the separately rounded sum of all earlier ranges.
 * Both are within 1e-12 (relative) of the sequential fp64 sum, but they are rounded differently,
 * so across a range boundary out[i+1] can fall below out[i] + in[i+1] by an ulp or two of the
 * running total; with non-negative input the result is still non-decreasing except where that
 * difference exceeds in[i+1] (inputs below ~1e-16 of the total). */
size_t gear_hip_scan_workspace_bytes(int64_t n);
int gear_hip_scan_f32_f64(const float *in, double *out, int64_t n, void *workspace,
                          size_t workspace_bytes, void *stream);

/* gear_hip_scan_f32_f64 for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses with a frozen memory pool.  It has no counterpart in
 * the reference.  The range sums that the other entry point keeps in the caller's workspace live
 * in a static device array inside the library (about 2 MiB per GPU, held until the process ends);
 * the call allocates and frees nothing.  Same result, bit for bit, as gear_hip_scan_f32_f64.
 * n <= gear_hip_scan_static_max_n() (2^27 = 134 217 728), else GEAR_HIP_ERANGE.
 * The array's address is looked up once per device, by gear_hip_set_device or by the first call
 * on that device; a first call on a stream that is being captured cannot look it up and returns
 * GEAR_HIP_ENOTREADY (call gear_hip_set_device, or once outside the capture, first).
 * All calls on one GPU share the array.  Outside graph capture the library orders them itself:
 * a call's kernels wait (on the device, through an event) for the kernels of the previous static
 * call on that GPU, whatever stream or host thread that one came from.  Captured calls are not
 * ordered by the library: graphs that hold one must not run at the same time as another static
 * call on that GPU, or the two race on the array; use the workspace form there. */
int64_t gear_hip_scan_static_max_n(void);
int gear_hip_scan_f32_f64_static(const float *in, double *out, int64_t n, void *stream);

/* Incremental form for the online priority path (priorities of a few trajectories change between
 * batches: SharedMemoryIndexServer::update, src/index/server.cc:175-180, and
 * WeightUpdateRequestArray, src/index/request.cc:41-75; the reference has no prefix to maintain).
 * Preconditions: the last call on (in, out, workspace) was gear_hip_scan_f32_f64 or this function
 * with the same n, and since then only in[first_changed .. n) changed.  Then out[i] is
 * recomputed from the start of the range that holds first_changed onwards, reusing the range sums
 * kept in the workspace; the result is bit-identical to a full gear_hip_scan_f32_f64.
 * first_changed >= n: nothing to do; first_changed = 0: a full scan. */
int gear_hip_rescan_f32_f64(const float *in, double *out, int64_t n, int64_t first_changed,
                            void *workspace, size_t workspace_bytes, void *stream);

/* The same scan (fp64 accumulation) with the result rounded to fp32 on output: the signature of
 * the reference's binding, prefix_sum(FloatTensor input, FloatTensor output)
 * (src/cuda/one_dim_prefix_sum.cu:246-278). */
int gear_hip_scan_f32_f32(const float *in, float *out, int64_t n, void *workspace,
                          size_t workspace_bytes, void *stream);

/* Same scan over int64 weights (trajectory lengths, include/index/set.h:42), exact in int64
 * (two's complement: weights of either sign, sums wrap like int64 additions).
 * Used for length-weighted trajectory sampling (benchmark config 3).
 * n <= 2^40. */
int gear_hip_scan_i64(const int64_t *in, int64_t *out, int64_t n, void *workspace,
                      size_t workspace_bytes, void *stream);

/* Sum of n fp32 values accumulated in fp64, written to out[0] (device) as fp32 and, when
 * out_f64 is not NULL, as fp64 to out_f64[0].  Deterministic (fixed reduction tree).
 * Replaces gear::cuda::launch_sum / one_dimension_sum (src/cuda/one_dim_sum.cu:22-99;
 * libgear.core.sum, :102-104), which uses fp32 atomics on the default stream.
 * workspace: gear_hip_sum_workspace_bytes(n) bytes on the device. */
size_t gear_hip_sum_workspace_bytes(int64_t n);
int gear_hip_sum_f32(const float *in, int64_t n, float *out, double *out_f64, void *workspace,
                     size_t workspace_bytes, void *stream);

/* Batched upper_bound of draws in an fp64 inclusive prefix array:
 *     idx_out[j] = min( #{ i : prefix[i] <= t_j }, n-1 )
 * with t_j = (double) u[j]                       when unit_uniforms == 0 (u in [0, total)),
 *      t_j = (double) u[j] * prefix[n-1]         when unit_uniforms != 0 (u in [0, 1)).
 * This is the "binary search of seeded uniforms" half of the weighted sampler (no kernel in
 * the reference; it stands where WeightedSampler calls torch.multinomial,
 * gear/sampler/global_sampler.py:170).
 * Optional importance weights (both or neither of priorities / weights_out non-NULL):
 *     w_j = ( n * priorities[idx_j] / prefix[n-1] ) ^ (-beta), computed in fp64;
 *     weights_out[j] = (float)( w_j / max_j w_j ).
 * workspace: gear_hip_search_workspace_bytes(num) bytes on the device (only used for weights;
 * may be NULL/0 when weights_out is NULL). */
size_t gear_hip_search_workspace_bytes(int64_t num);
int gear_hip_upper_bound_f64(const double *prefix, int64_t n, const float *u, int64_t num,
                             int unit_uniforms, int64_t *idx_out, const float *priorities,
                             double beta, float *weights_out, void *workspace,
                             size_t workspace_bytes, void *stream);

/* The sampler of one batch in one call: draws searched in the fp64 prefix (as
 * gear_hip_upper_bound_f64), the found indices sorted ascending -- what every sampler of the
 * reference returns, torch.sort(...).values, gear/sampler/global_sampler.py:131,172,195-199 --
 * and, when trajectory_length > 0, split like gear_hip_split_step_index into idxs/tss/lens
 * (lens may be NULL).  sorted_out may be NULL when trajectory_length > 0.
 * Up to 4096 draws take two launches (search over many workgroups, then the ranking sort,
 * which also splits); larger batches use the multi-pass radix sort.
 * workspace: gear_hip_sample_workspace_bytes(num) bytes on the device. */
size_t gear_hip_sample_workspace_bytes(int64_t num);
int gear_hip_sample_sorted_f64(const double *prefix, int64_t n, const float *u, int64_t num,
                               int unit_uniforms, int64_t *sorted_out, int64_t trajectory_length,
                               int64_t modulo, int64_t *idxs, int64_t *tss, int64_t *lens,
                               void *workspace, size_t workspace_bytes, void *stream);

/* Batch selection with the look-ups the loader performs before it can gather, in one call.
 * For a batch of positions into the loader's index array, sorted ascending, the entry at sorted
 * place r with position p yields
 *     sampled_out[r] = index_table ? index_table[p] : p      (0 for p outside [0, index_n))
 *     local_out[r]   = sampled_out[r] - index_offset
 *     lens_out[r]    = lengths_table[local_out[r]]            (0 outside [0, lengths_n))
 * Any of the three outputs may be NULL (not all); lens_out needs lengths_table.  This replaces,
 * for a sampler whose index array ascends (then sort(indices[p]) == indices[sort(p)]), the chain
 * torch.sort(concat_indices[draws]) (gear/sampler/global_sampler.py:131,172,196),
 * indices - index_offset and iset.timesteps[indices.cpu()] on the host
 * (gear/loader/offline_loader.py:161-177): up to 4096 positions take ONE launch after the search
 * (the ranking sort does the look-ups of the entry it places), more take the radix sort and an
 * element-wise launch.
 *   gear_hip_sample_lookup_f64  positions = upper_bound of the draws u in the fp64 prefix, as
 *                               gear_hip_upper_bound_f64 (index_table, when given, has n entries)
 *   gear_hip_sample_lookup_i64  the same in an int64 prefix (a sampler over lengths), u as for
 *                               gear_hip_upper_bound_i64; with starts_out, also the start of a
 *                               window of `window` steps inside the entry's recorded length:
 *                               starts_out[r] = floor(start_uniforms[r] * (lens[r] - window + 1)),
 *                               0 where the length is below the window (start_uniforms: num
 *                               doubles in [0, 1); needs lengths_table; starts_out may be NULL)
 *   gear_hip_sort_lookup_i64    positions given (uniform draws), each in [0, bound)
 *   gear_hip_lookup_i64         positions given and already in the wanted order (the top-k's
 *                               index-ordered selection): look-ups only, no workspace
 * workspace: gear_hip_sample_workspace_bytes(num) bytes on the device. */
int gear_hip_sample_lookup_f64(const double *prefix, int64_t n, const float *u, int64_t num,
                               int unit_uniforms, const int64_t *index_table,
                               int64_t index_offset, const int64_t *lengths_table,
                               int64_t lengths_n, int64_t *sampled_out, int64_t *local_out,
                               int64_t *lens_out, void *workspace, size_t workspace_bytes,
                               void *stream);
int gear_hip_sample_lookup_i64(const int64_t *prefix, int64_t n, const void *u, int64_t num,
                               int unit_uniforms, const int64_t *index_table,
                               int64_t index_offset, const int64_t *lengths_table,
                               int64_t lengths_n, int64_t *sampled_out, int64_t *local_out,
                               int64_t *lens_out, const double *start_uniforms, int64_t window,
                               int64_t *starts_out, void *workspace, size_t workspace_bytes,
                               void *stream);
int gear_hip_sort_lookup_i64(const int64_t *positions, int64_t num, int64_t bound,
                             const int64_t *index_table, int64_t index_n, int64_t index_offset,
                             const int64_t *lengths_table, int64_t lengths_n,
                             int64_t *sampled_out, int64_t *local_out, int64_t *lens_out,
                             void *workspace, size_t workspace_bytes, void *stream);
int gear_hip_lookup_i64(const int64_t *positions, int64_t num, const int64_t *index_table,
                        int64_t index_n, int64_t index_offset, const int64_t *lengths_table,
                        int64_t lengths_n, int64_t *sampled_out, int64_t *local_out,
                        int64_t *lens_out, void *stream);

/* Same search in an int64 prefix array (exact): t_j = floor(u[j] * prefix[n-1]) with u fp64 in
 * [0,1) when unit_uniforms != 0, else t_j = (int64) u[j] taken from an int64 array passed
 * through `u` (cast).  idx_out[j] = min(#{i : prefix[i] <= t_j}, n-1). */
int gear_hip_upper_bound_i64(const int64_t *prefix, int64_t n, const void *u, int64_t num,
                             int unit_uniforms, int64_t *idx_out, void *stream);

/* ---- sort / top-k / priority update ------------------------------------------------------- */

/* Ascending LSD radix sort of `num` int64 keys (non-negative, < 2^key_bits) with an optional
 * int64 payload, stable.  keys_out/vals_out must not alias the inputs.
 * Replaces the torch.sort of sampled indices in every sampler
 * (gear/sampler/global_sampler.py:131,172,195-199) and the unfinished
 * include/cuda/sort.cuh:19-122.
 * workspace: gear_hip_sort_workspace_bytes(num) bytes on the device. */
size_t gear_hip_sort_workspace_bytes(int64_t num);
int gear_hip_sort_i64(const int64_t *keys_in, int64_t *keys_out, const int64_t *vals_in,
                      int64_t *vals_out, int64_t num, int key_bits, void *workspace,
                      size_t workspace_bytes, void *stream);

/* Top-k of fp32 priorities, largest first; among equal priorities the smaller index wins
 * (i.e. the first k entries of a stable descending sort).  NaN is not a valid priority.
 * Replaces torch.topk(weights, k, largest=True) of TopKSampler
 * (gear/sampler/global_sampler.py:195-199) and the dead include/cuda/sort.cuh.
 *   sorted_by_value != 0: values_out/indices_out ordered by (value desc, index asc)
 *   sorted_by_value == 0: the same set ordered by index ascending (what TopKSampler returns
 *                         after its torch.sort of the indices)
 * values_out may be NULL.  1 <= k <= n < 2^31.
 * The priorities are normally read once: a sample of 2048 of them places a bound safely below
 * the k-th largest, the one pass over the array lists everything above the bound, and the exact
 * selection runs on those lists.  Where a list overflows (clustered maxima, masses of ties) the
 * later steps read that part of the array again; where the bound fails (fewer than k entries
 * above it: a sample that misleads) two of them read all of it again and look for the threshold
 * among the entries below the bound.  The result is the same either way.
 * workspace: gear_hip_topk_workspace_bytes(n, k) bytes on the device, 256-byte aligned; its
 * contents need not be initialised (the call clears what it needs on `stream`). */
size_t gear_hip_topk_workspace_bytes(int64_t n, int64_t k);
int gear_hip_topk_f32(const float *priorities, int64_t n, int64_t k, int sorted_by_value,
                      float *values_out, int64_t *indices_out, void *workspace,
                      size_t workspace_bytes, void *stream);

/* The same selection for a caller that repeats it on a slowly changing array (the priority
 * maintenance of a replay buffer between batches: TopKSampler.sync_sample on every step,
 * gear/sampler/global_sampler.py:175-203, after the updates of src/index/request.cc:41-51).
 * Every call leaves in the workspace the bound the NEXT call can start from: the boundary at or
 * below the 2k-th largest priority, taken from this call's exact counts.  This form takes that
 * bound up instead of drawing a sample when `workspace` was last used by gear_hip_topk_f32 or
 * this function with the same n, k and order (a mark in the workspace says so; anything else in
 * it, and a call whose own bound failed, lead to a sample as in gear_hip_topk_f32).  The bound
 * only decides how the work is done: however stale it is, the result equals gear_hip_topk_f32's
 * bit for bit (too high: the entries below it are searched as described above; too low: lists
 * overflow and those parts of the array are read again). */
int gear_hip_topk_f32_warm(const float *priorities, int64_t n, int64_t k, int sorted_by_value,
                           float *values_out, int64_t *indices_out, void *workspace,
                           size_t workspace_bytes, void *stream);

/* Priority update  weights[idx[j]] = values[j], j in [0,num).
 * Replaces the host loop over Indexset::set_weight (include/index/set.h:245-247) and fixes the
 * semantics of WeightUpdateRequestArray::update (src/index/request.cc:41-51): when an index
 * occurs more than once the LAST occurrence wins.
 *   unique_indices != 0: caller guarantees no duplicates; plain scatter, no workspace needed.
 *   unique_indices == 0: duplicates resolved deterministically with a stable radix sort of the
 *                        indices; workspace of gear_hip_scatter_workspace_bytes(num) bytes.
 * Indices outside [0,n) are ignored. */
size_t gear_hip_scatter_workspace_bytes(int64_t num);
int gear_hip_scatter_f32(float *weights, int64_t n, const int64_t *idx, const float *values,
                         int64_t num, int unique_indices, void *workspace,
                         size_t workspace_bytes, void *stream);

/* The same update for int64 tables: timesteps[idx[j]] = values[j] (the trajectory lengths that
 * travel with the priorities in a weight-update request, src/index/server.cc:175-180,
 * Indexset::set_timestep, include/index/set.h:242-244).  Same workspace query. */
int gear_hip_scatter_i64(int64_t *table, int64_t n, const int64_t *idx, const int64_t *values,
                         int64_t num, int unique_indices, void *workspace, size_t workspace_bytes,
                         void *stream);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif

#ifdef __cplusplus
}
#endif
#endif /* GEAR_HIP_H_ */
