/**
 *  @brief Thin C ABI over the gfx950 (MI355X) HIP kernels for packed batched dot products.
 *  @file include/numkong_amd/hip_abi.h
 *
 *  Everything in this header is plain C: pointers, sizes and integer codes, no HIP or torch types.
 *  The C host layer (numkong_amd/csrc/numkong.c, dispatch_*.c, gfx950.c) is the only intended caller;
 *  it builds the reference-compatible `nk_dots_*` entry points declared in <numkong_amd/dots.h> on top.
 *
 *  All `*_async` calls enqueue work on `stream` (a `hipStream_t` passed as `void *`, NULL = default
 *  stream), require DEVICE-accessible pointers and do not synchronise. They return 0 on success or a
 *  non-zero HIP error code; `nk_hip_last_error()` returns a thread-local description of the last failure.
 *
 *  `dtype` arguments take the `nk_dtype_t` codes of <numkong_amd/dots.h> (reference:
 *  include/numkong/types.h:923-952): nk_i8_k, nk_u8_k, nk_bf16_k, nk_f16_k, nk_e4m3_k, nk_e5m2_k, nk_e2m3_k, nk_e3m2_k,
 *  nk_i4_k, nk_u4_k, nk_f32_k, nk_f64_k (every kind), and nk_u1_k (the dot-product kinds). Depth counts dimensions, so
 *  4-bit values or bits for the sub-byte types; f32 and f64 write 8-byte f64 outputs, distances included.
 */
#ifndef NUMKONG_AMD_HIP_ABI_H
#define NUMKONG_AMD_HIP_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#pragma GCC visibility push(default)

/** Number of visible HIP devices; 0 when there is no usable GPU (never raises). */
int nk_hip_device_count(void);

/** 0 = plain host memory, 1 = device memory, 2 = host memory the device can address (pinned/managed). */
int nk_hip_pointer_kind(void const *ptr);

/** Device allocation helpers used by the host layer to stage host-resident operands. */
int nk_hip_malloc(void **ptr, size_t bytes);
int nk_hip_free(void *ptr);
int nk_hip_memcpy_h2d(void *dst, void const *src, size_t bytes, void *stream);
int nk_hip_memcpy_d2h(void *dst, void const *src, size_t bytes, void *stream);
int nk_hip_memcpy2d_h2d(void *dst, size_t dst_pitch, void const *src, size_t src_pitch, size_t width_bytes,
                        size_t rows, void *stream);
int nk_hip_memcpy2d_d2h(void *dst, size_t dst_pitch, void const *src, size_t src_pitch, size_t width_bytes,
                        size_t rows, void *stream);
int nk_hip_stream_synchronize(void *stream);

/**
 *  Per-thread state of the synchronous entry points, so that host threads calling at the same time (the reference's
 *  callers hand 64-row slices of A to a thread each against one shared packed B, python/matrix.c:466-483) neither share
 *  a stream nor allocate per call. Everything is created on first use by the calling thread and released when the
 *  thread ends or by `nk_hip_thread_release`.
 *   - `nk_hip_thread_stream(which)`, which = 0 or 1: the thread's own streams (blocking streams at the default
 *     priority: ordered against the legacy default stream, independent of each other). NULL on failure.
 *   - `nk_hip_thread_buffer(slot, pinned, bytes, &ptr)`: a staging buffer of at least `bytes` (device memory, or pinned
 *     host memory when `pinned` is non-zero) that lives in slot 0..7 until a larger one is asked for there.
 *   - `nk_hip_thread_trim(slot_bytes, total_bytes)`: frees the thread's staging buffers larger than `slot_bytes`, then
 *     all of them if more than `total_bytes` are still held.
 *   - `nk_hip_event_record / _synchronize`, `nk_hip_stream_wait_event`: the thread's events 0..7 (waiting for one
 *     that was never recorded returns at once).
 */
void *nk_hip_thread_stream(int which);
int nk_hip_thread_buffer(int slot, int pinned, size_t bytes, void **ptr);
size_t nk_hip_thread_cached_bytes(void);
void nk_hip_thread_release(void);
void nk_hip_thread_trim(size_t slot_bytes, size_t total_bytes);
int nk_hip_event_record(int which, void *stream);
int nk_hip_event_synchronize(int which);
int nk_hip_stream_wait_event(void *stream, int which);

/**
 *  Device copies of packed images that the caller keeps in host memory (what `malloc(nk_dots_packed_size_T(n, k))`
 *  gives a caller of the reference's interface), looked up by the number the image's pack call left in its header.
 *  A cached copy is always complete: it enters the cache only after every transfer into it has finished.
 *   - `claim`: 1 = cached, `*device_image` is the copy and the caller counts as a user until `release`; 2 = not cached,
 *     and an entry is now reserved for the caller, who uploads a copy into `nk_hip_malloc` memory, waits for the
 *     transfers, and calls `publish` (1: the cache owns the copy, the caller is its first user; 0: not taken, the caller
 *     frees it) or, on failure, `abandon`; other threads that claim the same image meanwhile wait for that upload
 *     instead of making their own; 0 = not cacheable (no header, over the budget, every entry in use): the caller
 *     works with a private copy and frees it.
 *   - `find`: the lookup alone, never waits (1 = cached and counted as a user).
 *   - `adopt`: hands the cache a complete copy made some other way (the pack call's own output); 1 = taken, the caller
 *     is its first user; 0 = not taken (also when a copy of the same image is cached already), the caller frees it.
 *  Copies nobody is using are dropped, least recently used first, beyond 4 images or NK_AMD_IMAGE_CACHE_BYTES
 *  (default 8 GiB); `clear` drops all of them.
 */
int nk_hip_image_cache_find(void const *host_image, size_t total_bytes, void **device_image);
int nk_hip_image_cache_claim(void const *host_image, size_t total_bytes, void **device_image);
int nk_hip_image_cache_publish(void const *host_image, size_t total_bytes, void *device_image);
void nk_hip_image_cache_abandon(void const *host_image, size_t total_bytes);
int nk_hip_image_cache_adopt(void const *host_image, size_t total_bytes, void *device_image);
void nk_hip_image_cache_release(void *device_image);
void nk_hip_image_cache_clear(void);

/**
 *  Bytes of the gfx950 packed image of an (n x k) B matrix: 64-byte header, MFMA-fragment tiles,
 *  per-column compensation terms, per-column sums of squares (f32 / f64: header, k-major f64 values, f64 sums of squares). Replaces `nk_dots_packed_size_<T>_<isa>`
 *  (reference: include/numkong/dots/serial.h:245-271). Returns 0 for an unsupported dtype or when
 *  n or k do not fit 32 bits.
 */
size_t nk_hip_dots_packed_size(int dtype, size_t n, size_t k);

/**
 *  Pack row-major B (n rows of k elements, `b_stride` bytes apart) into `b_packed`.
 *  Replaces `nk_dots_pack_<T>_<isa>` (reference: include/numkong/dots/serial.h:286-333).
 */
int nk_hip_dots_pack_async(int dtype, void const *b, size_t n, size_t k, size_t b_stride, void *b_packed,
                           void *stream);

/**
 *  C[m x n] = A[m x k] * B^T with widened accumulators (i32 / u32 / f32; f64 for f32 and f64 inputs), C overwritten.
 *  Replaces `nk_dots_packed_<T>_<isa>` (reference: include/numkong/dots/serial.h:520-1072).
 *  A packed image whose header does not match (dtype, n, k) makes every C element all ones (0xFF bytes).
 */
int nk_hip_dots_packed_async(int dtype, void const *a, void const *b_packed, void *c, size_t m, size_t n,
                             size_t k, size_t a_stride, size_t c_stride, void *stream);

/**
 *  Distances instead of dot products, in one pass: C[i][j] = angular (metric 1) or euclidean (metric 2) distance
 *  between row i of A and row j of B, as f32 (f64 for f32 and f64 inputs), from the same MFMA product, the per-column sums of squares that
 *  `nk_hip_dots_pack_async` leaves in the image and the per-row sums of squares gathered while A is staged.
 *  Replaces `nk_angulars_packed_<T>_<isa>` / `nk_euclideans_packed_<T>_<isa>`
 *  (reference: include/numkong/dots/serial.h:2756-2800, include/numkong/spatial/serial.h:257-344).
 */
int nk_hip_spatials_packed_async(int dtype, int metric, void const *a, void const *b_packed, void *c, size_t m,
                                 size_t n, size_t k, size_t a_stride, size_t c_stride, void *stream);

/**
 *  All pairs of one set of `n` vectors: result[i][j] for i in [row_start, row_start + row_count) and j >= i only,
 *  the dot product (metric 0), angular (1) or euclidean (2) distance of vectors i and j; distances on the diagonal
 *  are exactly 0. The vectors from the 32-row boundary at or below `row_start` to the end are packed into the
 *  workspace as the B of an ordinary product, the window's rows are its A, and a tile list (built on the device, in
 *  the workspace too) leaves out the tiles left of the diagonal. `workspace`: device memory, 256-byte aligned, at
 *  least `nk_hip_symmetric_workspace_size` bytes for the same arguments; in use until the stream has run the call.
 *  Replaces `nk_dots_symmetric_<T>_<isa>`, `nk_angulars_symmetric_<T>_<isa>`, `nk_euclideans_symmetric_<T>_<isa>`
 *  (reference: include/numkong/dots/serial.h:2361-2435, 2802-2878).
 */
size_t nk_hip_symmetric_workspace_size(int dtype, size_t n, size_t k, size_t row_start, size_t row_count);
int nk_hip_symmetric_async(int dtype, int metric, void const *vectors, size_t n, size_t k, size_t stride, void *result,
                           size_t result_stride, size_t row_start, size_t row_count, void *workspace,
                           size_t workspace_bytes, void *stream);

/**
 *  `nk_hip_symmetric_async` without a workspace argument and without any allocation: for callers that cannot call
 *  hipMalloc (code under HIP graph capture, tight serving loops, harnesses that forbid it). The workspace is a fixed
 *  array of `nk_hip_symmetric_static_capacity()` bytes (32 MiB) in device memory that the library holds on every GPU it
 *  runs on; a call whose `nk_hip_symmetric_workspace_size` is larger fails with a message saying so. All calls on one
 *  GPU share that array: calls that overlap there (two streams, two threads) race. No counterpart in the reference.
 */
size_t nk_hip_symmetric_static_capacity(void);
int nk_hip_symmetric_static_async(int dtype, int metric, void const *vectors, size_t n, size_t k, size_t stride,
                                  void *result, size_t result_stride, size_t row_start, size_t row_count, void *stream);

/** Fill the m x n block of 32-bit outputs with `value` (used for the 0xFF error convention). */
int nk_hip_fill_rows_async(void *c, size_t m, size_t n, size_t c_stride, uint32_t value, void *stream);

/** TEST HOOK, not part of the product interface: forces the tile shape of the calling thread's launches (0 = the
 *  heuristic picks; 1..5 = 256x256, 128x256, 128x128, 64x128, 128x512; bit 7: a forced shape may still split a
 *  triangle; bits 8..27: spread of the workgroups' start times in 10 ns ticks, plus one; bits 28..29: 1 = outputs
 *  stored past the caches, 2 = through them, whatever the alignment of C; bit 30: A is staged through registers also
 *  where it would go straight into LDS). The tests use it to run every shape, both kinds of store and both kinds of
 *  staging over the same cases; thread-local, so it never reaches another thread's calls. */
void nk_hip_set_tile_config(int config);

/** Thread-local text of the last failure in this layer ("" if none). */
char const *nk_hip_last_error(void);

#pragma GCC visibility pop

#ifdef __cplusplus
}
#endif

#endif // NUMKONG_AMD_HIP_ABI_H
