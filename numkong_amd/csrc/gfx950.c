/**
 *  @brief Host side of the gfx950 backend: operand placement, staging, the reference's error convention.
 *  @file numkong_amd/csrc/gfx950.c
 *
 *  Defines `nk_dots_packed_size_<T>_gfx950`, `nk_dots_pack_<T>_gfx950`, `nk_dots_packed_<T>_gfx950`, the packed
 *  distances and the symmetric kinds on top of them: the backend-suffixed kernels that dispatch_<T>.c binds, in the way the reference names its per-ISA
 *  kernels (include/numkong/dots.h:361-1877). Plain C over the thin HIP ABI of <numkong_amd/hip_abi.h>.
 *
 *  The reference's kernels take caller-owned pointers and return nothing (include/numkong/dots.h:84-98);
 *  so do these. A pointer the GPU can address is used in place; a plain host pointer is staged through pinned and
 *  device buffers that the calling thread keeps between calls (up to 1 GiB; the hidden allocations of this library,
 *  with the device copies of host-resident packed images). Every call runs on streams of the calling thread, so
 *  threads that call at the same time do not wait for each other, and is complete when it returns.
 *  Failures follow c/numkong.c:195-216: size 0, pack is a no-op, the product fills C with 0xFF.
 */
#define _GNU_SOURCE /* sysconf */
#include <pthread.h>
#include <stdatomic.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include "dispatch.h"
#include "numkong_amd/hip_abi.h"

static _Thread_local char nk_amd_error_[256] = "";

static void nk_amd_set_error_(char const *where) {
    char const *detail = nk_hip_last_error();
    snprintf(nk_amd_error_, sizeof(nk_amd_error_), "%s: %s", where, detail && detail[0] ? detail : "failed");
}

char const *nk_amd_last_error(void) { return nk_amd_error_; }

/** Bytes of one row of `k` elements: eight 1-bit or two 4-bit values to a byte, whole bytes (cast/serial.h:519-538). */
static size_t nk_amd_row_bytes_(nk_dtype_t dtype, size_t k) {
    switch (dtype) {
    case nk_u1_k: return (k + 7) / 8;
    case nk_i4_k:
    case nk_u4_k: return (k + 1) / 2;
    case nk_i8_k:
    case nk_u8_k:
    case nk_e4m3_k:
    case nk_e5m2_k:
    case nk_e2m3_k:
    case nk_e3m2_k: return k;
    case nk_f16_k:
    case nk_bf16_k: return k * 2;
    case nk_f32_k: return k * 4;
    case nk_f64_k: return k * 8;
    default: return 0;
    }
}

/** Bytes of one output: f64 for the two wide types, 32 bits for everything else on this path. */
static size_t nk_amd_output_bytes_(nk_dtype_t dtype) { return dtype == nk_f32_k || dtype == nk_f64_k ? 8 : 4; }

static size_t nk_amd_round_up_(size_t x, size_t to) { return (x + to - 1) / to * to; }

/** 0xFF over the m x n outputs only: the reference stub writes n * 8 bytes per row (c/numkong.c:209-216),
 *  which overruns 4-byte outputs; the convention is kept, the overrun is not (`out_bytes` per output). */
static void nk_amd_fill_error_(void *c, int c_kind, size_t m, size_t n, size_t c_stride, size_t out_bytes) {
    if (!c || !m || !n) return;
    if (c_kind == 1) { /* (as 32-bit words: two per f64 output) */
        void *stream = nk_hip_thread_stream(0);
        if (nk_hip_fill_rows_async(c, m, n * out_bytes / 4, c_stride, 0xFFFFFFFFu, stream) == 0) nk_hip_stream_synchronize(stream);
        return;
    }
    for (size_t row = 0; row < m; ++row) memset((char *)c + row * c_stride, 0xFF, n * out_bytes);
}

int nk_amd_dots_pack_async(nk_dtype_t dtype, void const *b, nk_size_t n, nk_size_t k, nk_size_t b_stride,
                           void *b_packed, void *stream) {
    return nk_hip_dots_pack_async((int)dtype, b, n, k, b_stride, b_packed, stream);
}

int nk_amd_dots_packed_async(nk_dtype_t dtype, void const *a, void const *b_packed, void *c, nk_size_t m, nk_size_t n,
                             nk_size_t k, nk_size_t a_stride, nk_size_t c_stride, void *stream) {
    return nk_hip_dots_packed_async((int)dtype, a, b_packed, c, m, n, k, a_stride, c_stride, stream);
}

int nk_amd_spatials_packed_async(nk_kernel_kind_t kind, nk_dtype_t dtype, void const *a, void const *b_packed, void *c,
                                 nk_size_t m, nk_size_t n, nk_size_t k, nk_size_t a_stride, nk_size_t c_stride,
                                 void *stream) {
    int const metric = kind == nk_kernel_angulars_packed_k ? 1 : (kind == nk_kernel_euclideans_packed_k ? 2 : 0);
    return nk_hip_spatials_packed_async((int)dtype, metric, a, b_packed, c, m, n, k, a_stride, c_stride, stream);
}

/** Is there a GPU? Asked of the runtime until the answer is yes, then remembered (devices do not go away). */
static int nk_amd_have_device_(void) {
    static _Atomic int seen = 0;
    if (atomic_load_explicit(&seen, memory_order_relaxed)) return 1;
    if (nk_hip_device_count() <= 0) return 0;
    atomic_store_explicit(&seen, 1, memory_order_relaxed);
    return 1;
}

static nk_size_t nk_amd_packed_size_(nk_dtype_t dtype, nk_size_t n, nk_size_t k) {
    return nk_hip_dots_packed_size((int)dtype, n, k);
}

#pragma region Staging of host operands

/*  Plain host memory reaches the GPU through pinned bounce buffers that the calling thread keeps between calls
 *  (hip_abi.h: nk_hip_thread_buffer), in pieces, so that the copy into the bounce buffer, the transfer and whatever the
 *  GPU does with the previous piece overlap. Copies of 16 MiB and more between pageable and pinned memory are split
 *  over a few helper threads (started once, then kept): one core moves about 10 GB/s, the link several times that.
 *  Pinned slots: 0, 1 uploads; 2, 3 downloads; 4, 5 row chunks of A; 6, 7 row chunks of C. Events: the same numbers
 *  for the slot's last transfer (4, 5: everything queued for a row chunk); 6: the packed image is on the device. */
enum {
    nk_amd_piece_bytes_k = 8u << 20,      /* one bounce-buffer piece of a plain upload or download */
    nk_amd_chunk_bytes_k = 32u << 20,     /* what a row chunk of the product moves in one direction, about */
    nk_amd_parallel_copy_k = 16u << 20,   /* host copies from this size on get helper threads */
};
static size_t const nk_amd_keep_slot_k = (size_t)256 << 20; /* the largest staging buffer a thread keeps between calls */
static size_t const nk_amd_keep_cached_k = (size_t)2 << 30; /* all the staging memory a thread may keep between calls */
enum { nk_amd_slot_a_k = 0, nk_amd_slot_c_k = 2, nk_amd_slot_b_k = 4, nk_amd_slot_image_k = 5, nk_amd_slot_result_k = 6 };

typedef struct {
    char *dst;
    char const *src;
    size_t dst_stride, src_stride, width, rows;
} nk_amd_copy_job_t_;

static void nk_amd_copy_job_run_(nk_amd_copy_job_t_ const *job) {
    for (size_t row = 0; row < job->rows; ++row) memcpy(job->dst + row * job->dst_stride, job->src + row * job->src_stride, job->width);
}

static int nk_amd_copy_threads_(void) {
    static _Atomic int cached = 0;
    int threads = atomic_load_explicit(&cached, memory_order_relaxed);
    if (threads) return threads;
    char const *text = getenv("NK_AMD_COPY_THREADS");
    long const online = sysconf(_SC_NPROCESSORS_ONLN);
    threads = text ? atoi(text) : (int)(online / 2);
    threads = threads < 1 ? 1 : (threads > 8 ? 8 : threads);
    atomic_store_explicit(&cached, threads, memory_order_relaxed);
    return threads;
}

/*  Helper threads for large host copies: started once, on the first large copy, and kept (detached, asleep on a
 *  condition variable between copies). Callers from any thread queue jobs under one lock and wait for their own. */
enum { nk_amd_copy_queue_k = 64 };
typedef struct {
    nk_amd_copy_job_t_ job;
    _Atomic int *pending; /* the caller's count of jobs not finished yet */
} nk_amd_queued_copy_t_;
static pthread_mutex_t nk_amd_copy_lock_ = PTHREAD_MUTEX_INITIALIZER;
static pthread_cond_t nk_amd_copy_work_ = PTHREAD_COND_INITIALIZER, nk_amd_copy_done_ = PTHREAD_COND_INITIALIZER;
static nk_amd_queued_copy_t_ nk_amd_copy_queue_[nk_amd_copy_queue_k];
static int nk_amd_copy_head_ = 0, nk_amd_copy_count_ = 0, nk_amd_copy_helpers_ = 0;

static void *nk_amd_copy_helper_(void *unused) {
    (void)unused;
    pthread_mutex_lock(&nk_amd_copy_lock_);
    for (;;) {
        while (!nk_amd_copy_count_) pthread_cond_wait(&nk_amd_copy_work_, &nk_amd_copy_lock_);
        nk_amd_queued_copy_t_ const taken = nk_amd_copy_queue_[nk_amd_copy_head_];
        nk_amd_copy_head_ = (nk_amd_copy_head_ + 1) % nk_amd_copy_queue_k, nk_amd_copy_count_--;
        pthread_mutex_unlock(&nk_amd_copy_lock_);
        nk_amd_copy_job_run_(&taken.job);
        pthread_mutex_lock(&nk_amd_copy_lock_);
        if (atomic_fetch_sub_explicit(taken.pending, 1, memory_order_acq_rel) == 1) pthread_cond_broadcast(&nk_amd_copy_done_);
    }
    return NULL;
}

/** Hands `job` to a helper; 0 when there is none to take it (the caller then copies it itself). */
static int nk_amd_copy_queue_job_(nk_amd_copy_job_t_ const *job, _Atomic int *pending, int wanted_helpers) {
    int queued = 0;
    pthread_mutex_lock(&nk_amd_copy_lock_);
    while (nk_amd_copy_helpers_ < wanted_helpers) { /* (started on first use, never more than 7) */
        pthread_t helper;
        pthread_attr_t attributes;
        if (pthread_attr_init(&attributes) != 0) break;
        pthread_attr_setdetachstate(&attributes, PTHREAD_CREATE_DETACHED);
        int const failed = pthread_create(&helper, &attributes, nk_amd_copy_helper_, NULL);
        pthread_attr_destroy(&attributes);
        if (failed) break;
        nk_amd_copy_helpers_++;
    }
    if (nk_amd_copy_helpers_ > 0 && nk_amd_copy_count_ < nk_amd_copy_queue_k) {
        int const at = (nk_amd_copy_head_ + nk_amd_copy_count_) % nk_amd_copy_queue_k;
        nk_amd_copy_queue_[at].job = *job, nk_amd_copy_queue_[at].pending = pending;
        atomic_fetch_add_explicit(pending, 1, memory_order_relaxed);
        nk_amd_copy_count_++, queued = 1;
        pthread_cond_signal(&nk_amd_copy_work_);
    }
    pthread_mutex_unlock(&nk_amd_copy_lock_);
    return queued;
}

/** `rows` runs of `width` bytes between host buffers, on this thread and, for large copies, the helpers. */
static void nk_amd_copy_rows_(void *dst, size_t dst_stride, void const *src, size_t src_stride, size_t width, size_t rows) {
    if (!width || !rows) return;
    if (dst_stride == width && src_stride == width && width != (1u << 16) && rows > 1) {
        /* one run of bytes: cut it into 64 KiB rows, which divide evenly among the threads, and a tail */
        size_t const total = width * rows, unit = 1u << 16;
        nk_amd_copy_rows_(dst, unit, src, unit, unit, total / unit);
        memcpy((char *)dst + total / unit * unit, (char const *)src + total / unit * unit, total % unit);
        return;
    }
    int threads = width * rows >= nk_amd_parallel_copy_k ? nk_amd_copy_threads_() : 1;
    if ((size_t)threads > rows) threads = (int)rows;
    nk_amd_copy_job_t_ jobs[8];
    _Atomic int pending = 0;
    int queued[8] = {0};
    size_t const share = (rows + (size_t)threads - 1) / (size_t)threads;
    for (int t = 0; t < threads; ++t) {
        size_t const first = (size_t)t * share, last = first + share < rows ? first + share : rows;
        jobs[t].dst = (char *)dst + first * dst_stride, jobs[t].src = (char const *)src + first * src_stride;
        jobs[t].dst_stride = dst_stride, jobs[t].src_stride = src_stride, jobs[t].width = width;
        jobs[t].rows = first < last ? last - first : 0;
        if (t > 0 && jobs[t].rows) queued[t] = nk_amd_copy_queue_job_(&jobs[t], &pending, threads - 1);
    }
    for (int t = 0; t < threads; ++t)
        if (t == 0 || !queued[t]) nk_amd_copy_job_run_(&jobs[t]); /* this thread's share, and any no helper could take */
    if (threads > 1) {
        pthread_mutex_lock(&nk_amd_copy_lock_);
        while (atomic_load_explicit(&pending, memory_order_acquire) > 0) pthread_cond_wait(&nk_amd_copy_done_, &nk_amd_copy_lock_);
        pthread_mutex_unlock(&nk_amd_copy_lock_);
    }
}

/** Host rows -> device rows on `stream`, through pinned pieces 0 and 1. Returns with the last transfers in flight. */
static int nk_amd_upload_(void *dst, size_t dst_pitch, void const *src, size_t src_pitch, size_t width, size_t rows,
                          void *stream) {
    if (!width || !rows) return 0;
    size_t piece_rows = nk_amd_piece_bytes_k / width;
    piece_rows = piece_rows < 1 ? 1 : (piece_rows > rows ? rows : piece_rows);
    int status = 0;
    for (size_t first = 0, piece = 0; first < rows && !status; first += piece_rows, ++piece) {
        int const slot = (int)(piece & 1);
        size_t const count = rows - first < piece_rows ? rows - first : piece_rows;
        void *bounce = NULL;
        if ((status = nk_hip_event_synchronize(slot))) break; /* the transfer that last used this piece is done */
        if ((status = nk_hip_thread_buffer(slot, 1, piece_rows * width, &bounce))) break;
        nk_amd_copy_rows_(bounce, width, (char const *)src + first * src_pitch, src_pitch, width, count);
        status = nk_hip_memcpy2d_h2d((char *)dst + first * dst_pitch, dst_pitch, bounce, width, width, count, stream);
        if (!status) status = nk_hip_event_record(slot, stream);
    }
    return status;
}

/** Device rows -> host rows, through pinned pieces 2 and 3; complete on return. */
static int nk_amd_download_(void *dst, size_t dst_pitch, void const *src, size_t src_pitch, size_t width, size_t rows,
                            void *stream) {
    if (!width || !rows) return 0;
    size_t piece_rows = nk_amd_piece_bytes_k / width;
    piece_rows = piece_rows < 1 ? 1 : (piece_rows > rows ? rows : piece_rows);
    size_t const pieces = (rows + piece_rows - 1) / piece_rows;
    void *bounce[2] = {NULL, NULL};
    int status = nk_hip_thread_buffer(2, 1, piece_rows * width, &bounce[0]);
    if (!status) status = nk_hip_thread_buffer(3, 1, piece_rows * width, &bounce[1]);
    /* piece p is queued before piece p - 1 is copied out of its bounce buffer */
    for (size_t piece = 0; piece <= pieces && !status; ++piece) {
        if (piece < pieces) {
            size_t const first = piece * piece_rows, count = rows - first < piece_rows ? rows - first : piece_rows;
            status = nk_hip_memcpy2d_d2h(bounce[piece & 1], width, (char const *)src + first * src_pitch, src_pitch, width, count, stream);
            if (!status) status = nk_hip_event_record(2 + (int)(piece & 1), stream);
        }
        if (piece > 0 && !status) {
            size_t const first = (piece - 1) * piece_rows, count = rows - first < piece_rows ? rows - first : piece_rows;
            status = nk_hip_event_synchronize(2 + (int)((piece - 1) & 1));
            if (!status) nk_amd_copy_rows_((char *)dst + first * dst_pitch, dst_pitch, bounce[(piece - 1) & 1], width, width, count);
        }
    }
    return status;
}

/** The same for one run of bytes (a packed image), taken as rows of 1 MiB and a tail. */
static int nk_amd_upload_flat_(void *dst, void const *src, size_t bytes, void *stream) {
    size_t const unit = 1u << 20, whole = bytes / unit;
    int status = nk_amd_upload_(dst, unit, src, unit, unit, whole, stream);
    if (!status) status = nk_amd_upload_((char *)dst + whole * unit, bytes % unit, (char const *)src + whole * unit, bytes % unit, bytes % unit, 1, stream);
    return status;
}
static int nk_amd_download_flat_(void *dst, void const *src, size_t bytes, void *stream) {
    size_t const unit = 1u << 20, whole = bytes / unit;
    int status = nk_amd_download_(dst, unit, src, unit, unit, whole, stream);
    if (!status) status = nk_amd_download_((char *)dst + whole * unit, bytes % unit, (char const *)src + whole * unit, bytes % unit, bytes % unit, 1, stream);
    return status;
}

/** What a synchronous call that staged something leaves behind: nothing in flight, and no more staging memory than a
 *  thread should keep (buffers past 256 MiB each go at once, everything once the thread holds more than 2 GiB). */
static void nk_amd_settle_(void) {
    (void)nk_hip_stream_synchronize(nk_hip_thread_stream(0));
    (void)nk_hip_stream_synchronize(nk_hip_thread_stream(1));
    nk_hip_thread_trim(nk_amd_keep_slot_k, nk_amd_keep_cached_k);
}

/**
 *  The packed image where the GPU can read it. A device (or device-addressable) image is used in place. A host image
 *  is looked up among the device copies of earlier calls and uploaded on `stream` when it is new; `*owned` is then 1
 *  for a copy this call must free and 2 for one to hand back to the cache (nk_amd_drop_image_).
 */
static int nk_amd_image_on_device_(void const *b_packed, int p_kind, size_t total, void *stream, void const **device, int *owned) {
    *owned = 0, *device = b_packed;
    if (p_kind != 0) return 0;
    void *copy = NULL;
    int const claimed = nk_hip_image_cache_claim(b_packed, total, &copy);
    if (claimed == 1) {
        *device = copy, *owned = 2;
        return 0;
    }
    int status = nk_hip_malloc(&copy, total);
    if (!status) {
        status = nk_amd_upload_flat_(copy, b_packed, total, stream);
        /* a copy that other threads can find must be complete: their streams are not ordered behind this one */
        if (claimed == 2 || status) status = nk_hip_stream_synchronize(stream) || status;
        if (status) nk_hip_free(copy);
    }
    if (status) {
        if (claimed == 2) nk_hip_image_cache_abandon(b_packed, total);
        return status;
    }
    *device = copy;
    *owned = claimed == 2 && nk_hip_image_cache_publish(b_packed, total, copy) ? 2 : 1;
    return 0;
}
static void nk_amd_drop_image_(void const *device, int owned) {
    if (owned == 2) nk_hip_image_cache_release((void *)device);
    if (owned == 1) nk_hip_free((void *)device);
}

#pragma endregion Staging of host operands

static void nk_amd_pack_(nk_dtype_t dtype, void const *b, nk_size_t n, nk_size_t k, nk_size_t b_stride,
                         void *b_packed) {
    nk_amd_error_[0] = 0;
    size_t const total = nk_hip_dots_packed_size((int)dtype, n, k);
    if (!total || !b_packed) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_pack: unsupported dtype or dimensions");
        return;
    }
    if (!nk_amd_have_device_()) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_pack: no HIP device");
        return;
    }
    void *stream = nk_hip_thread_stream(0);
    int const b_kind = (n && k) ? nk_hip_pointer_kind(b) : 1;
    int const p_kind = nk_hip_pointer_kind(b_packed);
    void *staged_b = NULL, *staged_p = NULL;
    void const *device_b = b;
    void *device_p = b_packed;
    size_t device_b_stride = b_stride;
    int status = stream ? 0 : -1;

    if (!status && b_kind == 0) {
        size_t const row_bytes = nk_amd_row_bytes_(dtype, k);
        device_b_stride = nk_amd_round_up_(row_bytes, 16);
        status = nk_hip_thread_buffer(nk_amd_slot_b_k, 0, n * device_b_stride, &staged_b);
        if (!status) status = nk_amd_upload_(staged_b, device_b_stride, b, b_stride, row_bytes, n, stream);
        device_b = staged_b;
    }
    if (!status && p_kind == 0) { /* (a buffer of its own: the device copy outlives the call, as the cached image) */
        status = nk_hip_malloc(&staged_p, total);
        device_p = staged_p;
    }
    if (!status) status = nk_hip_dots_pack_async((int)dtype, device_b, n, k, device_b_stride, device_p, stream);
    if (!status && staged_p) status = nk_amd_download_flat_(b_packed, staged_p, total, stream);
    if (!status) status = nk_hip_stream_synchronize(stream);
    if (status) nk_amd_set_error_("nk_dots_pack");
    if (staged_p) {
        /* the host image is what the caller multiplies with next: its device copy is kept for those calls */
        if (!status && nk_hip_image_cache_adopt(b_packed, total, staged_p)) nk_hip_image_cache_release(staged_p);
        else nk_hip_free(staged_p);
    }
    if (staged_b || staged_p || status) nk_amd_settle_();
}

/** `metric`: 0 dot products, 1 angular distances, 2 euclidean distances; outputs are 4 bytes wide, 8 for f32 and f64 inputs. */
static void nk_amd_packed_(nk_dtype_t dtype, int metric, void const *a, void const *b_packed, void *c, nk_size_t m,
                           nk_size_t n, nk_size_t k, nk_size_t a_stride, nk_size_t c_stride) {
    nk_amd_error_[0] = 0;
    if (!m || !n) return;
    size_t const out_bytes = nk_amd_output_bytes_(dtype);
    size_t const total = nk_hip_dots_packed_size((int)dtype, n, k);
    if (!nk_amd_have_device_()) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_packed: no HIP device");
        nk_amd_fill_error_(c, 0, m, n, c_stride, out_bytes);
        return;
    }
    /* where each operand lives: asked once per pointer and call */
    int const c_kind = nk_hip_pointer_kind(c);
    if (!total || !b_packed || !c) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_packed: unsupported dtype or dimensions");
        nk_amd_fill_error_(c, c_kind, m, n, c_stride, out_bytes);
        return;
    }
    int const a_kind = k ? nk_hip_pointer_kind(a) : 1;
    int const p_kind = nk_hip_pointer_kind(b_packed);
    void *stream = nk_hip_thread_stream(0);
    if (stream && a_kind != 0 && c_kind != 0 && p_kind != 0) {
        /* Everything where the GPU reads it: one launch on the thread's first stream, one wait for it. Nothing was
         * staged, so there is nothing else to wait for or to tidy up. */
        int status = metric == 0 ? nk_hip_dots_packed_async((int)dtype, a, b_packed, c, m, n, k, a_stride, c_stride, stream)
                                 : nk_hip_spatials_packed_async((int)dtype, metric, a, b_packed, c, m, n, k, a_stride, c_stride, stream);
        if (!status) status = nk_hip_stream_synchronize(stream);
        if (status) {
            nk_amd_set_error_("nk_dots_packed");
            (void)nk_hip_stream_synchronize(stream);
            nk_amd_fill_error_(c, c_kind, m, n, c_stride, out_bytes);
        }
        return;
    }
    void *streams[2] = {stream, nk_hip_thread_stream(1)};
    void const *device_p = b_packed;
    int image_owned = 0;
    int status = streams[0] && streams[1] ? 0 : -1;
    if (!status) status = nk_amd_image_on_device_(b_packed, p_kind, total, streams[0], &device_p, &image_owned);

    size_t const row_bytes = nk_amd_row_bytes_(dtype, k);
    size_t const a_pitch = nk_amd_round_up_(row_bytes, 16), c_pitch = nk_amd_round_up_(n * out_bytes, 16);
    if (!status && a_kind != 0 && c_kind != 0) { /* only the image was in host memory: one launch behind its upload */
        status = metric == 0 ? nk_hip_dots_packed_async((int)dtype, a, device_p, c, m, n, k, a_stride, c_stride, streams[0])
                             : nk_hip_spatials_packed_async((int)dtype, metric, a, device_p, c, m, n, k, a_stride, c_stride, streams[0]);
    }
    else if (!status) {
        /* Rows of A go up and rows of C come down in chunks, alternating between the thread's two streams, so that
         * the upload of one chunk, the product of the one before it and the copy of the one before that out of its
         * bounce buffer run at the same time. A chunk moves about 32 MiB in its heavier direction, in whole tiles of
         * the product kernels where that many rows are at least one; rows so long that 64 of them pass 256 MiB (the
         * largest buffer a thread keeps) go in fewer, down to one at a time. */
        size_t const heavier = (a_kind == 0 ? a_pitch : 0) > (c_kind == 0 ? c_pitch : 0) ? a_pitch : c_pitch;
        size_t const pitch = heavier ? heavier : 1;
        size_t chunk = nk_amd_chunk_bytes_k / pitch;
        if (chunk >= 256) chunk = chunk / 256 * 256;
        else if (chunk < 64) chunk = 64 * pitch <= nk_amd_keep_slot_k ? 64 : (nk_amd_keep_slot_k / pitch ? nk_amd_keep_slot_k / pitch : 1);
        if (chunk > m) chunk = m;
        size_t const chunks = (m + chunk - 1) / chunk;
        void *device_a[2] = {NULL, NULL}, *device_c[2] = {NULL, NULL}, *bounce_a[2] = {NULL, NULL}, *bounce_c[2] = {NULL, NULL};
        for (int half = 0; half < 2 && !status; ++half) {
            if (a_kind == 0) status = nk_hip_thread_buffer(nk_amd_slot_a_k + half, 0, chunk * a_pitch, &device_a[half]);
            if (!status && a_kind == 0) status = nk_hip_thread_buffer(4 + half, 1, chunk * a_pitch, &bounce_a[half]);
            if (!status && c_kind == 0) status = nk_hip_thread_buffer(nk_amd_slot_c_k + half, 0, chunk * c_pitch, &device_c[half]);
            if (!status && c_kind == 0) status = nk_hip_thread_buffer(6 + half, 1, chunk * c_pitch, &bounce_c[half]);
        }
        /* the image may still be on its way up stream 0: stream 1 waits for it */
        if (!status) status = nk_hip_event_record(6, streams[0]);
        if (!status) status = nk_hip_stream_wait_event(streams[1], 6);
        for (size_t at = 0; at <= chunks && !status; ++at) {
            if (at < chunks) {
                int const half = (int)(at & 1);
                size_t const first = at * chunk, rows = m - first < chunk ? m - first : chunk;
                void const *chunk_a = (char const *)a + first * a_stride;
                void *chunk_c = (char *)c + first * c_stride;
                size_t chunk_a_stride = a_stride, chunk_c_stride = c_stride;
                if (a_kind == 0) { /* (this half's buffers were last used two chunks ago: drained below) */
                    nk_amd_copy_rows_(bounce_a[half], a_pitch, chunk_a, a_stride, row_bytes, rows);
                    status = nk_hip_memcpy_h2d(device_a[half], bounce_a[half], rows * a_pitch, streams[half]);
                    chunk_a = device_a[half], chunk_a_stride = a_pitch;
                }
                if (c_kind == 0) chunk_c = device_c[half], chunk_c_stride = c_pitch;
                if (!status)
                    status = metric == 0 ? nk_hip_dots_packed_async((int)dtype, chunk_a, device_p, chunk_c, rows, n, k, chunk_a_stride, chunk_c_stride, streams[half])
                                         : nk_hip_spatials_packed_async((int)dtype, metric, chunk_a, device_p, chunk_c, rows, n, k, chunk_a_stride, chunk_c_stride, streams[half]);
                if (!status && c_kind == 0) status = nk_hip_memcpy_d2h(bounce_c[half], device_c[half], rows * c_pitch, streams[half]);
                if (!status) status = nk_hip_event_record(4 + half, streams[half]);
            }
            if (at > 0 && !status) { /* the chunk before: wait for it and hand its rows of C to the caller */
                int const half = (int)((at - 1) & 1);
                size_t const first = (at - 1) * chunk, rows = m - first < chunk ? m - first : chunk;
                status = nk_hip_event_synchronize(4 + half);
                if (!status && c_kind == 0) nk_amd_copy_rows_((char *)c + first * c_stride, c_stride, bounce_c[half], c_pitch, n * out_bytes, rows);
            }
        }
    }
    if (!status) status = nk_hip_stream_synchronize(streams[0]);
    if (!status) status = nk_hip_stream_synchronize(streams[1]);
    if (status) {
        nk_amd_set_error_("nk_dots_packed");
        nk_amd_settle_();
        nk_amd_fill_error_(c, c_kind, m, n, c_stride, out_bytes);
    }
    nk_amd_drop_image_(device_p, image_owned);
    nk_amd_settle_();
}

nk_size_t nk_amd_symmetric_workspace_size(nk_dtype_t dtype, nk_size_t vectors_count, nk_size_t depth,
                                          nk_size_t row_start, nk_size_t row_count) {
    return nk_hip_symmetric_workspace_size((int)dtype, vectors_count, depth, row_start, row_count);
}

static int nk_amd_symmetric_metric_(nk_kernel_kind_t kind) {
    switch (kind) {
    case nk_kernel_dots_symmetric_k: return 0;
    case nk_kernel_angulars_symmetric_k: return 1;
    case nk_kernel_euclideans_symmetric_k: return 2;
    default: return -1;
    }
}

int nk_amd_symmetric_async(nk_kernel_kind_t kind, nk_dtype_t dtype, void const *vectors, nk_size_t vectors_count,
                           nk_size_t depth, nk_size_t stride, void *result, nk_size_t result_stride, nk_size_t row_start,
                           nk_size_t row_count, void *workspace, nk_size_t workspace_bytes, void *stream) {
    return nk_hip_symmetric_async((int)dtype, nk_amd_symmetric_metric_(kind), vectors, vectors_count, depth, stride,
                                  result, result_stride, row_start, row_count, workspace, workspace_bytes, stream);
}

nk_size_t nk_amd_symmetric_static_capacity(void) { return nk_hip_symmetric_static_capacity(); }

int nk_amd_symmetric_static_async(nk_kernel_kind_t kind, nk_dtype_t dtype, void const *vectors, nk_size_t vectors_count,
                                  nk_size_t depth, nk_size_t stride, void *result, nk_size_t result_stride,
                                  nk_size_t row_start, nk_size_t row_count, void *stream) {
    return nk_hip_symmetric_static_async((int)dtype, nk_amd_symmetric_metric_(kind), vectors, vectors_count, depth, stride,
                                         result, result_stride, row_start, row_count, stream);
}

/** 0xFF over the whole n x n result, as the reference's stub does (c/numkong.c:218-227), 4 bytes per output. */
static void nk_amd_fill_symmetric_error_(void *result, int kind, size_t n, size_t result_stride, size_t out_bytes) {
    nk_amd_fill_error_(result, kind, n, n, result_stride, out_bytes);
}

/**
 *  The symmetric kinds: rows [row_start, row_start + row_count) of the upper triangle of the n x n result.
 *  Host operands are staged: the vectors from the window's first 32-row boundary on, and the window of the result
 *  both ways, so that what the kernel does not write (left of the diagonal) comes back as the caller had it.
 */
static void nk_amd_symmetric_(nk_dtype_t dtype, int metric, void const *vectors, nk_size_t n, nk_size_t k,
                              nk_size_t stride, void *result, nk_size_t result_stride, nk_size_t row_start,
                              nk_size_t row_count) {
    nk_amd_error_[0] = 0;
    if (!n || !row_count || row_start >= n) return;
    size_t const out_bytes = nk_amd_output_bytes_(dtype);
    if (!nk_amd_have_device_()) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_symmetric: no HIP device");
        nk_amd_fill_symmetric_error_(result, 0, n, result_stride, out_bytes);
        return;
    }
    int const r_kind = nk_hip_pointer_kind(result);
    size_t const workspace_bytes = nk_hip_symmetric_workspace_size((int)dtype, n, k, row_start, row_count);
    if (!workspace_bytes || !result) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_symmetric: unsupported dtype or dimensions");
        nk_amd_fill_symmetric_error_(result, r_kind, n, result_stride, out_bytes);
        return;
    }
    size_t const row_end = row_count < n - row_start ? row_start + row_count : n;
    size_t const first = row_start / 32 * 32; /* vectors and result columns from here on take part */
    int const v_kind = k ? nk_hip_pointer_kind(vectors) : 1;
    void *stream = nk_hip_thread_stream(0);
    void *staged_v = NULL, *staged_r = NULL, *workspace = NULL;
    /* device views, addressed as if they started at vector 0 / result element (0, 0) */
    char const *device_v = (char const *)vectors;
    char *device_r = (char *)result;
    size_t device_stride = stride, device_r_stride = result_stride;
    int status = stream ? nk_hip_thread_buffer(nk_amd_slot_image_k, 0, workspace_bytes + 256, &workspace) : -1;
    if (!status) workspace = (void *)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);

    if (!status && v_kind == 0) {
        size_t const row_bytes = nk_amd_row_bytes_(dtype, k);
        device_stride = nk_amd_round_up_(row_bytes, 16);
        status = nk_hip_thread_buffer(nk_amd_slot_b_k, 0, (n - first) * device_stride, &staged_v);
        if (!status)
            status = nk_amd_upload_(staged_v, device_stride, (char const *)vectors + first * stride, stride, row_bytes,
                                    n - first, stream);
        device_v = (char const *)staged_v - first * device_stride;
    }
    char *host_window = (char *)result + row_start * result_stride + first * out_bytes;
    if (!status && r_kind == 0) {
        device_r_stride = nk_amd_round_up_((n - first) * out_bytes, 16);
        status = nk_hip_thread_buffer(nk_amd_slot_result_k, 0, (row_end - row_start) * device_r_stride, &staged_r);
        if (!status)
            status = nk_amd_upload_(staged_r, device_r_stride, host_window, result_stride, (n - first) * out_bytes,
                                    row_end - row_start, stream);
        device_r = (char *)staged_r - row_start * device_r_stride - first * out_bytes;
    }
    if (!status)
        status = nk_hip_symmetric_async((int)dtype, metric, device_v, n, k, device_stride, device_r, device_r_stride,
                                        row_start, row_count, workspace, workspace_bytes, stream);
    if (!status && staged_r)
        status = nk_amd_download_(host_window, result_stride, staged_r, device_r_stride, (n - first) * out_bytes,
                                  row_end - row_start, stream);
    if (!status) status = nk_hip_stream_synchronize(stream);
    if (status) {
        nk_amd_set_error_("nk_dots_symmetric");
        nk_amd_settle_();
        nk_amd_fill_symmetric_error_(result, r_kind, n, result_stride, out_bytes);
    }
    nk_amd_settle_();
}

#define NK_AMD_DEFINE_BACKEND_DOTS_(T, in_t, out_t)                                                                     \
    nk_size_t nk_dots_packed_size_##T##_gfx950(nk_size_t width, nk_size_t depth) {                                 \
        return nk_amd_packed_size_(nk_##T##_k, width, depth);                                                      \
    }                                                                                                              \
    void nk_dots_pack_##T##_gfx950(in_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,            \
                                   void *b_packed) {                                                               \
        nk_amd_pack_(nk_##T##_k, b, width, depth, b_stride, b_packed);                                             \
    }                                                                                                              \
    void nk_dots_packed_##T##_gfx950(in_t const *a, void const *b_packed, out_t *c, nk_size_t height,              \
                                     nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride) {   \
        nk_amd_packed_(nk_##T##_k, 0, a, b_packed, c, height, width, depth, a_stride, c_stride);                   \
    }                                                                                                              \
    void nk_dots_symmetric_##T##_gfx950(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,             \
                                        nk_size_t stride, out_t *result, nk_size_t result_stride,                  \
                                        nk_size_t row_start, nk_size_t row_count) {                                \
        nk_amd_symmetric_(nk_##T##_k, 0, vectors, vectors_count, depth, stride, result, result_stride, row_start,  \
                          row_count);                                                                              \
    }

#define NK_AMD_DEFINE_BACKEND_DISTANCES_(T, in_t, r_t)                                                                 \
    void nk_angulars_packed_##T##_gfx950(in_t const *a, void const *b_packed, r_t *c, nk_size_t height,       \
                                         nk_size_t width, nk_size_t depth, nk_size_t a_stride,                     \
                                         nk_size_t c_stride) {                                                     \
        nk_amd_packed_(nk_##T##_k, 1, a, b_packed, c, height, width, depth, a_stride, c_stride);                   \
    }                                                                                                              \
    void nk_euclideans_packed_##T##_gfx950(in_t const *a, void const *b_packed, r_t *c, nk_size_t height,     \
                                           nk_size_t width, nk_size_t depth, nk_size_t a_stride,                   \
                                           nk_size_t c_stride) {                                                   \
        nk_amd_packed_(nk_##T##_k, 2, a, b_packed, c, height, width, depth, a_stride, c_stride);                   \
    }                                                                                                              \
    void nk_angulars_symmetric_##T##_gfx950(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,         \
                                            nk_size_t stride, r_t *result, nk_size_t result_stride,           \
                                            nk_size_t row_start, nk_size_t row_count) {                            \
        nk_amd_symmetric_(nk_##T##_k, 1, vectors, vectors_count, depth, stride, result, result_stride, row_start,  \
                          row_count);                                                                              \
    }                                                                                                              \
    void nk_euclideans_symmetric_##T##_gfx950(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,       \
                                              nk_size_t stride, r_t *result, nk_size_t result_stride,         \
                                              nk_size_t row_start, nk_size_t row_count) {                          \
        nk_amd_symmetric_(nk_##T##_k, 2, vectors, vectors_count, depth, stride, result, result_stride, row_start,  \
                          row_count);                                                                              \
    }

NK_AMD_DEFINE_BACKEND_DOTS_(i8, nk_i8_t, nk_i32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(i8, nk_i8_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(u8, nk_u8_t, nk_u32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(u8, nk_u8_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(bf16, nk_bf16_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(bf16, nk_bf16_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(f16, nk_f16_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(f16, nk_f16_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(e4m3, nk_e4m3_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(e4m3, nk_e4m3_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(e5m2, nk_e5m2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(e5m2, nk_e5m2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(e2m3, nk_e2m3_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(e2m3, nk_e2m3_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(e3m2, nk_e3m2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(e3m2, nk_e3m2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(i4, nk_i4x2_t, nk_i32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(i4, nk_i4x2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(u4, nk_u4x2_t, nk_u32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(u4, nk_u4x2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(u1, nk_u1x8_t, nk_u32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(f32, nk_f32_t, nk_f64_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(f32, nk_f32_t, nk_f64_t)
NK_AMD_DEFINE_BACKEND_DOTS_(f64, nk_f64_t, nk_f64_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(f64, nk_f64_t, nk_f64_t)
