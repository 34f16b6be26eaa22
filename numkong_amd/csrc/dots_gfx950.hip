/**
 *  @brief Plain-C entry points of the gfx950 backend: device memory, packing, the products and their symmetric forms.
 *  @file numkong_amd/csrc/dots_gfx950.hip
 *
 *  Exports the functions of <numkong_amd/hip_abi.h>; the reference-compatible API is built on top of them in C
 *  (gfx950.c). The kernels are in dots_gfx950.hpp; the product kernels of each element type are instantiated in a
 *  translation unit of their own (dots_gfx950_<T>.hip) and reached through nk_gfx950::launch_<T>.
 */
#include "dots_gfx950.hpp"

#include <pthread.h>
#include <time.h>
#include <unistd.h>

#include <stdlib.h>

#include <initializer_list>
#include <new>

namespace nk_gfx950 {

static thread_local int t_forced_config = 0;
int forced_tile_config() { return t_forced_config; }

uint64_t next_image_nonce() {
    static std::atomic<uint64_t> counter {0};
    static uint64_t const base = [] {
        struct timespec now;
        clock_gettime(CLOCK_REALTIME, &now);
        return (uint64_t)now.tv_sec * 1000000007ull ^ (uint64_t)now.tv_nsec << 20 ^ (uint64_t)getpid() << 44;
    }();
    uint64_t x = base + 0x9E3779B97F4A7C15ull * (counter.fetch_add(1, std::memory_order_relaxed) + 1); // (splitmix64)
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    x ^= x >> 31;
    return x ? x : 1;
}

int compute_unit_count() {
    static std::atomic<int> cached {0};
    int units = cached.load(std::memory_order_relaxed);
    if (units) return units;
    int device = 0;
    hipDeviceProp_t properties;
    if (hipGetDevice(&device) != hipSuccess || hipGetDeviceProperties(&properties, device) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    cached.store(properties.multiProcessorCount, std::memory_order_relaxed);
    return properties.multiProcessorCount;
}

} // namespace nk_gfx950

namespace {

thread_local char g_last_error[256] = "";

int fail(hipError_t e, char const *what) {
    snprintf(g_last_error, sizeof(g_last_error), "%s: %s", what, hipGetErrorString(e));
    (void)hipGetLastError();
    return (int)e ? (int)e : -1;
}
int fail_msg(char const *what) {
    snprintf(g_last_error, sizeof(g_last_error), "%s", what);
    return -1;
}

/**
 *  What a host thread keeps between synchronous calls: its streams, the events that order its staging pipeline, and
 *  device and pinned staging buffers that only ever grow. Created on first use, released when the thread ends (a
 *  pthread key's destructor: it runs for threads that exit, not at process exit, when the HIP runtime may already be
 *  gone).
 */
constexpr int kThreadStreams = 2, kThreadEvents = 8, kThreadSlots = 8;
struct CachedBuffer {
    void *ptr = nullptr;
    size_t bytes = 0;
};
struct ThreadContext {
    hipStream_t stream[kThreadStreams] = {};
    hipEvent_t event[kThreadEvents] = {};
    CachedBuffer device[kThreadSlots], pinned[kThreadSlots];
    void release(bool everything) {
        for (int slot = 0; slot < kThreadSlots; ++slot) {
            if (device[slot].ptr) (void)hipFree(device[slot].ptr);
            if (pinned[slot].ptr) (void)hipHostFree(pinned[slot].ptr);
            device[slot] = CachedBuffer(), pinned[slot] = CachedBuffer();
        }
        if (!everything) return;
        for (hipEvent_t &e : event)
            if (e) (void)hipEventDestroy(e), e = nullptr;
        for (hipStream_t &s : stream)
            if (s) (void)hipStreamDestroy(s), s = nullptr;
        (void)hipGetLastError();
    }
};
pthread_key_t g_context_key;
pthread_once_t g_context_once = PTHREAD_ONCE_INIT;
void destroy_thread_context(void *raw) {
    ThreadContext *context = (ThreadContext *)raw;
    context->release(true);
    delete context;
}
void make_context_key() { (void)pthread_key_create(&g_context_key, destroy_thread_context); }
ThreadContext *thread_context() {
    (void)pthread_once(&g_context_once, make_context_key);
    ThreadContext *context = (ThreadContext *)pthread_getspecific(g_context_key);
    if (!context) {
        context = new (std::nothrow) ThreadContext();
        if (context && pthread_setspecific(g_context_key, context) != 0) {
            delete context;
            context = nullptr;
        }
    }
    return context;
}

} // namespace

extern "C" {

int nk_hip_device_count(void) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return count;
}

int nk_hip_pointer_kind(void const *ptr) {
    if (!ptr) return 0;
    hipPointerAttribute_t attributes;
    memset(&attributes, 0, sizeof(attributes));
    if (hipPointerGetAttributes(&attributes, ptr) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    switch (attributes.type) {
    case hipMemoryTypeDevice: return 1;
    case hipMemoryTypeHost:
    case hipMemoryTypeManaged: return 2;
    default: return 0;
    }
}

int nk_hip_malloc(void **ptr, size_t bytes) {
    hipError_t e = hipMalloc(ptr, bytes ? bytes : 1);
    return e == hipSuccess ? 0 : fail(e, "hipMalloc");
}
int nk_hip_free(void *ptr) {
    hipError_t e = hipFree(ptr);
    return e == hipSuccess ? 0 : fail(e, "hipFree");
}

void *nk_hip_thread_stream(int which) {
    ThreadContext *context = thread_context();
    if (!context || which < 0 || which >= kThreadStreams) return nullptr;
    if (!context->stream[which]) {
        // (a blocking stream at the default priority: ordered against the legacy default stream in both directions,
        // so operands produced there are complete before this work starts, and independent of other threads' streams)
        hipError_t e = hipStreamCreateWithFlags(&context->stream[which], hipStreamDefault);
        if (e != hipSuccess) {
            context->stream[which] = nullptr;
            fail(e, "hipStreamCreateWithFlags");
            return nullptr;
        }
    }
    return (void *)context->stream[which];
}

int nk_hip_thread_buffer(int slot, int pinned, size_t bytes, void **ptr) {
    ThreadContext *context = thread_context();
    if (!context || slot < 0 || slot >= kThreadSlots) return fail_msg("nk_hip_thread_buffer: no such slot");
    CachedBuffer &buffer = pinned ? context->pinned[slot] : context->device[slot];
    if (buffer.bytes < bytes) {
        hipError_t e = hipSuccess;
        if (buffer.ptr) e = pinned ? hipHostFree(buffer.ptr) : hipFree(buffer.ptr);
        buffer.ptr = nullptr, buffer.bytes = 0;
        if (e != hipSuccess) return fail(e, "nk_hip_thread_buffer (release)");
        size_t const rounded = (bytes + 0xFFFFF) & ~(size_t)0xFFFFF; // whole MiB: a slightly larger call does not reallocate
        e = pinned ? hipHostMalloc(&buffer.ptr, rounded, hipHostMallocDefault) : hipMalloc(&buffer.ptr, rounded);
        if (e != hipSuccess) {
            buffer.ptr = nullptr;
            return fail(e, pinned ? "hipHostMalloc" : "hipMalloc");
        }
        buffer.bytes = rounded;
    }
    *ptr = buffer.ptr;
    return 0;
}

size_t nk_hip_thread_cached_bytes(void) {
    ThreadContext *context = thread_context();
    size_t total = 0;
    if (context)
        for (int slot = 0; slot < kThreadSlots; ++slot) total += context->device[slot].bytes + context->pinned[slot].bytes;
    return total;
}

void nk_hip_thread_release(void) {
    ThreadContext *context = thread_context();
    if (context) context->release(false);
}

void nk_hip_thread_trim(size_t slot_bytes, size_t total_bytes) {
    ThreadContext *context = thread_context();
    if (!context) return;
    size_t kept = 0;
    for (int slot = 0; slot < kThreadSlots; ++slot)
        for (CachedBuffer *buffer : {&context->device[slot], &context->pinned[slot]}) {
            if (buffer->bytes > slot_bytes) {
                if (buffer->ptr) (void)(buffer == &context->pinned[slot] ? hipHostFree(buffer->ptr) : hipFree(buffer->ptr));
                *buffer = CachedBuffer();
            }
            kept += buffer->bytes;
        }
    if (kept > total_bytes) context->release(false);
    (void)hipGetLastError();
}

int nk_hip_event_record(int which, void *stream) {
    ThreadContext *context = thread_context();
    if (!context || which < 0 || which >= kThreadEvents) return fail_msg("nk_hip_event_record: no such event");
    if (!context->event[which]) {
        hipError_t e = hipEventCreateWithFlags(&context->event[which], hipEventDisableTiming);
        if (e != hipSuccess) {
            context->event[which] = nullptr;
            return fail(e, "hipEventCreateWithFlags");
        }
    }
    hipError_t e = hipEventRecord(context->event[which], (hipStream_t)stream);
    return e == hipSuccess ? 0 : fail(e, "hipEventRecord");
}
int nk_hip_event_synchronize(int which) {
    ThreadContext *context = thread_context();
    if (!context || which < 0 || which >= kThreadEvents) return fail_msg("nk_hip_event_synchronize: no such event");
    if (!context->event[which]) return 0; // never recorded: nothing to wait for
    hipError_t e = hipEventSynchronize(context->event[which]);
    return e == hipSuccess ? 0 : fail(e, "hipEventSynchronize");
}
int nk_hip_stream_wait_event(void *stream, int which) {
    ThreadContext *context = thread_context();
    if (!context || which < 0 || which >= kThreadEvents || !context->event[which]) return fail_msg("nk_hip_stream_wait_event: no such event");
    hipError_t e = hipStreamWaitEvent((hipStream_t)stream, context->event[which], 0);
    return e == hipSuccess ? 0 : fail(e, "hipStreamWaitEvent");
}
int nk_hip_memcpy_h2d(void *dst, void const *src, size_t bytes, void *stream) {
    if (!bytes) return 0;
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream);
    return e == hipSuccess ? 0 : fail(e, "hipMemcpyAsync(H2D)");
}
int nk_hip_memcpy_d2h(void *dst, void const *src, size_t bytes, void *stream) {
    if (!bytes) return 0;
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream);
    return e == hipSuccess ? 0 : fail(e, "hipMemcpyAsync(D2H)");
}
int nk_hip_memcpy2d_h2d(void *dst, size_t dst_pitch, void const *src, size_t src_pitch, size_t width_bytes,
                        size_t rows, void *stream) {
    if (!width_bytes || !rows) return 0;
    hipError_t e = hipMemcpy2DAsync(dst, dst_pitch, src, src_pitch, width_bytes, rows, hipMemcpyHostToDevice,
                                    (hipStream_t)stream);
    return e == hipSuccess ? 0 : fail(e, "hipMemcpy2DAsync(H2D)");
}
int nk_hip_memcpy2d_d2h(void *dst, size_t dst_pitch, void const *src, size_t src_pitch, size_t width_bytes,
                        size_t rows, void *stream) {
    if (!width_bytes || !rows) return 0;
    hipError_t e = hipMemcpy2DAsync(dst, dst_pitch, src, src_pitch, width_bytes, rows, hipMemcpyDeviceToHost,
                                    (hipStream_t)stream);
    return e == hipSuccess ? 0 : fail(e, "hipMemcpy2DAsync(D2H)");
}
int nk_hip_stream_synchronize(void *stream) {
    hipError_t e = hipStreamSynchronize((hipStream_t)stream);
    return e == hipSuccess ? 0 : fail(e, "hipStreamSynchronize");
}

/**
 *  Device copies of packed images that live in host memory. A caller of the reference's interface allocates the image
 *  with malloc, so every product would have to upload it again; instead the upload is kept and found again by the
 *  number that the pack call left in the image's header (images are opaque: only a pack call changes one, and every
 *  pack call leaves a new number). Least recently used copies that no call is using are dropped beyond 4 entries or
 *  `budget` bytes. An entry is either ready (`device` set: a complete copy, every transfer into it finished) or
 *  loading (reserved by the one thread that uploads it; the others that ask for the same image wait for it).
 */
namespace {
struct CachedImage {
    uint64_t nonce, total_bytes, last_use;
    uint32_t dtype, n, k;
    void *device;
    int users;
    int loading;
};
constexpr int kCachedImages = 4;
CachedImage g_images[kCachedImages];
uint64_t g_image_clock = 0;
pthread_mutex_t g_image_lock = PTHREAD_MUTEX_INITIALIZER;
pthread_cond_t g_image_loaded = PTHREAD_COND_INITIALIZER;
size_t image_budget() {
    static size_t const budget = [] {
        char const *text = getenv("NK_AMD_IMAGE_CACHE_BYTES");
        return text ? (size_t)strtoull(text, nullptr, 10) : (size_t)8 << 30;
    }();
    return budget;
}
bool header_of_host_image(void const *image, size_t total_bytes, PackedHeader &h) {
    if (!image || total_bytes < sizeof(PackedHeader)) return false;
    memcpy(&h, image, sizeof(h));
    return h.magic == kMagic && h.version == kVersion && h.nonce != 0 && h.total_bytes == total_bytes;
}
/** The entry of this image, ready or loading (the lock is held). */
CachedImage *entry_of(PackedHeader const &h, size_t total_bytes) {
    for (CachedImage &entry : g_images)
        if ((entry.device || entry.loading) && entry.nonce == h.nonce && entry.total_bytes == total_bytes &&
            entry.dtype == h.dtype && entry.n == h.n && entry.k == h.k)
            return &entry;
    return nullptr;
}
/** A free entry with `total_bytes` of the budget to go with it, dropping least recently used copies that nobody is
 *  using (into `dropped`, for the caller to free once the lock is released); NULL when everything is in use. */
CachedImage *room_for(size_t total_bytes, void *(&dropped)[kCachedImages]) {
    for (;;) {
        size_t held = 0;
        CachedImage *vacant = nullptr, *oldest = nullptr;
        for (CachedImage &entry : g_images) {
            if (!entry.device && !entry.loading) { vacant = vacant ? vacant : &entry; continue; }
            held += entry.total_bytes;
            if (entry.device && !entry.users && (!oldest || entry.last_use < oldest->last_use)) oldest = &entry;
        }
        if (vacant && held + total_bytes <= image_budget()) return vacant;
        if (!oldest) return nullptr;
        for (void *&slot : dropped)
            if (!slot) { slot = oldest->device; break; }
        oldest->device = nullptr;
    }
}
void free_dropped(void *(&dropped)[kCachedImages]) {
    for (void *image : dropped)
        if (image) (void)hipFree(image);
}
} // namespace

int nk_hip_image_cache_find(void const *host_image, size_t total_bytes, void **device_image) {
    PackedHeader h;
    *device_image = nullptr;
    if (!header_of_host_image(host_image, total_bytes, h)) return 0;
    int found = 0;
    pthread_mutex_lock(&g_image_lock);
    CachedImage *entry = entry_of(h, total_bytes);
    if (entry && entry->device) {
        entry->users++, entry->last_use = ++g_image_clock;
        *device_image = entry->device, found = 1;
    }
    pthread_mutex_unlock(&g_image_lock);
    return found;
}

int nk_hip_image_cache_claim(void const *host_image, size_t total_bytes, void **device_image) {
    PackedHeader h;
    *device_image = nullptr;
    if (!header_of_host_image(host_image, total_bytes, h) || total_bytes > image_budget()) return 0;
    void *dropped[kCachedImages] = {};
    int outcome = 0;
    pthread_mutex_lock(&g_image_lock);
    for (;;) {
        CachedImage *entry = entry_of(h, total_bytes);
        if (entry && entry->device) {
            entry->users++, entry->last_use = ++g_image_clock;
            *device_image = entry->device, outcome = 1;
            break;
        }
        if (entry) { // another thread is uploading this very image: its copy will do
            pthread_cond_wait(&g_image_loaded, &g_image_lock);
            continue;
        }
        CachedImage *vacant = room_for(total_bytes, dropped);
        if (vacant) *vacant = CachedImage {h.nonce, total_bytes, ++g_image_clock, h.dtype, h.n, h.k, nullptr, 1, 1}, outcome = 2;
        break;
    }
    pthread_mutex_unlock(&g_image_lock);
    free_dropped(dropped);
    return outcome;
}

int nk_hip_image_cache_publish(void const *host_image, size_t total_bytes, void *device_image) {
    PackedHeader h;
    if (!device_image || !header_of_host_image(host_image, total_bytes, h)) return 0;
    int published = 0;
    pthread_mutex_lock(&g_image_lock);
    CachedImage *entry = entry_of(h, total_bytes);
    if (entry && entry->loading && !entry->device) {
        entry->device = device_image, entry->loading = 0, entry->last_use = ++g_image_clock; // (users stays 1: the uploader)
        published = 1;
    }
    pthread_cond_broadcast(&g_image_loaded);
    pthread_mutex_unlock(&g_image_lock);
    return published;
}

void nk_hip_image_cache_abandon(void const *host_image, size_t total_bytes) {
    PackedHeader h;
    if (!header_of_host_image(host_image, total_bytes, h)) return;
    pthread_mutex_lock(&g_image_lock);
    CachedImage *entry = entry_of(h, total_bytes);
    if (entry && entry->loading && !entry->device) *entry = CachedImage {};
    pthread_cond_broadcast(&g_image_loaded); // (one of those waiting takes over the upload)
    pthread_mutex_unlock(&g_image_lock);
}

int nk_hip_image_cache_adopt(void const *host_image, size_t total_bytes, void *device_image) {
    PackedHeader h;
    if (!device_image || !header_of_host_image(host_image, total_bytes, h) || total_bytes > image_budget()) return 0;
    void *dropped[kCachedImages] = {};
    int adopted = 0;
    pthread_mutex_lock(&g_image_lock);
    if (!entry_of(h, total_bytes)) { // (a copy of this image that is there already, or on its way, is enough)
        CachedImage *vacant = room_for(total_bytes, dropped);
        if (vacant) *vacant = CachedImage {h.nonce, total_bytes, ++g_image_clock, h.dtype, h.n, h.k, device_image, 1, 0}, adopted = 1;
    }
    pthread_mutex_unlock(&g_image_lock);
    free_dropped(dropped);
    return adopted;
}

void nk_hip_image_cache_release(void *device_image) {
    pthread_mutex_lock(&g_image_lock);
    for (CachedImage &entry : g_images)
        if (entry.device == device_image && entry.users > 0) entry.users--;
    pthread_mutex_unlock(&g_image_lock);
}

void nk_hip_image_cache_clear(void) {
    void *dropped[kCachedImages] = {};
    pthread_mutex_lock(&g_image_lock);
    for (int i = 0; i < kCachedImages; ++i)
        if (g_images[i].device && !g_images[i].users) dropped[i] = g_images[i].device, g_images[i].device = nullptr;
    pthread_mutex_unlock(&g_image_lock);
    free_dropped(dropped);
}

size_t nk_hip_dots_packed_size(int dtype, size_t n, size_t k) {
    WideGeometry wide;
    if (wide_geometry(dtype, n, k, wide)) return (size_t)wide.total_bytes;
    Geometry g;
    if (!make_geometry(dtype, n, k, g)) return 0;
    return (size_t)g.total_bytes;
}

/** `terms`: also the per-column terms after the tiles (only the u8 product and the distances read them). */
static int pack_async(int dtype, void const *b, size_t n, size_t k, size_t b_stride, void *b_packed, void *stream_,
                      bool terms) {
    hipStream_t stream = (hipStream_t)stream_;
    Geometry g;
    bool const wide = dtype == kF32 || dtype == kF64;
    if (!wide && !make_geometry(dtype, n, k, g)) return fail_msg("nk_hip_dots_pack: unsupported dtype or dimensions");
    if (!b_packed || ((uintptr_t)b_packed & 15)) return fail_msg("nk_hip_dots_pack: b_packed must be 16-byte aligned");
    if (n && k && !b) return fail_msg("nk_hip_dots_pack: b is NULL");
    if (wide) {
        hipError_t const status = wide_pack(dtype, b, n, k, b_stride, b_packed, stream);
        return status == hipSuccess ? 0 : fail(status, "nk_hip_dots_pack (f32 / f64)");
    }
    if (elem_bits_of(dtype) == 16 && (((uintptr_t)b | b_stride) & 1)) return fail_msg("nk_hip_dots_pack: 16-bit B is misaligned");

    PackedHeader h;
    memset(&h, 0, sizeof(h));
    h.magic = kMagic, h.version = kVersion, h.dtype = (uint32_t)dtype, h.elem_bytes = g.packed_bytes;
    h.n = g.n, h.k = g.k, h.n_tiles = g.n_tiles, h.k_chunks = g.k_chunks;
    h.nonce = next_image_nonce();
    h.sums_offset = sizeof(PackedHeader) + g.data_bytes;
    h.norms_offset = h.sums_offset + g.sums_bytes;
    h.total_bytes = g.total_bytes;

    uint8_t *image = (uint8_t *)b_packed;
    uint8_t *data = image + sizeof(PackedHeader);
    uint32_t *sums = (uint32_t *)(data + g.data_bytes);
    uint32_t *norms = sums + (uint64_t)g.n_tiles * kTileRows;
    hipError_t e = hipSuccess;
    if (!(g.n_tiles && g.k_chunks)) { // nothing to pack: the header alone
        hipLaunchKernelGGL(write_header_kernel, dim3(1), dim3(64), 0, stream, (PackedHeader *)image, h);
        if ((e = hipGetLastError()) != hipSuccess) return fail(e, "write_header_kernel");
    }
    if (g.n_tiles && g.k_chunks) {
        uint32_t const xr = dtype == kU8 ? 0x80808080u : 0u;
        // by how the source is widened and by what the image then holds (see pack_kernel)
        typedef void (*pack_fn)(uint8_t const *, uint64_t, uint32_t, uint64_t, uint32_t, uint32_t, uint8_t *, uint32_t *,
                                uint32_t *, int, uint32_t, int, PackedHeader);
        pack_fn kernel = nullptr;
        switch (widen_kind_of(dtype, k)) {
        case 0: kernel = dtype == kI8 ? pack_kernel<0, 0> : (dtype == kU8 ? pack_kernel<0, 1> : (dtype == kBF16 ? pack_kernel<0, 2> : pack_kernel<0, 3>)); break;
        case 1: kernel = kE4M3ViaBF16 ? pack_kernel<1, 2> : pack_kernel<1, 3>; break;
        case 2: kernel = pack_kernel<2, 3>; break;
        case 3: kernel = pack_kernel<3, 0>; break;
        case 4: kernel = pack_kernel<4, 3>; break;
        case 5: kernel = pack_kernel<5, 0>; break;
        case 6: kernel = pack_kernel<6, 0>; break;
        case 7: kernel = pack_kernel<7, 4>; break;
        default: kernel = pack_kernel<8, 3>; break;
        }
        hipLaunchKernelGGL(kernel, dim3(g.n_tiles), dim3(kPackThreads), 0, stream, (uint8_t const *)b, (uint64_t)b_stride, g.n,
                           g.k_src_bytes, g.k_chunks, g.k, data, sums, norms, widest_load(b, b_stride), xr, terms ? 1 : 0, h);
        e = hipGetLastError();
        if (e != hipSuccess) return fail(e, "pack_kernel");
    }
    else if (g.n_tiles && terms) { // no depth at all: the terms are zeros
        uint64_t const count = 2 * (uint64_t)g.n_tiles * kTileRows; // both arrays, back to back
        hipLaunchKernelGGL(fill_u32_kernel, dim3((uint32_t)((count + 255) / 256)), dim3(256), 0, stream, sums, count, 0u);
        e = hipGetLastError();
        if (e != hipSuccess) return fail(e, "fill_u32_kernel");
    }
    return 0;
}

int nk_hip_dots_pack_async(int dtype, void const *b, size_t n, size_t k, size_t b_stride, void *b_packed,
                           void *stream) {
    return pack_async(dtype, b, n, k, b_stride, b_packed, stream, true);
}

int nk_hip_fill_rows_async(void *c, size_t m, size_t n, size_t c_stride, uint32_t value, void *stream) {
    if (!m || !n) return 0;
    if (m > 0x7FFFFFFFull || n > 0x7FFFFFFFull) return fail_msg("nk_hip_fill_rows: dimensions too large");
    uint64_t const count = (uint64_t)m * n;
    uint64_t const blocks = (count + 255) / 256;
    if (blocks > 0x7FFFFFFFull) return fail_msg("nk_hip_fill_rows: matrix too large");
    hipLaunchKernelGGL(fill_rows_kernel, dim3((uint32_t)blocks), dim3(256), 0, (hipStream_t)stream, (uint8_t *)c,
                       (uint32_t)m, (uint32_t)n, (uint64_t)c_stride, value, 0u, 0u);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : fail(e, "fill_rows_kernel");
}

/** `triangle`: NULL for the full m x n product; otherwise only the outputs with col >= row + shift are computed
 *  and stored, over a tile list built in that scratch memory. */
static int product_async(int dtype, int metric, void const *a, void const *b_packed, void *c, size_t m, size_t n,
                         size_t k, size_t a_stride, size_t c_stride, void *stream_,
                         TriangleScratch const *triangle = nullptr, uint32_t shift = 0) {
    hipStream_t stream = (hipStream_t)stream_;
    if (!m || !n) return 0;
    if (dtype == kF32 || dtype == kF64) { // f64 results, a kernel of their own
        if (!c || !b_packed || (k && !a)) return fail_msg("nk_hip_dots_packed: NULL operand");
        hipError_t const status = wide_product(dtype, a, b_packed, c, m, n, k, a_stride, c_stride, stream, triangle != nullptr, shift, metric);
        return status == hipSuccess ? 0 : fail(status, "nk_hip_dots_packed (f32 / f64)");
    }
    Geometry geo;
    if (!make_geometry(dtype, n, k, geo)) return fail_msg("nk_hip_dots_packed: unsupported dtype or dimensions");
    if (m > 0x7FFFFFFFull) return fail_msg("nk_hip_dots_packed: too many rows");
    if (!c || ((uintptr_t)c & 3) || (c_stride & 3)) return fail_msg("nk_hip_dots_packed: c must be 4-byte aligned");
    if (!b_packed || ((uintptr_t)b_packed & 15)) return fail_msg("nk_hip_dots_packed: b_packed must be 16-byte aligned");
    if (k == 0 && !triangle) return nk_hip_fill_rows_async(c, m, n, c_stride, 0u, stream_);
    if (k == 0) {
        uint64_t const blocks = ((uint64_t)m * n + 255) / 256;
        if (blocks > 0x7FFFFFFFull) return fail_msg("nk_hip_dots_symmetric: matrix too large");
        hipLaunchKernelGGL(fill_rows_kernel, dim3((uint32_t)blocks), dim3(256), 0, stream, (uint8_t *)c, (uint32_t)m,
                           (uint32_t)n, (uint64_t)c_stride, 0u, shift, 0xFFFFFFFFu);
        hipError_t const e = hipGetLastError();
        return e == hipSuccess ? 0 : fail(e, "fill_rows_kernel");
    }
    if (!a) return fail_msg("nk_hip_dots_packed: a is NULL");
    if (elem_bits_of(dtype) == 16 && (((uintptr_t)a | a_stride) & 1)) return fail_msg("nk_hip_dots_packed: 16-bit A is misaligned");

    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.a = (uint8_t const *)a, g.bp = (uint8_t const *)b_packed, g.c = (uint8_t *)c;
    g.a_stride = a_stride, g.c_stride = c_stride, g.k_src_bytes = geo.k_src_bytes;
    g.m = (uint32_t)m, g.n = geo.n, g.k = geo.k, g.n_tiles = geo.n_tiles, g.k_chunks = geo.k_chunks;
    g.avec = widest_load(a, a_stride);
    g.metric = metric;
    if (triangle) g.tri_shift = shift, g.tri_mask = 0xFFFFFFFFu;
    {
        // Stages between accumulator folds: about an eighth of the depth, even, between 2 and 16.
        uint32_t const eighth = (g.k_chunks / kStageChunks / 8) & ~1u;
        g.chunk_stages = eighth < 2 ? 2 : (eighth > 16 ? 16 : eighth);
    }

    hipError_t e;
    switch (dtype) {
    case kI8: e = launch_i8(g, stream, triangle); break;
    case kU8: e = launch_u8(g, stream, triangle); break;
    case kBF16: e = launch_bf16(g, stream, triangle); break;
    case kF16: e = launch_f16(g, stream, triangle); break;
    case kE4M3: e = launch_e4m3(g, stream, triangle); break;
    case kE5M2: e = launch_e5m2(g, stream, triangle); break;
    case kE2M3: e = launch_e2m3(g, stream, triangle); break;
    case kE3M2: e = launch_e3m2(g, stream, triangle); break;
    case kI4: e = launch_i4(g, stream, triangle); break;
    case kU4: e = launch_u4(g, stream, triangle); break;
    case kU1: e = launch_u1(g, stream, triangle); break;
    default: return fail_msg("nk_hip_dots_packed: unsupported dtype");
    }
    return e == hipSuccess ? 0 : fail(e, "dots_packed_kernel");
}

int nk_hip_dots_packed_async(int dtype, void const *a, void const *b_packed, void *c, size_t m, size_t n, size_t k,
                             size_t a_stride, size_t c_stride, void *stream) {
    return product_async(dtype, 0, a, b_packed, c, m, n, k, a_stride, c_stride, stream);
}

int nk_hip_spatials_packed_async(int dtype, int metric, void const *a, void const *b_packed, void *c, size_t m, size_t n,
                                 size_t k, size_t a_stride, size_t c_stride, void *stream) {
    if (metric != 1 && metric != 2) return fail_msg("nk_hip_spatials_packed: metric must be 1 (angular) or 2 (euclidean)");
    return product_async(dtype, metric, a, b_packed, c, m, n, k, a_stride, c_stride, stream);
}

/** What one symmetric call covers: rows [row_start, row_end) of the result, and of those the columns from
 *  `col_begin` (the start of the 32-row tile of the packed image that holds row_start) to the end. */
struct SymmetricWindow {
    size_t row_end, col_begin, columns, image_bytes, scratch_bytes;
};
static bool symmetric_window(int dtype, size_t n, size_t k, size_t row_start, size_t row_count, SymmetricWindow &w) {
    w.row_end = row_count < n - row_start ? row_start + row_count : n;
    w.col_begin = row_start / kTileRows * kTileRows;
    w.columns = n - w.col_begin;
    w.scratch_bytes = 0;
    WideGeometry wide;
    if (wide_geometry(dtype, w.columns, k, wide)) { // (no tile lists: that kernel walks the full grid and skips tiles)
        w.image_bytes = (size_t)((wide.total_bytes + 255) & ~255ull);
        return true;
    }
    Geometry geo;
    if (!make_geometry(dtype, w.columns, k, geo)) return false;
    w.image_bytes = (size_t)((geo.total_bytes + 255) & ~255ull);
    uint32_t const shift = (uint32_t)(row_start - w.col_begin);
    for (int c = 1; c < kConfigCount; ++c) {
        size_t const bytes = triangle_scratch_bytes(w.row_end - row_start, w.columns, kConfigs[c].tm * 32,
                                                    kConfigs[c].tn * 128, shift);
        if (bytes > w.scratch_bytes) w.scratch_bytes = bytes;
    }
    w.scratch_bytes = 2 * ((w.scratch_bytes + 7) & ~(size_t)7); // room for the lists of two launches (see launch_typed)
    return true;
}

size_t nk_hip_symmetric_workspace_size(int dtype, size_t n, size_t k, size_t row_start, size_t row_count) {
    if (row_start >= n || !row_count) return 0;
    SymmetricWindow w;
    if (!symmetric_window(dtype, n, k, row_start, row_count, w)) return 0;
    return w.image_bytes + w.scratch_bytes;
}

int nk_hip_symmetric_async(int dtype, int metric, void const *vectors, size_t n, size_t k, size_t stride, void *result,
                           size_t result_stride, size_t row_start, size_t row_count, void *workspace,
                           size_t workspace_bytes, void *stream) {
    if (metric < 0 || metric > 2) return fail_msg("nk_hip_symmetric: metric must be 0 (dots), 1 (angular) or 2 (euclidean)");
    if (row_start >= n || !row_count) return 0;
    SymmetricWindow w;
    if (!symmetric_window(dtype, n, k, row_start, row_count, w)) return fail_msg("nk_hip_symmetric: unsupported dtype or dimensions");
    if (!workspace || ((uintptr_t)workspace & 255)) return fail_msg("nk_hip_symmetric: workspace must be 256-byte aligned");
    if (workspace_bytes < w.image_bytes + w.scratch_bytes) return fail_msg("nk_hip_symmetric: workspace too small");
    size_t const out_bytes = dtype == kF32 || dtype == kF64 ? 8 : 4;
    if (!result || (((uintptr_t)result | result_stride) & (out_bytes - 1))) return fail_msg("nk_hip_symmetric: result is misaligned");
    if (k && !vectors) return fail_msg("nk_hip_symmetric: vectors is NULL");
    // The columns of the window, packed as the B of an ordinary product; the rows of the window are its A.
    uint8_t const *rows = (uint8_t const *)vectors;
    int status = pack_async(dtype, rows + w.col_begin * stride, w.columns, k, stride, workspace, stream,
                            metric != 0 || dtype == kU8);
    if (status) return status;
    TriangleScratch const scratch = {(uint32_t *)((uint8_t *)workspace + w.image_bytes), w.scratch_bytes};
    uint8_t *c = (uint8_t *)result + row_start * result_stride + w.col_begin * out_bytes;
    return product_async(dtype, metric, rows + row_start * stride, workspace, c, w.row_end - row_start, w.columns, k, stride,
                         result_stride, stream, &scratch, (uint32_t)(row_start - w.col_begin));
}

/**
 *  The symmetric kinds for callers that cannot allocate: the workspace is a fixed array in device memory that belongs
 *  to the library (each GPU the library runs on holds its own copy until the process ends), found once per device by
 *  its symbol. Calls that overlap on one GPU share it and race; the array keeps the last call's contents, and nothing
 *  in this path expects zeros there (the pack kernels write every byte of the image they read, padding included, and
 *  the tile lists are written before they are read).
 */
constexpr size_t kStaticWorkspaceBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticWorkspaceBytes];

constexpr int kMaxDevices = 64;
static std::atomic<void *> g_scratch_of_device[kMaxDevices];

/** The address of `scratch` on the current device (the array's name is a host-side stand-in, not a device address). */
static int static_workspace(void **workspace) {
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return fail(e, "hipGetDevice");
    if (device < 0 || device >= kMaxDevices) return fail_msg("nk_hip_symmetric_static: device index out of range");
    void *ptr = g_scratch_of_device[device].load(std::memory_order_acquire);
    if (!ptr) {
        e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) return fail(e, "hipGetSymbolAddress(scratch)");
        g_scratch_of_device[device].store(ptr, std::memory_order_release);
    }
    *workspace = ptr;
    return 0;
}

size_t nk_hip_symmetric_static_capacity(void) { return kStaticWorkspaceBytes; }

int nk_hip_symmetric_static_async(int dtype, int metric, void const *vectors, size_t n, size_t k, size_t stride,
                                  void *result, size_t result_stride, size_t row_start, size_t row_count, void *stream) {
    if (row_start >= n || !row_count) return 0;
    size_t const needed = nk_hip_symmetric_workspace_size(dtype, n, k, row_start, row_count);
    if (!needed) return fail_msg("nk_hip_symmetric_static: unsupported dtype or dimensions");
    if (needed > kStaticWorkspaceBytes) {
        snprintf(g_last_error, sizeof(g_last_error),
                 "nk_hip_symmetric_static: this call needs %zu bytes of workspace, the built-in one holds %zu; use "
                 "nk_hip_symmetric_async with a workspace of the caller's",
                 needed, kStaticWorkspaceBytes);
        return -1;
    }
    void *workspace = nullptr;
    int const status = static_workspace(&workspace);
    if (status) return status;
    return nk_hip_symmetric_async(dtype, metric, vectors, n, k, stride, result, result_stride, row_start, row_count,
                                  workspace, kStaticWorkspaceBytes, stream);
}

void nk_hip_set_tile_config(int config) {
    t_forced_config = config; // (bits 0..6 the shape; bit 7: a forced shape may still hand the narrow end of a triangle to small tiles; bits 8..27: start spread in 10 ns ticks + 1; bits 28..29: kind of store; bit 30: no staging straight into LDS)
}

char const *nk_hip_last_error(void) { return g_last_error; }

} // extern "C"
