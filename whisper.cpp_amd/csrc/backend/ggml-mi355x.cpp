// The five ggml-backend vtables for MI355X (ggml/src/ggml-backend-impl.h:17-207 of the whisper.cpp tree)
// and the two dynamic-loading entry points (ggml-backend-impl.h:215-218).  Host-side only: device memory
// comes from hipMalloc, transfers are hipMemcpy on the backend's stream, all arithmetic goes through the
// kernel C ABI declared in mi355x_kernels.h.
#include "backend.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <chrono>

// ------------------------------------------------------------------------------------------------------
// device discovery
// ------------------------------------------------------------------------------------------------------

static std::vector<int> & gfx950_devices() {
    static std::vector<int> devs = [] {
        std::vector<int> v;
        int n = 0;
        if (hipGetDeviceCount(&n) != hipSuccess) { (void) hipGetLastError(); return v; }
        for (int i = 0; i < n; ++i) if (mi355x_device_is_gfx950(i) == 1) v.push_back(i);
        return v;
    }();
    return devs;
}

static bool env_flag(const char * name, bool dflt) {
    const char * v = getenv(name);
    if (!v || !*v) return dflt;
    return atoi(v) != 0;
}

// live backend contexts, so that options and statistics can address all of them at once (backend == NULL) and the
// buffer-level transfers can find the host mirrors of graph outputs
static std::mutex                        g_live_mutex;
static std::vector<mi355x_backend_ctx *> g_live;
static std::map<std::string, mi355x_kernel_stat> g_retired_stats;   // statistics of backends that were freed
static int64_t g_retired_counters[MI355X_N_COUNTERS] = {};

// ------------------------------------------------------------------------------------------------------
// host <-> device transfers of the buffer interface
//
// A decode step uploads three or four small inputs (token ids, positions, the attention mask) and downloads 1 MB of
// logits.  hipMemcpy from pageable memory costs 11 us for 20 bytes and 33 us for 64 KB on this system, because the
// runtime stages and waits; copying into a pinned ring and queueing the transfer on the null stream returns in 2 us.
// The ordering ggml relies on is kept by the streams: every backend instance's stream is a blocking stream, so work
// queued on it later starts after the transfer, and the transfer starts after the kernels queued before it; reads
// back go through the same null stream.  The caller's memory is free for reuse on return, as set_tensor promises.
//
// Downloads: a graph's result that the host fetches in several pieces (a decode step's logits, which whisper_decode reads
// row by row with one blocking ggml_backend_tensor_get per beam, src/whisper.cpp:2960-2966) is, once that has been seen, copied
// into pinned memory at the end of every graph_compute that produces it — as its last node or as a flagged output, the two kinds of
// tensor whose memory still holds their value when the graph is over — in one transfer on the backend's stream
// (mi355x_backend_ctx::mirror_outputs); get_tensor serves slices of it from there — a memcpy — until something writes
// the tensor or the next graph runs.  Compute-buffer addresses are stable from step to step (ggml/src/ggml-alloc.c:816-914),
// which is what makes "the tensor at this address" a usable key.  Everything else is a plain hipMemcpy.
// ------------------------------------------------------------------------------------------------------

// [lo, hi): the bytes the host has asked for so far; reads: get_tensor calls on it since the last graph
struct wanted_download { int device; const void * data; size_t size, lo, hi; int reads; };
static std::mutex                   g_wanted_mutex;
static std::vector<wanted_download> g_wanted;            // a handful of entries: the outputs the host reads back

bool mi355x_download_is_wanted(int device, const void * data, size_t size, size_t * lo, size_t * hi) {
    std::lock_guard<std::mutex> lock(g_wanted_mutex);
    for (wanted_download & w : g_wanted) if (w.device == device && w.data == data && w.size == size) {
        // One transfer into pinned memory and a memcpy per read beats blocking copies when the host reads the result in
        // several pieces (the five rows of a 5-beam step: 132 us against 213 us per graph measured); a single read is
        // faster as one blocking copy (by 10 us per step).  So: mirror when the last graph's result was read more than once.
        const int reads = w.reads;
        w.reads = 0;
        *lo = w.lo; *hi = w.hi;
        return reads >= 2;
    }
    return false;
}

static void count_download(int device, const void * data) {
    std::lock_guard<std::mutex> lock(g_wanted_mutex);
    for (wanted_download & w : g_wanted) if (w.device == device && w.data == data) w.reads += 1;
}

// the host fetched [offset, offset + len) of the tensor (data, size)
static void want_download(int device, const void * data, size_t size, size_t offset, size_t len) {
    std::lock_guard<std::mutex> lock(g_wanted_mutex);
    for (wanted_download & w : g_wanted) if (w.device == device && w.data == data && w.size == size) {
        w.lo = std::min(w.lo, offset); w.hi = std::max(w.hi, offset + len); w.reads += 1;
        return;
    }
    if (g_wanted.size() >= 64) g_wanted.erase(g_wanted.begin());
    g_wanted.push_back({ device, data, size, offset, offset + len, 1 });
}

// a buffer is going away: nothing at its addresses is wanted any more
static void forget_downloads(int device, const void * begin, size_t size) {
    std::lock_guard<std::mutex> lock(g_wanted_mutex);
    const char * b = (const char *) begin;
    for (size_t i = 0; i < g_wanted.size();) {
        if (g_wanted[i].device == device && (const char *) g_wanted[i].data >= b && (const char *) g_wanted[i].data < b + size) g_wanted.erase(g_wanted.begin() + (long) i); else ++i;
    }
}

// [data + offset, + size) of a tensor from the host mirror of a backend instance on this device; false: not mirrored
static bool download_from_mirror(int device, const struct ggml_tensor * tensor, void * data, size_t offset, size_t size) {
    // Find the entry under the locks, wait for its transfer without them (a host thread that reads one state's logits must
    // not hold up the options, statistics and buffer writes of every other state for a whole graph), then look again: a
    // write may have retired the mirror meanwhile.
    for (int attempt = 0; attempt < 2; ++attempt) {
        hipEvent_t done = nullptr;
        {
            std::lock_guard<std::mutex> live(g_live_mutex);
            for (mi355x_backend_ctx * ctx : g_live) {
                if (ctx->device != device) continue;
                std::lock_guard<std::mutex> lock(ctx->mirror_mutex);
                for (const mi355x_backend_ctx::mirror_entry & e : ctx->mirror) {
                    if (e.dev != (const char *) tensor->data || offset < e.lo || offset + size > e.lo + e.size) continue;
                    if (attempt == 0 && hipEventQuery(ctx->mirror_done) != hipSuccess) { (void) hipGetLastError(); done = ctx->mirror_done; break; }
                    if (attempt == 1 && hipEventQuery(ctx->mirror_done) != hipSuccess) { (void) hipGetLastError(); return false; }
                    memcpy(data, ctx->mirror_host + e.off + (offset - e.lo), size);
                    ctx->counters[4] += 1;
                    return true;
                }
                if (done) break;
            }
        }
        if (!done) return false;
        // (the event belongs to a live instance; an instance is freed only after its host thread stopped calling into it, and a
        // destroyed event makes the wait fail, which sends the read down the plain copy path)
        if (hipEventSynchronize(done) != hipSuccess) { (void) hipGetLastError(); return false; }
    }
    return false;
}

// something writes [begin, begin + size) on this device: mirrors of that range are stale
static void drop_mirrors(int device, const void * begin, size_t size) {
    std::lock_guard<std::mutex> live(g_live_mutex);
    for (mi355x_backend_ctx * ctx : g_live) if (ctx->device == device) ctx->mirror_drop(begin, size);
}

#define STAGE_RING_BYTES   (8u << 20)
#define STAGE_UPLOAD_MAX   (512u << 10)      // larger uploads (model weights) take the runtime's own path

struct staging_ring {
    std::mutex m;
    char *     base = nullptr;
    size_t     head = 0;
    bool       failed = false;
};
static staging_ring g_rings[64];             // per device, pinned for the life of the process

static staging_ring * ring_of(int device) {
    if (device < 0 || device >= 64) return nullptr;
    staging_ring & r = g_rings[device];
    std::lock_guard<std::mutex> lock(r.m);             // two states of one context may make their first upload at once
    if (!r.base && !r.failed) {
        void * p = nullptr;
        const bool ok = hipHostMalloc(&p, STAGE_RING_BYTES, hipHostMallocDefault) == hipSuccess && p;
        if (ok) r.base = (char *) p; else { (void) hipGetLastError(); r.failed = true; }
    }
    return r.base ? &r : nullptr;
}

// the current device is `device`
static bool upload(int device, void * dst, const void * src, size_t size) {
    if (size == 0) return true;
    if (size <= STAGE_UPLOAD_MAX) {
        if (staging_ring * r = ring_of(device)) {
            std::lock_guard<std::mutex> lock(r->m);
            const size_t need = (size + 255) & ~(size_t) 255;
            if (r->head + need > STAGE_RING_BYTES) {        // wrapped: the transfers queued from the ring must have left it
                if (hipStreamSynchronize(nullptr) != hipSuccess) { (void) hipGetLastError(); return false; }
                r->head = 0;
            }
            memcpy(r->base + r->head, src, size);
            if (hipMemcpyAsync(dst, r->base + r->head, size, hipMemcpyHostToDevice, nullptr) == hipSuccess) { r->head += need; return true; }
            (void) hipGetLastError();
        }
    }
    return hipMemcpy(dst, src, size, hipMemcpyHostToDevice) == hipSuccess;
}

// ------------------------------------------------------------------------------------------------------
// buffer  (ggml_backend_buffer_i, ggml-backend-impl.h:41-58)
// ------------------------------------------------------------------------------------------------------

const void * mi355x_buffer_ctx::weight_image(const struct ggml_tensor * w, hipStream_t stream, int kind) {
    std::lock_guard<std::mutex> lock(image_mutex);
    if ((uintptr_t) w->data & 1) return nullptr;
    const uintptr_t key = (uintptr_t) w->data | (uintptr_t) kind;
    auto it = images.find(key);
    if (it != images.end()) {
        const mi355x_weight_image & im = it->second;
        if (im.type == (int) w->type && im.ne0 == w->ne[0] && im.ne1 == w->ne[1]) return im.f16;
        (void) hipFree(im.f16);                       // same address, another tensor: the buffer was laid out anew
        images.erase(it);
    }
    mi355x_weight_image im = { nullptr, ggml_nbytes(w), (int) w->type, w->ne[0], w->ne[1] };
    const int64_t n = w->ne[0] * w->ne[1];
    const size_t bytes = kind == MI355X_IMAGE_TILES ? mi355x_q8_0_tiles_size(w->ne[0], w->ne[1]) : (size_t) n * 2;
    if (!bytes) return nullptr;
    if (hipMalloc(&im.f16, bytes) != hipSuccess || !im.f16) {
        (void) hipGetLastError();
        static bool warned = false;
        if (!warned) { warned = true; GGML_LOG_WARN("ggml-mi355x: no memory for the %s of %s (%.1f MiB); it is multiplied from its block rows\n", kind == MI355X_IMAGE_TILES ? "tiles" : "f16 image", w->name, bytes / 1048576.0); }
        return nullptr;
    }
    int rc;
    if (kind == MI355X_IMAGE_TILES) {
        mi355x_tensor t = {};
        t.data = w->data; t.type = (int) w->type;
        for (int i = 0; i < 4; ++i) { t.ne[i] = w->ne[i]; t.nb[i] = w->nb[i]; }
        rc = mi355x_q8_0_tiles_pack(&t, im.f16, stream);
    } else {
        rc = mi355x_dequantize_row_f16((int) w->type, w->data, im.f16, n, stream);
    }
    if (rc != MI355X_OK) { (void) hipFree(im.f16); return nullptr; }
    // The image is shared by every backend instance that uses these weights (whisper_full_parallel: one instance and one
    // stream per state), so it is complete before anyone can find it: once per weight matrix.
    if (hipStreamSynchronize(stream) != hipSuccess) { (void) hipGetLastError(); (void) hipFree(im.f16); return nullptr; }
    images.emplace(key, im);
    return im.f16;
}

void mi355x_buffer_ctx::drop_images(const void * begin, size_t nbytes) {
    std::lock_guard<std::mutex> lock(image_mutex);
    const uintptr_t b = (uintptr_t) begin, e = b + nbytes;
    for (auto it = images.begin(); it != images.end();) {
        const uintptr_t at = it->first & ~(uintptr_t) 1;                // (the lowest bit of the key is the kind of image)
        if (at < e && b < at + it->second.src_bytes) { (void) hipFree(it->second.f16); it = images.erase(it); }   // hipFree waits for the device
        else ++it;
    }
}

void mi355x_buffer_ctx::drop_all_images() {
    std::lock_guard<std::mutex> lock(image_mutex);
    for (auto & kv : images) (void) hipFree(kv.second.f16);
    images.clear();
}

static void buffer_free(ggml_backend_buffer_t buffer) {
    mi355x_buffer_ctx * ctx = (mi355x_buffer_ctx *) buffer->context;
    HIP_TRY(hipSetDevice(ctx->device), (void) 0);
    HIP_TRY(hipDeviceSynchronize(), (void) 0);
    ctx->drop_all_images();
    drop_mirrors(ctx->device, ctx->base, ctx->size);
    forget_downloads(ctx->device, ctx->base, ctx->size);
    HIP_TRY(hipFree(ctx->base), (void) 0);
    delete ctx;
}

static void * buffer_get_base(ggml_backend_buffer_t buffer) {
    return ((mi355x_buffer_ctx *) buffer->context)->base;
}

static enum ggml_status buffer_init_tensor(ggml_backend_buffer_t, struct ggml_tensor *) {
    return GGML_STATUS_SUCCESS;   // tensors need no per-tensor state
}

// Buffer-level transfers are synchronous (the scheduler synchronizes the backend before it calls them,
// ggml/src/ggml-backend.cpp:1371-1375); they run on the null stream, which orders itself against the
// backend's (blocking) stream.
static void buffer_memset_tensor(ggml_backend_buffer_t buffer, struct ggml_tensor * tensor, uint8_t value, size_t offset, size_t size) {
    mi355x_buffer_ctx * ctx = (mi355x_buffer_ctx *) buffer->context;
    HIP_TRY(hipSetDevice(ctx->device), return);
    ctx->drop_images((char *) tensor->data + offset, size);
    drop_mirrors(ctx->device, (char *) tensor->data + offset, size);
    ctx->unwritten.written((char *) tensor->data + offset, size);
    HIP_TRY(hipMemset((char *) tensor->data + offset, value, size), return);
    HIP_TRY(hipStreamSynchronize(nullptr), return);
}

static void buffer_set_tensor(ggml_backend_buffer_t buffer, struct ggml_tensor * tensor, const void * data, size_t offset, size_t size) {
    mi355x_buffer_ctx * ctx = (mi355x_buffer_ctx *) buffer->context;
    HIP_TRY(hipSetDevice(ctx->device), return);
    ctx->drop_images((char *) tensor->data + offset, size);
    drop_mirrors(ctx->device, (char *) tensor->data + offset, size);
    ctx->unwritten.written((char *) tensor->data + offset, size);
    if (!upload(ctx->device, (char *) tensor->data + offset, data, size)) {
        GGML_LOG_ERROR("ggml-mi355x: upload of %zu bytes into %s failed: %s\n", size, tensor->name, hipGetErrorString(hipGetLastError()));
    }
}

// A download or copy of memory whose value a launch folded away (the graph came in pieces and the walker saw no reader):
// say so, and hand over NaN patterns instead of whatever the memory held.
static bool refuse_stale_read(mi355x_buffer_ctx * ctx, const struct ggml_tensor * tensor, size_t offset, size_t size, const char * what) {
    char name[48];
    if (!ctx->unwritten.stale((const char *) tensor->data + offset, size, name)) return false;
    GGML_LOG_ERROR("ggml-mi355x: %s of %s reads memory of %s, which an earlier launch folded into its consumer and never stored "
                   "(a graph handed over in pieces?); the data is replaced by NaN. GGML_MI355X_FUSE=0 stores every result\n", what, tensor->name, name);
    return true;
}

static void buffer_get_tensor(ggml_backend_buffer_t buffer, const struct ggml_tensor * tensor, void * data, size_t offset, size_t size) {
    mi355x_buffer_ctx * ctx = (mi355x_buffer_ctx *) buffer->context;
    if (refuse_stale_read(ctx, tensor, offset, size, "a download")) { memset(data, 0xff, size); return; }
    if (download_from_mirror(ctx->device, tensor, data, offset, size)) { count_download(ctx->device, tensor->data); return; }
    HIP_TRY(hipSetDevice(ctx->device), return);
    HIP_TRY(hipMemcpy(data, (const char *) tensor->data + offset, size, hipMemcpyDeviceToHost), return);
    // a result that the host reads back (whisper.cpp does not flag its logits as an output: they are the graph's last node,
    // src/whisper.cpp:2953): from the next graph on it is mirrored in pinned memory
    static const bool no_mirror = env_flag("GGML_MI355X_NO_MIRROR", false);
    if (!no_mirror && buffer->usage != GGML_BACKEND_BUFFER_USAGE_WEIGHTS && !tensor->view_src && ggml_is_contiguous(tensor) &&
        ggml_nbytes(tensor) <= MI355X_MIRROR_MAX) want_download(ctx->device, tensor->data, ggml_nbytes(tensor), offset, size);
    std::lock_guard<std::mutex> live(g_live_mutex);
    for (mi355x_backend_ctx * b : g_live) if (b->device == ctx->device) { b->counters[5] += 1; break; }
}

static bool buffer_is_mi355x(ggml_backend_buffer_t buffer) { return buffer && buffer->iface.get_base == buffer_get_base; }
bool mi355x_buffer_is_ours(ggml_backend_buffer_t buffer) { return buffer_is_mi355x(buffer); }

static bool buffer_cpy_tensor(ggml_backend_buffer_t buffer, const struct ggml_tensor * src, struct ggml_tensor * dst) {
    mi355x_buffer_ctx * ctx = (mi355x_buffer_ctx *) buffer->context;
    ggml_backend_buffer_t sbuf = src->view_src ? src->view_src->buffer : src->buffer;
    if (!ggml_is_contiguous(src) || !ggml_is_contiguous(dst) || ggml_nbytes(src) != ggml_nbytes(dst)) return false;
    HIP_TRY(hipSetDevice(ctx->device), return false);
    ctx->drop_images(dst->data, ggml_nbytes(dst));
    drop_mirrors(ctx->device, dst->data, ggml_nbytes(dst));
    ctx->unwritten.written(dst->data, ggml_nbytes(dst));
    if (buffer_is_mi355x(sbuf)) {
        if (refuse_stale_read((mi355x_buffer_ctx *) sbuf->context, src, 0, ggml_nbytes(src), "a copy")) {
            HIP_TRY(hipMemset(dst->data, 0xff, ggml_nbytes(dst)), return false);
            HIP_TRY(hipStreamSynchronize(nullptr), return false);
            return true;
        }
        const int sdev = ((mi355x_buffer_ctx *) sbuf->context)->device;
        if (sdev != ctx->device) {                          // uploads queued on the other device's null stream come first
            HIP_TRY(hipSetDevice(sdev), return false);
            HIP_TRY(hipStreamSynchronize(nullptr), return false);
            HIP_TRY(hipSetDevice(ctx->device), return false);
        }
        HIP_TRY(hipMemcpy(dst->data, src->data, ggml_nbytes(src), hipMemcpyDeviceToDevice), return false);
        HIP_TRY(hipStreamSynchronize(nullptr), return false);
        return true;
    }
    if (sbuf && ggml_backend_buffer_is_host(sbuf)) return upload(ctx->device, dst->data, src->data, ggml_nbytes(src));
    return false;
}

static void buffer_clear(ggml_backend_buffer_t buffer, uint8_t value) {
    mi355x_buffer_ctx * ctx = (mi355x_buffer_ctx *) buffer->context;
    HIP_TRY(hipSetDevice(ctx->device), return);
    ctx->drop_all_images();
    drop_mirrors(ctx->device, ctx->base, ctx->size);
    ctx->unwritten.clear();
    HIP_TRY(hipMemset(ctx->base, value, ctx->size), return);
    HIP_TRY(hipDeviceSynchronize(), return);
}

static const struct ggml_backend_buffer_i mi355x_buffer_iface = {
    /* .free_buffer   = */ buffer_free,
    /* .get_base      = */ buffer_get_base,
    /* .init_tensor   = */ buffer_init_tensor,
    /* .memset_tensor = */ buffer_memset_tensor,
    /* .set_tensor    = */ buffer_set_tensor,
    /* .get_tensor    = */ buffer_get_tensor,
    /* .cpy_tensor    = */ buffer_cpy_tensor,
    /* .clear         = */ buffer_clear,
    /* .reset         = */ NULL,
};

// ------------------------------------------------------------------------------------------------------
// buffer type  (ggml_backend_buffer_type_i, ggml-backend-impl.h:17-29)
// ------------------------------------------------------------------------------------------------------

static const char * buft_get_name(ggml_backend_buffer_type_t buft) {
    return ((mi355x_device_ctx *) buft->device->context)->name.c_str();
}

static ggml_backend_buffer_t buft_alloc_buffer(ggml_backend_buffer_type_t buft, size_t size) {
    mi355x_device_ctx * dev = (mi355x_device_ctx *) buft->device->context;
    HIP_TRY(hipSetDevice(dev->device), return NULL);
    void * base = nullptr;
    const size_t alloc = size ? size : 1;
    hipError_t err = hipMalloc(&base, alloc);
    if (err != hipSuccess || !base) {
        (void) hipGetLastError();
        GGML_LOG_ERROR("ggml-mi355x: allocating %.2f MiB on device %d failed: %s\n", alloc / 1048576.0, dev->device, hipGetErrorString(err));
        return NULL;
    }
    mi355x_buffer_ctx * ctx = new mi355x_buffer_ctx;
    ctx->device = dev->device; ctx->base = base; ctx->size = size;
    return ggml_backend_buffer_init(buft, mi355x_buffer_iface, ctx, size);
}

static size_t buft_get_alignment(ggml_backend_buffer_type_t) { return MI355X_BUFFER_ALIGN; }

static size_t buft_get_max_size(ggml_backend_buffer_type_t buft) {
    mi355x_device_ctx * dev = (mi355x_device_ctx *) buft->device->context;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev->device) != hipSuccess) { (void) hipGetLastError(); return SIZE_MAX; }
    return prop.totalGlobalMem;
}

// No kernel reads past the last block of a row or the last row of a tensor, so tensors need no padding.
static size_t buft_get_alloc_size(ggml_backend_buffer_type_t, const struct ggml_tensor * tensor) {
    return ggml_nbytes(tensor);
}

static bool buft_is_host(ggml_backend_buffer_type_t) { return false; }

static const struct ggml_backend_buffer_type_i mi355x_buft_iface = {
    /* .get_name       = */ buft_get_name,
    /* .alloc_buffer   = */ buft_alloc_buffer,
    /* .get_alignment  = */ buft_get_alignment,
    /* .get_max_size   = */ buft_get_max_size,
    /* .get_alloc_size = */ buft_get_alloc_size,
    /* .is_host        = */ buft_is_host,
};

// ------------------------------------------------------------------------------------------------------
// host buffer type  (ggml_backend_device_i::get_host_buffer_type, ggml-backend-impl.h:160): host memory that the device
// reads and writes at full PCIe speed — pinned with hipHostMalloc — behind ggml's own host-buffer interface, so that every
// CPU-side user (ggml_backend_tensor_set / _get are memcpy, the CPU backend computes on it) sees an ordinary host buffer.
// A host that stages its graph inputs or results there spares the runtime its own staging copy on every transfer.
// ------------------------------------------------------------------------------------------------------

static const char * host_buft_get_name(ggml_backend_buffer_type_t) { return GGML_MI355X_NAME "_Host"; }

static void host_buffer_free(ggml_backend_buffer_t buffer) {
    if (hipHostFree(buffer->context) != hipSuccess) (void) hipGetLastError();
}

static ggml_backend_buffer_t host_buft_alloc_buffer(ggml_backend_buffer_type_t buft, size_t size) {
    void * p = nullptr;
    if (hipHostMalloc(&p, size ? size : 1, hipHostMallocDefault) != hipSuccess || !p) {
        (void) hipGetLastError();
        GGML_LOG_WARN("ggml-mi355x: could not pin %.2f MiB of host memory; the buffer is ordinary host memory\n", size / 1048576.0);
        return ggml_backend_buft_alloc_buffer(ggml_backend_cpu_buffer_type(), size);
    }
    ggml_backend_buffer_t buffer = ggml_backend_cpu_buffer_from_ptr(p, size);     // host-buffer vtable over memory of ours
    buffer->buft = buft;
    buffer->iface.free_buffer = host_buffer_free;                                 // its context is the pointer
    return buffer;
}

static size_t host_buft_get_alignment(ggml_backend_buffer_type_t) { return ggml_backend_buft_get_alignment(ggml_backend_cpu_buffer_type()); }
static bool   host_buft_is_host(ggml_backend_buffer_type_t) { return true; }

static const struct ggml_backend_buffer_type_i mi355x_host_buft_iface = {
    /* .get_name       = */ host_buft_get_name,
    /* .alloc_buffer   = */ host_buft_alloc_buffer,
    /* .get_alignment  = */ host_buft_get_alignment,
    /* .get_max_size   = */ NULL,
    /* .get_alloc_size = */ NULL,
    /* .is_host        = */ host_buft_is_host,
};

// ------------------------------------------------------------------------------------------------------
// backend / stream  (ggml_backend_i, ggml-backend-impl.h:87-117)
// ------------------------------------------------------------------------------------------------------


static ggml_guid_t backend_guid() {
    static ggml_guid guid = { 0x4d, 0x49, 0x33, 0x35, 0x35, 0x58, 0x2d, 0x67, 0x66, 0x78, 0x39, 0x35, 0x30, 0x2d, 0x76, 0x31 };
    return &guid;
}

static const char * backend_get_name(ggml_backend_t backend) {
    return ((mi355x_backend_ctx *) backend->context)->name.c_str();
}

static void backend_synchronize(ggml_backend_t backend) {
    mi355x_backend_ctx * ctx = (mi355x_backend_ctx *) backend->context;
    const auto t0 = std::chrono::steady_clock::now();
    HIP_TRY(hipSetDevice(ctx->device), return);
    HIP_TRY(hipStreamSynchronize(ctx->stream), return);
    ctx->counters[7] += std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - t0).count();
    if (!ctx->pending.empty()) ctx->drain_events();
}

static void backend_free(ggml_backend_t backend) {
    mi355x_backend_ctx * ctx = (mi355x_backend_ctx *) backend->context;
    backend_synchronize(backend);
    {
        std::lock_guard<std::mutex> lock(g_live_mutex);
        g_live.erase(std::remove(g_live.begin(), g_live.end(), ctx), g_live.end());
        for (auto & kv : ctx->stats) {
            auto & s = g_retired_stats[kv.first];
            s.calls += kv.second.calls; s.ms += kv.second.ms; s.bytes += kv.second.bytes; s.flops += kv.second.flops;
        }
        for (int i = 0; i < MI355X_N_COUNTERS; ++i) {
            if (i == 9) g_retired_counters[i] = std::max(g_retired_counters[i], ctx->counters[i]); else g_retired_counters[i] += ctx->counters[i];
        }
    }
    for (hipEvent_t e : ctx->event_pool) (void) hipEventDestroy(e);
    if (ctx->ws_base) (void) hipFree(ctx->ws_base);
    if (ctx->mirror_host) (void) hipHostFree(ctx->mirror_host);
    if (ctx->mirror_done) (void) hipEventDestroy(ctx->mirror_done);
    if (ctx->stream) (void) hipStreamDestroy(ctx->stream);
    delete ctx;
    delete backend;
}

static void backend_set_tensor_async(ggml_backend_t backend, struct ggml_tensor * tensor, const void * data, size_t offset, size_t size) {
    mi355x_backend_ctx * ctx = (mi355x_backend_ctx *) backend->context;
    HIP_TRY(hipSetDevice(ctx->device), return);
    ggml_backend_buffer_t buf = tensor->view_src ? tensor->view_src->buffer : tensor->buffer;
    if (buffer_is_mi355x(buf)) {
        mi355x_buffer_ctx * bctx = (mi355x_buffer_ctx *) buf->context;
        bctx->drop_images((char *) tensor->data + offset, size);
        bctx->unwritten.written((char *) tensor->data + offset, size);
    }
    drop_mirrors(ctx->device, (char *) tensor->data + offset, size);          // (of every instance on the device, like the buffer-level writers)
    HIP_TRY(hipMemcpyAsync((char *) tensor->data + offset, data, size, hipMemcpyHostToDevice, ctx->stream), return);
}

static void backend_get_tensor_async(ggml_backend_t backend, const struct ggml_tensor * tensor, void * data, size_t offset, size_t size) {
    mi355x_backend_ctx * ctx = (mi355x_backend_ctx *) backend->context;
    HIP_TRY(hipSetDevice(ctx->device), return);
    ggml_backend_buffer_t buf = tensor->view_src ? tensor->view_src->buffer : tensor->buffer;
    if (buffer_is_mi355x(buf) && refuse_stale_read((mi355x_buffer_ctx *) buf->context, tensor, offset, size, "a download")) { memset(data, 0xff, size); return; }
    HIP_TRY(hipMemcpyAsync(data, (const char *) tensor->data + offset, size, hipMemcpyDeviceToHost, ctx->stream), return);
}

static enum ggml_status backend_graph_compute(ggml_backend_t backend, struct ggml_cgraph * cgraph) {
    return mi355x_graph_compute((mi355x_backend_ctx *) backend->context, cgraph);
}

static const struct ggml_backend_i mi355x_backend_iface = {
    /* .get_name           = */ backend_get_name,
    /* .free               = */ backend_free,
    /* .set_tensor_async   = */ backend_set_tensor_async,
    /* .get_tensor_async   = */ backend_get_tensor_async,
    /* .cpy_tensor_async   = */ NULL,
    /* .synchronize        = */ backend_synchronize,
    /* .graph_plan_create  = */ NULL,
    /* .graph_plan_free    = */ NULL,
    /* .graph_plan_update  = */ NULL,
    /* .graph_plan_compute = */ NULL,
    /* .graph_compute      = */ backend_graph_compute,
    /* .event_record       = */ NULL,
    /* .event_wait         = */ NULL,
};

// ------------------------------------------------------------------------------------------------------
// device  (ggml_backend_device_i, ggml-backend-impl.h:137-179)
// ------------------------------------------------------------------------------------------------------

static const char * device_get_name(ggml_backend_dev_t dev)        { return ((mi355x_device_ctx *) dev->context)->name.c_str(); }
static const char * device_get_description(ggml_backend_dev_t dev) { return ((mi355x_device_ctx *) dev->context)->description.c_str(); }

static void device_get_memory(ggml_backend_dev_t dev, size_t * free, size_t * total) {
    mi355x_device_ctx * ctx = (mi355x_device_ctx *) dev->context;
    *free = 0; *total = 0;
    HIP_TRY(hipSetDevice(ctx->device), return);
    HIP_TRY(hipMemGetInfo(free, total), return);
}

static enum ggml_backend_dev_type device_get_type(ggml_backend_dev_t) { return GGML_BACKEND_DEVICE_TYPE_GPU; }

static void device_get_props(ggml_backend_dev_t dev, struct ggml_backend_dev_props * props) {
    props->name        = device_get_name(dev);
    props->description = device_get_description(dev);
    props->type        = device_get_type(dev);
    device_get_memory(dev, &props->memory_free, &props->memory_total);
    props->caps = { /* async */ false, /* host_buffer */ true, /* buffer_from_host_ptr */ false, /* events */ false };
}

static ggml_backend_t device_init_backend(ggml_backend_dev_t dev, const char *) {
    mi355x_device_ctx * dctx = (mi355x_device_ctx *) dev->context;
    HIP_TRY(hipSetDevice(dctx->device), return NULL);
    mi355x_backend_ctx * ctx = new mi355x_backend_ctx;
    ctx->device  = dctx->device;
    ctx->name    = dctx->name;
    ctx->fuse    = env_flag("GGML_MI355X_FUSE", true);
    ctx->profile = env_flag("GGML_MI355X_PROFILE", false);
    ctx->exact   = env_flag("GGML_MI355X_EXACT", false);
    if (const char * e = getenv("GGML_MI355X_FA_ACCUM")) { const int v = atoi(e); if (v >= 0 && v <= 3) ctx->fa_accum = v; }
    if (const char * e = getenv("GGML_MI355X_FA_CHAIN")) { const int v = atoi(e); if (v >= 0 && v <= 2) ctx->fa_chain = v; }
    ctx->weight_images = env_flag("GGML_MI355X_WEIGHT_IMAGES", true);
    ctx->dead_f32 = env_flag("GGML_MI355X_DEAD_F32", true);
    ctx->check_reads = env_flag("GGML_MI355X_CHECK_READS", true);
    ctx->debug   = env_flag("GGML_MI355X_DEBUG", false);
    // default priority, blocking with respect to the null stream used by the buffer-level copies
    HIP_TRY(hipStreamCreate(&ctx->stream), { delete ctx; return NULL; });
    ggml_backend_t backend = new ggml_backend{
        /* .guid    = */ backend_guid(),
        /* .iface   = */ mi355x_backend_iface,
        /* .device  = */ dev,
        /* .context = */ ctx,
    };
    {
        std::lock_guard<std::mutex> lock(g_live_mutex);
        g_live.push_back(ctx);
    }
    return backend;
}

static ggml_backend_buffer_type_t device_get_buffer_type(ggml_backend_dev_t dev);
static ggml_backend_buffer_type_t device_get_host_buffer_type(ggml_backend_dev_t dev);

static bool device_supports_op(ggml_backend_dev_t, const struct ggml_tensor * op) { return mi355x_supports_op(op); }

static bool device_supports_buft(ggml_backend_dev_t dev, ggml_backend_buffer_type_t buft) {
    return buft->iface.get_name == buft_get_name && buft->device == dev;
}

static bool device_offload_op(ggml_backend_dev_t, const struct ggml_tensor *) { return false; }

static const struct ggml_backend_device_i mi355x_device_iface = {
    /* .get_name             = */ device_get_name,
    /* .get_description      = */ device_get_description,
    /* .get_memory           = */ device_get_memory,
    /* .get_type             = */ device_get_type,
    /* .get_props            = */ device_get_props,
    /* .init_backend         = */ device_init_backend,
    /* .get_buffer_type      = */ device_get_buffer_type,
    /* .get_host_buffer_type = */ device_get_host_buffer_type,
    /* .buffer_from_host_ptr = */ NULL,
    /* .supports_op          = */ device_supports_op,
    /* .supports_buft        = */ device_supports_buft,
    /* .offload_op           = */ device_offload_op,
    /* .event_new            = */ NULL,
    /* .event_free           = */ NULL,
    /* .event_synchronize    = */ NULL,
};

// ------------------------------------------------------------------------------------------------------
// reg  (ggml_backend_reg_i, ggml-backend-impl.h:191-207)
// ------------------------------------------------------------------------------------------------------

struct mi355x_reg_ctx {
    std::vector<ggml_backend_device>      devices;
    std::vector<ggml_backend_buffer_type> bufts;
    std::vector<ggml_backend_buffer_type> host_bufts;
};

static const char * reg_get_name(ggml_backend_reg_t) { return GGML_MI355X_NAME; }

static size_t reg_get_device_count(ggml_backend_reg_t reg) { return ((mi355x_reg_ctx *) reg->context)->devices.size(); }

static ggml_backend_dev_t reg_get_device(ggml_backend_reg_t reg, size_t index) {
    mi355x_reg_ctx * ctx = (mi355x_reg_ctx *) reg->context;
    return index < ctx->devices.size() ? &ctx->devices[index] : NULL;
}

static struct ggml_backend_feature * get_features(ggml_backend_reg_t) {
    static struct ggml_backend_feature features[] = {
        { "GFX950",   "1" },
        { "MFMA_F16", "1" },
        { "DOT4_I8",  "1" },
        { NULL, NULL },
    };
    return features;
}

static void ctx_synchronize(mi355x_backend_ctx * ctx) {
    if (hipSetDevice(ctx->device) != hipSuccess || hipStreamSynchronize(ctx->stream) != hipSuccess) { (void) hipGetLastError(); return; }
    if (!ctx->pending.empty()) ctx->drain_events();
}

// backend == NULL addresses every live MI355X backend of the process
static int set_option(ggml_backend_t backend, const char * name, int value) {
    if (!name || (backend && !ggml_backend_is_mi355x(backend))) return -1;
    const bool is_fuse = strcmp(name, "fuse") == 0, is_profile = strcmp(name, "profile") == 0, is_exact = strcmp(name, "exact") == 0;
    const bool is_accum = strcmp(name, "fa_accum") == 0, is_chain = strcmp(name, "fa_chain") == 0;
    if (!is_fuse && !is_profile && !is_exact && !is_accum && !is_chain) return -1;
    if (is_accum && (value < 0 || value > 3)) return -1;
    if (is_chain && (value < 0 || value > 2)) return -1;
    std::lock_guard<std::mutex> lock(g_live_mutex);
    for (mi355x_backend_ctx * ctx : g_live) {
        if (backend && ctx != (mi355x_backend_ctx *) backend->context) continue;
        if (is_fuse) ctx->fuse = value != 0;
        else if (is_exact) ctx->exact = value != 0;
        else if (is_accum) ctx->fa_accum = value;
        else if (is_chain) ctx->fa_chain = value;
        else { ctx_synchronize(ctx); ctx->profile = value != 0; }
    }
    return 0;
}

static size_t get_stats(ggml_backend_t backend, char * buf, size_t size, int reset) {
    if (backend && !ggml_backend_is_mi355x(backend)) return 0;
    std::map<std::string, mi355x_kernel_stat> total;
    {
        std::lock_guard<std::mutex> lock(g_live_mutex);
        auto add = [&](const std::map<std::string, mi355x_kernel_stat> & m) {
            for (auto & kv : m) {
                auto & s = total[kv.first];
                s.calls += kv.second.calls; s.ms += kv.second.ms; s.bytes += kv.second.bytes; s.flops += kv.second.flops;
            }
        };
        for (mi355x_backend_ctx * ctx : g_live) {
            if (backend && ctx != (mi355x_backend_ctx *) backend->context) continue;
            ctx_synchronize(ctx);
            add(ctx->stats);
            if (reset) ctx->stats.clear();
        }
        if (!backend) { add(g_retired_stats); if (reset) g_retired_stats.clear(); }
    }
    std::string s = "[";
    bool first = true;
    for (auto & kv : total) {
        char line[512];
        snprintf(line, sizeof(line), "%s{\"kernel\": \"%s\", \"calls\": %lld, \"ms\": %.6f, \"bytes\": %.0f, \"flops\": %.0f}",
                 first ? "" : ", ", kv.first.c_str(), (long long) kv.second.calls, kv.second.ms, kv.second.bytes, kv.second.flops);
        s += line; first = false;
    }
    s += "]";
    if (buf && size) { const size_t n = s.size() < size - 1 ? s.size() : size - 1; memcpy(buf, s.data(), n); buf[n] = 0; }
    return s.size() + 1;
}

// graph_compute calls, graph nodes received, nodes that are not views or empty, kernel launches, downloads served from the
// host mirror, downloads by hipMemcpy — since the last reset
static void get_counters(ggml_backend_t backend, int64_t out[MI355X_N_COUNTERS], int reset) {
    for (int i = 0; i < MI355X_N_COUNTERS; ++i) out[i] = 0;
    if (backend && !ggml_backend_is_mi355x(backend)) return;
    std::lock_guard<std::mutex> lock(g_live_mutex);
    for (mi355x_backend_ctx * ctx : g_live) {
        if (backend && ctx != (mi355x_backend_ctx *) backend->context) continue;
        for (int i = 0; i < MI355X_N_COUNTERS; ++i) {
            if (i == 9) out[i] = std::max(out[i], ctx->counters[i]); else out[i] += ctx->counters[i];      // (9 is a maximum)
            if (reset) ctx->counters[i] = 0;
        }
    }
    if (!backend) for (int i = 0; i < MI355X_N_COUNTERS; ++i) {
        if (i == 9) out[i] = std::max(out[i], g_retired_counters[i]); else out[i] += g_retired_counters[i];
        if (reset) g_retired_counters[i] = 0;
    }
}

// host-memory front of mi355x_log_mel_spectrogram: one allocation for samples, filter bank, result and workspace, the
// null stream, blocking copies.  Called once per audio file, next to milliseconds of host work it replaces.
static int64_t log_mel(int device, const float * samples, int64_t n_samples, const float * filters, int n_mel, float * mel, int64_t mel_capacity, float * device_ms) {
    const int64_t n_len = mi355x_log_mel_n_len(n_samples);
    const size_t ws_bytes = mi355x_log_mel_workspace_size(n_mel);
    if (!samples || !filters || n_len <= 0) return MI355X_ERR_INVALID;
    if (!ws_bytes) return MI355X_ERR_UNSUPPORTED;
    if (!mel) return n_len;
    if (mel_capacity < n_len * n_mel) return MI355X_ERR_INVALID;
    HIP_TRY(hipSetDevice(device), return MI355X_ERR_HIP);
    auto pad = [](size_t b) { return (b + 255) / 256 * 256; };
    const size_t b_s = pad((size_t) n_samples * 4), b_f = pad((size_t) n_mel * 201 * 4), b_m = pad((size_t) n_len * n_mel * 4);
    char * base = nullptr;
    HIP_TRY(hipMalloc((void **) &base, b_s + b_f + b_m + ws_bytes), return MI355X_ERR_HIP);
    int64_t rc = MI355X_ERR_HIP;
    if (hipMemcpy(base, samples, (size_t) n_samples * 4, hipMemcpyHostToDevice) == hipSuccess &&
        hipMemcpy(base + b_s, filters, (size_t) n_mel * 201 * 4, hipMemcpyHostToDevice) == hipSuccess) {
        hipEvent_t e0 = nullptr, e1 = nullptr;
        if (device_ms && (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)) { (void) hipGetLastError(); device_ms = nullptr; }
        if (device_ms) (void) hipEventRecord(e0, nullptr);
        rc = mi355x_log_mel_spectrogram((const float *) base, n_samples, (const float *)(base + b_s), n_mel, (float *)(base + b_s + b_f),
                                        base + b_s + b_f + b_m, ws_bytes, nullptr);
        if (device_ms) {
            (void) hipEventRecord(e1, nullptr);
            if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(device_ms, e0, e1) != hipSuccess) { (void) hipGetLastError(); *device_ms = -1.0f; }
        }
        if (e0) (void) hipEventDestroy(e0);
        if (e1) (void) hipEventDestroy(e1);
        if (rc == MI355X_OK) rc = hipMemcpy(mel, base + b_s + b_f, (size_t) n_len * n_mel * 4, hipMemcpyDeviceToHost) == hipSuccess ? n_len : (int64_t) MI355X_ERR_HIP;
    }
    if (rc == MI355X_ERR_HIP) (void) hipGetLastError();
    (void) hipFree(base);
    return rc;
}

static void * reg_get_proc_address(ggml_backend_reg_t, const char * name) {
    if (!name) return NULL;
    if (strcmp(name, "ggml_backend_get_features") == 0)      return (void *) get_features;
    if (strcmp(name, "ggml_backend_mi355x_set_option") == 0) return (void *) set_option;
    if (strcmp(name, "ggml_backend_mi355x_get_stats") == 0)  return (void *) get_stats;
    if (strcmp(name, "ggml_backend_mi355x_get_counters") == 0) return (void *) get_counters;
    if (strcmp(name, "ggml_backend_mi355x_log_mel") == 0)    return (void *) log_mel;
    return NULL;
}

static const struct ggml_backend_reg_i mi355x_reg_iface = {
    /* .get_name         = */ reg_get_name,
    /* .get_device_count = */ reg_get_device_count,
    /* .get_device       = */ reg_get_device,
    /* .get_proc_address = */ reg_get_proc_address,
};

static ggml_backend_buffer_type_t device_get_buffer_type(ggml_backend_dev_t dev) {
    mi355x_reg_ctx * rctx = (mi355x_reg_ctx *) dev->reg->context;
    for (size_t i = 0; i < rctx->devices.size(); ++i) if (&rctx->devices[i] == dev) return &rctx->bufts[i];
    return NULL;
}

static ggml_backend_buffer_type_t device_get_host_buffer_type(ggml_backend_dev_t dev) {
    mi355x_reg_ctx * rctx = (mi355x_reg_ctx *) dev->reg->context;
    for (size_t i = 0; i < rctx->devices.size(); ++i) if (&rctx->devices[i] == dev) return &rctx->host_bufts[i];
    return NULL;
}

// ------------------------------------------------------------------------------------------------------
// public entry points
// ------------------------------------------------------------------------------------------------------

extern "C" {

ggml_backend_reg_t ggml_backend_mi355x_reg(void) {
    static struct ggml_backend_reg reg;
    static std::once_flag once;
    std::call_once(once, [] {
        mi355x_reg_ctx * ctx = new mi355x_reg_ctx;   // lives as long as the process, like the registry itself
        const std::vector<int> & devs = gfx950_devices();
        ctx->devices.reserve(devs.size());
        ctx->bufts.reserve(devs.size());
        ctx->host_bufts.reserve(devs.size());
        reg = { GGML_BACKEND_API_VERSION, mi355x_reg_iface, ctx };
        for (size_t i = 0; i < devs.size(); ++i) {
            mi355x_device_ctx * d = new mi355x_device_ctx;
            d->device = devs[i];
            d->name   = std::string(GGML_MI355X_NAME) + std::to_string(i);
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, devs[i]) == hipSuccess) d->description = std::string(prop.name) + " (" + prop.gcnArchName + ")";
            else { (void) hipGetLastError(); d->description = "AMD Instinct MI355X"; }
            ctx->devices.push_back({ mi355x_device_iface, &reg, d });
            ctx->bufts.push_back({ mi355x_buft_iface, &ctx->devices.back(), NULL });
            ctx->host_bufts.push_back({ mi355x_host_buft_iface, &ctx->devices.back(), NULL });
        }
    });
    return &reg;
}

int ggml_backend_mi355x_get_device_count(void) { return (int) gfx950_devices().size(); }

ggml_backend_t ggml_backend_mi355x_init(int device) {
    ggml_backend_reg_t reg = ggml_backend_mi355x_reg();
    ggml_backend_dev_t dev = reg_get_device(reg, (size_t) device);
    return dev ? device_init_backend(dev, NULL) : NULL;
}

bool ggml_backend_is_mi355x(ggml_backend_t backend) {
    return backend != NULL && backend->iface.graph_compute == backend_graph_compute;
}

ggml_backend_buffer_type_t ggml_backend_mi355x_buffer_type(int device) {
    ggml_backend_reg_t reg = ggml_backend_mi355x_reg();
    ggml_backend_dev_t dev = reg_get_device(reg, (size_t) device);
    return dev ? device_get_buffer_type(dev) : NULL;
}

// ggml_backend_registry::load_backend (ggml/src/ggml-backend-reg.cpp:227-271) rejects a library whose score is 0
int ggml_backend_score(void) { return gfx950_devices().empty() ? 0 : 100; }

ggml_backend_reg_t ggml_backend_init(void) { return ggml_backend_mi355x_reg(); }

} // extern "C"
