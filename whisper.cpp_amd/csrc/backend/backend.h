// Internal declarations shared by the ggml-mi355x backend sources.
#pragma once

#include <hip/hip_runtime.h>

#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "ggml.h"
#include "ggml-backend.h"
#include "ggml-backend-impl.h"
#include "ggml-impl.h"

#include "ggml-mi355x.h"
#include "mi355x_kernels.h"
#include "range_set.h"

#define MI355X_BUFFER_ALIGN 256
#define MI355X_N_COUNTERS   10
#define MI355X_MIRROR_MAX   (4u << 20)       // outputs larger than this are never mirrored (an encoder's states stay on the device)

#define HIP_TRY(expr, on_fail)                                                                            \
    do {                                                                                                  \
        hipError_t err_ = (expr);                                                                         \
        if (err_ != hipSuccess) {                                                                         \
            GGML_LOG_ERROR("ggml-mi355x: %s failed: %s (%s:%d)\n", #expr, hipGetErrorString(err_), __FILE__, __LINE__); \
            (void) hipGetLastError();                                                                     \
            on_fail;                                                                                      \
        }                                                                                                 \
    } while (0)

struct mi355x_device_ctx {
    int         device;        // HIP ordinal
    std::string name;          // "MI355X0"
    std::string description;   // marketing name from the driver
};

// A second form of a quantized weight tensor, kept beside it in HBM:
//   MI355X_IMAGE_F16     rows of f16(d * q), operand of the MFMA GEMM
//   MI355X_IMAGE_TILES   Q8_0 blocks in the order of mi355x_q8_0_tiles_pack, operand of the few-column product over a
//                        matrix long enough to be a stream (the vocabulary projection)
enum { MI355X_IMAGE_F16 = 0, MI355X_IMAGE_TILES = 1 };
struct mi355x_weight_image {
    void * f16;        // device memory (F16: ne0 * ne1 halves)
    size_t src_bytes;  // bytes of the tensor it mirrors
    int    type;
    int64_t ne0, ne1;
};

struct mi355x_buffer_ctx {
    int    device;
    void * base;
    size_t size;
    // Weight buffers keep, next to a Q5_0 / Q8_0 matrix that is multiplied with many columns at once, its f16 image:
    // 2 bytes per weight more HBM, so that the GEMM streams matrix-core operands instead of unpacking the same blocks
    // in every workgroup and on every call.  Keyed by the tensor's data address; anything that writes into the buffer
    // drops the images it overlaps.  (Key: the address with the kind of image in its lowest bit — block rows start at
    // even addresses.)
    std::mutex                               image_mutex;
    std::map<uintptr_t, mi355x_weight_image> images;

    // Results of graph nodes in this buffer that no launch stored (folded into their consumer, or kept only as the next
    // product's activation image): a later read of such memory is refused, see range_set.h.
    mi355x_range_set unwritten;

    const void * weight_image(const struct ggml_tensor * w, hipStream_t stream, int kind = MI355X_IMAGE_F16);   // NULL: none could be made
    void         drop_images(const void * begin, size_t size);
    void         drop_all_images();
};

bool mi355x_buffer_is_ours(ggml_backend_buffer_t buffer);

struct mi355x_kernel_stat {
    int64_t calls = 0;
    double  ms    = 0.0;
    double  bytes = 0.0;
    double  flops = 0.0;
};

struct mi355x_pending_event {
    hipEvent_t  start, stop;
    const char *name;
    double      bytes, flops;
};

struct mi355x_backend_ctx {
    int         device;
    std::string name;
    hipStream_t stream = nullptr;
    bool        fuse    = true;
    bool        profile = false;
    bool        debug   = false;   // log what every MUL_MAT launch folds in (GGML_MI355X_DEBUG=1)
    int         fa_accum = 0;           // V accumulation of attention: 0 the reference's sequence (f32 fma, f16 store, key by key);
                                        // bit 0: f32 accumulators (matrix cores) for more than 8 queries, bit 1: f32
                                        // accumulators for a decode step's few queries
    int         fa_chain = 2;           // the f16 key-by-key step: 2 one fused f16 multiply-add on the factor rounded to f16 (the reference's
                                        // builds with f16 vector units) in every launch, 1 only where a launch has more than 8 queries,
                                        // 0 f32 fma then f16 store (its x86 build) everywhere
    bool        dead_f32 = true;        // a result whose only reader is the next launch's activation image is not also written as f32
                                        // (GGML_MI355X_DEAD_F32=0: always write it)
    bool        check_reads = true;     // refuse to read memory whose value a launch folded away (GGML_MI355X_CHECK_READS=0 turns the
                                        // bookkeeping off)
    bool        pieces = false;         // a graph turned out to arrive in pieces (a later piece read a result that an earlier one had
                                        // folded away): from then on every result is stored, whatever the visible readers say
    bool        weight_images = true;   // keep f16 images of quantized GEMM weights (GGML_MI355X_WEIGHT_IMAGES=0 turns it off)
    bool        exact   = false;   // true: f32 attention accumulators and un-rounded GEMM activations instead of the
                                   // reference's f16-sequential / Q8_0-rounded arithmetic

    // scratch for the kernels (grow-only), and which activations its Q8_0-rounded copy currently mirrors
    void *       ws_base  = nullptr;   // the allocation: two slots of ws_size bytes
    void *       ws       = nullptr;   // the current slot (where the cached activation image lives)
    size_t       ws_size  = 0;         // bytes per slot
    int          ws_slot  = 0;
    const void * image_only = nullptr; // the tensor (of this graph) whose producer wrote its image into the workspace and nothing else
    const void * ws_x     = nullptr;
    int          ws_x_mode = 0;
    int64_t      ws_x_ne[4] = {0, 0, 0, 0};
    size_t       ws_x_nb[4] = {0, 0, 0, 0};
    bool         reserve_workspace(size_t size);

    // what graph_compute was handed and did, always counted: calls, nodes of the graphs as received, nodes that are not
    // views or empty (each of them is carried out by some launch), kernel launches
    int64_t      counters[MI355X_N_COUNTERS] = {};

    // Host mirror of graph outputs (the logits of a decode step): tensors flagged GGML_TENSOR_FLAG_OUTPUT that the host has
    // downloaded before are copied into pinned memory at the end of graph_compute, on the stream, in one transfer each;
    // get_tensor then serves any slice of them from there until something writes the tensor or the next graph runs.
    struct mirror_entry { const char * dev; size_t lo, size, off; };    // bytes [lo, lo + size) of the tensor at `dev`, at `off` in the block
    std::mutex                mirror_mutex;
    char *                    mirror_host = nullptr;      // pinned
    size_t                    mirror_cap  = 0;
    std::vector<mirror_entry> mirror;                     // what the pinned block holds of the last graph's outputs
    hipEvent_t                mirror_done = nullptr;      // recorded behind the transfers
    void mirror_outputs(struct ggml_cgraph * cgraph);     // end of graph_compute
    void mirror_drop(const void * begin, size_t size);    // a write into [begin, begin + size)

    // profiling
    std::vector<mi355x_pending_event>         pending;
    std::vector<hipEvent_t>                   event_pool;
    std::map<std::string, mi355x_kernel_stat> stats;

    hipEvent_t take_event();
    void       drain_events();           // call after the stream has been synchronized
};

// ggml-mi355x.cpp: has the host downloaded the tensor at this address before (so that mirroring it pays)?
bool mi355x_download_is_wanted(int device, const void * data, size_t size, size_t * lo, size_t * hi);

// graph.cpp
enum ggml_status mi355x_graph_compute(mi355x_backend_ctx * ctx, struct ggml_cgraph * cgraph);
bool             mi355x_supports_op(const struct ggml_tensor * op);
