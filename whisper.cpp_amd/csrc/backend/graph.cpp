// graph_compute for the MI355X backend: walks the nodes of a ggml graph in order on one HIP stream and
// launches the hand-written kernels through their C ABI.  Takes the place of
// ggml_backend_cpu_graph_compute -> ggml_graph_compute -> ggml_compute_forward
// (ggml/src/ggml-cpu/ggml-cpu.cpp:149-169, ggml/src/ggml-cpu/ggml-cpu.c:3111, 1722).
//
// Neighbouring nodes that whisper always emits together are folded into one launch when the
// intermediate result has no other reader in the graph:
//     NORM -> MUL(w) -> ADD(b)                                    (src/whisper.cpp:2116-2121)
//     MUL_MAT [-> ADD(bias)] [-> GELU | -> SCALE | -> ADD(resid)]  (src/whisper.cpp:2126-2249)
//     MUL_MAT [-> ADD | -> SCALE] -> CPY(f32 -> f16, dense)        (src/whisper.cpp:2316-2351, 2564-2601)
#include "backend.h"

#include <stdlib.h>
#include <string.h>
#include <algorithm>
#include <string>
#include <chrono>
#include <unordered_map>

static mi355x_tensor to_view(const ggml_tensor * t) {
    mi355x_tensor v;
    v.data = t->data;
    v.type = (int32_t) t->type;   // numeric values are shared with enum mi355x_type
    v._pad = 0;
    for (int i = 0; i < 4; ++i) { v.ne[i] = t->ne[i]; v.nb[i] = t->nb[i]; }
    return v;
}

static bool type_in(enum ggml_type t, std::initializer_list<enum ggml_type> set) {
    for (auto s : set) if (s == t) return true;
    return false;
}

static bool is_view_op(enum ggml_op op) {
    return op == GGML_OP_NONE || op == GGML_OP_RESHAPE || op == GGML_OP_VIEW || op == GGML_OP_PERMUTE || op == GGML_OP_TRANSPOSE;
}

// ------------------------------------------------------------------------------------------------------
// supports_op: true only for (op, types, layout) tuples that have a kernel; everything else is left to the
// scheduler's CPU fallback (ggml/src/ggml-backend.cpp:1013-1034).
// ------------------------------------------------------------------------------------------------------

// GGML_MI355X_DECLINE=GELU,SCALE: ops (ggml_op_name, or ggml_unary_op_name for unary ops) that supports_op turns down although
// a kernel exists.  The scheduler then places them on the CPU backend and every graph reaches this backend as several
// ggml_graph_view pieces with copies in between (ggml/src/ggml-backend.cpp:1013-1034, 1196-1215) — the way to exercise that
// contract with whisper's own graphs.
static bool declined(const struct ggml_tensor * op) {
    static const std::string list = [] { const char * e = getenv("GGML_MI355X_DECLINE"); return std::string(e ? e : ""); }();
    if (list.empty() || is_view_op(op->op)) return false;
    const char * name = op->op == GGML_OP_UNARY ? ggml_unary_op_name(ggml_get_unary_op(op)) : ggml_op_name(op->op);
    const size_t len = strlen(name);
    for (size_t at = 0; at < list.size();) {
        size_t end = list.find(',', at);
        if (end == std::string::npos) end = list.size();
        if (end - at == len && list.compare(at, len, name) == 0) return true;
        at = end + 1;
    }
    return false;
}

bool mi355x_supports_op(const struct ggml_tensor * op) {
    const ggml_tensor * s0 = op->src[0];
    const ggml_tensor * s1 = op->src[1];
    if (declined(op)) return false;
    switch (op->op) {
        case GGML_OP_NONE: case GGML_OP_RESHAPE: case GGML_OP_VIEW: case GGML_OP_PERMUTE: case GGML_OP_TRANSPOSE:
            return true;
        case GGML_OP_MUL_MAT:
            if (!type_in(s0->type, {GGML_TYPE_Q5_0, GGML_TYPE_Q8_0, GGML_TYPE_F16, GGML_TYPE_F32})) return false;
            if (!(s1->type == GGML_TYPE_F32 || (s1->type == GGML_TYPE_F16 && s0->type == GGML_TYPE_F16))) return false;
            if (op->type != GGML_TYPE_F32) return false;
            return s0->nb[0] == ggml_type_size(s0->type) && s1->nb[0] == ggml_type_size(s1->type) && op->nb[0] == sizeof(float);
        case GGML_OP_ADD: case GGML_OP_MUL:
            return s0->type == GGML_TYPE_F32 && s1->type == GGML_TYPE_F32 && op->type == GGML_TYPE_F32;
        case GGML_OP_SCALE:
            return s0->type == GGML_TYPE_F32 && op->type == GGML_TYPE_F32;
        case GGML_OP_UNARY:
            return ggml_get_unary_op(op) == GGML_UNARY_OP_GELU && s0->type == GGML_TYPE_F32 && op->type == GGML_TYPE_F32;
        case GGML_OP_NORM:
            return s0->type == GGML_TYPE_F32 && op->type == GGML_TYPE_F32 && s0->nb[0] == sizeof(float) && op->nb[0] == sizeof(float);
        case GGML_OP_SOFT_MAX: {
            float max_bias; memcpy(&max_bias, (const float *) op->op_params + 1, sizeof(float));
            if (max_bias != 0.0f) return false;
            if (s1 && !type_in(s1->type, {GGML_TYPE_F32, GGML_TYPE_F16})) return false;
            return s0->type == GGML_TYPE_F32 && op->type == GGML_TYPE_F32 && s0->nb[0] == sizeof(float) && op->nb[0] == sizeof(float);
        }
        case GGML_OP_CPY: case GGML_OP_CONT: case GGML_OP_DUP: {
            const ggml_tensor * d = op->op == GGML_OP_CPY ? s1 : op;
            if (type_in(s0->type, {GGML_TYPE_F32, GGML_TYPE_F16}) && type_in(d->type, {GGML_TYPE_F32, GGML_TYPE_F16})) return true;
            return s0->type == d->type && ggml_is_contiguous(s0) && ggml_is_contiguous(d) &&
                   type_in(s0->type, {GGML_TYPE_I32, GGML_TYPE_Q5_0, GGML_TYPE_Q8_0});
        }
        case GGML_OP_GET_ROWS:
            return type_in(s0->type, {GGML_TYPE_Q5_0, GGML_TYPE_Q8_0, GGML_TYPE_F16, GGML_TYPE_F32}) &&
                   s1->type == GGML_TYPE_I32 && op->type == GGML_TYPE_F32 && s1->ne[0] * s1->ne[1] * s1->ne[2] <= 65535;
        case GGML_OP_IM2COL: {
            const int32_t is_2d = op->op_params[6];
            return is_2d == 0 && op->type == GGML_TYPE_F16 && s1->type == GGML_TYPE_F32 && s1->nb[0] == sizeof(float) && s1->ne[3] == 1;
        }
        case GGML_OP_FLASH_ATTN_EXT: {
            const ggml_tensor * k = op->src[1], * v = op->src[2], * m = op->src[3];
            float max_bias, softcap;
            memcpy(&max_bias, (const float *) op->op_params + 1, sizeof(float));
            memcpy(&softcap,  (const float *) op->op_params + 2, sizeof(float));
            if (max_bias != 0.0f || softcap != 0.0f) return false;
            if (s0->type != GGML_TYPE_F32 || k->type != GGML_TYPE_F16 || v->type != GGML_TYPE_F16) return false;
            if (m && m->type != GGML_TYPE_F16) return false;
            return s0->ne[0] == 64 && k->ne[0] == 64 && v->ne[0] == 64;
        }
        case GGML_OP_CONCAT:
            return s0->type == GGML_TYPE_F32 && s1->type == GGML_TYPE_F32 && op->type == GGML_TYPE_F32;
        default:
            return false;
    }
}

// ------------------------------------------------------------------------------------------------------
// profiling helpers
// ------------------------------------------------------------------------------------------------------

hipEvent_t mi355x_backend_ctx::take_event() {
    if (!event_pool.empty()) { hipEvent_t e = event_pool.back(); event_pool.pop_back(); return e; }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) { (void) hipGetLastError(); return nullptr; }
    return e;
}

void mi355x_backend_ctx::drain_events() {
    for (auto & p : pending) {
        float ms = 0.0f;
        if (p.start && p.stop && hipEventElapsedTime(&ms, p.start, p.stop) == hipSuccess) {
            auto & s = stats[p.name];
            s.calls += 1; s.ms += ms; s.bytes += p.bytes; s.flops += p.flops;
        } else {
            (void) hipGetLastError();
        }
        if (p.start) event_pool.push_back(p.start);
        if (p.stop)  event_pool.push_back(p.stop);
    }
    pending.clear();
}

// Two slots of `size` bytes each: a product reads its activation image from one while its epilogue may already write the
// next product's image into the other.
bool mi355x_backend_ctx::reserve_workspace(size_t size) {
    if (size <= ws_size) return true;
    // Grow: the slots keep their contents (an activation image that a producer left there may be the only copy of its values,
    // see image_only), so the old block is copied over before it goes.
    const size_t want = (size + size / 2 + 255) / 256 * 256;
    void * fresh = nullptr;
    if (hipMalloc(&fresh, 2 * want) != hipSuccess) { (void) hipGetLastError(); return false; }
    bool ok = true;
    if (ws_base) {
        ok = hipMemcpyAsync(fresh, ws_base, ws_size, hipMemcpyDeviceToDevice, stream) == hipSuccess &&
             hipMemcpyAsync((char *) fresh + want, (char *) ws_base + ws_size, ws_size, hipMemcpyDeviceToDevice, stream) == hipSuccess;
    }
    // the stream may still be reading the old block
    ok = hipStreamSynchronize(stream) == hipSuccess && ok;
    if (!ok) { (void) hipGetLastError(); (void) hipFree(fresh); return false; }
    if (ws_base) (void) hipFree(ws_base);
    ws_base = fresh;
    ws_size = want;
    ws = (char *) ws_base + (size_t) ws_slot * ws_size;
    return true;
}

// Queue the download of those results of this graph that the host is known to read (whisper_decode reads the logits row by row
// with blocking ggml_backend_tensor_get calls, src/whisper.cpp:2960-2966): one transfer per tensor into pinned memory,
// behind the graph on the same stream, so that it is over when the host's synchronize returns.
void mi355x_backend_ctx::mirror_outputs(struct ggml_cgraph * cgraph) {
    std::lock_guard<std::mutex> lock(mirror_mutex);
    size_t used = 0;
    for (int i = 0; i < cgraph->n_nodes; ++i) {
        const ggml_tensor * n = cgraph->nodes[i];
        // only tensors whose memory the allocator cannot have handed on by the end of the graph
        if (!((n->flags & GGML_TENSOR_FLAG_OUTPUT) || i == cgraph->n_nodes - 1) || !n->data || n->view_src || ggml_is_empty(n) || !ggml_is_contiguous(n)) continue;
        size_t lo = 0, hi = 0;                            // the part of it the host has asked for (one row of five, or all)
        if (ggml_nbytes(n) > MI355X_MIRROR_MAX || !mi355x_download_is_wanted(device, n->data, ggml_nbytes(n), &lo, &hi) || hi <= lo) continue;
        const size_t size = hi - lo;
        const size_t off = (used + 255) & ~(size_t) 255;
        if (off + size > mirror_cap) {
            if (!mirror.empty()) continue;                 // transfers into the block are queued: it cannot move now
            if (hipStreamSynchronize(stream) != hipSuccess) { (void) hipGetLastError(); return; }
            if (mirror_host) (void) hipHostFree(mirror_host);
            mirror_host = nullptr; mirror_cap = 0;
            const size_t want = std::max<size_t>(2 * (off + size), 2u << 20);
            void * p = nullptr;
            if (hipHostMalloc(&p, want, hipHostMallocDefault) != hipSuccess || !p) { (void) hipGetLastError(); return; }
            mirror_host = (char *) p; mirror_cap = want;
        }
        if (hipMemcpyAsync(mirror_host + off, (const char *) n->data + lo, size, hipMemcpyDeviceToHost, stream) != hipSuccess) { (void) hipGetLastError(); continue; }
        mirror.push_back({ (const char *) n->data, lo, size, off });
        used = off + size;
    }
    if (mirror.empty()) return;
    if (!mirror_done && hipEventCreateWithFlags(&mirror_done, hipEventDisableTiming) != hipSuccess) { (void) hipGetLastError(); mirror_done = nullptr; }
    if (!mirror_done || hipEventRecord(mirror_done, stream) != hipSuccess) { (void) hipGetLastError(); mirror.clear(); }
}

void mi355x_backend_ctx::mirror_drop(const void * begin, size_t size) {
    std::lock_guard<std::mutex> lock(mirror_mutex);
    const char * b = (const char *) begin;
    for (size_t i = 0; i < mirror.size();) {
        if (mirror[i].dev + mirror[i].lo < b + size && b < mirror[i].dev + mirror[i].lo + mirror[i].size) mirror.erase(mirror.begin() + (long) i); else ++i;
    }
}

namespace {

struct launch_scope {   // brackets one kernel launch with events when profiling
    mi355x_backend_ctx * ctx;
    mi355x_pending_event ev;
    bool on;
    launch_scope(mi355x_backend_ctx * c, const char * name, double bytes, double flops) : ctx(c), on(c->profile) {
        ctx->counters[3] += 1;
        if (!on) return;
        ev.name = name; ev.bytes = bytes; ev.flops = flops;
        ev.start = ctx->take_event(); ev.stop = ctx->take_event();
        if (ev.start) (void) hipEventRecord(ev.start, ctx->stream);
    }
    ~launch_scope() {
        if (!on) return;
        if (ev.stop) (void) hipEventRecord(ev.stop, ctx->stream);
        ctx->pending.push_back(ev);
    }
    void cancel() { ctx->counters[3] -= 1; on = false; }   // nothing was launched after all
};

double nbytes_of(const ggml_tensor * t) { return t ? (double) ggml_nbytes(t) : 0.0; }

bool ranges_overlap(const ggml_tensor * a, const ggml_tensor * b) {
    const char * a0 = (const char *) a->data, * b0 = (const char *) b->data;
    return a0 < b0 + ggml_nbytes(b) && b0 < a0 + ggml_nbytes(a);
}

// row vector [ne0] that repeats over the rows of `like`
bool is_row_vector_of(const ggml_tensor * v, const ggml_tensor * like) {
    return v->type == GGML_TYPE_F32 && v->ne[0] == like->ne[0] && v->ne[1] == 1 && v->ne[2] == 1 && v->ne[3] == 1 && v->nb[0] == sizeof(float);
}

struct graph_runner {
    mi355x_backend_ctx * ctx;
    ggml_cgraph *        g;
    std::unordered_map<const ggml_tensor *, int> readers;   // how many nodes of this graph read a tensor

    graph_runner(mi355x_backend_ctx * c, ggml_cgraph * cg) : ctx(c), g(cg) {
        if (!ctx->fuse) return;
        readers.reserve((size_t) g->n_nodes * 2);
        for (int i = 0; i < g->n_nodes; ++i) {
            const ggml_tensor * n = g->nodes[i];
            // each distinct tensor a node touches (sources and the tensor it is a view of) counts once
            const ggml_tensor * seen[GGML_MAX_SRC + 1]; int ns = 0;
            for (int s = 0; s <= GGML_MAX_SRC; ++s) {
                const ggml_tensor * t = s < GGML_MAX_SRC ? n->src[s] : n->view_src;
                if (!t) continue;
                bool dup = false;
                for (int k = 0; k < ns; ++k) dup = dup || seen[k] == t;
                if (!dup) { seen[ns++] = t; readers[t] += 1; }
            }
        }
    }

    // `t` is read by exactly one node of the graph and is not a graph output
    bool only_feeds_next(const ggml_tensor * t) const {
        if ((t->flags & GGML_TENSOR_FLAG_OUTPUT) || ctx->pieces) return false;
        auto it = readers.find(t);
        return it != readers.end() && it->second == 1;
    }

    ggml_tensor * node_at(int i) const { return i < g->n_nodes ? g->nodes[i] : nullptr; }

    // Results of the launch in progress that it does not store: intermediate values folded into the launch, and results
    // kept only as the next product's activation image.  graph_compute books them as holding no value (range_set.h).
    bool few_query_attention = false;   // the graph holds an attention node with at most 8 queries: a decode step
    std::vector<const ggml_tensor *> not_stored;
    // activations that the launch in progress took from their image in the workspace: it does not read their memory
    std::vector<const ggml_tensor *> from_image;
    // the nodes [i, i + used) folded into one launch whose result lands in `out`
    void fold_nodes(int i, int used, const ggml_tensor * out) {
        for (int k = i; k < i + used; ++k) {
            const ggml_tensor * n = g->nodes[k];
            if (n != out && !is_view_op(n->op) && !ggml_is_empty(n)) not_stored.push_back(n);
        }
    }

    // every reader of `key` is a product over it (src1), and they are the next launches, one after the other, each with
    // whatever it folds in; none but the last of them replaces the workspace image by one of its own result.  Only then
    // can the producer of `key` write the image and nothing else: the image is there for each of them.
    bool readers_are_the_next_products(const ggml_tensor * key, int from) const {
        if (ctx->pieces) return false;
        auto it = readers.find(key);
        const int want = it == readers.end() ? 0 : it->second;
        int served = 0, j = from;
        while (served < want) {
            while (node_at(j) && (is_view_op(node_at(j)->op) || ggml_is_empty(node_at(j)))) {
                if (node_at(j)->src[0] == key || node_at(j)->view_src == key) return false;     // a view of it: another way to read it
                ++j;
            }
            const ggml_tensor * n = node_at(j);
            if (!n || n->op != GGML_OP_MUL_MAT || n->src[1] != key || n->src[0] == key) return false;
            const mm_chain c = plan_chain(j);
            ++served;
            j += c.used;
            if (served < want && image_consumer(c.out, j) != nullptr) return false;            // its epilogue would put another image in place
        }
        return want > 0;
    }

    // ---- MUL_MAT and what can be folded behind it --------------------------------------------------------
    struct mm_chain {
        ggml_tensor *       mm;
        const ggml_tensor * w, * x;
        mi355x_epilogue     epi;
        ggml_tensor *       out;       // tensor that receives the fused result
        int                 used;      // nodes consumed, starting at the MUL_MAT
    };

    mm_chain plan_chain(int i) const {
        ggml_tensor * mm = g->nodes[i];
        const ggml_tensor * w = mm->src[0], * x = mm->src[1];
        mi355x_epilogue epi = { 0, 1.0f, nullptr, nullptr, nullptr };
        ggml_tensor * last = mm;       // node whose value the fused kernel produces
        ggml_tensor * out  = mm;
        int used = 1;

        if (ctx->fuse && mm->ne[2] == 1 && mm->ne[3] == 1 && ggml_is_contiguous(mm)) {
            auto same_layout = [&](const ggml_tensor * t) {
                return t->type == GGML_TYPE_F32 && ggml_are_same_shape(t, mm) && ggml_is_contiguous(t);
            };
            // Views are no-ops for the device, so they can be stepped over while looking for the next link: a dense
            // RESHAPE of the running result becomes the running result (ggml_conv_1d reshapes its MUL_MAT,
            // ggml/src/ggml.c:3899); a view of anything else (the cache slice a CPY is about to write, src/whisper.cpp:2155)
            // is simply skipped.  A view of the running result that is not such a reshape ends the chain.
            auto hop_views = [&]() {
                ggml_tensor * t = node_at(i + used);
                while (t && is_view_op(t->op)) {
                    const bool of_last = t->src[0] == last || t->view_src == last;
                    if (of_last) {
                        if (t->op == GGML_OP_RESHAPE && only_feeds_next(last) && ggml_is_contiguous(t)) last = t; else return (ggml_tensor *) nullptr;
                    }
                    ++used; t = node_at(i + used);
                }
                return t;
            };
            ggml_tensor * n = hop_views();
            // + bias
            if (n && n->op == GGML_OP_ADD && n->src[0] == last && only_feeds_next(last) && same_layout(n) && n->src[1]->type == GGML_TYPE_F32) {
                const ggml_tensor * b = n->src[1];
                if (is_row_vector_of(b, mm)) {
                    epi.flags |= MI355X_EPI_BIAS; epi.bias = b->data; last = n; ++used;
                } else if (b->ne[0] == 1 && b->ne[1] == mm->ne[1] && b->ne[2] == 1 && b->ne[3] == 1 && ggml_is_contiguous(b)) {
                    epi.flags |= MI355X_EPI_BIAS_COL; epi.bias = b->data; last = n; ++used;   // conv bias [1, d]
                }
                n = hop_views();
            }
            // + activation / scale / residual (at most one of them)
            if (n && n->src[0] == last && only_feeds_next(last) && same_layout(n)) {
                if (n->op == GGML_OP_UNARY && ggml_get_unary_op(n) == GGML_UNARY_OP_GELU) {
                    epi.flags |= MI355X_EPI_GELU; last = n; ++used;
                } else if (n->op == GGML_OP_SCALE) {
                    epi.flags |= MI355X_EPI_SCALE; memcpy(&epi.scale, n->op_params, sizeof(float)); last = n; ++used;
                } else if (n->op == GGML_OP_ADD && same_layout(n->src[1]) && n->src[1] != last) {
                    epi.flags |= MI355X_EPI_RESIDUAL; epi.residual = n->src[1]->data; last = n; ++used;
                }
                n = hop_views();
            }
            // views stepped over after the last folded link stay in the graph walk (they are no-ops there, too)
            out = last;
            // + store as f16 (K/V cache writes)
            if (n && n->op == GGML_OP_CPY && n->src[0] == last && only_feeds_next(last) && !(epi.flags & MI355X_EPI_RESIDUAL) &&
                n->src[1]->type == GGML_TYPE_F16 && ggml_is_contiguous(n->src[1]) && ggml_nelements(n->src[1]) == ggml_nelements(mm)) {
                epi.flags |= MI355X_EPI_OUT_F16; out = n; ++used;
            }
            // the folded result must not land on memory the kernel is still reading
            if (used > 1 && (ranges_overlap(out, x) || ranges_overlap(out, w))) {
                epi = { 0, 1.0f, nullptr, nullptr, nullptr }; out = mm; used = 1;
            }
        }
        return { mm, w, x, epi, out, used };
    }

    // operand descriptors of a planned chain; a quantized weight matrix that meets many columns is replaced by its f16
    // image, kept beside it in HBM (then MI355X_MM_ACT_Q8_0 goes into `mm_flags`)
    struct mm_operands { mi355x_tensor vw, vx, vd; int mm_flags; const char * kernel_name; const void * tiles; };
    mm_operands describe(const mm_chain & c) const {
        mm_operands o;
        o.vw = to_view(c.w); o.vx = to_view(c.x); o.vd = to_view(c.mm);
        o.vd.data = c.out->data;
        if (c.epi.flags & MI355X_EPI_OUT_F16) {
            o.vd.type = MI355X_TYPE_F16;
            o.vd.nb[0] = 2; o.vd.nb[1] = 2 * (size_t) c.mm->ne[0]; o.vd.nb[2] = o.vd.nb[1] * c.mm->ne[1]; o.vd.nb[3] = o.vd.nb[2];
        }
        o.kernel_name = mi355x_mul_mat_kernel_name(&o.vw, &o.vx);
        o.mm_flags = ctx->exact ? MI355X_MM_EXACT_ACT : 0;
        const ggml_tensor * w = c.w;
        if (ctx->weight_images && ggml_is_quantized(w->type) && w->ne[2] == 1 && w->ne[3] == 1 && ggml_is_contiguous(w) && !w->view_src &&
            w->buffer && w->buffer->usage == GGML_BACKEND_BUFFER_USAGE_WEIGHTS && mi355x_buffer_is_ours(w->buffer) &&
            strncmp(o.kernel_name, "mul_mat.gemm", 12) == 0) {
            const void * image = ((mi355x_buffer_ctx *) w->buffer->context)->weight_image(w, ctx->stream);
            if (image) {
                o.vw.data = (void *) image; o.vw.type = MI355X_TYPE_F16;
                o.vw.nb[0] = 2; o.vw.nb[1] = 2 * (size_t) w->ne[0]; o.vw.nb[2] = o.vw.nb[1] * (size_t) w->ne[1]; o.vw.nb[3] = o.vw.nb[2];
                o.mm_flags |= MI355X_MM_ACT_Q8_0;
            }
        }
        // the few-column product over a Q8_0 matrix of tens of MB (the logits over the vocabulary) reads a copy of it in
        // matrix-core order
        o.tiles = nullptr;
        if (ctx->weight_images && w->type == GGML_TYPE_Q8_0 && nbytes_of(w) >= 32e6 && w->ne[2] == 1 && w->ne[3] == 1 && ggml_is_contiguous(w) &&
            !w->view_src && w->buffer && w->buffer->usage == GGML_BACKEND_BUFFER_USAGE_WEIGHTS && mi355x_buffer_is_ours(w->buffer) &&
            strcmp(o.kernel_name, "mul_mat.gemv_q8_0") == 0 && !(c.epi.flags & ~MI355X_EPI_OUT_F16) && c.x->type == GGML_TYPE_F32 &&
            c.mm->ne[2] == 1 && c.mm->ne[3] == 1 && mi355x_q8_0_tiles_size(w->ne[0], w->ne[1]) > 0) {
            o.tiles = ((mi355x_buffer_ctx *) w->buffer->context)->weight_image(w, ctx->stream, MI355X_IMAGE_TILES);
        }
        return o;
    }

    // The GEMM first brings src1 to f16 (rounded to Q8_0 on the way when the weights are quantized) in the workspace, the
    // few-column product over quantized weights brings it to Q8_0; consecutive MUL_MATs over the same activations share
    // that copy.  Runs (and times) the conversion when the workspace
    // does not hold it yet; returns the MM flags to add (WS_READY), or -1 with `status` set.
    int prepare_src1(const mm_chain & c, const mm_operands & o, size_t need, int & status) {
        if (!need) return 0;
        if (!ctx->reserve_workspace(need)) { status = MI355X_ERR_WORKSPACE; return -1; }
        const ggml_tensor * x = c.x;
        if (x->type != GGML_TYPE_F32) return 0;
        const bool gemv = strncmp(o.kernel_name, "mul_mat.gemv", 12) == 0;
        const int mode = gemv ? 2 : (ggml_is_quantized(c.w->type) && !ctx->exact) ? 1 : 0;       // 1: f16 rounded to Q8_0, 2: Q8_0 itself
        const bool hit = ctx->ws_x == x->data && ctx->ws_x_mode == mode && memcmp(ctx->ws_x_ne, x->ne, sizeof(x->ne)) == 0 &&
                         memcmp(ctx->ws_x_nb, x->nb, sizeof(x->nb)) == 0;
        ctx->ws_x = x->data; ctx->ws_x_mode = mode; memcpy(ctx->ws_x_ne, x->ne, sizeof(x->ne)); memcpy(ctx->ws_x_nb, x->nb, sizeof(x->nb));
        cached_x = x;
        if (!hit && ctx->image_only == (const void *) x) {
            // the producer of these activations wrote nothing but their image, and the image is gone: a planner error, not
            // something to paper over with a conversion of memory that was never written
            GGML_LOG_ERROR("ggml-mi355x: the activation image of %s was dropped before %s read it\n", x->name, c.mm->name);
            status = MI355X_ERR_INVALID;
            return -1;
        }
        if (hit) from_image.push_back(x);
        if (!hit) {
            mi355x_epilogue prep = c.epi;                 // same call as the product itself, stopped after the conversion
            prep.flags |= o.mm_flags | MI355X_MM_PREPARE_ONLY;
            launch_scope ls(ctx, gemv ? "mul_mat.src1_to_q8_0" : "mul_mat.src1_to_f16", nbytes_of(x) * (gemv ? 1.3125 : 1.5), 0.0);
            status = mi355x_mul_mat(&o.vw, &o.vx, &o.vd, &prep, ctx->ws, ctx->ws_size, ctx->stream);
            if (status != MI355X_OK) return -1;
        }
        return MI355X_MM_WS_READY;
    }

    static double chain_flops(const mm_chain & c) { return 2.0 * c.mm->ne[0] * c.mm->ne[1] * c.w->ne[0] * (double) c.mm->ne[2] * c.mm->ne[3]; }
    static double chain_bytes(const mm_chain & c) {
        return nbytes_of(c.w) + nbytes_of(c.x) + (double) ggml_nelements(c.mm) * ((c.epi.flags & MI355X_EPI_OUT_F16) ? 2 : 4) +
               ((c.epi.flags & MI355X_EPI_RESIDUAL) ? nbytes_of(c.mm) : 0.0);
    }

    // A LayerNorm of a decode step (a handful of rows) whose result only feeds few-column products is not launched when
    // it is met: it is held here and goes out inside the launch of those products (mi355x_norm_mul_mat_group).  If the
    // next node to execute turns out to be something else, or the fused form does not take the shapes, it runs on its own
    // after all (flush_norm).
    struct held_norm {
        bool active = false;
        const ggml_tensor * src = nullptr, * out = nullptr, * key = nullptr;
        float eps = 0.0f; const float * w = nullptr, * b = nullptr;
        bool affine = false;
    } held;

    // The embedding of a decode step's tokens (GET_ROWS, GET_ROWS, ADD: a handful of rows) that only feeds a LayerNorm is
    // held the same way: if that LayerNorm ends up inside the launch of its products, the rows are made there
    // (mi355x_embed_norm_mul_mat_group); in every other case the embedding runs on its own first (flush_embed).
    struct held_embed {
        bool active = false;
        const ggml_tensor * tok = nullptr, * tok_ids = nullptr, * pos = nullptr, * pos_ids = nullptr, * out = nullptr;
    } emb;

    int flush_embed() {
        if (!emb.active) return MI355X_OK;
        emb.active = false;
        mi355x_tensor a = to_view(emb.tok), ia = to_view(emb.tok_ids), b = to_view(emb.pos), ib = to_view(emb.pos_ids), d = to_view(emb.out);
        launch_scope ls(ctx, "get_rows_add", 3.0 * nbytes_of(emb.out), 0.0);
        const int rc = mi355x_get_rows_add(&a, &ia, &b, &ib, &d, ctx->stream);
        note_write(emb.out);
        return rc;
    }

    int flush_norm() {
        if (const int rc = flush_embed()) return rc;        // (a held embedding is the held LayerNorm's source)
        if (!held.active) return MI355X_OK;
        held.active = false;
        mi355x_tensor vs = to_view(held.src), vd = to_view(held.out);
        const size_t image_bytes = (size_t)(held.out->ne[0] * held.out->ne[1] + held.out->ne[0] / 32 * held.out->ne[1] * 8);
        bool emit = ctx->reserve_workspace(image_bytes + 256);
        int status;
        {
            launch_scope ls(ctx, held.affine ? (emit ? "norm_affine_emit" : "norm_affine") : "norm", nbytes_of(held.src) + nbytes_of(held.out) + (emit ? image_bytes : 0), 0.0);
            status = emit ? mi355x_norm_emit_q8_0(&vs, &vd, held.eps, held.w, held.b, ctx->ws, ctx->stream) : mi355x_norm(&vs, &vd, held.eps, held.w, held.b, ctx->stream);
        }
        if (emit && status == MI355X_ERR_UNSUPPORTED) { emit = false; status = mi355x_norm(&vs, &vd, held.eps, held.w, held.b, ctx->stream); }
        note_write(held.out);
        if (emit && status == MI355X_OK) workspace_holds(held.key, ctx->ws_slot, 2);
        return status;
    }

    // Products that follow each other over the same activations with weights of one shape (Q, K, V of a layer; the
    // cross-attention K / V of all decoder layers) go out as one launch.  Returns the nodes consumed, 0 if no group formed.
    // With a held LayerNorm over these activations the launch includes it, and one product is group enough.
    int run_mul_mat_group(int i, const mm_chain & first, const mm_operands & o0, int & status) {
        // (the few-column form: a decode step's Q, K and V over quantized weights, up to 8 products)
        const bool gemv = strncmp(o0.kernel_name, "mul_mat.gemv", 12) == 0;
        if (!ctx->fuse || first.mm->ne[2] != 1 || first.mm->ne[3] != 1) return 0;
        if (gemv) {
            if (mi355x_mul_mat_workspace_size(&o0.vw, &o0.vx) == 0) return 0;
        } else if (o0.vw.type != MI355X_TYPE_F16 || strncmp(o0.kernel_name, "mul_mat.gemm", 12) != 0 || first.w->ne[0] % 256 != 0) return 0;
        std::vector<mm_chain>    chains{ first };
        std::vector<mm_operands> ops{ o0 };
        int end = i + first.used;                       // first node after the group
        while ((int) chains.size() < (gemv ? 8 : 64)) {
            int j = end;
            while (node_at(j) && (is_view_op(node_at(j)->op) || ggml_is_empty(node_at(j)))) ++j;
            ggml_tensor * n = node_at(j);
            if (!n || n->op != GGML_OP_MUL_MAT || n->src[1] != first.x || n->src[0]->type != first.w->type ||
                !ggml_are_same_shape(n->src[0], first.w) || !ggml_are_same_shape(n, first.mm)) break;
            mm_chain c = plan_chain(j);
            mm_operands o = describe(c);
            if (o.vw.type != o0.vw.type || o.mm_flags != o0.mm_flags || o.vw.nb[1] != o0.vw.nb[1]) break;
            // nothing in the group may read what another member writes
            bool clash = false;
            for (const mm_chain & p : chains) {
                clash = clash || ranges_overlap(c.out, p.out) || ranges_overlap(p.out, c.w);
                for (int k = j; k < j + c.used; ++k)
                    for (int s = 0; s < GGML_MAX_SRC; ++s)
                        if (g->nodes[k]->src[s] && !is_view_op(g->nodes[k]->op)) clash = clash || ranges_overlap(p.out, g->nodes[k]->src[s]);
            }
            if (clash) break;
            chains.push_back(c); ops.push_back(o);
            end = j + c.used;
        }
        // (not for the product over the vocabulary: 70 MB of weights hide no prologue, and its time stays a GEMV's time)
        const bool with_norm = held.active && gemv && held.key == first.x && nbytes_of(first.w) < 32e6;
        if (chains.size() < 2 && !with_norm) return 0;

        const size_t need = mi355x_mul_mat_workspace_size(&o0.vw, &o0.vx);
        std::vector<mi355x_mul_mat_item> items(chains.size());
        double flops = 0.0, bytes = 0.0;
        for (size_t k = 0; k < chains.size(); ++k) {
            items[k] = { &ops[k].vw, &ops[k].vd, &chains[k].epi };
            flops += chain_flops(chains[k]); bytes += chain_bytes(chains[k]) - (k ? nbytes_of(first.x) : 0.0);
        }
        if (with_norm) {
            // A single product whose result (the FFN's first matrix with its GELU) feeds nothing but the few-column product that
            // is launched next also leaves it quantized to Q8_0, in the other workspace slot: that product's quantization pass —
            // a launch on the step's critical path — is not needed then.
            const ggml_tensor * q8_key = nullptr;
            size_t need_all = need;
            if (chains.size() == 1 && !(chains[0].epi.flags & MI355X_EPI_OUT_F16) && chains[0].out->ne[0] % 32 == 0) {
                q8_key = image_consumer(chains[0].out, end, true);
                if (q8_key && !next_is_product_over(q8_key, end)) q8_key = nullptr;
                if (q8_key) need_all = std::max(need, (size_t)(chains[0].out->ne[0] * chains[0].out->ne[1] + chains[0].out->ne[0] / 32 * chains[0].out->ne[1] * 8) + 256);
            }
            if (!ctx->reserve_workspace(need_all)) { status = MI355X_ERR_WORKSPACE; return end - i; }
            mi355x_tensor vs = to_view(held.src), vn = to_view(held.out);
            if (q8_key) { chains[0].epi.flags |= MI355X_EPI_EMIT_Q8_0; chains[0].epi.image = slot_ptr(ctx->ws_slot ^ 1); }
            auto launch = [&](bool embed) {
                mi355x_tensor vt, vti, vp, vpi;
                if (embed) { vt = to_view(emb.tok); vti = to_view(emb.tok_ids); vp = to_view(emb.pos); vpi = to_view(emb.pos_ids); }
                auto call = [&]() {
                    return embed ? mi355x_embed_norm_mul_mat_group(&vt, &vti, &vp, &vpi, &vs, &vn, held.eps, held.w, held.b, items.data(), (int) items.size(), ctx->ws, ctx->ws_size, ctx->stream)
                                 : mi355x_norm_mul_mat_group(&vs, &vn, held.eps, held.w, held.b, items.data(), (int) items.size(), ctx->ws, ctx->ws_size, ctx->stream);
                };
                int r = call();
                if (r == MI355X_ERR_UNSUPPORTED && q8_key) {
                    chains[0].epi.flags &= ~MI355X_EPI_EMIT_Q8_0; chains[0].epi.image = nullptr; q8_key = nullptr;
                    r = call();
                }
                return r;
            };
            int rc = MI355X_ERR_UNSUPPORTED;
            if (emb.active) {                               // (then held.src is the embedding: nothing has written it yet)
                launch_scope ls(ctx, "embed_norm_mul_mat.gemv", bytes + 3.0 * nbytes_of(held.src) + nbytes_of(held.out), flops);
                rc = launch(true);
                if (rc == MI355X_ERR_UNSUPPORTED) ls.cancel();
                else { emb.active = false; note_write(emb.out); }
            }
            if (rc == MI355X_ERR_UNSUPPORTED) {
                if ((rc = flush_embed()) != MI355X_OK) { status = rc; return end - i; }
                launch_scope ls(ctx, "norm_mul_mat.gemv", bytes + nbytes_of(held.src) + nbytes_of(held.out), flops);
                rc = launch(false);
                if (rc == MI355X_ERR_UNSUPPORTED) ls.cancel();
            }
            if (rc == MI355X_ERR_UNSUPPORTED) return 0;      // the caller lets the LayerNorm run on its own and takes the usual path
            held.active = false;
            status = rc;
            note_write(held.out);
            if (rc == MI355X_OK) workspace_holds(held.key, ctx->ws_slot, 2);
            for (const mm_chain & c : chains) { note_write(c.out); fold_nodes((int)(std::find(g->nodes + i, g->nodes + end, c.mm) - g->nodes), c.used, c.out); }
            if (rc == MI355X_OK && q8_key) workspace_holds(q8_key, ctx->ws_slot ^ 1, 2);       // (after note_write: the image is of what was just written)
            return end - i;
        }
        const int ready = prepare_src1(first, o0, need, status);
        if (ready < 0) return end - i;
        int rc;
        {
            launch_scope ls(ctx, gemv ? "mul_mat.gemv_group" : "mul_mat.gemm_group", bytes, flops);
            rc = mi355x_mul_mat_group(items.data(), (int) items.size(), &o0.vx, o0.mm_flags | ready, ctx->ws, ctx->ws_size, ctx->stream);
        }
        if (rc == MI355X_ERR_UNSUPPORTED) return 0;     // the single-product path takes them one by one
        status = rc;
        if (ctx->debug) GGML_LOG_INFO("ggml-mi355x: %s of %zu starting at %s, %d nodes\n", gemv ? "mul_mat.gemv_group" : "mul_mat.gemm_group", chains.size(), first.mm->name, end - i);
        for (const mm_chain & c : chains) { note_write(c.out); fold_nodes((int)(std::find(g->nodes + i, g->nodes + end, c.mm) - g->nodes), c.used, c.out); }
        return end - i;
    }

    // returns the number of nodes consumed
    int run_mul_mat(int i, int & status) {
        const mm_chain c = plan_chain(i);
        mm_operands o = describe(c);
        if (const int grouped = run_mul_mat_group(i, c, o, status)) return grouped;
        // the decoder's last LayerNorm, held, in front of the logits over the tile-ordered vocabulary matrix: one launch, the
        // LayerNorm under the 7 us the first tile rows take to arrive
        if (held.active && held.key == c.x && o.tiles && !emb.active &&
            ctx->reserve_workspace((size_t)(c.x->ne[0] * c.x->ne[1] + c.x->ne[0] / 32 * c.x->ne[1] * 8) + 256)) {
            mi355x_tensor vs = to_view(held.src), vn = to_view(held.out);
            int rc;
            {
                launch_scope ls(ctx, "norm_mul_mat.gemv_q8_0.vocab", chain_bytes(c) + nbytes_of(held.src) + nbytes_of(held.out), chain_flops(c));
                rc = mi355x_norm_mul_mat_q8_0_tiles(o.tiles, c.w->ne[0], c.w->ne[1], &vs, &vn, held.eps, held.w, held.b, &o.vd,
                                                    c.epi.flags & MI355X_EPI_OUT_F16, ctx->ws, ctx->ws_size, ctx->stream);
                if (rc == MI355X_ERR_UNSUPPORTED) ls.cancel();
            }
            if (rc != MI355X_ERR_UNSUPPORTED) {
                held.active = false;
                status = rc;
                note_write(held.out);
                if (rc == MI355X_OK) workspace_holds(held.key, ctx->ws_slot, 2);
                note_write(c.out);
                fold_nodes(i, c.used, c.out);
                return c.used;
            }
        }
        if (held.active && (status = flush_norm()) != MI355X_OK) return c.used;

        mi355x_epilogue epi = c.epi;
        epi.flags |= o.mm_flags;
        size_t need = mi355x_mul_mat_workspace_size(&o.vw, &o.vx);
        // when the result feeds nothing but products that round it to Q8_0 (the FFN's second matrix after the first), the
        // epilogue writes that image into the workspace slot this product is not reading from
        const ggml_tensor * key = nullptr;
        if (!(epi.flags & MI355X_EPI_OUT_F16) && c.mm->ne[2] == 1 && c.mm->ne[3] == 1 && strncmp(o.kernel_name, "mul_mat.gemm", 12) == 0) {
            key = image_consumer(c.out, i + c.used);
            if (key) need = std::max(need, (size_t) ggml_nelements(c.out) * 2 + 256);
        }
        const int ready = prepare_src1(c, o, need, status);
        if (ready < 0) return c.used;
        epi.flags |= ready;
        if (key && ctx->ws_base) { epi.flags |= MI355X_EPI_EMIT_F16; epi.image = slot_ptr(ctx->ws_slot ^ 1); } else key = nullptr;
        // ... and nothing else when the product that takes the image is the very next launch: the f32 values would have no reader
        const bool image_only = key && ctx->dead_f32 && readers_are_the_next_products(key, i + c.used);
        if (image_only) epi.flags |= MI355X_EPI_IMAGE_ONLY;
        if (ctx->debug) {
            GGML_LOG_INFO("ggml-mi355x: %s %s [%lld x %lld x %lld] folds %d nodes, flags 0x%x\n", o.kernel_name, c.mm->name,
                          (long long) c.mm->ne[0], (long long) c.mm->ne[1], (long long) c.w->ne[0], c.used, epi.flags);
        }
        // the statistics keep the one few-column product that streams tens of MB (the logits over the vocabulary) apart
        // from the many that are over in the latency of a launch
        const char * scope = o.kernel_name;
        if (nbytes_of(c.w) >= 32e6) {
            if (strcmp(scope, "mul_mat.gemv_q8_0") == 0) scope = "mul_mat.gemv_q8_0.vocab";
            else if (strcmp(scope, "mul_mat.gemv_q5_0") == 0) scope = "mul_mat.gemv_q5_0.vocab";
        }
        {
            launch_scope ls(ctx, scope, chain_bytes(c), chain_flops(c));
            status = MI355X_ERR_UNSUPPORTED;
            if (o.tiles && !key) {
                status = mi355x_mul_mat_q8_0_tiles(o.tiles, c.w->ne[0], c.w->ne[1], &o.vx, &o.vd,
                                                   epi.flags & (MI355X_EPI_OUT_F16 | MI355X_MM_WS_READY), ctx->ws, ctx->ws_size, ctx->stream);
            }
            if (status == MI355X_ERR_UNSUPPORTED)       // (a K the tiles kernel is not built for)
            status = mi355x_mul_mat(&o.vw, &o.vx, &o.vd, epi.flags ? &epi : nullptr, ctx->ws, ctx->ws_size, ctx->stream);
            if (key && status == MI355X_ERR_UNSUPPORTED) {          // shapes the epilogue cannot emit for: plain product
                epi.flags &= ~(MI355X_EPI_EMIT_F16 | MI355X_EPI_IMAGE_ONLY); key = nullptr;
                status = mi355x_mul_mat(&o.vw, &o.vx, &o.vd, epi.flags ? &epi : nullptr, ctx->ws, ctx->ws_size, ctx->stream);
            }
        }
        note_write(c.out);
        fold_nodes(i, c.used, c.out);
        if (key && status == MI355X_OK) { workspace_holds(key, ctx->ws_slot ^ 1); if (image_only && (epi.flags & MI355X_EPI_IMAGE_ONLY)) { ctx->image_only = key; not_stored.push_back(c.out); } }
        return c.used;
    }

    // When everything that reads `out` (produced just before node `from`) — directly, or through one dense 2-d RESHAPE of
    // it — is a many-column product with quantized weights, the producer can leave the Q8_0-rounded f16 image those
    // products want in the workspace and they skip their conversion pass.  Returns the tensor the products name as src1.
    // `few`: the same question for the few-column products, which read their activations as Q8_0 from the workspace.
    const ggml_tensor * image_consumer(const ggml_tensor * out, int from, bool few = false) const {
        if (!ctx->fuse || ctx->exact || (out->flags & GGML_TENSOR_FLAG_OUTPUT) || !ggml_is_contiguous(out)) return nullptr;
        const ggml_tensor * key = out;
        for (int hop = 0; hop < 2; ++hop) {
            auto it = readers.find(key);
            const int want = it == readers.end() ? 0 : it->second;
            if (want == 0) return nullptr;
            int seen = 0;
            const ggml_tensor * reshape = nullptr;
            for (int j = from; j < g->n_nodes && seen < want; ++j) {
                const ggml_tensor * n = g->nodes[j];
                bool reads = n->view_src == key;
                for (int k = 0; k < GGML_MAX_SRC; ++k) reads = reads || n->src[k] == key;
                if (!reads) continue;
                ++seen;
                if (n->op == GGML_OP_MUL_MAT && n->src[1] == key && n->src[0] != key && ggml_is_quantized(n->src[0]->type)) {
                    if (!few) continue;
                    mi355x_tensor vw = to_view(n->src[0]), vx = to_view(key);
                    if (mi355x_mul_mat_workspace_size(&vw, &vx) > 0 && strncmp(mi355x_mul_mat_kernel_name(&vw, &vx), "mul_mat.gemv", 12) == 0) continue;
                    return nullptr;
                }
                if (want == 1 && hop == 0 && n->op == GGML_OP_RESHAPE && n->src[0] == key && ggml_is_contiguous(n) && !(n->flags & GGML_TENSOR_FLAG_OUTPUT)) { reshape = n; continue; }
                return nullptr;
            }
            if (seen != want) return nullptr;
            if (!reshape) break;
            key = reshape;
        }
        if (key->ne[2] != 1 || key->ne[3] != 1 || (key->ne[1] <= MI355X_GEMV_MAX_COLS) != few || key->ne[0] % 32 != 0) return nullptr;
        return key;
    }
    void * slot_ptr(int slot) const { return (char *) ctx->ws_base + (size_t) slot * ctx->ws_size; }
    // the image of `key` now sits in `slot`, which becomes the current one
    void workspace_holds(const ggml_tensor * key, int slot, int mode = 1) {
        ctx->ws_slot = slot; ctx->ws = slot_ptr(slot);
        ctx->ws_x = key->data; ctx->ws_x_mode = mode; memcpy(ctx->ws_x_ne, key->ne, sizeof(key->ne)); memcpy(ctx->ws_x_nb, key->nb, sizeof(key->nb));
        cached_x = key;
    }

    // ---- NORM [-> MUL(w) -> ADD(b)] ---------------------------------------------------------------------
    int run_norm(int i, int & status) {
        ggml_tensor * nm = g->nodes[i];
        float eps; memcpy(&eps, nm->op_params, sizeof(float));
        const float * w = nullptr, * b = nullptr;
        ggml_tensor * out = nm;
        int used = 1;
        if (ctx->fuse) {
            ggml_tensor * mul = node_at(i + 1), * add = node_at(i + 2);
            if (mul && add && mul->op == GGML_OP_MUL && add->op == GGML_OP_ADD &&
                mul->src[0] == nm && add->src[0] == mul && only_feeds_next(nm) && only_feeds_next(mul) &&
                is_row_vector_of(mul->src[1], nm) && is_row_vector_of(add->src[1], nm) &&
                ggml_are_same_shape(add, nm) && add->type == GGML_TYPE_F32 && add->nb[0] == sizeof(float)) {
                w = (const float *) mul->src[1]->data; b = (const float *) add->src[1]->data;
                out = add; used = 3;
            }
        }
        mi355x_tensor vs = to_view(nm->src[0]), vd = to_view(out);
        // When everything that reads the result is a many-column product with quantized weights, the kernel also leaves
        // the Q8_0-rounded f16 image those products want in the workspace, and they skip their conversion pass.
        // (A decode step's few-column products read Q8_0 itself; then the kernel leaves that.)
        const ggml_tensor * key = out->ne[0] <= 2048 ? image_consumer(out, i + used) : nullptr;
        int mode = 1;
        if (!key && out->ne[0] <= 2048 && (key = image_consumer(out, i + used, true))) mode = 2;
        if (mode == 2 && nm->src[0]->ne[2] == 1 && nm->src[0]->ne[3] == 1 && next_is_product_over(key, i + used)) {
            held.active = true; held.src = nm->src[0]; held.out = out; held.key = key; held.eps = eps; held.w = w; held.b = b; held.affine = used == 3;
            fold_nodes(i, used, out);
            return used;
        }
        if ((status = flush_embed()) != MI355X_OK) return used;
        const size_t image_bytes = mode == 1 ? (size_t)(out->ne[0] * out->ne[1] * 2) : (size_t)(out->ne[0] * out->ne[1] + out->ne[0] / 32 * out->ne[1] * 8);
        bool emit = key && ctx->reserve_workspace(image_bytes + 256);
        // the image and nothing else when the product that takes it is the very next launch: the f32 rows would have no reader
        const bool image_only = emit && mode == 1 && ctx->dead_f32 && readers_are_the_next_products(key, i + used);
        {
            launch_scope ls(ctx, used == 3 ? (emit ? "norm_affine_emit" : "norm_affine") : "norm", nbytes_of(nm->src[0]) + (image_only ? 0 : nbytes_of(out)) + (emit ? image_bytes : 0), 0.0);
            mi355x_tensor vo = vd;
            if (image_only) vo.data = nullptr;
            status = !emit ? mi355x_norm(&vs, &vd, eps, w, b, ctx->stream)
                   : mode == 1 ? mi355x_norm_emit_f16(&vs, &vo, eps, w, b, ctx->ws, ctx->stream) : mi355x_norm_emit_q8_0(&vs, &vd, eps, w, b, ctx->ws, ctx->stream);
        }
        if (emit && status == MI355X_ERR_UNSUPPORTED) { emit = false; status = mi355x_norm(&vs, &vd, eps, w, b, ctx->stream); }
        note_write(out);
        fold_nodes(i, used, out);
        if (emit && status == MI355X_OK) { workspace_holds(key, ctx->ws_slot, mode); if (image_only) { ctx->image_only = key; not_stored.push_back(out); } }
        return used;
    }

    // the next node that executes (views and empty nodes skipped) is a MUL_MAT with `key` as src1
    bool next_is_product_over(const ggml_tensor * key, int from) const {
        int j = from;
        while (node_at(j) && (is_view_op(node_at(j)->op) || ggml_is_empty(node_at(j)))) ++j;
        const ggml_tensor * n = node_at(j);
        return n && n->op == GGML_OP_MUL_MAT && n->src[1] == key;
    }

    // A decode step casts its f32 mask to f16 (src/whisper.cpp:2523) right in front of its first FLASH_ATTN_EXT node.  When
    // that node runs on the few-query kernel, the cast is not launched — it is a launch on the step's critical path — and
    // the attention launch rounds the f32 values itself and leaves the f16 copy behind for the later layers' nodes
    // (mi355x_flash_attn_ext_cast_mask).  The f32 tensor is read in the launch that takes the cast's place, so the
    // allocator's reuse of its memory after the cast (ggml/src/ggml-alloc.c:640-667) is not a concern.
    const ggml_tensor * cast_dst = nullptr, * cast_src = nullptr;          // a cast that the next attention node carries out

    bool next_attention_casts(int i) const {
        const ggml_tensor * n = g->nodes[i], * s0 = n->src[0];
        if (!ctx->fuse || ctx->exact || (ctx->fa_accum & 2) || n->src[1] != n || s0->type != GGML_TYPE_F32 || n->type != GGML_TYPE_F16 ||
            (n->flags & GGML_TENSOR_FLAG_OUTPUT) || !ggml_is_contiguous(s0) || !ggml_is_contiguous(n) || !ggml_are_same_shape(s0, n) ||
            n->ne[2] != 1 || n->ne[3] != 1 || n->view_src) return false;
        int j = i + 1;
        while (node_at(j) && (is_view_op(node_at(j)->op) || ggml_is_empty(node_at(j)))) {
            if (node_at(j)->src[0] == n || node_at(j)->view_src == n) return false;       // a view of the copy: someone else reads it
            ++j;
        }
        const ggml_tensor * r = node_at(j);
        if (!r || r->op != GGML_OP_FLASH_ATTN_EXT || r->src[3] != n || r->src[0]->ne[1] > n->ne[1]) return false;
        // The allocator frees the f32 mask after the cast (ggml/src/ggml-alloc.c:612-667) and may place the attention node's
        // own output there: its workgroups would then overwrite mask rows that others are still reading.  (The f16 copy
        // is a source of the attention node, so the allocator keeps that apart from the output by itself.)
        if (ranges_overlap(r, s0) || ranges_overlap(r, n)) return false;
        mi355x_tensor vq = to_view(r->src[0]), vk = to_view(r->src[1]);
        return strcmp(mi355x_flash_attn_ext_kernel_name(&vq, &vk, MI355X_FA_F16_SEQ), "flash_attn.seq_row") == 0;
    }

    // the workspace copy of the activations goes stale when something overwrites them
    const ggml_tensor * cached_x = nullptr;
    void note_write(const ggml_tensor * out) {
        if (cached_x && ctx->ws_x && ranges_overlap(out, cached_x)) { ctx->ws_x = nullptr; cached_x = nullptr; }
    }

    int run_node(int i, int & status) {
        ggml_tensor * n = g->nodes[i];
        status = MI355X_OK;
        if (ggml_is_empty(n) || is_view_op(n->op)) return 1;
        const ggml_tensor * s0 = n->src[0], * s1 = n->src[1];
        if (held.active && !(n->op == GGML_OP_MUL_MAT && s1 == held.key) && (status = flush_norm()) != MI355X_OK) return 1;
        if (emb.active && !held.active && !(n->op == GGML_OP_NORM && s0 == emb.out) && (status = flush_embed()) != MI355X_OK) return 1;
        if (n->op != GGML_OP_MUL_MAT && n->op != GGML_OP_NORM) note_write(n->op == GGML_OP_CPY ? s1 : n);
        switch (n->op) {
            case GGML_OP_MUL_MAT: return run_mul_mat(i, status);
            case GGML_OP_NORM:    return run_norm(i, status);
            case GGML_OP_ADD: case GGML_OP_MUL: {
                mi355x_tensor a = to_view(s0), b = to_view(s1), d = to_view(n);
                launch_scope ls(ctx, n->op == GGML_OP_ADD ? "add" : "mul", nbytes_of(s0) + nbytes_of(s1) + nbytes_of(n), 0.0);
                status = mi355x_binary(n->op == GGML_OP_ADD ? 0 : 1, &a, &b, &d, ctx->stream);
                return 1;
            }
            case GGML_OP_SCALE: {
                float s; memcpy(&s, n->op_params, sizeof(float));
                mi355x_tensor a = to_view(s0), d = to_view(n);
                launch_scope ls(ctx, "scale", nbytes_of(s0) + nbytes_of(n), 0.0);
                status = mi355x_scale(&a, &d, s, ctx->stream);
                return 1;
            }
            case GGML_OP_UNARY: {
                if (ggml_get_unary_op(n) != GGML_UNARY_OP_GELU) { status = MI355X_ERR_UNSUPPORTED; return 1; }
                mi355x_tensor a = to_view(s0), d = to_view(n);
                launch_scope ls(ctx, "gelu", nbytes_of(s0) + nbytes_of(n), 0.0);
                status = mi355x_gelu(&a, &d, ctx->stream);
                return 1;
            }
            case GGML_OP_SOFT_MAX: {
                float scale; memcpy(&scale, n->op_params, sizeof(float));
                mi355x_tensor a = to_view(s0), d = to_view(n), m;
                if (s1) m = to_view(s1);
                launch_scope ls(ctx, "soft_max", nbytes_of(s0) + nbytes_of(s1) + nbytes_of(n), 0.0);
                status = mi355x_soft_max(&a, s1 ? &m : nullptr, &d, scale, ctx->stream);
                return 1;
            }
            case GGML_OP_CPY: case GGML_OP_CONT: case GGML_OP_DUP: {
                if (n->op == GGML_OP_CPY && next_attention_casts(i)) { cast_dst = n; cast_src = s0; return 1; }
                const ggml_tensor * dt = n->op == GGML_OP_CPY ? s1 : n;
                mi355x_tensor a = to_view(s0), d = to_view(dt);
                launch_scope ls(ctx, "cpy", nbytes_of(s0) + nbytes_of(dt), 0.0);
                status = mi355x_cpy(&a, &d, ctx->stream);
                return 1;
            }
            case GGML_OP_GET_ROWS: {
                // token embedding + positional embedding of a decoder input (src/whisper.cpp:2526-2529): GET_ROWS, GET_ROWS, ADD
                // as one launch when the two gathered tensors feed nothing else
                if (ctx->fuse && only_feeds_next(n) && s1->ne[1] == 1 && s1->ne[2] == 1 && s1->ne[3] == 1) {
                    int j = i + 1;
                    while (node_at(j) && (is_view_op(node_at(j)->op) || ggml_is_empty(node_at(j)))) ++j;
                    ggml_tensor * g2 = node_at(j);
                    int k = j + 1;
                    while (node_at(k) && (is_view_op(node_at(k)->op) || ggml_is_empty(node_at(k)))) ++k;
                    ggml_tensor * add = node_at(k);
                    if (g2 && add && g2->op == GGML_OP_GET_ROWS && add->op == GGML_OP_ADD && only_feeds_next(g2) && g2->src[0]->type == GGML_TYPE_F32 &&
                        ((add->src[0] == n && add->src[1] == g2) || (add->src[0] == g2 && add->src[1] == n)) &&
                        ggml_are_same_shape(n, g2) && ggml_are_same_shape(n, add) && add->type == GGML_TYPE_F32 && ggml_is_contiguous(add) &&
                        g2->src[1]->ne[0] == s1->ne[0] && g2->src[1]->ne[1] == 1 && g2->src[1]->ne[2] == 1 && g2->src[1]->ne[3] == 1) {
                        bool plain = true;                  // nothing between the three nodes may be a view of the gathered tensors
                        for (int v = i + 1; v < k; ++v) plain = plain && (v == j || (node_at(v)->src[0] != n && node_at(v)->view_src != n && node_at(v)->src[0] != g2 && node_at(v)->view_src != g2));
                        // a handful of rows that the next launch normalizes: held, to be made inside that launch if it comes to one
                        int nx = k + 1;
                        while (node_at(nx) && (is_view_op(node_at(nx)->op) || ggml_is_empty(node_at(nx)))) ++nx;
                        if (plain && add->ne[1] <= 8 && add->ne[2] == 1 && add->ne[3] == 1 && (s0->type == GGML_TYPE_Q8_0 || s0->type == GGML_TYPE_Q5_0 || s0->type == GGML_TYPE_F16) &&
                            node_at(nx) && node_at(nx)->op == GGML_OP_NORM && node_at(nx)->src[0] == add) {
                            emb.active = true; emb.tok = s0; emb.tok_ids = s1; emb.pos = g2->src[0]; emb.pos_ids = g2->src[1]; emb.out = add;
                            note_write(add); fold_nodes(i, k - i + 1, add);
                            return k - i + 1;
                        }
                        if (plain) {
                            mi355x_tensor a = to_view(s0), ia = to_view(s1), b = to_view(g2->src[0]), ib = to_view(g2->src[1]), d = to_view(add);
                            int rc;
                            {
                                launch_scope ls(ctx, "get_rows_add", 3.0 * nbytes_of(add), 0.0);
                                rc = mi355x_get_rows_add(&a, &ia, &b, &ib, &d, ctx->stream);
                            }
                            if (rc != MI355X_ERR_UNSUPPORTED) { status = rc; note_write(add); fold_nodes(i, k - i + 1, add); return k - i + 1; }
                        }
                    }
                }
                mi355x_tensor a = to_view(s0), b = to_view(s1), d = to_view(n);
                launch_scope ls(ctx, "get_rows", 2.0 * nbytes_of(n), 0.0);
                status = mi355x_get_rows(&a, &b, &d, ctx->stream);
                return 1;
            }
            case GGML_OP_IM2COL: {
                const int32_t * p = n->op_params;   // s0, s1, p0, p1, d0, d1, is_2D (ggml/src/ggml.c:3849)
                mi355x_tensor a = to_view(s1), d = to_view(n);
                launch_scope ls(ctx, "im2col", nbytes_of(s1) + nbytes_of(n), 0.0);
                status = mi355x_im2col_1d(&a, &d, (int) s0->ne[0], p[0], p[2], p[4], ctx->stream);
                return 1;
            }
            case GGML_OP_FLASH_ATTN_EXT: {
                const ggml_tensor * k = n->src[1], * v = n->src[2], * m = n->src[3];
                const ggml_tensor * m16 = nullptr;          // the f16 copy this launch leaves behind
                if (m && m == cast_dst) { m16 = m; m = cast_src; cast_dst = cast_src = nullptr; }
                float scale; memcpy(&scale, n->op_params, sizeof(float));
                mi355x_tensor vq = to_view(s0), vk = to_view(k), vv = to_view(v), vm, vd = to_view(n);
                if (m) vm = to_view(m);
                if (s0->ne[1] <= 8) { few_query_attention = true; if (m) ctx->counters[9] = std::max<int64_t>(ctx->counters[9], k->ne[1]); }
                const double flops = 4.0 * s0->ne[1] * k->ne[1] * 64.0 * s0->ne[2] * s0->ne[3];
                const double bytes = (double) ggml_nelements(s0) * 4 + 2.0 * (double) k->ne[0] * k->ne[1] * k->ne[2] * k->ne[3] * 2 + nbytes_of(n);
                // the accumulation option, bit 0: more than 8 queries, bit 1: a decode step's few queries
                const bool f32_accum = s0->ne[1] > 8 ? (ctx->fa_accum & 1) != 0 : (ctx->fa_accum & 2) != 0;
                const int mode = ctx->exact || f32_accum ? MI355X_FA_F32 : ctx->fa_chain == 2 || (ctx->fa_chain == 1 && s0->ne[1] > 8) ? MI355X_FA_F16_PK : MI355X_FA_F16_SEQ;
                const char * name = mi355x_flash_attn_ext_kernel_name(&vq, &vk, mode);
                // the output projection that follows takes its Q8_0-rounded activations from the attention kernel itself
                const bool emits = !ctx->exact && (strncmp(name, "flash_attn.seq_tile", 19) == 0 || strcmp(name, "flash_attn.mfma_f32") == 0);
                const ggml_tensor * key = emits ? image_consumer(n, i + 1) : nullptr;
                // (a decode step's projection reads Q8_0 itself, written by the few-query kernel)
                int form = 1;
                if (!key && !ctx->exact && strncmp(name, "flash_attn.seq_row", 18) == 0 && (key = image_consumer(n, i + 1, true))) form = 2;
                const size_t image_bytes = form == 1 ? (size_t) ggml_nelements(n) * 2 : (size_t) ggml_nelements(n) / 32 * 40;
                if (key && !ctx->reserve_workspace(image_bytes + 256)) key = nullptr;
                // ... and only the image when the projection is the very next launch: the f32 rows would have no reader
                const bool image_only = key && form == 1 && ctx->dead_f32 && strncmp(name, "flash_attn.seq_tile", 19) == 0 && readers_are_the_next_products(key, i + 1);
                if (image_only) vd.data = nullptr;
                {
                    launch_scope ls(ctx, name, bytes - (image_only ? nbytes_of(n) : 0) + (key ? image_bytes : 0), flops);
                    const int flags = mode | (!key ? 0 : form == 1 ? MI355X_FA_EMIT_F16 : MI355X_FA_EMIT_Q8_0);
                    if (m16) {
                        mi355x_tensor vm16 = to_view(m16);
                        status = mi355x_flash_attn_ext_cast_mask(&vq, &vk, &vv, &vm, &vm16, &vd, scale, flags, key ? ctx->ws : nullptr, key ? ctx->ws_size : 0, ctx->stream);
                    } else
                    status = mi355x_flash_attn_ext(&vq, &vk, &vv, m ? &vm : nullptr, &vd, scale, flags,
                                                   key ? ctx->ws : nullptr, key ? ctx->ws_size : 0, ctx->stream);
                }
                if (key && status == MI355X_OK) { workspace_holds(key, ctx->ws_slot, form); if (image_only) { ctx->image_only = key; not_stored.push_back(n); } }
                return 1;
            }
            case GGML_OP_CONCAT: {
                mi355x_tensor a = to_view(s0), b = to_view(s1), d = to_view(n);
                launch_scope ls(ctx, "concat", 2.0 * nbytes_of(n), 0.0);
                status = mi355x_concat(&a, &b, &d, n->op_params[0], ctx->stream);
                return 1;
            }
            default:
                status = MI355X_ERR_UNSUPPORTED;
                return 1;
        }
    }
};

} // namespace

static mi355x_buffer_ctx * buffer_ctx_of(const ggml_tensor * t) {
    ggml_backend_buffer_t b = t->buffer ? t->buffer : t->view_src ? t->view_src->buffer : nullptr;
    return mi355x_buffer_is_ours(b) ? (mi355x_buffer_ctx *) b->context : nullptr;
}

// The nodes [i, i + used) went out as one launch.  What they read from outside the launch must hold a value; what they
// did not store holds none from now on; everything else they produced does.  False: a source was memory that an earlier
// launch had left unwritten — the graph reaches this backend in pieces, and the piece before had no sight of this reader.
static bool book_reads_and_writes(mi355x_backend_ctx * ctx, const ggml_cgraph * g, int i, int used, const std::vector<const ggml_tensor *> & not_stored,
                                  const std::vector<const ggml_tensor *> & from_image) {
    for (int k = i; k < i + used; ++k) {
        const ggml_tensor * n = g->nodes[k];
        if (is_view_op(n->op) || ggml_is_empty(n)) continue;
        for (int s = 0; s < GGML_MAX_SRC; ++s) {
            const ggml_tensor * src = n->src[s];
            if (!src || !src->data) continue;
            const ggml_tensor * root = src;
            while (root->view_src) root = root->view_src;
            bool inside = false;                          // produced by this very launch
            for (int j = i; j < k && !inside; ++j) inside = g->nodes[j] == src || g->nodes[j] == root;
            if (inside || (n->op == GGML_OP_CPY && s == 1)) continue;       // (a CPY's second source is its destination)
            if (n->op == GGML_OP_MUL_MAT && s == 1 && std::find(from_image.begin(), from_image.end(), src) != from_image.end()) continue;
            mi355x_buffer_ctx * b = buffer_ctx_of(src);
            char name[48];
            if (b && b->unwritten.stale(src->data, ggml_nbytes(src), name)) {
                GGML_LOG_ERROR("ggml-mi355x: %s (%s) reads %s, which lies in memory of %s: an earlier launch folded that result into its consumer "
                               "and never stored it. The graph reaches this backend in pieces; from now on this instance stores every result "
                               "(run the graph again)\n", ggml_op_desc(n), n->name, src->name, name);
                ctx->pieces = true;
                return false;
            }
        }
    }
    for (const ggml_tensor * t : not_stored) if (mi355x_buffer_ctx * b = buffer_ctx_of(t)) b->unwritten.add(t->data, ggml_nbytes(t), t->name);
    for (int k = i; k < i + used; ++k) {
        const ggml_tensor * n = g->nodes[k];
        if (is_view_op(n->op) || ggml_is_empty(n) || std::find(not_stored.begin(), not_stored.end(), n) != not_stored.end()) continue;
        const ggml_tensor * w = n->op == GGML_OP_CPY ? n->src[1] : n;
        if (mi355x_buffer_ctx * b = buffer_ctx_of(w)) b->unwritten.written(w->data, ggml_nbytes(w));
    }
    return true;
}

static int64_t host_now_ns() {
    return std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

enum ggml_status mi355x_graph_compute(mi355x_backend_ctx * ctx, struct ggml_cgraph * cgraph) {
    struct host_timer {                                    // host time spent planning and queueing, into counters[6]
        mi355x_backend_ctx * c; int64_t t0;
        ~host_timer() { c->counters[6] += host_now_ns() - t0; }
    } timer{ ctx, host_now_ns() };
    HIP_TRY(hipSetDevice(ctx->device), return GGML_STATUS_FAILED);
    ctx->ws_x = nullptr;   // tensors may have been rewritten between graphs
    ctx->image_only = nullptr;
    { std::lock_guard<std::mutex> lock(ctx->mirror_mutex); ctx->mirror.clear(); }      // this graph may write anywhere in the compute buffer
    ctx->counters[0] += 1;
    ctx->counters[1] += cgraph->n_nodes;
    for (int i = 0; i < cgraph->n_nodes; ++i) ctx->counters[2] += !(ggml_is_empty(cgraph->nodes[i]) || is_view_op(cgraph->nodes[i]->op));
    graph_runner run(ctx, cgraph);
    for (int i = 0; i < cgraph->n_nodes;) {
        int status = MI355X_OK;
        run.not_stored.clear(); run.from_image.clear();
        const int used = run.run_node(i, status);
        if (status != MI355X_OK) {
            const ggml_tensor * n = cgraph->nodes[i];
            GGML_LOG_ERROR("ggml-mi355x: %s (%s) failed: %s\n", ggml_op_desc(n), n->name, mi355x_status_string(status));
            return GGML_STATUS_FAILED;
        }
        if (ctx->check_reads && !book_reads_and_writes(ctx, cgraph, i, used, run.not_stored, run.from_image)) return GGML_STATUS_FAILED;
        i += used;
    }
    if (const int status = run.flush_norm()) {               // a LayerNorm at the very end of a graph
        GGML_LOG_ERROR("ggml-mi355x: trailing NORM failed: %s\n", mi355x_status_string(status));
        return GGML_STATUS_FAILED;
    }
    ctx->counters[8] += run.few_query_attention;
    ctx->mirror_outputs(cgraph);
    return GGML_STATUS_SUCCESS;
}
