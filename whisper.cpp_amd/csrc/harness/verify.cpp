// Per-node parity inside the real whisper graphs.
//
// whisper.cpp keeps its scheduler and backends private, so the harness hooks in one level lower: it loads the
// MI355X plugin by hand, replaces the device's init_backend with a wrapper that swaps the new backend's
// graph_compute for verifying_graph_compute below, and only then registers the plugin
// (ggml_backend_register, ggml/src/ggml-backend-impl.h:210).  verifying_graph_compute runs every node of every graph
// on the MI355X backend on its own (so nothing is fused), then copies that node's *device-side inputs* to the host,
// evaluates the same node with ggml's CPU backend, and compares the two results — the per-op NMSE of
// test-backend-ops, but on the operands the model really produces, layouts and aliasing included.
#include "verify.h"

#include <dlfcn.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <map>
#include <string>
#include <vector>

#include "ggml.h"
#include "ggml-alloc.h"
#include "ggml-backend.h"
#include "ggml-backend-impl.h"
#include "ggml-cpu.h"
#include "ggml-impl.h"

#include "synth_model.h"

namespace verify {

namespace {

struct node_stat { int64_t count = 0; double worst = 0, sum = 0; int64_t n_bad = 0; std::string worst_name; };

ggml_backend_t (*g_orig_init_backend)(ggml_backend_dev_t, const char *) = nullptr;
enum ggml_status (*g_orig_graph_compute)(ggml_backend_t, struct ggml_cgraph *) = nullptr;
ggml_backend_t g_cpu = nullptr;
std::map<std::string, node_stat> g_stats;
std::vector<std::string> g_bad_lines, g_exact_lines;
double g_tol = 5e-4;
bool   g_enabled = true;

bool is_view_op(enum ggml_op op) {
    return op == GGML_OP_NONE || op == GGML_OP_RESHAPE || op == GGML_OP_VIEW || op == GGML_OP_PERMUTE || op == GGML_OP_TRANSPOSE;
}

// 64-byte aligned byte buffer (ggml_backend_cpu_buffer_from_ptr insists on TENSOR_ALIGNMENT)
struct abuf {
    uint8_t * p = nullptr;
    size_t    n = 0;
    abuf() = default;
    explicit abuf(size_t size) { resize(size); }
    abuf(const abuf &) = delete;
    abuf & operator=(const abuf &) = delete;
    abuf(abuf && o) noexcept : p(o.p), n(o.n) { o.p = nullptr; o.n = 0; }
    ~abuf() { free(p); }
    void resize(size_t size) { free(p); p = nullptr; n = size; if (posix_memalign((void **) &p, 64, size ? size : 64) != 0) p = nullptr; else memset(p, 0, size ? size : 64); }
    uint8_t * data() { return p; }
    const uint8_t * data() const { return p; }
    size_t size() const { return n; }
};

// host copy of a (possibly strided) device tensor: same ne / nb over a private byte buffer
struct host_copy {
    ggml_tensor * t = nullptr;
    abuf bytes;
};

ggml_tensor * clone_meta(ggml_context * ctx, const ggml_tensor * s) {
    ggml_tensor * h = ggml_new_tensor(ctx, s->type, GGML_MAX_DIMS, s->ne);   // no_alloc context: metadata only
    for (int i = 0; i < GGML_MAX_DIMS; ++i) h->nb[i] = s->nb[i];
    memcpy(h->op_params, s->op_params, sizeof(h->op_params));
    ggml_set_name(h, s->name);
    return h;
}

double nmse_of(const ggml_tensor * t, const abuf & a, const abuf & b, int64_t * n_mismatch) {
    // walk logical elements (the tensors may be strided); candidate a vs reference b share the layout
    double num = 0, den = 0;
    *n_mismatch = 0;
    const size_t ts = ggml_type_size(t->type);
    for (int64_t i3 = 0; i3 < t->ne[3]; ++i3) for (int64_t i2 = 0; i2 < t->ne[2]; ++i2) for (int64_t i1 = 0; i1 < t->ne[1]; ++i1)
        for (int64_t i0 = 0; i0 < t->ne[0]; ++i0) {
            const size_t off = i0 * t->nb[0] + i1 * t->nb[1] + i2 * t->nb[2] + i3 * t->nb[3];
            float x, y;
            if (t->type == GGML_TYPE_F32) { memcpy(&x, a.data() + off, 4); memcpy(&y, b.data() + off, 4); }
            else if (t->type == GGML_TYPE_F16) { uint16_t hx, hy; memcpy(&hx, a.data() + off, 2); memcpy(&hy, b.data() + off, 2); x = synth::f16_to_f32(hx); y = synth::f16_to_f32(hy); }
            else { x = memcmp(a.data() + off, b.data() + off, ts) == 0 ? 0.0f : 1.0f; y = 0.0f; if (x != 0.0f) ++*n_mismatch; continue; }
            if (!std::isfinite(x) || !std::isfinite(y)) { if (!((std::isnan(x) && std::isnan(y)) || x == y)) ++*n_mismatch; continue; }
            const double d = (double) x - y; num += d * d; den += (double) y * y;
        }
    return den > 0 ? num / den : (num > 0 ? INFINITY : 0.0);
}

// softmax(scale * q.k + mask) @ v in double precision from the snapshotted operands (q rounded to f16 as both backends do):
// tells which of the two backends is the one that is off when they disagree
void exact_flash_attn(const ggml_tensor * n, const ggml_tensor * q, const ggml_tensor * k, const ggml_tensor * v, const ggml_tensor * m,
                      std::vector<double> & out) {
    float scale; memcpy(&scale, n->op_params, sizeof(float));
    const int64_t D = q->ne[0], N = q->ne[1], H = q->ne[2], KV = k->ne[1];
    out.assign((size_t)(D * H * N), 0.0);
    std::vector<double> s((size_t) KV);
    for (int64_t h = 0; h < H; ++h) for (int64_t i = 0; i < N; ++i) {
        const float * qp = (const float *)((const char *) q->data + i * q->nb[1] + h * q->nb[2]);
        const int64_t hk = h / (H / k->ne[2]), hv = h / (H / v->ne[2]);
        double mx = -INFINITY;
        for (int64_t c = 0; c < KV; ++c) {
            const float mv = m ? synth::f16_to_f32(*(const uint16_t *)((const char *) m->data + i * m->nb[1] + c * 2)) : 0.0f;
            if (mv == -INFINITY) { s[(size_t) c] = -INFINITY; continue; }
            const uint16_t * kp = (const uint16_t *)((const char *) k->data + c * k->nb[1] + hk * k->nb[2]);
            double a = 0;
            for (int64_t e = 0; e < D; ++e) a += (double) synth::f16_to_f32(synth::f32_to_f16(qp[e])) * synth::f16_to_f32(kp[e]);
            s[(size_t) c] = a * scale + mv; mx = fmax(mx, s[(size_t) c]);
        }
        double S = 0;
        for (int64_t c = 0; c < KV; ++c) { s[(size_t) c] = s[(size_t) c] == -INFINITY ? 0.0 : exp(s[(size_t) c] - mx); S += s[(size_t) c]; }
        for (int64_t c = 0; c < KV; ++c) {
            if (s[(size_t) c] == 0.0) continue;
            const uint16_t * vp = (const uint16_t *)((const char *) v->data + c * v->nb[1] + hv * v->nb[2]);
            for (int64_t e = 0; e < D; ++e) out[(size_t)((i * H + h) * D + e)] += s[(size_t) c] * synth::f16_to_f32(vp[e]);
        }
        for (int64_t e = 0; e < D; ++e) out[(size_t)((i * H + h) * D + e)] /= S;
    }
}

double nmse_vs_exact(const abuf & got, const std::vector<double> & exact) {
    double num = 0, den = 0;
    const float * g = (const float *) got.data();
    for (size_t i = 0; i < exact.size(); ++i) { const double d = g[i] - exact[i]; num += d * d; den += exact[i] * exact[i]; }
    return den > 0 ? num / den : 0;
}

// Inputs are snapshotted before the device runs the node (an in-place node overwrites one of them), the device
// result is read after.
struct pending_node {
    ggml_context * ctx = nullptr;
    ggml_tensor *  n   = nullptr;
    ggml_tensor *  hn  = nullptr;
    std::vector<host_copy> srcs;
};

pending_node snapshot_inputs(ggml_tensor * n) {
    pending_node p;
    ggml_init_params ip = { ggml_tensor_overhead() * 16 + ggml_graph_overhead_custom(8, false), nullptr, true };
    p.ctx = ggml_init(ip);
    p.n = n;
    p.srcs.resize(GGML_MAX_SRC);
    p.hn = clone_meta(p.ctx, n);
    p.hn->op = n->op;
    p.hn->flags = n->flags;
    for (int s = 0; s < GGML_MAX_SRC; ++s) {
        if (!n->src[s]) continue;
        p.srcs[s].t = clone_meta(p.ctx, n->src[s]);
        p.srcs[s].bytes.resize(ggml_nbytes(n->src[s]));
        ggml_backend_tensor_get(n->src[s], p.srcs[s].bytes.data(), 0, p.srcs[s].bytes.size());
        p.srcs[s].t->data = p.srcs[s].bytes.data();
        p.hn->src[s] = p.srcs[s].t;
    }
    return p;
}

void verify_node(pending_node & p) {
    ggml_tensor * n = p.n, * hn = p.hn;
    std::vector<host_copy> & srcs = p.srcs;
    // the tensor that receives the result: for CPY it is src[1] (the node is a view of it)
    const ggml_tensor * dev_out = n->op == GGML_OP_CPY ? n->src[1] : n;
    abuf ref(ggml_nbytes(dev_out)), got(ggml_nbytes(dev_out));
    ggml_backend_tensor_get(dev_out, got.data(), 0, got.size());
    // CPY writes every element of its destination view, so the snapshot of src[1] is a valid canvas
    hn->data = n->op == GGML_OP_CPY ? (void *) srcs[1].bytes.data() : (void *) ref.data();
    ggml_backend_buffer_t wrap_out = ggml_backend_cpu_buffer_from_ptr(hn->data, n->op == GGML_OP_CPY ? srcs[1].bytes.size() : ref.size());
    hn->buffer = wrap_out;
    std::vector<ggml_backend_buffer_t> wraps;
    for (int s = 0; s < GGML_MAX_SRC; ++s) if (srcs[s].t) {
        ggml_backend_buffer_t w = (n->op == GGML_OP_CPY && s == 1) ? wrap_out : ggml_backend_cpu_buffer_from_ptr(srcs[s].bytes.data(), srcs[s].bytes.size());
        srcs[s].t->buffer = w;
        if (w != wrap_out) wraps.push_back(w);
    }
    ggml_cgraph * gf = ggml_new_graph_custom(p.ctx, 8, false);
    ggml_build_forward_expand(gf, hn);
    const bool ok = ggml_backend_graph_compute(g_cpu, gf) == GGML_STATUS_SUCCESS;
    const abuf & refbytes = n->op == GGML_OP_CPY ? srcs[1].bytes : ref;

    int64_t mism = 0;
    const double nmse = ok ? nmse_of(dev_out, got, refbytes, &mism) : INFINITY;
    std::string key = ggml_op_desc(n);
    if (n->op == GGML_OP_MUL_MAT) key += std::string("(") + ggml_type_name(n->src[0]->type) + (n->ne[1] <= 8 ? ",gemv)" : ",gemm)");
    node_stat & st = g_stats[key];
    st.count++; st.sum += std::isfinite(nmse) ? nmse : 0;
    if (st.worst_name.empty() || nmse > st.worst) { st.worst = nmse; st.worst_name = n->name; }
    if (!(nmse <= g_tol) || mism) {
        st.n_bad++;
        if (g_bad_lines.size() < 40) {
            char line[512];
            snprintf(line, sizeof(line), "{\"bad_node\": \"%s\", \"op\": \"%s\", \"nmse\": %.3e, \"mismatch\": %lld, \"ne\": [%lld, %lld, %lld, %lld]}",
                     n->name, key.c_str(), nmse, (long long) mism, (long long) n->ne[0], (long long) n->ne[1], (long long) n->ne[2], (long long) n->ne[3]);
            g_bad_lines.push_back(line);
        }
    }
    if (n->op == GGML_OP_FLASH_ATTN_EXT && n->ne[3] == 1 && g_exact_lines.size() < 24) {
        std::vector<double> exact;
        exact_flash_attn(n, srcs[0].t, srcs[1].t, srcs[2].t, srcs[3].t, exact);
        char line[512];
        snprintf(line, sizeof(line), "{\"flash_attn_vs_exact_f64\": \"%s\", \"n\": %lld, \"kv\": %lld, \"mi355x_nmse\": %.3e, \"cpu_nmse\": %.3e, \"mi355x_vs_cpu_nmse\": %.3e}",
                 n->name, (long long) n->ne[2], (long long) n->src[1]->ne[1], nmse_vs_exact(got, exact), nmse_vs_exact(ref, exact), nmse);
        g_exact_lines.push_back(line);
    }
    for (ggml_backend_buffer_t w : wraps) ggml_backend_buffer_free(w);
    ggml_backend_buffer_free(wrap_out);
    ggml_free(p.ctx);
}

enum ggml_status verifying_graph_compute(ggml_backend_t backend, struct ggml_cgraph * cgraph) {
    if (!g_enabled) return g_orig_graph_compute(backend, cgraph);
    for (int i = 0; i < cgraph->n_nodes; ++i) {
        ggml_tensor * n = cgraph->nodes[i];
        if (ggml_is_empty(n) || is_view_op(n->op)) continue;
        ggml_backend_synchronize(backend);
        pending_node p = snapshot_inputs(n);
        struct ggml_cgraph one = ggml_graph_view(cgraph, i, i + 1);
        const enum ggml_status st = g_orig_graph_compute(backend, &one);
        if (st != GGML_STATUS_SUCCESS) { ggml_free(p.ctx); return st; }
        ggml_backend_synchronize(backend);
        verify_node(p);
    }
    return GGML_STATUS_SUCCESS;
}

ggml_backend_t hooked_init_backend(ggml_backend_dev_t dev, const char * params) {
    ggml_backend_t b = g_orig_init_backend(dev, params);
    if (b) {
        g_orig_graph_compute = b->iface.graph_compute;
        b->iface.graph_compute = verifying_graph_compute;
    }
    return b;
}

} // namespace

ggml_backend_reg_t load_plugin_hooked(const std::string & path) {
    void * h = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
    if (!h) { fprintf(stderr, "verify: dlopen %s: %s\n", path.c_str(), dlerror()); return nullptr; }
    auto score = (int (*)(void)) dlsym(h, "ggml_backend_score");
    auto init  = (ggml_backend_reg_t (*)(void)) dlsym(h, "ggml_backend_init");
    if (!init || (score && score() == 0)) return nullptr;
    ggml_backend_reg_t reg = init();
    if (!reg || reg->api_version != GGML_BACKEND_API_VERSION || ggml_backend_reg_dev_count(reg) == 0) return nullptr;
    ggml_backend_dev_t dev = ggml_backend_reg_dev_get(reg, 0);
    g_orig_init_backend = dev->iface.init_backend;
    dev->iface.init_backend = hooked_init_backend;
    g_cpu = ggml_backend_cpu_init();
    ggml_backend_register(reg);
    return reg;
}

void set_threads(int n) { if (g_cpu) ggml_backend_cpu_set_n_threads(g_cpu, n); }
void set_enabled(bool on) { g_enabled = on; }
void set_tolerance(double tol) { g_tol = tol; }

int report(const char * phase) {
    int n_bad = 0;
    for (const std::string & l : g_bad_lines) printf("%s\n", l.c_str());
    for (const std::string & l : g_exact_lines) printf("%s\n", l.c_str());
    for (auto & kv : g_stats) {
        printf("{\"phase\": \"%s\", \"op\": \"%s\", \"nodes\": %lld, \"worst_nmse\": %.3e, \"mean_nmse\": %.3e, \"worst_node\": \"%s\", \"over_tol\": %lld, \"tol\": %.1e}\n",
               phase, kv.first.c_str(), (long long) kv.second.count, kv.second.worst, kv.second.sum / std::max<int64_t>(1, kv.second.count),
               kv.second.worst_name.c_str(), (long long) kv.second.n_bad, g_tol);
        n_bad += (int) kv.second.n_bad;
    }
    g_stats.clear(); g_bad_lines.clear(); g_exact_lines.clear();
    return n_bad;
}

} // namespace verify
