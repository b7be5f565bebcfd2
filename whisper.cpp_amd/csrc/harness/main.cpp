// mi355x-harness: drives the unmodified whisper.cpp host libraries with the MI355X backend plugged in
// through ggml_backend_load(), next to ggml's own CPU backend on the same inputs.  Every subcommand prints
// one JSON object per line on stdout; diagnostics go to stderr.
//
//   info                                      devices, features, supports_op table
//   gen    --arch A --ftype T --out F         write a synthetic model file
//   selftest                                  the writer's quantizers / f16 conversion vs the reference's, byte for byte
//   ops    [--filter S] [--quick] [--threads N] [--reps R] [--cpu-only]
//                                             per-op parity (NMSE / bit-exactness) and timing, CPU vs MI355X
//   model  --model F [--steps 32] [--batch B] [--kv-to N] [--seed S] [--threads N]
//                                             whole-model parity: logits NMSE and greedy ids, teacher-forced; one split per graph
//   full   --model F [--beam 1|5] [--max-tokens 24] [--seconds 30] [--threads N] [--dtw] [--processors N] [--gpu-mel]
//                                             whisper_full() end to end (PCM -> mel -> encode -> search) on both backends
//   mel    --model F [--seconds 30] [--reps 20] [--threads N]
//                                             the log-mel front end: device path through the plugin vs whisper_pcm_to_mel
//   verify --model F [--steps 3] [--threads N]
//                                             per-node parity inside the real whisper graphs (unfused), CPU vs MI355X
//   download                                  the pinned host mirror of results the host reads back, and the pinned host buffer type
//   bench  --model F --what encoder|decoder|whisper-bench --backend gpu|cpu [--threads N] [--reps R] [--profile]
//                                             timings with the whisper-bench protocol (examples/bench/bench.cpp:108-138)
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <map>
#include <string>
#include <thread>
#include <vector>

#include "ggml.h"
#include "ggml-alloc.h"
#include "ggml-backend.h"
#include "ggml-cpu.h"
#include "ggml-impl.h"
#include "whisper.h"

#include "ggml-mi355x.h"
#include "op_cases.h"
#include "synth_model.h"
#include "verify.h"
#include "../backend/range_set.h"

// ---------------------------------------------------------------------------------------------------------------
// small utilities
// ---------------------------------------------------------------------------------------------------------------

static double now_ms() {
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

struct args {
    std::map<std::string, std::string> kv;
    bool has(const std::string & k) const { return kv.count(k) != 0; }
    std::string str(const std::string & k, const std::string & d = "") const { auto it = kv.find(k); return it == kv.end() ? d : it->second; }
    int num(const std::string & k, int d) const { auto it = kv.find(k); return it == kv.end() ? d : atoi(it->second.c_str()); }
};

static args parse_args(int argc, char ** argv, int first) {
    args a;
    for (int i = first; i < argc; ++i) {
        std::string k = argv[i];
        if (k.rfind("--", 0) != 0) continue;
        k = k.substr(2);
        if (i + 1 < argc && strncmp(argv[i + 1], "--", 2) != 0) a.kv[k] = argv[++i];
        else a.kv[k] = "1";
    }
    return a;
}

// The scheduler's own account of how it split a graph (GGML_SCHED_DEBUG=1: ggml_backend_sched_print_assignments,
// ggml/src/ggml-backend.cpp:791-802, one "## SPLIT #i: <backend> # n inputs" line per split), counted while enabled.
static bool g_count_splits = false;
static int  g_splits_total = 0, g_splits_not_on_device = 0;

static void quiet_log(enum ggml_log_level level, const char * text, void *) {
    static const bool verbose = getenv("GGML_MI355X_DEBUG") != nullptr;
    if (g_count_splits) {
        if (const char * p = strstr(text, "## SPLIT #")) {
            ++g_splits_total;
            const char * colon = strchr(p, ':');
            if (!colon || strncmp(colon + 2, GGML_MI355X_NAME, strlen(GGML_MI355X_NAME)) != 0) ++g_splits_not_on_device;
        }
    }
    if (level == GGML_LOG_LEVEL_ERROR || level == GGML_LOG_LEVEL_WARN || (verbose && strncmp(text, "ggml-mi355x", 11) == 0)) fputs(text, stderr);
}

static std::string self_dir() {
    char buf[4096];
    ssize_t n = readlink("/proc/self/exe", buf, sizeof(buf) - 1);
    if (n <= 0) return ".";
    buf[n] = 0;
    std::string s(buf);
    return s.substr(0, s.find_last_of('/'));
}

// the plugin sits next to this binary
static ggml_backend_reg_t load_plugin(bool required) {
    const char * env = getenv("GGML_MI355X_PLUGIN");
    const std::string path = env ? env : self_dir() + "/libggml-mi355x.so";
    ggml_backend_reg_t reg = ggml_backend_load(path.c_str());
    if (!reg && required) fprintf(stderr, "harness: could not load %s (no gfx950 device, or the library is missing)\n", path.c_str());
    return reg;
}

static ggml_backend_t init_gpu_backend(ggml_backend_reg_t reg) {
    if (!reg || ggml_backend_reg_dev_count(reg) == 0) return nullptr;
    return ggml_backend_dev_init(ggml_backend_reg_dev_get(reg, 0), nullptr);
}

static int default_threads() {
    const char * e = getenv("OMP_NUM_THREADS");
    if (e && atoi(e) > 0) return atoi(e);
    int n = (int) std::thread::hardware_concurrency();
    return n > 0 ? std::min(n, 16) : 4;
}

static std::string json_escape(const std::string & s) {
    std::string o;
    for (char c : s) { if (c == '"' || c == '\\') o += '\\'; o += c; }
    return o;
}

// ---------------------------------------------------------------------------------------------------------------
// comparing two result buffers
// ---------------------------------------------------------------------------------------------------------------

struct cmp_result { double nmse, max_abs; bool bit_exact; int64_t n, n_nonfinite_mismatch; };

static std::vector<float> to_f32(const std::vector<uint8_t> & raw, ggml_type type, int64_t n) {
    std::vector<float> out((size_t) n);
    if (type == GGML_TYPE_F32) memcpy(out.data(), raw.data(), (size_t) n * 4);
    else if (type == GGML_TYPE_F16) {
        const uint16_t * h = (const uint16_t *) raw.data();
        for (int64_t i = 0; i < n; ++i) out[(size_t) i] = synth::f16_to_f32(h[i]);
    } else out.assign((size_t) n, 0.0f);
    return out;
}

static cmp_result compare(const std::vector<uint8_t> & a, const std::vector<uint8_t> & b, ggml_type type, int64_t n) {
    cmp_result r{};
    r.n = n;
    r.bit_exact = a.size() == b.size() && memcmp(a.data(), b.data(), a.size()) == 0;
    const std::vector<float> fa = to_f32(a, type, n), fb = to_f32(b, type, n);
    double num = 0, den = 0, mx = 0;
    for (int64_t i = 0; i < n; ++i) {
        const float x = fa[(size_t) i], y = fb[(size_t) i];    // x: candidate, y: reference
        if (!std::isfinite(x) || !std::isfinite(y)) {
            if (!((std::isnan(x) && std::isnan(y)) || x == y)) r.n_nonfinite_mismatch++;
            continue;
        }
        const double d = (double) x - y;
        num += d * d; den += (double) y * y; mx = std::max(mx, fabs(d));
    }
    r.nmse = den > 0 ? num / den : (num > 0 ? INFINITY : 0.0);
    r.max_abs = mx;
    return r;
}

// ---------------------------------------------------------------------------------------------------------------
// ops: one case on one backend
// ---------------------------------------------------------------------------------------------------------------

static uint64_t name_seed(const std::string & s) {
    uint64_t h = 1469598103934665603ull;
    for (char c : s) { h ^= (uint8_t) c; h *= 1099511628211ull; }
    return h;
}

static void fill_input(const ops::input & in, const std::string & case_name) {
    ggml_tensor * t = in.t;
    const int64_t n = ggml_nelements(t);
    const uint64_t seed = name_seed(case_name + "/" + t->name);
    std::vector<uint8_t> data;
    switch (in.kind) {
        case ops::FILL_NORMAL:
            data = synth::random_tensor((int) t->type, n, seed, in.scale, in.offset);
            break;
        case ops::FILL_ZERO_TAIL: {
            data = synth::random_tensor((int) t->type, n, seed, in.scale, in.offset);
            const size_t keep = (size_t)(in.range * in.rows) * ggml_type_size(t->type);
            if (keep < data.size()) memset(data.data() + keep, 0, data.size() - keep);
        } break;
        case ops::FILL_IDS: {
            data.resize((size_t) n * 4);
            int32_t * ids = (int32_t *) data.data();
            const bool all = n == in.range;     // "every row once", in a shuffled-looking but fixed order
            for (int64_t i = 0; i < n; ++i) ids[i] = all ? (int32_t)((i * 2654435761ull + 17) % (uint64_t) in.range)
                                                         : (int32_t)((seed + (uint64_t) i * 7919ull) % (uint64_t) in.range);
        } break;
        case ops::FILL_MASK: {
            const int64_t kv = t->ne[0], nrow = t->ne[1];
            std::vector<float> m((size_t) n, -INFINITY);
            for (int64_t r = 0; r < std::min(nrow, in.rows); ++r)
                for (int64_t k = 0; k < kv; ++k) {
                    bool ok;
                    if (in.range == 2) ok = k <= kv - in.rows + r;                         // causal
                    else               ok = k < (kv + 1) / 2 || (k % in.rows) == r;        // beam-style cell ownership
                    if (ok) m[(size_t)(r * kv + k)] = 0.0f;
                }
            if (t->type == GGML_TYPE_F32) { data.resize((size_t) n * 4); memcpy(data.data(), m.data(), data.size()); }
            else { data.resize((size_t) n * 2); uint16_t * h = (uint16_t *) data.data(); for (int64_t i = 0; i < n; ++i) h[i] = synth::f32_to_f16(m[(size_t) i]); }
        } break;
    }
    ggml_backend_tensor_set(t, data.data(), 0, ggml_nbytes(t));
}

struct run_out { std::vector<uint8_t> data; ggml_type type; int64_t n; double ms; bool ok; };

static run_out run_case(const ops::op_case & c, ggml_backend_t backend, int reps) {
    run_out out{};
    ggml_init_params ip = { ggml_tensor_overhead() * 256 + ggml_graph_overhead(), nullptr, true };
    ggml_context * ctx = ggml_init(ip);
    ops::built b = c.build(ctx);
    ggml_cgraph * gf = ggml_new_graph(ctx);
    for (ggml_tensor * r : b.roots) ggml_build_forward_expand(gf, r);
    ggml_backend_buffer_t buf = ggml_backend_alloc_ctx_tensors(ctx, backend);
    if (!buf) { fprintf(stderr, "harness: allocation failed for %s\n", c.name.c_str()); ggml_free(ctx); return out; }
    for (const ops::input & in : b.inputs) fill_input(in, c.name);
    bool ok = ggml_backend_graph_compute(backend, gf) == GGML_STATUS_SUCCESS;      // first run doubles as warm-up
    out.type = b.result->type; out.n = ggml_nelements(b.result);
    out.data.resize(ggml_nbytes(b.result));
    if (ok) ggml_backend_tensor_get(b.result, out.data.data(), 0, out.data.size());
    double best = 1e30;
    const bool rerunnable = b.result->op != GGML_OP_NONE || true;   // inputs are never overwritten by these graphs' roots
    for (int r = 0; ok && rerunnable && r < reps; ++r) {
        const double t0 = now_ms();
        ok = ggml_backend_graph_compute(backend, gf) == GGML_STATUS_SUCCESS;
        best = std::min(best, now_ms() - t0);
    }
    out.ms = reps > 0 ? best : 0.0;
    out.ok = ok;
    ggml_backend_buffer_free(buf);
    ggml_free(ctx);
    return out;
}

static int cmd_ops(const args & a) {
    const bool cpu_only = a.has("cpu-only");
    ggml_backend_reg_t reg = cpu_only ? nullptr : load_plugin(true);
    ggml_backend_t gpu = init_gpu_backend(reg);
    if (!cpu_only && !gpu) { printf("{\"error\": \"no MI355X backend\"}\n"); return 2; }
    ggml_backend_t cpu = ggml_backend_cpu_init();
    const int threads = a.num("threads", default_threads());
    ggml_backend_cpu_set_n_threads(cpu, threads);
    const int reps = a.num("reps", 3);
    const std::string filter = a.str("filter");
    const bool quick = a.has("quick");
    int n_fail = 0, n_run = 0;
    for (const ops::op_case & c : ops::all_cases()) {
        if (!filter.empty() && c.name.find(filter) == std::string::npos) continue;
        if (quick && c.heavy) continue;
        fprintf(stderr, "case %s\n", c.name.c_str()); fflush(stderr);
        run_out rc = run_case(c, cpu, a.has("time-cpu") ? reps : 0);
        if (cpu_only) {
            printf("{\"case\": \"%s\", \"op\": \"%s\", \"cpu_ok\": %s, \"n\": %lld}\n", c.name.c_str(), c.op.c_str(), rc.ok ? "true" : "false", (long long) rc.n);
            ++n_run; continue;
        }
        run_out rg = run_case(c, gpu, reps);
        cmp_result r = compare(rg.data, rc.data, rc.type, rc.n);
        const bool pass = rg.ok && rc.ok && r.n_nonfinite_mismatch == 0 && (c.bit_exact ? r.bit_exact : r.nmse <= c.nmse_tol);
        if (!pass) ++n_fail;
        ++n_run;
        printf("{\"case\": \"%s\", \"op\": \"%s\", \"pass\": %s, \"nmse\": %.3e, \"max_abs\": %.3e, \"bit_exact\": %s, \"want_bit_exact\": %s, "
               "\"nmse_tol\": %.1e, \"nonfinite_mismatch\": %lld, \"n\": %lld, \"gpu_ms\": %.4f, \"cpu_ms\": %.4f, \"cpu_threads\": %d, "
               "\"flops\": %.0f, \"bytes\": %.0f}\n",
               c.name.c_str(), c.op.c_str(), pass ? "true" : "false", r.nmse, r.max_abs, r.bit_exact ? "true" : "false",
               c.bit_exact ? "true" : "false", c.nmse_tol, (long long) r.n_nonfinite_mismatch, (long long) r.n, rg.ms, rc.ms, threads, c.flops, c.bytes);
        fflush(stdout);
    }
    printf("{\"summary\": \"ops\", \"run\": %d, \"failed\": %d}\n", n_run, n_fail);
    if (gpu) ggml_backend_free(gpu);
    ggml_backend_free(cpu);
    return n_fail ? 1 : 0;
}

// ---------------------------------------------------------------------------------------------------------------
// pieces: graphs that reach the backend as ggml_graph_view slices, the way the scheduler hands over the splits of a graph
// (ggml/src/ggml-backend.cpp:1252, 1377-1440), and a reader of a result that is not the product next to its producer
// ---------------------------------------------------------------------------------------------------------------

namespace {
struct ln_products {
    ggml_context * ctx = nullptr;
    ggml_cgraph * gf = nullptr;
    ggml_backend_buffer_t buf = nullptr;
    ggml_tensor * ln = nullptr, * y1 = nullptr, * y2 = nullptr, * y3 = nullptr;
    int n_first = 0;                    // nodes up to and including y1 (and y2 when present)
};
// ln = LayerNorm(x) * w + b;  y1 = W1 ln;  [y2 = W2 y1;]  y3 = W3 ln  — quantized weights, `cols` columns
ln_products build_ln_products(ggml_backend_t backend, bool with_y2, int64_t cols) {
    ln_products p;
    ggml_init_params ip = { ggml_tensor_overhead() * 64 + ggml_graph_overhead(), nullptr, true };
    p.ctx = ggml_init(ip);
    const int64_t K = 256;
    ggml_tensor * x  = ggml_new_tensor_2d(p.ctx, GGML_TYPE_F32, K, cols);  ggml_set_name(x, "x");
    ggml_tensor * w  = ggml_new_tensor_1d(p.ctx, GGML_TYPE_F32, K);        ggml_set_name(w, "ln_w");
    ggml_tensor * b  = ggml_new_tensor_1d(p.ctx, GGML_TYPE_F32, K);        ggml_set_name(b, "ln_b");
    ggml_tensor * W1 = ggml_new_tensor_2d(p.ctx, GGML_TYPE_Q8_0, K, K);    ggml_set_name(W1, "W1");
    ggml_tensor * W2 = ggml_new_tensor_2d(p.ctx, GGML_TYPE_Q8_0, K, K);    ggml_set_name(W2, "W2");
    ggml_tensor * W3 = ggml_new_tensor_2d(p.ctx, GGML_TYPE_Q8_0, K, 320);  ggml_set_name(W3, "W3");
    p.ln = ggml_add(p.ctx, ggml_mul(p.ctx, ggml_norm(p.ctx, x, 1e-5f), w), b); ggml_set_name(p.ln, "ln");
    p.y1 = ggml_mul_mat(p.ctx, W1, p.ln); ggml_set_name(p.y1, "y1");
    if (with_y2) { p.y2 = ggml_mul_mat(p.ctx, W2, p.y1); ggml_set_name(p.y2, "y2"); }
    p.y3 = ggml_mul_mat(p.ctx, W3, p.ln); ggml_set_name(p.y3, "y3");
    p.gf = ggml_new_graph(p.ctx);
    ggml_build_forward_expand(p.gf, with_y2 ? p.y2 : p.y1);
    p.n_first = ggml_graph_n_nodes(p.gf);
    ggml_build_forward_expand(p.gf, p.y3);
    p.buf = ggml_backend_alloc_ctx_tensors(p.ctx, backend);
    const std::string tag = "pieces";
    for (const ops::input & in : { ops::input{ x, ops::FILL_NORMAL, 1.0f, 0.3f }, ops::input{ w, ops::FILL_NORMAL, 0.1f, 1.0f }, ops::input{ b, ops::FILL_NORMAL, 0.1f },
                                   ops::input{ W1, ops::FILL_NORMAL, 0.05f }, ops::input{ W2, ops::FILL_NORMAL, 0.05f }, ops::input{ W3, ops::FILL_NORMAL, 0.05f } })
        fill_input(in, tag);
    return p;
}
std::vector<uint8_t> fetch(ggml_tensor * t) { std::vector<uint8_t> v(ggml_nbytes(t)); ggml_backend_tensor_get(t, v.data(), 0, v.size()); return v; }
void release(ln_products & p) { ggml_backend_buffer_free(p.buf); ggml_free(p.ctx); }
}

static int cmd_pieces(const args & a) {
    ggml_backend_reg_t reg = load_plugin(true);
    ggml_backend_t gpu = init_gpu_backend(reg);
    if (!gpu) { printf("{\"error\": \"no MI355X backend\"}\n"); return 2; }
    ggml_backend_t cpu = ggml_backend_cpu_init();
    ggml_backend_cpu_set_n_threads(cpu, a.num("threads", default_threads()));
    int bad = 0;
    for (int64_t cols : { (int64_t) 64, (int64_t) 5 }) {
        // (1) one graph: the LayerNorm's result is read by the product next to it and by a later one, with a product in between
        //     whose own result goes on as an activation image — the later one must still find its activations
        {
            ln_products pc = build_ln_products(cpu, true, cols), pg = build_ln_products(gpu, true, cols);
            const bool okc = ggml_backend_graph_compute(cpu, pc.gf) == GGML_STATUS_SUCCESS, okg = ggml_backend_graph_compute(gpu, pg.gf) == GGML_STATUS_SUCCESS;
            const cmp_result r2 = compare(fetch(pg.y2), fetch(pc.y2), GGML_TYPE_F32, ggml_nelements(pc.y2));
            const cmp_result r3 = compare(fetch(pg.y3), fetch(pc.y3), GGML_TYPE_F32, ggml_nelements(pc.y3));
            const bool pass = okc && okg && r2.nmse <= 5e-4 && r3.nmse <= 5e-4 && r2.n_nonfinite_mismatch == 0 && r3.n_nonfinite_mismatch == 0;
            bad += !pass;
            printf("{\"pieces\": \"late_reader_in_one_graph\", \"cols\": %lld, \"nmse_y2\": %.3e, \"nmse_y3\": %.3e, \"pass\": %s}\n", (long long) cols, r2.nmse, r3.nmse, pass ? "true" : "false");
            release(pc); release(pg);
        }
        // (2) the same two readers in two pieces: the first piece shows one reader of the LayerNorm's result, and with many
        //     columns the backend then keeps only the activation image.  The second piece must not read the memory that was
        //     never written: the graph fails, the instance switches to storing everything, and the repeat is correct.
        {
            ln_products pc = build_ln_products(cpu, false, cols), pg = build_ln_products(gpu, false, cols);
            const bool okc = ggml_backend_graph_compute(cpu, pc.gf) == GGML_STATUS_SUCCESS;
            ggml_cgraph first = ggml_graph_view(pg.gf, 0, pg.n_first), second = ggml_graph_view(pg.gf, pg.n_first, ggml_graph_n_nodes(pg.gf));
            const int s1 = (int) ggml_backend_graph_compute(gpu, &first), s2 = (int) ggml_backend_graph_compute(gpu, &second);
            // the LayerNorm's rows themselves: NaN patterns from a download of memory without a value, if it was refused
            const std::vector<uint8_t> ln_bytes = fetch(pg.ln);
            bool ln_poisoned = true;
            for (uint8_t v : ln_bytes) ln_poisoned = ln_poisoned && v == 0xff;
            const int t1 = (int) ggml_backend_graph_compute(gpu, &first), t2 = (int) ggml_backend_graph_compute(gpu, &second);
            const cmp_result r1 = compare(fetch(pg.y1), fetch(pc.y1), GGML_TYPE_F32, ggml_nelements(pc.y1));
            const cmp_result r3 = compare(fetch(pg.y3), fetch(pc.y3), GGML_TYPE_F32, ggml_nelements(pc.y3));
            const cmp_result rl = compare(fetch(pg.ln), fetch(pc.ln), GGML_TYPE_F32, ggml_nelements(pc.ln));
            // few columns: the decode-step kernels always store the LayerNorm's rows, so nothing is refused there
            const bool refused = s1 == GGML_STATUS_SUCCESS && s2 == GGML_STATUS_FAILED && ln_poisoned;
            const bool straight = s1 == GGML_STATUS_SUCCESS && s2 == GGML_STATUS_SUCCESS && !ln_poisoned;
            const bool pass = okc && (cols > 8 ? refused : straight) && t1 == GGML_STATUS_SUCCESS && t2 == GGML_STATUS_SUCCESS &&
                              r1.nmse <= 5e-4 && r3.nmse <= 5e-4 && rl.nmse <= 1e-6 && r3.n_nonfinite_mismatch == 0;
            bad += !pass;
            printf("{\"pieces\": \"late_reader_in_the_next_piece\", \"cols\": %lld, \"first_try\": [%d, %d], \"download_poisoned\": %s, \"second_try\": [%d, %d], "
                   "\"nmse_y1\": %.3e, \"nmse_y3\": %.3e, \"nmse_ln\": %.3e, \"pass\": %s}\n", (long long) cols, s1, s2, ln_poisoned ? "true" : "false", t1, t2,
                   r1.nmse, r3.nmse, rl.nmse, pass ? "true" : "false");
            release(pc); release(pg);
        }
        // the instance now stores everything; a fresh one for the next round
        ggml_backend_free(gpu);
        gpu = init_gpu_backend(reg);
    }
    printf("{\"summary\": \"pieces\", \"failed\": %d}\n", bad);
    ggml_backend_free(gpu); ggml_backend_free(cpu);
    return bad ? 1 : 0;
}

// ---------------------------------------------------------------------------------------------------------------
// info
// ---------------------------------------------------------------------------------------------------------------

static int cmd_info(const args &) {
    ggml_backend_reg_t reg = load_plugin(false);
    printf("{\"plugin_loaded\": %s, \"n_registered_devices\": %zu", reg ? "true" : "false", ggml_backend_dev_count());
    if (reg) {
        printf(", \"reg\": \"%s\", \"devices\": [", ggml_backend_reg_name(reg));
        for (size_t i = 0; i < ggml_backend_reg_dev_count(reg); ++i) {
            ggml_backend_dev_t dev = ggml_backend_reg_dev_get(reg, i);
            size_t fr = 0, tot = 0; ggml_backend_dev_memory(dev, &fr, &tot);
            printf("%s{\"name\": \"%s\", \"description\": \"%s\", \"type\": %d, \"free\": %zu, \"total\": %zu}", i ? ", " : "",
                   ggml_backend_dev_name(dev), json_escape(ggml_backend_dev_description(dev)).c_str(), (int) ggml_backend_dev_type(dev), fr, tot);
        }
        printf("]");
        auto feat = (ggml_backend_get_features_t) ggml_backend_reg_get_proc_address(reg, "ggml_backend_get_features");
        if (feat) {
            printf(", \"features\": {");
            bool first = true;
            for (ggml_backend_feature * f = feat(reg); f->name; ++f) { printf("%s\"%s\": \"%s\"", first ? "" : ", ", f->name, f->value); first = false; }
            printf("}");
        }
    }
    printf("}\n");
    return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// selftest: the synthetic-model writer's own quantizers and f16 conversion against the reference's (byte equality)
// ---------------------------------------------------------------------------------------------------------------

static int cmd_selftest(const args &) {
    { ggml_init_params ip = { 1024, nullptr, false }; ggml_free(ggml_init(ip)); }   // fills ggml's f16 -> f32 table
    const int64_t n = 32 * 4096;
    std::vector<float> x((size_t) n);
    for (int64_t i = 0; i < n; ++i) x[(size_t) i] = 0.02f * synth::normal_at(99, (uint64_t) i) * (i % 977 == 0 ? 40.0f : 1.0f);
    for (int64_t i = 0; i < 64; ++i) x[(size_t) i] = 0.0f;                       // all-zero blocks
    x[100] = 1e-9f; x[200] = -65504.0f; x[300] = 3.0e38f;                          // tiny, f16 max, beyond f16
    int bad = 0;
    for (int type : { (int) GGML_TYPE_Q5_0, (int) GGML_TYPE_Q8_0 }) {
        const size_t bytes = (size_t)(n / 32) * (type == GGML_TYPE_Q5_0 ? 22 : 34);
        std::vector<uint8_t> mine(bytes), ref(bytes);
        if (type == GGML_TYPE_Q5_0) synth::quantize_q5_0(x.data(), mine.data(), n); else synth::quantize_q8_0(x.data(), mine.data(), n);
        ggml_quantize_chunk((ggml_type) type, x.data(), ref.data(), 0, 1, n, nullptr);
        const bool same = memcmp(mine.data(), ref.data(), bytes) == 0;
        bad += !same;
        printf("{\"selftest\": \"quantize_%s_vs_ggml_quantize_chunk\", \"bytes\": %zu, \"identical\": %s}\n", ggml_type_name((ggml_type) type), bytes, same ? "true" : "false");
    }
    {
        int64_t diff = 0;
        for (uint32_t h = 0; h < 65536; ++h) {
            const float f = ggml_fp16_to_fp32((ggml_fp16_t) h), g = synth::f16_to_f32((uint16_t) h);
            if (memcmp(&f, &g, 4) != 0 && !(std::isnan(f) && std::isnan(g))) ++diff;
        }
        for (int64_t i = 0; i < n; ++i) {
            const float v = x[(size_t) i] * 1000.0f;
            if ((uint16_t) ggml_fp32_to_fp16(v) != synth::f32_to_f16(v)) ++diff;
        }
        bad += diff != 0;
        printf("{\"selftest\": \"f16_conversions_vs_ggml\", \"mismatches\": %lld}\n", (long long) diff);
    }
    {
        // the plugin's bookkeeping of device memory that holds no value (results folded into their consumer): add, trim,
        // split and lookup on plain addresses
        mi355x_range_set set;
        char * base = (char *) 0x10000;
        char name[48];
        int wrong = 0;
        wrong += set.stale(base, 100);                                            // empty set
        set.add(base + 100, 100, "a");                                              // [100, 200)
        set.add(base + 120, 30, "inside");                                          // already covered
        wrong += set.size() != 1;
        wrong += !set.stale(base + 150, 1, name) || strcmp(name, "a") != 0;
        wrong += set.stale(base, 100) || set.stale(base + 200, 50);                  // touching is not overlapping
        wrong += !set.stale(base + 50, 51) || !set.stale(base + 199, 10);
        set.written(base + 140, 20);                                                // a hole: [100, 140) and [160, 200)
        wrong += set.size() != 2 || set.stale(base + 140, 20) || !set.stale(base + 139, 1) || !set.stale(base + 160, 1);
        set.written(base + 90, 20);                                                 // trims the front: [110, 140)
        wrong += set.stale(base + 100, 10) || !set.stale(base + 110, 1);
        set.written(base + 190, 100);                                               // trims the back: [160, 190)
        wrong += set.stale(base + 190, 10) || !set.stale(base + 189, 1);
        set.add(base + 1000, 10, "b");
        set.written(base, 195);                                                     // covers both pieces of "a", leaves "b"
        wrong += set.size() != 1 || !set.stale(base + 1005, 1, name) || strcmp(name, "b") != 0 || set.stale(base + 100, 100);
        set.written(base + 1000, 10);
        wrong += set.size() != 0 || set.stale(base + 1000, 10);
        set.add(base, 10, "c"); set.clear();
        wrong += set.size() != 0;
        bad += wrong != 0;
        printf("{\"selftest\": \"unwritten_range_bookkeeping\", \"wrong\": %d}\n", wrong);
    }
    printf("{\"summary\": \"selftest\", \"failed\": %d}\n", bad);
    return bad ? 1 : 0;
}

// ---------------------------------------------------------------------------------------------------------------
// gen
// ---------------------------------------------------------------------------------------------------------------

static int cmd_gen(const args & a) {
    const synth::arch * arch = synth::find_arch(a.str("arch", "base"));
    const int ftype = synth::ftype_from_name(a.str("ftype", "q5_0"));
    const std::string out = a.str("out");
    if (!arch || ftype < 0 || out.empty()) { fprintf(stderr, "usage: gen --arch micro|tiny|base|large-v3|large-v3-turbo --ftype f16|q8_0|q5_0 --out FILE [--seed N]\n"); return 2; }
    const double t0 = now_ms();
    const bool ok = synth::write_model(out, *arch, ftype, (uint64_t) a.num("seed", 1234));
    printf("{\"gen\": \"%s\", \"arch\": \"%s\", \"ftype\": \"%s\", \"ok\": %s, \"ms\": %.1f}\n", out.c_str(), arch->name, a.str("ftype", "q5_0").c_str(), ok ? "true" : "false", now_ms() - t0);
    return ok ? 0 : 1;
}

// ---------------------------------------------------------------------------------------------------------------
// whisper contexts
// ---------------------------------------------------------------------------------------------------------------

static bool g_flash_attn = true;   // --no-flash-attn: whisper.cpp's default graphs (KQ MUL_MAT, SOFT_MAX, KQV MUL_MAT; src/whisper.cpp:3620)

static int  g_processors = 1;
static bool g_gpu_mel = false; // --gpu-mel: the GPU run takes its log-mel from the plugin ("ggml_backend_mi355x_log_mel") instead of whisper_pcm_to_mel
static ggml_backend_mi355x_log_mel_t g_log_mel = nullptr;
static std::string g_model_path;
static double g_mel_ms = -1.0;
static bool g_dtw = false;     // --dtw: token-level timestamps from the cross-attention of the top alignment heads (needs --no-flash-attn)

static whisper_context * open_model(const std::string & path, bool use_gpu) {
    whisper_context_params cp = whisper_context_default_params();
    cp.use_gpu    = use_gpu;
    cp.flash_attn = g_flash_attn;
    if (g_dtw) {
        cp.dtw_token_timestamps = true;
        cp.dtw_aheads_preset    = WHISPER_AHEADS_N_TOP_MOST;
        cp.dtw_n_top            = 2;
    }
    return whisper_init_from_file_with_params(path.c_str(), cp);
}

static int argmax(const float * v, int n, float * margin) {
    int best = 0; float b1 = -INFINITY, b2 = -INFINITY;
    for (int i = 0; i < n; ++i) {
        if (v[i] > b1) { b2 = b1; b1 = v[i]; best = i; } else if (v[i] > b2) b2 = v[i];
    }
    if (margin) *margin = b1 - b2;
    return best;
}

// whole-model parity: both contexts encode the same synthetic mel, then decode the same token history step by step
// (teacher-forced with the CPU's greedy choices so that one flipped argmax cannot cascade); per step compares the
// logits of every row.  --batch B feeds B tokens per step after the prompt (the shape of a B-beam search step: B rows
// through every product, B queries per attention node) — the B greedy ids of the step before — and --kv-to N keeps
// stepping until the self-attention cache holds N positions (448 = n_text_ctx fills it).
//
// Also checks that nothing left the device: the scheduler reports its splits (GGML_SCHED_DEBUG=1) and the plugin counts
// the graphs and nodes it was handed; every graph whisper computes must be one split on the MI355X device.
static int cmd_model(const args & a) {
    const std::string path = a.str("model");
    const int threads = a.num("threads", default_threads()), batch = std::max(1, a.num("batch", 1));
    if (path.empty()) { fprintf(stderr, "usage: model --model FILE [--steps N] [--batch B] [--kv-to N] [--seed S]\n"); return 2; }
    ggml_backend_reg_t reg = load_plugin(true);
    if (!reg) { printf("{\"error\": \"no MI355X backend\"}\n"); return 2; }
    auto get_counters = (ggml_backend_mi355x_get_counters_t) ggml_backend_reg_get_proc_address(reg, "ggml_backend_mi355x_get_counters");
    setenv("GGML_SCHED_DEBUG", "1", 1);                 // read when a scheduler is created (ggml/src/ggml-backend.cpp:1462)
    whisper_context * gpu = open_model(path, true);
    unsetenv("GGML_SCHED_DEBUG");
    whisper_context * cpu = open_model(path, false);
    if (!gpu || !cpu || !get_counters) { printf("{\"error\": \"model load failed\"}\n"); return 2; }
    const int n_mels = whisper_model_n_mels(cpu), n_vocab = whisper_n_vocab(cpu), n_text_ctx = whisper_n_text_ctx(cpu);
    const int kv_to = std::min(a.num("kv-to", 0), n_text_ctx);
    const int steps = a.num("steps", 32);
    const std::vector<float> mel = synth::synthetic_mel(n_mels, 3000, (uint64_t) a.num("seed", 7));
    whisper_set_mel(gpu, mel.data(), 3000, n_mels);
    whisper_set_mel(cpu, mel.data(), 3000, n_mels);

    // graphs whisper computes vs what the scheduler and the plugin saw, over the GPU context's calls
    int64_t graphs_expected = 0, cnt[GGML_MI355X_N_COUNTERS];
    get_counters(nullptr, cnt, 1);
    g_splits_total = g_splits_not_on_device = 0;

    double t0 = now_ms();
    g_count_splits = true;
    const int eg = whisper_encode(gpu, 0, threads);
    g_count_splits = false;
    graphs_expected += 3;                                // conv stem, encoder, cross-attention K / V (src/whisper.cpp:2362-2466)
    const double enc_gpu_ms = now_ms() - t0; t0 = now_ms();
    const int ec = whisper_encode(cpu, 0, threads);
    const double enc_cpu_ms = now_ms() - t0;
    if (eg != 0 || ec != 0) { printf("{\"error\": \"encode failed\", \"gpu\": %d, \"cpu\": %d}\n", eg, ec); return 1; }
    get_counters(nullptr, cnt, 0);
    const int64_t encode_nodes = cnt[1], encode_launches = cnt[3];

    // prompt: <|sot|> <|en|> <|transcribe|> <|notimestamps|>  (4-token batch: exercises the n_tokens > 1 path)
    std::vector<whisper_token> feed = { whisper_token_sot(cpu), whisper_token_lang(cpu, whisper_lang_id("en")),
                                        whisper_token_transcribe(cpu), whisper_token_not(cpu) };
    int n_past = 0, n_same = 0, n_total = 0, n_clear = 0, n_clear_same = 0, n_steps = 0;
    double worst_nmse = 0, min_margin = 1e30, sum_nmse = 0;
    bool all_ok = true;
    for (int s = 0; kv_to > 0 ? n_past < kv_to : s < steps; ++s) {
        if (n_past + (int) feed.size() > n_text_ctx) feed.resize((size_t)(n_text_ctx - n_past));
        if (kv_to > 0 && n_past + (int) feed.size() > kv_to) feed.resize((size_t)(kv_to - n_past));
        g_count_splits = true;
        const int rg = whisper_decode(gpu, feed.data(), (int) feed.size(), n_past, threads);
        g_count_splits = false;
        graphs_expected += 1;
        const int rc = whisper_decode(cpu, feed.data(), (int) feed.size(), n_past, threads);
        if (rg != 0 || rc != 0) { printf("{\"error\": \"decode failed\", \"step\": %d, \"gpu\": %d, \"cpu\": %d}\n", s, rg, rc); return 1; }
        // logits of every fed token are returned: every row is compared on its own
        const int rows = (int) feed.size();
        const float * lg = whisper_get_logits(gpu), * lc = whisper_get_logits(cpu);
        std::vector<whisper_token> next;
        double step_worst = 0, step_min_margin = 1e30, step_rms = 0;
        int step_same = 0, step_clear = 0, step_clear_same = 0;
        for (int r = 0; r < rows; ++r) {
            const float * g = lg + (size_t) r * n_vocab, * c = lc + (size_t) r * n_vocab;
            double num = 0, den = 0;
            for (int i = 0; i < n_vocab; ++i) { const double d = (double) g[i] - c[i]; num += d * d; den += (double) c[i] * c[i]; }
            const double nmse = den > 0 ? num / den : 0, rms_diff = sqrt(num / n_vocab);
            float margin = 0;
            const int tok_c = argmax(c, n_vocab, &margin), tok_g = argmax(g, n_vocab, nullptr);
            next.push_back(tok_c);
            // a row is "clear" when the reference's own top-1 / top-2 margin is more than six times the RMS difference between
            // the two logit vectors: then the two argmaxes can only differ through an error, not through rounding noise
            const bool clear = margin > 6.0 * rms_diff;
            const bool counted = batch > 1 || r == rows - 1;      // one-row mode: the prompt's earlier rows are compared, not sampled
            if (!(nmse <= 1e-3)) all_ok = false;
            step_worst = std::max(step_worst, nmse); step_rms = std::max(step_rms, rms_diff);
            if (counted) {
                step_min_margin = std::min(step_min_margin, (double) margin);
                step_same += tok_c == tok_g; step_clear += clear; step_clear_same += clear && tok_c == tok_g;
                n_same += tok_c == tok_g; ++n_total; n_clear += clear; n_clear_same += clear && tok_c == tok_g;
                sum_nmse += nmse;
            }
        }
        worst_nmse = std::max(worst_nmse, step_worst); min_margin = std::min(min_margin, step_min_margin);
        printf("{\"step\": %d, \"n_tokens\": %d, \"n_past\": %d, \"worst_row_logits_nmse\": %.3e, \"rows_ids_identical\": %d, \"rows_clear\": %d, "
               "\"rows_clear_identical\": %d, \"min_top1_top2_margin\": %.4e, \"max_logits_rms_diff\": %.4e}\n",
               s, rows, n_past, step_worst, step_same, step_clear, step_clear_same, step_min_margin, step_rms);
        n_past += rows; ++n_steps;
        if (batch > 1) { next.resize((size_t) std::min<int>(batch, (int) next.size())); while ((int) next.size() < batch) next.push_back(next.back()); feed = next; }
        else feed.assign(1, next.back());
    }
    get_counters(nullptr, cnt, 0);
    // one split per graph, all on the device, and the plugin was called exactly once per graph
    const bool one_split = g_splits_total == graphs_expected && g_splits_not_on_device == 0 && cnt[0] == graphs_expected;
    // pass: logits within the bound on every row, identical greedy ids on every row whose margin is clear of the noise
    // --pieces (with GGML_MI355X_DECLINE set): the graphs are expected to reach the plugin as several splits with CPU splits between
    const bool in_pieces = g_splits_total > graphs_expected && g_splits_not_on_device > 0 && cnt[0] > graphs_expected;
    const bool pass = all_ok && n_clear_same == n_clear && (a.has("pieces") ? in_pieces : one_split);
    printf("{\"summary\": \"model\", \"model\": \"%s\", \"batch\": %d, \"steps\": %d, \"kv_positions\": %d, \"rows\": %d, \"ids_identical\": %d, \"clear_steps\": %d, "
           "\"clear_ids_identical\": %d, \"worst_logits_nmse\": %.3e, \"mean_logits_nmse\": %.3e, \"min_top1_top2_margin\": %.4e, "
           "\"graphs\": %lld, \"sched_splits\": %d, \"sched_splits_not_on_device\": %d, \"plugin_graph_computes\": %lld, \"plugin_nodes\": %lld, "
           "\"plugin_launches\": %lld, \"encode_nodes\": %lld, \"encode_launches\": %lld, \"one_split_per_graph\": %s, "
           "\"encode_gpu_ms_first_call\": %.2f, \"encode_cpu_ms\": %.2f, \"cpu_threads\": %d, \"seed\": %d, \"pass\": %s}\n",
           json_escape(path).c_str(), batch, n_steps, n_past, n_total, n_same, n_clear, n_clear_same, worst_nmse, sum_nmse / std::max(1, n_total), min_margin,
           (long long) graphs_expected, g_splits_total, g_splits_not_on_device, (long long) cnt[0], (long long) cnt[1], (long long) cnt[3],
           (long long) encode_nodes, (long long) encode_launches, one_split ? "true" : "false",
           enc_gpu_ms, enc_cpu_ms, threads, a.num("seed", 7), pass ? "true" : "false");
    whisper_free(gpu); whisper_free(cpu);
    return pass ? 0 : 1;
}

// whisper_full() end to end on synthetic audio: log-mel on the host, encoder, then whisper's own greedy or beam search
// with its logits filters, timestamp rules and KV-cache bookkeeping.  Both backends see the same PCM; the token ids of
// the two transcripts are compared from the front (a random-init model's near-flat logits let one rounding flip an
// argmax, after which the two searches walk different histories, so only the common prefix is meaningful).
// the filter bank of a model file (the loader keeps its copy private): magic, 11 hyper-parameters, n_mel, n_fft, data
// (src/whisper.cpp:1522-1597)
static std::vector<float> read_filters(const std::string & path, int32_t * n_mel) {
    std::vector<float> filters;
    int32_t n_fft = 0;
    *n_mel = 0;
    if (FILE * f = fopen(path.c_str(), "rb")) {
        if (fseek(f, 4 + 11 * 4, SEEK_SET) == 0 && fread(n_mel, 4, 1, f) == 1 && fread(&n_fft, 4, 1, f) == 1 && n_fft == 201 && *n_mel > 0 && *n_mel <= 128) {
            filters.resize((size_t) *n_mel * n_fft);
            if (fread(filters.data(), 4, filters.size(), f) != filters.size()) filters.clear();
        }
        fclose(f);
    }
    return filters;
}

// fresh_state: the call runs on a state of its own (whisper_full_with_state), made for it and freed after it.  The search's
// first decoder keeps the generator it was given when its state was made (src/whisper.cpp:3481; the others are seeded in every
// call, :5583), so only calls on new states draw the same candidates.
static std::vector<whisper_token> run_full(whisper_context * ctx, const std::vector<float> & pcm, int beam, int max_tokens, int threads, int * rc, double * ms,
                                           std::vector<int64_t> * t_dtw = nullptr, bool use_gpu_mel = false, bool fresh_state = false) {
    whisper_full_params p = whisper_full_default_params(beam > 1 ? WHISPER_SAMPLING_BEAM_SEARCH : WHISPER_SAMPLING_GREEDY);
    p.n_threads = threads;
    p.print_progress = false; p.print_realtime = false; p.print_timestamps = false; p.print_special = false;
    p.language = "en"; p.translate = false;
    p.max_tokens = max_tokens;
    p.temperature_inc = 0.0f;                  // no temperature fallback: one pass per window
    p.suppress_blank = true;
    if (beam > 1) p.beam_search.beam_size = beam; else p.greedy.best_of = 1;
    const double t0 = now_ms();
    if (use_gpu_mel) {
        int32_t n_mel = 0;
        const std::vector<float> filters = read_filters(g_model_path, &n_mel);
        if (filters.empty()) { *rc = -100; *ms = 0; return {}; }
        const double m0 = now_ms();
        const int64_t n_len = g_log_mel(0, pcm.data(), (int64_t) pcm.size(), filters.data(), n_mel, nullptr, 0, nullptr);
        std::vector<float> mel(n_len > 0 ? (size_t) n_len * n_mel : 0);
        if (n_len <= 0 || g_log_mel(0, pcm.data(), (int64_t) pcm.size(), filters.data(), n_mel, mel.data(), (int64_t) mel.size(), nullptr) != n_len) { *rc = -101; *ms = 0; return {}; }
        g_mel_ms = now_ms() - m0;
        if (whisper_set_mel(ctx, mel.data(), (int) n_len, n_mel) != 0) { *rc = -102; *ms = 0; return {}; }
        *rc = whisper_full(ctx, p, nullptr, 0);          // no samples: transcribes from the mel it was given (src/whisper.cpp:5492)
    } else if (fresh_state) {
        std::vector<whisper_token> out;
        whisper_state * st = whisper_init_state(ctx);
        if (!st) { *rc = -103; *ms = 0; return out; }
        *rc = whisper_full_with_state(ctx, st, p, pcm.data(), (int) pcm.size());
        *ms = now_ms() - t0;
        if (*rc == 0)
            for (int i = 0; i < whisper_full_n_segments_from_state(st); ++i)
                for (int j = 0; j < whisper_full_n_tokens_from_state(st, i); ++j) out.push_back(whisper_full_get_token_id_from_state(st, i, j));
        whisper_free_state(st);
        return out;
    } else
    // --processors N: whisper_full_parallel splits the audio over N states, each with its own backend instance and host thread
    *rc = g_processors > 1 ? whisper_full_parallel(ctx, p, pcm.data(), (int) pcm.size(), g_processors) : whisper_full(ctx, p, pcm.data(), (int) pcm.size());
    *ms = now_ms() - t0;
    std::vector<whisper_token> out;
    if (*rc != 0) return out;
    const int nseg = whisper_full_n_segments(ctx);
    for (int i = 0; i < nseg; ++i)
        for (int j = 0; j < whisper_full_n_tokens(ctx, i); ++j) {
            out.push_back(whisper_full_get_token_id(ctx, i, j));
            if (t_dtw) t_dtw->push_back(whisper_full_get_token_data(ctx, i, j).t_dtw);
        }
    return out;
}

static int cmd_full(const args & a) {
    const std::string path = a.str("model");
    const int threads = a.num("threads", default_threads()), beam = a.num("beam", 1), max_tokens = a.num("max-tokens", 24);
    const int seconds = a.num("seconds", 30);
    if (path.empty()) { fprintf(stderr, "usage: full --model FILE [--beam N] [--max-tokens N] [--seconds N] [--gpu-mel]\n"); return 2; }
    ggml_backend_reg_t reg = load_plugin(true);
    if (!reg) { printf("{\"error\": \"no MI355X backend\"}\n"); return 2; }
    g_model_path = path;
    if (g_gpu_mel) {
        g_log_mel = (ggml_backend_mi355x_log_mel_t) ggml_backend_reg_get_proc_address(reg, "ggml_backend_mi355x_log_mel");
        if (!g_log_mel || g_processors > 1) { printf("{\"error\": \"--gpu-mel needs the plugin's log-mel entry and one processor\"}\n"); return 2; }
    }
    whisper_context * gpu = open_model(path, true);
    whisper_context * cpu = open_model(path, false);
    if (!gpu || !cpu) { printf("{\"error\": \"model load failed\"}\n"); return 2; }
    // a few drifting tones under noise, 16 kHz mono
    std::vector<float> pcm((size_t) seconds * WHISPER_SAMPLE_RATE);
    uint64_t st = 0x9E3779B97F4A7C15ull ^ (uint64_t) a.num("seed", 7);
    for (size_t i = 0; i < pcm.size(); ++i) {
        st = st * 6364136223846793005ull + 1442695040888963407ull;
        const double t = (double) i / WHISPER_SAMPLE_RATE;
        const double noise = ((double)(st >> 40) / (double)(1 << 24)) - 0.5;
        pcm[i] = (float)(0.25 * sin(2 * M_PI * (220.0 + 30.0 * t) * t) + 0.15 * sin(2 * M_PI * 1310.0 * t) + 0.1 * noise);
    }
    int rg = 0, rc = 0; double ms_g = 0, ms_c = 0;
    std::vector<int64_t> dg, dc;
    const std::vector<whisper_token> tg = run_full(gpu, pcm, beam, max_tokens, threads, &rg, &ms_g, &dg, g_gpu_mel);
    // --repeat: the same call once more on the device (greedy: no random draws).  The first run makes the weight images while
    // the states of a parallel run all start at once; the second finds them made: the two transcripts must be the same tokens.
    bool repeat_identical = true;
    if (a.has("repeat")) {
        int r2 = 0; double ms2 = 0;
        if (beam > 1 && g_processors == 1 && !g_gpu_mel) {
            // beam search: two calls on two new states (see run_full), compared with each other
            int r1 = 0; double ms1 = 0;
            const std::vector<whisper_token> one = run_full(gpu, pcm, beam, max_tokens, threads, &r1, &ms1, nullptr, false, true);
            const std::vector<whisper_token> two = run_full(gpu, pcm, beam, max_tokens, threads, &r2, &ms2, nullptr, false, true);
            repeat_identical = r1 == 0 && r2 == 0 && !one.empty() && one == two;
        } else {
            const std::vector<whisper_token> again = run_full(gpu, pcm, beam, max_tokens, threads, &r2, &ms2, nullptr, g_gpu_mel);
            repeat_identical = r2 == 0 && again == tg;
        }
    }
    const std::vector<whisper_token> tc = run_full(cpu, pcm, beam, max_tokens, threads, &rc, &ms_c, &dc);
    size_t same = 0;
    while (same < tg.size() && same < tc.size() && tg[same] == tc[same]) ++same;
    // DTW timestamps of the common prefix (only meaningful with --dtw; -1 otherwise)
    size_t dtw_same = 0;
    for (size_t i = 0; i < same; ++i) dtw_same += dg[i] == dc[i];
    std::string sg, sc;
    for (size_t i = 0; i < tg.size() && i < 16; ++i) sg += (i ? "," : "") + std::to_string(tg[i]);
    for (size_t i = 0; i < tc.size() && i < 16; ++i) sc += (i ? "," : "") + std::to_string(tc[i]);
    const bool pass = rg == 0 && rc == 0 && !tg.empty() && repeat_identical;
    printf("{\"summary\": \"full\", \"model\": \"%s\", \"beam\": %d, \"seconds\": %d, \"gpu_rc\": %d, \"cpu_rc\": %d, \"gpu_segments\": %d, \"cpu_segments\": %d, "
           "\"gpu_repeat_identical\": %s, "
           "\"gpu_tokens\": %zu, \"cpu_tokens\": %zu, \"common_prefix\": %zu, \"dtw\": %s, \"dtw_identical_in_prefix\": %zu, \"gpu_t_dtw_first\": %lld, "
           "\"gpu_first\": [%s], \"cpu_first\": [%s], \"gpu_ms\": %.1f, \"cpu_ms\": %.1f, \"gpu_mel\": %s, \"gpu_mel_ms\": %.3f, \"pass\": %s}\n",
           json_escape(path).c_str(), beam, seconds, rg, rc, rg == 0 ? whisper_full_n_segments(gpu) : -1, rc == 0 ? whisper_full_n_segments(cpu) : -1,
           repeat_identical ? "true" : "false", tg.size(), tc.size(), same, g_dtw ? "true" : "false", dtw_same, dg.empty() ? -1LL : (long long) dg[0], sg.c_str(), sc.c_str(), ms_g, ms_c, g_gpu_mel ? "true" : "false", g_mel_ms, pass ? "true" : "false");
    whisper_free(gpu); whisper_free(cpu);
    return pass ? 0 : 1;
}

// per-node parity on the graphs whisper builds: conv + encoder + cross, one prompt batch, a few single-token steps,
// one 5-token batch (the shape of a beam-search step)
static int cmd_verify(const args & a) {
    const std::string path = a.str("model");
    const int steps = a.num("steps", 3), threads = a.num("threads", default_threads());
    if (path.empty()) { fprintf(stderr, "usage: verify --model FILE [--steps N]\n"); return 2; }
    const char * env = getenv("GGML_MI355X_PLUGIN");
    if (!verify::load_plugin_hooked(env ? env : self_dir() + "/libggml-mi355x.so")) { printf("{\"error\": \"no MI355X backend\"}\n"); return 2; }
    verify::set_threads(threads);
    verify::set_enabled(false);                       // worst-case reserve graphs run on uninitialised data
    whisper_context * gpu = open_model(path, true);
    if (!gpu) { printf("{\"error\": \"model load failed\"}\n"); return 2; }
    verify::set_enabled(true);
    const int n_mels = whisper_model_n_mels(gpu);
    const std::vector<float> mel = synth::synthetic_mel(n_mels, 3000, (uint64_t) a.num("seed", 7));
    whisper_set_mel(gpu, mel.data(), 3000, n_mels);
    int bad = 0;
    if (whisper_encode(gpu, 0, threads) != 0) return 1;
    bad += verify::report("encode");
    std::vector<whisper_token> prompt = { whisper_token_sot(gpu), whisper_token_lang(gpu, whisper_lang_id("en")), whisper_token_transcribe(gpu), whisper_token_not(gpu) };
    if (whisper_decode(gpu, prompt.data(), (int) prompt.size(), 0, threads) != 0) return 1;
    bad += verify::report("decode_prompt4");
    int n_past = (int) prompt.size();
    for (int s = 0; s < steps; ++s) {
        float m; whisper_token t = argmax(whisper_get_logits(gpu), whisper_n_vocab(gpu), &m);
        if (whisper_decode(gpu, &t, 1, n_past++, threads) != 0) return 1;
    }
    bad += verify::report("decode_single");
    std::vector<whisper_token> five = { 11, 22, 33, 44, 55 };
    if (whisper_decode(gpu, five.data(), 5, n_past, threads) != 0) return 1;
    bad += verify::report("decode_batch5");
    printf("{\"summary\": \"verify\", \"model\": \"%s\", \"nodes_over_tol\": %d, \"pass\": %s}\n", json_escape(path).c_str(), bad, bad == 0 ? "true" : "false");
    whisper_free(gpu);
    return bad == 0 ? 0 : 1;
}

// ---------------------------------------------------------------------------------------------------------------
// bench
// ---------------------------------------------------------------------------------------------------------------

// whisper.h does not expose the backends of a state, so the options and statistics calls address every live MI355X
// backend of the process (backend == NULL).
static void plugin_set_option(ggml_backend_reg_t reg, const char * name, int value) {
    if (!reg) return;
    auto set = (ggml_backend_mi355x_set_option_t) ggml_backend_reg_get_proc_address(reg, "ggml_backend_mi355x_set_option");
    if (set) set(nullptr, name, value);
}

static std::string plugin_stats(ggml_backend_reg_t reg, bool reset) {
    if (!reg) return "[]";
    auto get = (ggml_backend_mi355x_get_stats_t) ggml_backend_reg_get_proc_address(reg, "ggml_backend_mi355x_get_stats");
    if (!get) return "[]";
    const size_t need = get(nullptr, nullptr, 0, 0);
    std::string s(need + 1, '\0');
    get(nullptr, &s[0], s.size(), reset ? 1 : 0);
    s.resize(strlen(s.c_str()));
    return s;
}

static double median(std::vector<double> v) {
    if (v.empty()) return 0;
    std::sort(v.begin(), v.end());
    return v[v.size() / 2];
}

static int cmd_bench(const args & a) {
    const std::string path = a.str("model"), what = a.str("what", "encoder"), be = a.str("backend", "gpu");
    const int threads = a.num("threads", default_threads()), reps = a.num("reps", 5), warmup = a.num("warmup", 2);
    if (path.empty()) { fprintf(stderr, "usage: bench --model FILE --what encoder|decoder|whisper-bench --backend gpu|cpu\n"); return 2; }
    const bool use_gpu = be == "gpu";
    ggml_backend_reg_t reg = use_gpu ? load_plugin(true) : nullptr;
    if (use_gpu && !reg) { printf("{\"error\": \"no MI355X backend\"}\n"); return 2; }
    const bool profile = use_gpu && a.has("profile");
    if (use_gpu && a.has("no-fuse")) setenv("GGML_MI355X_FUSE", "0", 1);
    whisper_context * ctx = open_model(path, use_gpu);
    if (!ctx) { printf("{\"error\": \"model load failed\"}\n"); return 2; }
    const int n_mels = whisper_model_n_mels(ctx);
    const std::vector<float> mel = synth::synthetic_mel(n_mels, 3000, 7);
    whisper_set_mel(ctx, mel.data(), 3000, n_mels);

    if (what == "encoder") {
        // `warmup` untimed windows, then exactly `reps` timed ones; afterwards, optionally, `profile-reps` more with every
        // kernel bracketed by HIP events on the backend's stream (these do not enter the timing above)
        const int prof_reps = use_gpu ? a.num("profile-reps", profile ? 3 : 0) : 0;
        for (int i = 0; i < warmup; ++i) if (whisper_encode(ctx, 0, threads) != 0) return 1;
        std::vector<double> wall, enc;
        const double t_all = now_ms();
        for (int i = 0; i < reps; ++i) {
            whisper_reset_timings(ctx);
            const double t0 = now_ms();
            if (whisper_encode(ctx, 0, threads) != 0) return 1;
            wall.push_back(now_ms() - t0);
            whisper_timings * t = whisper_get_timings(ctx);
            enc.push_back(t ? t->encode_ms : 0.0);
            delete t;
        }
        const double total_ms = now_ms() - t_all;
        std::string kernels = "[]";
        if (prof_reps > 0) {
            plugin_set_option(reg, "profile", 1); plugin_stats(reg, true);
            for (int i = 0; i < prof_reps; ++i) if (whisper_encode(ctx, 0, threads) != 0) return 1;
            kernels = plugin_stats(reg, true);
            plugin_set_option(reg, "profile", 0);
        }
        printf("{\"bench\": \"encoder\", \"backend\": \"%s\", \"threads\": %d, \"reps\": %d, \"warmup\": %d, \"total_ms\": %.4f, \"ms_per_step\": %.4f, "
               "\"encode_ms_median\": %.4f, \"encode_ms_min\": %.4f, \"wall_ms_median\": %.4f, \"profile_reps\": %d, \"kernels\": %s, \"model\": \"%s\"}\n",
               be.c_str(), threads, reps, warmup, total_ms, total_ms / std::max(1, reps), median(enc), *std::min_element(enc.begin(), enc.end()), median(wall),
               prof_reps, kernels.c_str(), json_escape(path).c_str());
    } else if (what == "decoder") {
        // 5-token batches with a growing self-attention cache: the per-step work of a 5-beam search
        // (src/whisper.cpp:6089-6117), driven through whisper_decode like the batch-5 leg of whisper-bench.
        // Step i places its tokens at positions kv_stride * i .. + batch - 1 (capped so that they fit the cache): with
        // --kv-stride 2 the 224 steps walk the self-attention cache up to its 448 positions.
        const int n_steps = a.num("steps", 224), batch = a.num("batch", 5), kv_stride = a.num("kv-stride", 1);
        const int n_text_ctx = whisper_n_text_ctx(ctx);
        auto past_of = [&](int i) { return std::min(kv_stride * i, n_text_ctx - batch); };
        if (whisper_encode(ctx, 0, threads) != 0) return 1;
        std::vector<whisper_token> tok((size_t) batch, 0);
        for (int i = 0; i < warmup; ++i) if (whisper_decode(ctx, tok.data(), batch, i, threads) != 0) return 1;
        std::vector<double> per_rep;
        for (int r = 0; r < reps; ++r) {
            const double t0 = now_ms();
            for (int i = 0; i < n_steps; ++i) {
                for (int j = 0; j < batch; ++j) tok[(size_t) j] = (whisper_token)((i * 131 + j * 17) % 50000);
                if (whisper_decode(ctx, tok.data(), batch, past_of(i), threads) != 0) return 1;
            }
            per_rep.push_back(now_ms() - t0);
        }
        const double ms = median(per_rep);
        std::string kernels = "[]";
        int64_t cnt[GGML_MI355X_N_COUNTERS] = {};
        if (use_gpu) {
            auto get_counters = (ggml_backend_mi355x_get_counters_t) ggml_backend_reg_get_proc_address(reg, "ggml_backend_mi355x_get_counters");
            if (get_counters) {                           // launches and downloads of one more pass, unprofiled
                get_counters(nullptr, cnt, 1);
                for (int i = 0; i < n_steps; ++i) if (whisper_decode(ctx, tok.data(), batch, past_of(i), threads) != 0) return 1;
                get_counters(nullptr, cnt, 1);
            }
        }
        if (profile) {
            plugin_set_option(reg, "profile", 1); plugin_stats(reg, true);
            for (int i = 0; i < n_steps; ++i) if (whisper_decode(ctx, tok.data(), batch, past_of(i), threads) != 0) return 1;
            kernels = plugin_stats(reg, true);
            plugin_set_option(reg, "profile", 0);
        }
        printf("{\"bench\": \"decoder\", \"backend\": \"%s\", \"threads\": %d, \"reps\": %d, \"steps\": %d, \"batch\": %d, \"kv_stride\": %d, \"max_kv_positions\": %d, "
               "\"total_ms_median\": %.3f, \"ms_per_step\": %.5f, \"ms_per_step_min\": %.5f, \"steps_per_s\": %.2f, \"batch_tokens_per_s\": %.2f, \"launches_per_step\": %.2f, "
               "\"downloads_from_mirror_per_step\": %.2f, \"downloads_by_copy_per_step\": %.2f, \"host_us_in_graph_compute_per_step\": %.2f, \"host_us_waiting_in_synchronize_per_step\": %.2f, \"profiled\": %s, \"kernels\": %s, \"model\": \"%s\"}\n",
               be.c_str(), threads, reps, n_steps, batch, kv_stride, past_of(n_steps - 1) + batch, ms, ms / n_steps, *std::min_element(per_rep.begin(), per_rep.end()) / n_steps,
               1000.0 * n_steps / ms, 1000.0 * n_steps * batch / ms, (double) cnt[3] / n_steps, (double) cnt[4] / n_steps, (double) cnt[5] / n_steps, cnt[6] / 1e3 / n_steps, cnt[7] / 1e3 / n_steps,
               profile ? "true" : "false", kernels.c_str(), json_escape(path).c_str());
    } else if (what == "full") {
        // whisper_full() as a user calls it: beam search with --beam beams (src/whisper.cpp:5781-5798: one KV cache for all beams,
        // per-row masks), up to n_text_ctx / 2 - 4 tokens per window, no temperature fallback, over synthetic audio.  Per pass:
        // wall time, whisper's own timings and its run counts (read from whisper_print_timings through the log callback: the
        // counts are not in whisper_timings), and from the plugin the number of decode-step graphs and the largest number of
        // keys a step's attention walked.
        const int beam = a.num("beam", 5), seconds = a.num("seconds", 30);
        std::vector<float> pcm((size_t) seconds * WHISPER_SAMPLE_RATE);
        uint64_t st = 0x9E3779B97F4A7C15ull ^ 7ull;
        for (size_t i = 0; i < pcm.size(); ++i) {
            st = st * 6364136223846793005ull + 1442695040888963407ull;
            const double t = (double) i / WHISPER_SAMPLE_RATE;
            const double noise = ((double)(st >> 40) / (double)(1 << 24)) - 0.5;
            pcm[i] = (float)(0.25 * sin(2 * M_PI * (220.0 + 30.0 * t) * t) + 0.15 * sin(2 * M_PI * 1310.0 * t) + 0.1 * noise);
        }
        whisper_full_params p = whisper_full_default_params(beam > 1 ? WHISPER_SAMPLING_BEAM_SEARCH : WHISPER_SAMPLING_GREEDY);
        p.n_threads = threads;
        p.print_progress = false; p.print_realtime = false; p.print_timestamps = false; p.print_special = false;
        p.language = "en"; p.translate = false;
        p.temperature_inc = 0.0f;
        if (beam > 1) p.beam_search.beam_size = beam; else p.greedy.best_of = 1;
        auto get_counters = use_gpu ? (ggml_backend_mi355x_get_counters_t) ggml_backend_reg_get_proc_address(reg, "ggml_backend_mi355x_get_counters") : nullptr;
        static std::string timing_log;
        auto collect = [](ggml_log_level, const char * text, void *) { timing_log += text; };
        auto run_count = [](const char * label) {          // "...   batchd time =   123.45 ms /   678 runs ..."
            const size_t at = timing_log.find(label);
            if (at == std::string::npos) return std::pair<double, long>(0.0, 0L);
            double ms = 0; long runs = 0;
            const size_t eq = timing_log.find('=', at);
            if (eq != std::string::npos) sscanf(timing_log.c_str() + eq + 1, " %lf ms / %ld", &ms, &runs);
            return std::pair<double, long>(ms, runs);
        };
        std::vector<double> wall;
        std::string last;
        for (int r = 0; r < warmup + reps; ++r) {
            int64_t cnt[GGML_MI355X_N_COUNTERS] = {};
            if (get_counters) get_counters(nullptr, cnt, 1);
            whisper_reset_timings(ctx);
            const double t0 = now_ms();
            if (whisper_full(ctx, p, pcm.data(), (int) pcm.size()) != 0) return 1;
            const double ms = now_ms() - t0;
            if (r < warmup) continue;
            wall.push_back(ms);
            if (get_counters) get_counters(nullptr, cnt, 0);
            timing_log.clear();
            whisper_log_set(collect, nullptr);
            whisper_print_timings(ctx);
            whisper_log_set(nullptr, nullptr);
            const auto enc = run_count("encode time"), dec = run_count("decode time"), bat = run_count("batchd time"), prm = run_count("prompt time"), smp = run_count("sample time");
            int tokens = 0;
            for (int i = 0; i < whisper_full_n_segments(ctx); ++i) tokens += whisper_full_n_tokens(ctx, i);
            // whisper counts a batched call's tokens as its runs (src/whisper.cpp: n_batchd += n_tokens); a step is one call
            const long steps = get_counters ? (long) cnt[8] : 0;
            char buf[1024];
            snprintf(buf, sizeof(buf), "\"wall_ms\": %.2f, \"encode_ms\": %.2f, \"encode_runs\": %ld, \"batchd_ms\": %.2f, \"batchd_token_runs\": %ld, \"decode_ms\": %.2f, "
                     "\"decode_runs\": %ld, \"prompt_ms\": %.2f, \"prompt_token_runs\": %ld, \"sample_ms\": %.2f, \"tokens_in_result\": %d, \"segments\": %d, "
                     "\"decode_step_graphs\": %ld, \"largest_n_kv\": %lld, \"ms_per_decode_step\": %.4f, \"launches\": %lld",
                     ms, enc.first, enc.second, bat.first, bat.second, dec.first, dec.second, prm.first, prm.second, smp.first, tokens, whisper_full_n_segments(ctx),
                     steps, (long long) cnt[9], steps > 0 ? (bat.first + dec.first) / steps : 0.0, (long long) cnt[3]);
            last = buf;
        }
        printf("{\"bench\": \"full\", \"backend\": \"%s\", \"threads\": %d, \"beam\": %d, \"seconds\": %d, \"reps\": %d, \"wall_ms_median\": %.2f, %s, \"model\": \"%s\"}\n",
               be.c_str(), threads, beam, seconds, reps, median(wall), last.c_str(), json_escape(path).c_str());
    } else {   // whisper-bench protocol, verbatim counts (examples/bench/bench.cpp:86-138)
        whisper_token tokens[512]; memset(tokens, 0, sizeof(tokens));
        if (whisper_encode(ctx, 0, threads) != 0) return 1;
        if (whisper_decode(ctx, tokens, 256, 0, threads) != 0) return 1;
        if (whisper_decode(ctx, tokens, 1, 256, threads) != 0) return 1;
        whisper_reset_timings(ctx);
        if (whisper_encode(ctx, 0, threads) != 0) return 1;
        for (int i = 0; i < 256; i++) if (whisper_decode(ctx, tokens, 1, i, threads) != 0) return 1;
        for (int i = 0; i < 64; i++)  if (whisper_decode(ctx, tokens, 5, 0, threads) != 0) return 1;
        for (int i = 0; i < 16; i++)  if (whisper_decode(ctx, tokens, 256, 0, threads) != 0) return 1;
        whisper_timings * t = whisper_get_timings(ctx);
        printf("{\"bench\": \"whisper-bench\", \"backend\": \"%s\", \"threads\": %d, \"encode_ms\": %.3f, \"decode_ms_per_token\": %.4f, "
               "\"batchd_ms_per_token\": %.4f, \"prompt_ms_per_token\": %.4f, \"model\": \"%s\"}\n",
               be.c_str(), threads, t->encode_ms, t->decode_ms, t->batchd_ms, t->prompt_ms, json_escape(path).c_str());   // already per token (src/whisper.cpp:4256-4260)
        delete t;
    }
    whisper_free(ctx);
    return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// copy: a plain device copy of known size (one CPY node, f32 -> f32, contiguous) — the yardstick the memory-traffic
// counters of a profiler are scaled by
// ---------------------------------------------------------------------------------------------------------------

// the log-mel front end of one window: the device path through the plugin (device time from HIP events, and the whole
// host-to-host call) beside whisper_pcm_to_mel on the host threads, same samples, same filter bank
static int cmd_mel(const args & a) {
    const std::string path = a.str("model");
    const int threads = a.num("threads", default_threads()), seconds = a.num("seconds", 30), reps = a.num("reps", 20);
    if (path.empty()) { fprintf(stderr, "usage: mel --model FILE [--seconds N] [--reps N] [--threads N]\n"); return 2; }
    ggml_backend_reg_t reg = load_plugin(true);
    auto fn = reg ? (ggml_backend_mi355x_log_mel_t) ggml_backend_reg_get_proc_address(reg, "ggml_backend_mi355x_log_mel") : nullptr;
    if (!fn) { printf("{\"error\": \"no MI355X backend\"}\n"); return 2; }
    int32_t n_mel = 0;
    const std::vector<float> filters = read_filters(path, &n_mel);
    whisper_context * cpu = open_model(path, false);
    if (filters.empty() || !cpu) { printf("{\"error\": \"model load failed\"}\n"); return 2; }
    std::vector<float> pcm((size_t) seconds * WHISPER_SAMPLE_RATE);
    uint64_t st = 0x9E3779B97F4A7C15ull;
    for (size_t i = 0; i < pcm.size(); ++i) {
        st = st * 6364136223846793005ull + 1442695040888963407ull;
        const double t = (double) i / WHISPER_SAMPLE_RATE;
        pcm[i] = (float)(0.25 * sin(2 * M_PI * (220.0 + 30.0 * t) * t) + 0.1 * (((double)(st >> 40) / (double)(1 << 24)) - 0.5));
    }
    const int64_t n_len = fn(0, pcm.data(), (int64_t) pcm.size(), filters.data(), n_mel, nullptr, 0, nullptr);
    std::vector<float> mel((size_t) n_len * n_mel);
    std::vector<double> dev, whole, host;
    for (int r = 0; r < reps + 2; ++r) {
        float ms = 0.0f;
        const double t0 = now_ms();
        if (fn(0, pcm.data(), (int64_t) pcm.size(), filters.data(), n_mel, mel.data(), (int64_t) mel.size(), &ms) != n_len) { printf("{\"error\": \"device log-mel failed\"}\n"); return 1; }
        if (r >= 2) { dev.push_back(ms); whole.push_back(now_ms() - t0); }
    }
    for (int r = 0; r < 5; ++r) {
        const double t0 = now_ms();
        if (whisper_pcm_to_mel(cpu, pcm.data(), (int) pcm.size(), threads) != 0) { printf("{\"error\": \"whisper_pcm_to_mel failed\"}\n"); return 1; }
        if (r >= 1) host.push_back(now_ms() - t0);
    }
    auto median = [](std::vector<double> v) { std::sort(v.begin(), v.end()); return v[v.size() / 2]; };
    // algorithmic bytes of the device work: samples in, mel out (the filter bank and the workspace stay in the caches)
    const double bytes = (double) pcm.size() * 4 + (double) mel.size() * 4;
    printf("{\"bench\": \"log_mel\", \"seconds\": %d, \"n_mel\": %d, \"n_len\": %lld, \"device_us\": %.2f, \"host_to_host_ms\": %.3f, "
           "\"cpu_ms\": %.3f, \"cpu_threads\": %d, \"algorithmic_mb\": %.3f, \"model\": \"%s\"}\n",
           seconds, n_mel, (long long) n_len, median(dev) * 1e3, median(whole), median(host), threads, bytes / 1e6, json_escape(path).c_str());
    whisper_free(cpu);
    return 0;
}

static int cmd_copy(const args & a) {
    const int64_t mib = a.num("mib", 256), reps = a.num("reps", 5);
    ggml_backend_reg_t reg = load_plugin(true);
    if (!reg) { printf("{\"error\": \"no MI355X backend\"}\n"); return 2; }
    ggml_backend_t be = ggml_backend_dev_init(ggml_backend_reg_dev_get(reg, 0), nullptr);
    if (!be) return 1;
    ggml_init_params ip = { ggml_tensor_overhead() * 8 + ggml_graph_overhead(), nullptr, true };
    ggml_context * ctx = ggml_init(ip);
    const int64_t n = mib * 1024 * 1024 / 4;
    ggml_tensor * src = ggml_new_tensor_1d(ctx, GGML_TYPE_F32, n), * dst = ggml_new_tensor_1d(ctx, GGML_TYPE_F32, n);
    ggml_tensor * cp = ggml_cpy(ctx, src, dst);
    ggml_cgraph * gf = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, cp);
    ggml_backend_buffer_t buf = ggml_backend_alloc_ctx_tensors(ctx, be);
    if (!buf) return 1;
    ggml_backend_buffer_clear(buf, 0);
    if (ggml_backend_graph_compute(be, gf) != GGML_STATUS_SUCCESS) return 1;
    const double t0 = now_ms();
    for (int i = 0; i < reps; ++i) if (ggml_backend_graph_compute(be, gf) != GGML_STATUS_SUCCESS) return 1;
    const double ms = (now_ms() - t0) / (double) reps;
    printf("{\"copy\": \"f32 contiguous\", \"bytes_read\": %lld, \"bytes_written\": %lld, \"launches\": %lld, \"ms_per_launch\": %.4f, \"gb_per_s\": %.1f}\n",
           (long long)(n * 4), (long long)(n * 4), (long long)(reps + 1), ms, 2.0 * n * 4 / ms / 1e6);
    ggml_backend_buffer_free(buf);
    ggml_free(ctx);
    ggml_backend_free(be);
    return 0;
}

// the host side of a step's boundary: results that the host reads back are mirrored in pinned memory after the first
// download and served from there until something writes them; and the device's pinned host buffer type
static int cmd_download(const args & a) {
    ggml_backend_reg_t reg = load_plugin(true);
    if (!reg) { printf("{\"error\": \"no MI355X backend\"}\n"); return 2; }
    ggml_backend_dev_t dev = ggml_backend_reg_dev_get(reg, 0);
    ggml_backend_t be = ggml_backend_dev_init(dev, nullptr);
    auto get_counters = (ggml_backend_mi355x_get_counters_t) ggml_backend_reg_get_proc_address(reg, "ggml_backend_mi355x_get_counters");
    if (!be || !get_counters) return 1;
    const int64_t n = a.num("n", 51866 * 5);            // the logits of a 5-beam step
    const int rows = 5;
    ggml_init_params ip = { ggml_tensor_overhead() * 8 + ggml_graph_overhead(), nullptr, true };
    ggml_context * ctx = ggml_init(ip);
    ggml_tensor * x = ggml_new_tensor_1d(ctx, GGML_TYPE_F32, n);
    ggml_tensor * y = ggml_scale(ctx, x, 2.0f);         // the graph's last node: what whisper's logits are (src/whisper.cpp:2953)
    ggml_cgraph * gf = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, y);
    ggml_backend_buffer_t buf = ggml_backend_alloc_ctx_tensors(ctx, be);
    if (!buf) return 1;
    std::vector<float> in1((size_t) n), in2((size_t) n), got((size_t) n), other((size_t) n);
    for (int64_t i = 0; i < n; ++i) { in1[(size_t) i] = synth::normal_at(5, (uint64_t) i); in2[(size_t) i] = synth::normal_at(6, (uint64_t) i); other[(size_t) i] = (float) i; }
    int64_t c[GGML_MI355X_N_COUNTERS];
    int bad = 0;
    auto fetch_rows = [&]() {                              // row by row, as whisper_decode does (src/whisper.cpp:2960-2966)
        std::fill(got.begin(), got.end(), -1.0f);
        const int64_t per = n / rows;
        for (int r = 0; r < rows; ++r) {
            const int64_t cnt = r == rows - 1 ? n - per * (rows - 1) : per;
            ggml_backend_tensor_get(y, got.data() + per * r, sizeof(float) * (size_t)(per * r), sizeof(float) * (size_t) cnt);
        }
    };
    auto expect = [&](const std::vector<float> & in, float f, const char * what, int64_t want_mirror, int64_t want_copy) {
        bool same = true;
        for (int64_t i = 0; i < n && same; ++i) same = got[(size_t) i] == in[(size_t) i] * f;
        get_counters(be, c, 1);
        const bool ok = same && c[4] == want_mirror && c[5] == want_copy;
        bad += !ok;
        printf("{\"download\": \"%s\", \"bytes_equal\": %s, \"from_mirror\": %lld, \"by_copy\": %lld, \"ok\": %s}\n", what, same ? "true" : "false", (long long) c[4], (long long) c[5], ok ? "true" : "false");
    };
    get_counters(be, c, 1);
    ggml_backend_tensor_set(x, in1.data(), 0, ggml_nbytes(x));
    if (ggml_backend_graph_compute(be, gf) != GGML_STATUS_SUCCESS) return 1;
    fetch_rows(); expect(in1, 2.0f, "first graph: blocking copies (the tensor is not known yet)", 0, rows);
    ggml_backend_tensor_set(x, in2.data(), 0, ggml_nbytes(x));
    if (ggml_backend_graph_compute(be, gf) != GGML_STATUS_SUCCESS) return 1;
    fetch_rows(); expect(in2, 2.0f, "second graph: served from the pinned mirror", rows, 0);
    fetch_rows(); expect(in2, 2.0f, "read again: still the mirror", rows, 0);
    ggml_backend_tensor_set(y, other.data(), 0, ggml_nbytes(y));               // the host overwrites the result
    fetch_rows(); expect(other, 1.0f, "after a write into the tensor: the mirror is stale, blocking copies", 0, rows);
    ggml_backend_tensor_set(y, in1.data(), sizeof(float) * 100, sizeof(float) * 50);   // (and a partial write, after a new graph)
    if (ggml_backend_graph_compute(be, gf) != GGML_STATUS_SUCCESS) return 1;
    ggml_backend_tensor_set(y, other.data(), sizeof(float) * 100, sizeof(float) * 50);
    fetch_rows();
    { std::vector<float> want((size_t) n); for (int64_t i = 0; i < n; ++i) want[(size_t) i] = (i >= 100 && i < 150) ? other[(size_t)(i - 100)] : 2.0f * in2[(size_t) i];
      expect(want, 1.0f, "after a partial write behind a new graph: blocking copies", 0, rows); }
    double t0 = now_ms();
    for (int i = 0; i < 50; ++i) { if (ggml_backend_graph_compute(be, gf) != GGML_STATUS_SUCCESS) return 1; fetch_rows(); }
    const double ms_mirror = (now_ms() - t0) / 50;
    expect(in2, 2.0f, "timed loop with the mirror", 50 * rows, 0);
    // a result that is read in one piece is not mirrored: one blocking copy is faster than a transfer plus a memcpy
    if (ggml_backend_graph_compute(be, gf) != GGML_STATUS_SUCCESS) return 1;
    ggml_backend_tensor_get(y, got.data(), 0, ggml_nbytes(y));
    expect(in2, 2.0f, "one read after a graph whose predecessor was read in pieces: the mirror", 1, 0);
    if (ggml_backend_graph_compute(be, gf) != GGML_STATUS_SUCCESS) return 1;
    ggml_backend_tensor_get(y, got.data(), 0, ggml_nbytes(y));
    expect(in2, 2.0f, "one read per graph: a blocking copy", 0, 1);

    // the pinned host buffer type: an ordinary host buffer for every CPU-side user, a source of device copies
    ggml_backend_buffer_type_t hbt = ggml_backend_dev_host_buffer_type(dev);
    bool host_ok = hbt && ggml_backend_buft_is_host(hbt);
    if (host_ok) {
        ggml_init_params ip2 = { ggml_tensor_overhead() * 4, nullptr, true };
        ggml_context * hctx = ggml_init(ip2);
        ggml_tensor * hx = ggml_new_tensor_1d(hctx, GGML_TYPE_F32, n);
        ggml_backend_buffer_t hbuf = ggml_backend_alloc_ctx_tensors_from_buft(hctx, hbt);
        host_ok = hbuf && ggml_backend_buffer_is_host(hbuf) && hx->data;
        if (host_ok) {
            memcpy(hx->data, in1.data(), ggml_nbytes(hx));            // host code writes it directly
            ggml_backend_tensor_copy(hx, x);                          // pinned host -> device
            if (ggml_backend_graph_compute(be, gf) != GGML_STATUS_SUCCESS) return 1;
            fetch_rows();
            for (int64_t i = 0; i < n && host_ok; ++i) host_ok = got[(size_t) i] == 2.0f * in1[(size_t) i];
            ggml_backend_tensor_copy(y, hx);                          // device -> pinned host
            ggml_backend_synchronize(be);
            for (int64_t i = 0; i < n && host_ok; ++i) host_ok = ((const float *) hx->data)[i] == 2.0f * in1[(size_t) i];
        }
        if (hbuf) ggml_backend_buffer_free(hbuf);
        ggml_free(hctx);
    }
    bad += !host_ok;
    ggml_backend_dev_props props; ggml_backend_dev_get_props(dev, &props);
    printf("{\"summary\": \"download\", \"failed\": %d, \"host_buffer_type\": \"%s\", \"host_buffer_ok\": %s, \"caps_host_buffer\": %s, \"ms_per_graph_and_5_reads_mirror\": %.4f, \"bytes\": %lld}\n",
           bad, hbt ? ggml_backend_buft_name(hbt) : "", host_ok ? "true" : "false", props.caps.host_buffer ? "true" : "false", ms_mirror, (long long)(n * 4));
    ggml_backend_buffer_free(buf);
    ggml_free(ctx);
    ggml_backend_free(be);
    return bad ? 1 : 0;
}

int main(int argc, char ** argv) {
    if (argc < 2) { fprintf(stderr, "usage: %s info|gen|selftest|ops|model|full|verify|bench|copy|mel|download [options]\n", argv[0]); return 2; }
    ggml_log_set(quiet_log, nullptr);
    whisper_log_set(quiet_log, nullptr);
    const std::string cmd = argv[1];
    const args a = parse_args(argc, argv, 2);
    if (a.has("no-flash-attn")) g_flash_attn = false;
    g_processors = a.num("processors", 1);
    g_gpu_mel = a.has("gpu-mel");
    if (a.has("dtw")) { g_dtw = true; g_flash_attn = false; }        // whisper.cpp turns DTW off under flash attention
    if (cmd == "info")  return cmd_info(a);
    if (cmd == "gen")   return cmd_gen(a);
    if (cmd == "selftest") return cmd_selftest(a);
    if (cmd == "ops")   return cmd_ops(a);
    if (cmd == "model") return cmd_model(a);
    if (cmd == "full")  return cmd_full(a);
    if (cmd == "verify") return cmd_verify(a);
    if (cmd == "bench") return cmd_bench(a);
    if (cmd == "copy")  return cmd_copy(a);
    if (cmd == "mel")   return cmd_mel(a);
    if (cmd == "download") return cmd_download(a);
    if (cmd == "pieces") return cmd_pieces(a);
    fprintf(stderr, "unknown command %s\n", cmd.c_str());
    return 2;
}
