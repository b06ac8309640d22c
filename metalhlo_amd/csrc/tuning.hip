// Autotuner and tuning table: the role of the reference's AutoTuner / TuningDatabase
// (Sources/MetalHLOCore/Tuning/AutoTuner.swift:12-103,301-458, TuningDatabase.swift:15-160).
//
// The search space is what the kernel library can actually launch for a problem:
//   gemm       the compiled GEMM kernels (tile shape x waves x LDS pipeline) that can serve it;
//   row        softmax / LayerNorm / RMSNorm launch forms: one wave per row with the parameters in
//              LDS (persistent grid, resident workgroups per CU searched) or a row split over the
//              waves of a workgroup (one or two rows per wave group, grid in address order or
//              persistent);
//   attention  the 128-row kernel, or the 256-row pipelined kernel with causal tiles unpaired / paired.
// A candidate that the problem's shape, the 160 KB of LDS or the register file rule out is not
// timed (the validity filter).  The measurement is HIP-event time of real launches on the
// caller's stream.  Results are kept per device (architecture name + compute units) and problem
// in a process-wide table that the entry points consult before their heuristics, and can be
// saved to / loaded from a text file (MHIP_TUNING_DB names one to load at first use).  Entries
// of other devices are kept and written back, never used.
#include <dlfcn.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "gemm_common.h"

namespace mhip {

bool gemm256_eligible(const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype, int bw = 256, bool any_tile_count = false);
bool gemm_stream_eligible(const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype);
bool gemm384_activation_ok(int act);
bool gemm_split_shape(const GemmArgs& g, int64_t batch, int* n_wide_out);

namespace {
struct Entry { std::string choice; float us; };
std::mutex g_mu;
std::map<std::string, Entry> g_table;     // "<op> <device> <problem...>" -> choice
bool g_env_loaded = false;
thread_local int g_forced_gemm = 0;
thread_local int g_forced_attention = 0;

// "gfx950/256": architecture name without its feature suffix, and the number of compute units
const std::string& device_key() {
    static std::mutex mu;
    static std::map<int, std::string> cache;
    std::lock_guard<std::mutex> lk(mu);
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = -1;
    auto it = cache.find(dev);
    if (it != cache.end()) return it->second;
    std::string key = "nodevice/0";
    hipDeviceProp_t p;
    if (dev >= 0 && hipGetDeviceProperties(&p, dev) == hipSuccess) {
        std::string arch = p.gcnArchName;
        arch = arch.substr(0, arch.find(':'));
        key = arch + "/" + std::to_string(p.multiProcessorCount);
    } else {
        (void)hipGetLastError();
    }
    return cache.emplace(dev, key).first->second;
}

std::string fmt(const char* f, ...) {
    char buf[256];
    va_list ap;
    va_start(ap, f);
    vsnprintf(buf, sizeof buf, f, ap);
    va_end(ap);
    return buf;
}

std::string gemm_key(int64_t M, int64_t N, int64_t K, int64_t B, int ta, int tb, int dt) {
    return fmt("gemm %s %lld %lld %lld %lld %d %d %d", device_key().c_str(), (long long)M, (long long)N, (long long)K,
               (long long)B, ta, tb, dt);
}
std::string row_key(int op, int dt, int64_t rows, int64_t cols, bool g, bool b) {
    return fmt("row %s %d %d %lld %lld %d %d", device_key().c_str(), op, dt, (long long)rows, (long long)cols, g ? 1 : 0, b ? 1 : 0);
}
std::string attention_key(int dt, int64_t bh, int64_t Sq, int64_t Skv, int64_t D, bool causal) {
    return fmt("attention %s %d %lld %lld %lld %lld %d", device_key().c_str(), dt, (long long)bh, (long long)Sq, (long long)Skv,
               (long long)D, causal ? 1 : 0);
}

bool valid_choice(const char* line, const std::string& choice) {
    int a = 0, b = 0, c = 0, d = 0;
    if (!strncmp(line, "gemm ", 5)) {
        const int v = atoi(choice.c_str());
        return v == 128 || v == 256 || (v >= 2560 && v <= 2570);
    }
    if (!strncmp(line, "row ", 4))
        return sscanf(choice.c_str(), "%d %d %d %d", &a, &b, &c, &d) == 4 && (a == 1 || a == 2) && (b == 1 || b == 2) &&
               (c == 0 || c == 1) && d >= 0 && d <= 64;
    if (!strncmp(line, "attention ", 10)) {
        const int v = atoi(choice.c_str());
        return v >= 1 && v <= 3;
    }
    return false;
}

// one entry per line: "<key> = <choice> @ <microseconds>"
int load_file(const char* path, bool quiet) {
    FILE* f = fopen(path, "r");
    if (!f) return quiet ? MHIP_OK : fail(MHIP_ERR_INVALID_ARGUMENT, "tuning: cannot open %s", path);
    char line[512];
    int st = MHIP_OK;
    while (fgets(line, sizeof line, f)) {
        if (line[0] == '#' || line[0] == '\n') continue;
        char* eq = strstr(line, " = ");
        char* at = eq ? strstr(eq, " @ ") : nullptr;
        float us = 0.f;
        if (!eq || !at || sscanf(at + 3, "%f", &us) != 1 || !valid_choice(line, std::string(eq + 3, at - eq - 3))) {
            st = quiet ? MHIP_OK : fail(MHIP_ERR_INVALID_ARGUMENT, "tuning: malformed line in %s: %s", path, line);
            break;
        }
        g_table[std::string(line, eq - line)] = Entry{std::string(eq + 3, at - eq - 3), us};
    }
    fclose(f);
    return st;
}

// The table that ships with the library: <directory of this shared object>/../tuning/<arch>_<CUs>.txt
// (for the device in use), written by `python -m metalhlo_amd.tune` on such a device.
std::string shipped_table_path() {
    Dl_info info;
    if (!dladdr(reinterpret_cast<const void*>(&shipped_table_path), &info) || !info.dli_fname) return "";
    std::string dir = info.dli_fname;
    const size_t slash = dir.rfind('/');
    dir = slash == std::string::npos ? "." : dir.substr(0, slash);
    std::string dev = device_key();
    std::replace(dev.begin(), dev.end(), '/', '_');
    return dir + "/../tuning/" + dev + ".txt";
}

// False when there is nothing to look up (no key is built then).  At first use the shipped table of
// the device is loaded, then the file MHIP_TUNING_DB names (its entries win); MHIP_TUNING_DB=none
// loads neither.
bool have_entries() {
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_env_loaded) {
        g_env_loaded = true;
        const char* p = getenv("MHIP_TUNING_DB");
        if (!p || strcmp(p, "none") != 0) {
            const std::string shipped = shipped_table_path();
            if (!shipped.empty()) load_file(shipped.c_str(), true);
            if (p && *p) load_file(p, true);
        }
    }
    return !g_table.empty();
}

bool lookup(const std::string& key, std::string* choice) {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_table.find(key);
    if (it == g_table.end()) return false;
    *choice = it->second.choice;
    return true;
}

void record(const std::string& key, const std::string& choice, float us) {
    std::lock_guard<std::mutex> lk(g_mu);
    g_table[key] = Entry{choice, us};
}

struct Timer {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    bool ok() { return hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess; }
    ~Timer() {
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
    }
    // mean microseconds of `iters` calls of fn() after two untimed ones; negative on failure
    template <typename F>
    float time(hipStream_t s, int iters, F&& fn) {
        for (int i = 0; i < 2; i++)
            if (fn() != MHIP_OK) return -1.f;
        (void)hipEventRecord(e0, s);
        for (int i = 0; i < iters; i++)
            if (fn() != MHIP_OK) return -1.f;
        (void)hipEventRecord(e1, s);
        float ms = 0.f;
        if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) {
            fail(MHIP_ERR_LAUNCH, "autotune: timing failed: %s", hipGetErrorString(hipGetLastError()));
            return -1.f;
        }
        return ms * 1000.f / (float)iters;
    }
};
}  // namespace

// Variant a tuned entry (or a running tuning pass) prescribes for this problem; 0 = none.
int tuned_gemm_variant(const GemmArgs& g, int64_t batch, int ta, int tb, int dtype) {
    if (g_forced_gemm) return g_forced_gemm;
    std::string c;
    if (!have_entries() || !lookup(gemm_key(g.M, g.N, g.K, batch, ta, tb, dtype), &c)) return 0;
    const int v = atoi(c.c_str());
    return (v == 128 || v == 256 || (v >= 2560 && v <= 2570)) ? v : 0;
}

bool tuned_row_launch(int op, int dtype, int64_t rows, int64_t cols, bool has_gamma, bool has_beta, RowLaunch* out) {
    std::string c;
    if (!have_entries() || !lookup(row_key(op, dtype, rows, cols, has_gamma, has_beta), &c)) return false;
    RowLaunch r;
    if (sscanf(c.c_str(), "%d %d %d %d", &r.kind, &r.r, &r.ordered, &r.per_cu) != 4) return false;
    if ((r.kind != 1 && r.kind != 2) || r.r < 1 || r.r > 2 || r.ordered < 0 || r.ordered > 1 || r.per_cu < 0 || r.per_cu > 64) return false;
    *out = r;
    return true;
}

int tuned_attention_variant(int dtype, int64_t batch_heads, int64_t Sq, int64_t Skv, int64_t D, bool causal) {
    if (g_forced_attention) return g_forced_attention;
    std::string c;
    if (!have_entries() || !lookup(attention_key(dtype, batch_heads, Sq, Skv, D, causal), &c)) return 0;
    const int v = atoi(c.c_str());
    return v >= 1 && v <= 3 ? v : 0;
}

}  // namespace mhip

using namespace mhip;

// GEMM candidates a problem can run (the validity filter: shape, alignment, LDS and tile count rules of each kernel).
static std::vector<int> gemm_candidates(const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype) {
    std::vector<int> out;
    for (int v : {128, 256, 2560, 2561, 2562, 2563, 2564, 2565, 2566, 2567, 2568, 2569, 2570}) {
        if ((v == 2560 || v == 2566) && !gemm256_eligible(g, batch, trans_a, trans_b, dtype)) continue;
        if ((v == 2561 || v == 2564 || v == 2565 || v == 2568) && !gemm256_eligible(g, batch, trans_a, trans_b, dtype, 128)) continue;
        if (v == 2570 && !(gemm256_eligible(g, batch, trans_a, trans_b, dtype, 288) && gemm384_activation_ok(g.act))) continue;
        if (v == 2569 && !gemm256_eligible(g, batch, trans_a, trans_b, dtype, 192)) continue;
        if (v == 2567 && !(gemm256_eligible(g, batch, trans_a, trans_b, dtype, 384) && gemm384_activation_ok(g.act))) continue;
        if (v == 2562 && !gemm_stream_eligible(g, batch, trans_a, trans_b, dtype)) continue;
        if (v == 2563 && !(gemm_split_shape(g, batch, nullptr) && gemm256_eligible(g, batch, trans_a, trans_b, dtype))) continue;
        out.push_back(v);
    }
    return out;
}

extern "C" int mhip_gemm_autotune(void* stream, const void* a, const void* b, const void* bias, void* c,
                                  int64_t M, int64_t N, int64_t K, int64_t batch, int64_t stride_a,
                                  int64_t stride_b, int64_t stride_c, int trans_a, int trans_b,
                                  int activation, int dtype, int iters, int* out_variant, float* out_us) {
    if (dtype != MHIP_BF16 && dtype != MHIP_F16)
        return fail(MHIP_ERR_UNSUPPORTED, "mhip_gemm_autotune: only the 16-bit MFMA kernels have variants");
    if (iters <= 0 || M <= 0 || N <= 0 || K <= 0 || batch <= 0 || !a || !b || !c)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_gemm_autotune: bad argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    if (!t.ok()) return fail(MHIP_ERR_LAUNCH, "mhip_gemm_autotune: cannot create events");
    GemmArgs g{};
    g.a = a; g.b = b; g.bias = bias; g.c = c;
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.lda = (int)(trans_a ? M : K); g.ldb = (int)(trans_b ? K : N);
    g.sa = stride_a; g.sb = stride_b; g.sc = stride_c;
    g.act = activation;
    const std::vector<int> cand = gemm_candidates(g, batch, trans_a, trans_b, dtype);
    std::vector<float> us(cand.size(), -1.f);
    // two passes over the candidates, the better time of each counts: the first candidates of the
    // first pass run on a device that is still raising its clocks
    for (int pass = 0; pass < 2; pass++)
        for (size_t i = 0; i < cand.size(); i++) {
            g_forced_gemm = cand[i];
            const float t_us = t.time(s, iters, [&] {
                return mhip_gemm(stream, a, b, bias, c, M, N, K, batch, stride_a, stride_b, stride_c, trans_a, trans_b, activation, dtype);
            });
            g_forced_gemm = 0;
            if (t_us < 0.f) return MHIP_ERR_LAUNCH;
            if (us[i] < 0.f || t_us < us[i]) us[i] = t_us;
        }
    size_t best = 0;
    for (size_t i = 1; i < cand.size(); i++)
        if (us[i] < us[best]) best = i;
    record(gemm_key(M, N, K, batch, trans_a, trans_b, dtype), std::to_string(cand[best]), us[best]);
    if (out_variant) *out_variant = cand[best];
    if (out_us) *out_us = us[best];
    return MHIP_OK;
}

// The same search with every launch timed on its own as a model finds its operands: `flush` is
// overwritten first (64 to 128 MB empty the L2s and leave most of the 256 MB memory-side cache, the
// state of weights that were written a millisecond ago; 512 MB and more empty both), then A is
// rewritten in place the way the kernel in front of a GEMM leaves its result, then one launch between
// two events.  The median of `iters` such launches decides.  A GEMM in a loop of its own finds both
// operands in the caches, which favours other tile widths and ring depths than a model does.
extern "C" int mhip_gemm_autotune_in_model(void* stream, const void* a, const void* b, const void* bias, void* c,
                                           int64_t M, int64_t N, int64_t K, int64_t batch, int64_t stride_a,
                                           int64_t stride_b, int64_t stride_c, int trans_a, int trans_b,
                                           int activation, int dtype, int iters, void* flush, int64_t flush_bytes,
                                           int* out_variant, float* out_us) {
    if (dtype != MHIP_BF16 && dtype != MHIP_F16)
        return fail(MHIP_ERR_UNSUPPORTED, "mhip_gemm_autotune_in_model: only the 16-bit MFMA kernels have variants");
    if (iters <= 0 || M <= 0 || N <= 0 || K <= 0 || batch <= 0 || !a || !b || !c || !flush || flush_bytes < (64ll << 20))
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_gemm_autotune_in_model: bad argument (the flush buffer needs at least 64 MB)");
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    if (!t.ok()) return fail(MHIP_ERR_LAUNCH, "mhip_gemm_autotune_in_model: cannot create events");
    GemmArgs g{};
    g.a = a; g.b = b; g.bias = bias; g.c = c;
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.lda = (int)(trans_a ? M : K); g.ldb = (int)(trans_b ? K : N);
    g.sa = stride_a; g.sb = stride_b; g.sc = stride_c;
    g.act = activation;
    const int64_t a_bytes = (batch == 1 || stride_a == M * K) ? M * K * batch * 2 : M * K * 2;
    int best = 0;
    float best_us = 0.f;
    std::vector<float> us(iters);
    for (int v : gemm_candidates(g, batch, trans_a, trans_b, dtype)) {
        for (int i = -1; i < iters; i++) {            // launch -1 is not counted
            if (mhip_fill(stream, flush, flush_bytes / 4, (uint64_t)(i + 2), 4) != MHIP_OK) return MHIP_ERR_LAUNCH;
            if (mhip_copy(stream, a, const_cast<void*>(a), a_bytes) != MHIP_OK) return MHIP_ERR_LAUNCH;
            (void)hipEventRecord(t.e0, s);
            g_forced_gemm = v;
            const int st = mhip_gemm(stream, a, b, bias, c, M, N, K, batch, stride_a, stride_b, stride_c, trans_a, trans_b, activation, dtype);
            g_forced_gemm = 0;
            if (st != MHIP_OK) return st;
            (void)hipEventRecord(t.e1, s);
            float ms = 0.f;
            if (hipEventSynchronize(t.e1) != hipSuccess || hipEventElapsedTime(&ms, t.e0, t.e1) != hipSuccess)
                return fail(MHIP_ERR_LAUNCH, "autotune: timing failed: %s", hipGetErrorString(hipGetLastError()));
            if (i >= 0) us[i] = ms * 1000.f;
        }
        std::sort(us.begin(), us.end());
        const float med = us[iters / 2];
        if (!best || med < best_us) { best = v; best_us = med; }
    }
    record(gemm_key(M, N, K, batch, trans_a, trans_b, dtype), std::to_string(best), best_us);
    if (out_variant) *out_variant = best;
    if (out_us) *out_us = best_us;
    return MHIP_OK;
}

// A search that times something larger than one kernel (a whole forward pass, say) records its
// result here: the GEMM problem's entry becomes `variant` (0 removes the entry).
extern "C" int mhip_tuning_set_gemm(int64_t M, int64_t N, int64_t K, int64_t batch, int trans_a, int trans_b, int dtype,
                                    int variant, float us) {
    const std::string key = gemm_key(M, N, K, batch, trans_a, trans_b, dtype);
    if (variant == 0) {
        std::lock_guard<std::mutex> lk(g_mu);
        g_table.erase(key);
        g_env_loaded = true;
        return MHIP_OK;
    }
    if (!valid_choice("gemm ", std::to_string(variant)))
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_tuning_set_gemm: %d is no kernel variant", variant);
    {
        std::lock_guard<std::mutex> lk(g_mu);
        g_env_loaded = true;
    }
    record(key, std::to_string(variant), us);
    return MHIP_OK;
}

extern "C" int mhip_row_autotune(void* stream, int op, const void* x, const void* gamma, const void* beta, void* y,
                                 int64_t rows, int64_t cols, float eps, int dtype, int iters, int* out_choice,
                                 float* out_us) {
    if (op < 0 || op > 2) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_row_autotune: operator %d (0 softmax, 1 LayerNorm, 2 RMSNorm)", op);
    if (iters <= 0 || rows <= 0 || cols <= 0 || !x || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_row_autotune: bad argument");
    const int elems = dtype == MHIP_F32 ? 4 : (dtype == MHIP_BF16 || dtype == MHIP_F16) ? 8 : 0;
    if (!elems) return fail(MHIP_ERR_UNSUPPORTED, "mhip_row_autotune: dtype %d (need f32, f16 or bf16)", dtype);
    auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (cols % elems || cols > 64 * 16 * elems || !al(x) || !al(y) || !al(gamma) || !al(beta))
        return fail(MHIP_ERR_UNSUPPORTED, "mhip_row_autotune: rows that are not 16-byte vectors (or too long for registers) have one launch form");
    if (op == 0) gamma = beta = nullptr;
    if (op == 2) beta = nullptr;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    if (!t.ok()) return fail(MHIP_ERR_LAUNCH, "mhip_row_autotune: cannot create events");
    const int64_t nvec = cols / elems;
    const size_t param_bytes = (size_t)cols * (dtype == MHIP_F32 ? 4 : 2) * ((gamma ? 1 : 0) + (beta ? 1 : 0));
    RowLaunch best;
    float best_us = -1.f;
    auto consider = [&](const RowLaunch& c) -> int {
        const float us = t.time(s, iters, [&] { return row_launch_as(op, c, stream, x, gamma, beta, y, rows, cols, eps, dtype); });
        if (us < 0.f) return MHIP_ERR_LAUNCH;
        if (best_us < 0.f || us < best_us) { best = c; best_us = us; }
        return MHIP_OK;
    };
    // one wave per row, parameters in LDS: resident workgroups per CU searched; the staged
    // parameters of every resident workgroup must fit the 160 KB of LDS
    for (int per_cu : {0, 2, 4, 6, 8}) {
        if (per_cu && param_bytes && (size_t)per_cu * (param_bytes + 512) > 160 * 1024 - 4096) continue;
        RowLaunch c; c.kind = 1; c.r = 1; c.ordered = 0; c.per_cu = per_cu;
        if (consider(c) != MHIP_OK) return MHIP_ERR_LAUNCH;
    }
    // a row split over the waves of a workgroup: needs more than one wave's worth of vectors
    if (nvec > 64) {
        for (int r : {1, 2})
            for (int ordered : {1, 0})
                for (int per_cu : {0, 8, 16}) {
                    if (ordered && per_cu) continue;            // a grid in address order has no residency to choose
                    RowLaunch c; c.kind = 2; c.r = r; c.ordered = ordered; c.per_cu = per_cu;
                    if (consider(c) != MHIP_OK) return MHIP_ERR_LAUNCH;
                }
    }
    record(row_key(op, dtype, rows, cols, gamma != nullptr, beta != nullptr),
           fmt("%d %d %d %d", best.kind, best.r, best.ordered, best.per_cu), best_us);
    if (out_choice) { out_choice[0] = best.kind; out_choice[1] = best.r; out_choice[2] = best.ordered; out_choice[3] = best.per_cu; }
    if (out_us) *out_us = best_us;
    return MHIP_OK;
}

extern "C" int mhip_attention_autotune(void* stream, const void* q, const void* k, const void* v, void* o, int64_t B,
                                       int64_t H, int64_t Sq, int64_t Skv, int64_t D, float scale, int is_causal,
                                       int dtype, int iters, int* out_variant, float* out_us) {
    if (dtype != MHIP_BF16 && dtype != MHIP_F16)
        return fail(MHIP_ERR_UNSUPPORTED, "mhip_attention_autotune: only the 16-bit MFMA kernels have variants");
    if (D != 64 && D != 128) return fail(MHIP_ERR_UNSUPPORTED, "mhip_attention_autotune: head size %lld has one kernel", (long long)D);
    if (iters <= 0 || B <= 0 || H <= 0 || Sq <= 0 || Skv <= 0 || !q || !k || !v || !o)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_attention_autotune: bad argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    Timer t;
    if (!t.ok()) return fail(MHIP_ERR_LAUNCH, "mhip_attention_autotune: cannot create events");
    int best = 0;
    float best_us = 0.f;
    for (int variant : {1, 2, 3}) {
        // validity: the 256-row kernel serves head size 128 and at least one full tile; pairing is a causal notion
        if (variant >= 2 && (D != 128 || Sq < 256)) continue;
        if (variant == 3 && !is_causal) continue;
        g_forced_attention = variant;
        const float us = t.time(s, iters, [&] {
            return mhip_flash_attention(stream, q, k, v, nullptr, o, B, H, Sq, Skv, D, scale, is_causal, 0, 0, dtype);
        });
        g_forced_attention = 0;
        if (us < 0.f) return MHIP_ERR_LAUNCH;
        if (!best || us < best_us) { best = variant; best_us = us; }
    }
    record(attention_key(dtype, B * H, Sq, Skv, D, is_causal != 0), std::to_string(best), best_us);
    if (out_variant) *out_variant = best;
    if (out_us) *out_us = best_us;
    return MHIP_OK;
}

extern "C" int mhip_tuning_save(const char* path) {
    if (!path) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_tuning_save: NULL path");
    FILE* f = fopen(path, "w");
    if (!f) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_tuning_save: cannot open %s", path);
    fprintf(f, "# <operator> <device: architecture/compute units> <problem> = <choice> @ <microseconds>\n"
               "#   gemm ... M N K batch trans_a trans_b dtype = kernel variant\n"
               "#   row ... operator dtype rows cols has_gamma has_beta = kind rows_per_group ordered per_cu\n"
               "#   attention ... dtype batch*heads Sq Skv D causal = kernel variant\n");
    std::lock_guard<std::mutex> lk(g_mu);
    for (auto& kv : g_table) fprintf(f, "%s = %s @ %.3f\n", kv.first.c_str(), kv.second.choice.c_str(), kv.second.us);
    fclose(f);
    return MHIP_OK;
}

extern "C" int mhip_tuning_load(const char* path) {
    if (!path) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_tuning_load: NULL path");
    std::lock_guard<std::mutex> lk(g_mu);
    return load_file(path, false);
}

extern "C" void mhip_tuning_clear(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    g_table.clear();
    g_env_loaded = true;        // an explicit clear also cancels the automatic load at first use
}

extern "C" int mhip_tuning_count(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    return (int)g_table.size();
}

extern "C" const char* mhip_tuning_device(void) { return device_key().c_str(); }
