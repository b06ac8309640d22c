// Autotuner for the GEMM kernel choice and its tuning table: the role of the
// reference's AutoTuner / TuningDatabase (Sources/MetalHLOCore/Tuning/AutoTuner.swift:
// 301-458, TuningDatabase.swift:15-160).  The search space here is the set of compiled
// GEMM kernels (tile shape x waves x LDS pipeline) that can serve a problem; the
// measurement is HIP-event time of real launches on the caller's stream.  Results are
// kept per (M, N, K, batch, layout, dtype) in a process-wide table that mhip_gemm
// consults before its heuristic, and can be saved to / loaded from a text file
// (MHIP_TUNING_DB names one to load at first use).
#include <stdio.h>
#include <string.h>

#include <map>
#include <mutex>
#include <tuple>

#include "gemm_common.h"

namespace mhip {

bool gemm256_eligible(const GemmArgs& g, int64_t batch, int dtype, int bw = 256);

namespace {
using Key = std::tuple<int64_t, int64_t, int64_t, int64_t, int, int, int>;
struct Entry { int variant; float us; };
std::mutex g_mu;
std::map<Key, Entry> g_table;
bool g_env_loaded = false;
thread_local int g_forced = 0;

int load_file(const char* path, bool quiet) {
    FILE* f = fopen(path, "r");
    if (!f) return quiet ? MHIP_OK : fail(MHIP_ERR_INVALID_ARGUMENT, "tuning: cannot open %s", path);
    char line[256];
    int st = MHIP_OK;
    while (fgets(line, sizeof line, f)) {
        if (line[0] == '#' || line[0] == '\n') continue;
        long long M, N, K, B;
        int ta, tb, dt, variant;
        float us;
        if (sscanf(line, "gemm %lld %lld %lld %lld %d %d %d %d %f", &M, &N, &K, &B, &ta, &tb, &dt, &variant, &us) != 9 ||
            (variant != 128 && variant != 256 && variant != 2560 && variant != 2561)) {
            st = quiet ? MHIP_OK : fail(MHIP_ERR_INVALID_ARGUMENT, "tuning: malformed line in %s: %s", path, line);
            break;
        }
        g_table[Key(M, N, K, B, ta, tb, dt)] = Entry{variant, us};
    }
    fclose(f);
    return st;
}
}  // namespace

// Variant a tuned entry (or a running tuning pass) prescribes for this problem; 0 = none.
int tuned_gemm_variant(const GemmArgs& g, int64_t batch, int ta, int tb, int dtype) {
    if (g_forced) return g_forced;
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_env_loaded) {
        g_env_loaded = true;
        const char* p = getenv("MHIP_TUNING_DB");
        if (p && *p) load_file(p, true);
    }
    if (g_table.empty()) return 0;
    auto it = g_table.find(Key(g.M, g.N, g.K, batch, ta, tb, dtype));
    return it == g_table.end() ? 0 : it->second.variant;
}

bool tuned_row_launch(int, int, int64_t, int64_t, bool, bool, RowLaunch*) { return false; }

}  // namespace mhip

using namespace mhip;

extern "C" int mhip_gemm_autotune(void* stream, const void* a, const void* b, const void* bias, void* c,
                                  int64_t M, int64_t N, int64_t K, int64_t batch, int64_t stride_a,
                                  int64_t stride_b, int64_t stride_c, int trans_a, int trans_b,
                                  int activation, int dtype, int iters, int* out_variant, float* out_us) {
    if (dtype != MHIP_BF16 && dtype != MHIP_F16)
        return fail(MHIP_ERR_UNSUPPORTED, "mhip_gemm_autotune: only the 16-bit MFMA kernels have variants");
    if (iters <= 0 || M <= 0 || N <= 0 || K <= 0 || batch <= 0 || !a || !b || !c)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_gemm_autotune: bad argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)
        return fail(MHIP_ERR_LAUNCH, "mhip_gemm_autotune: cannot create events");
    GemmArgs g{};
    g.a = a; g.b = b; g.bias = bias; g.c = c;
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.sa = stride_a; g.sb = stride_b; g.sc = stride_c;
    const int candidates[4] = {128, 256, 2560, 2561};
    int best = 0, st = MHIP_OK;
    float best_us = 0.f;
    for (int v : candidates) {
        if (v == 2560 && !gemm256_eligible(g, batch, dtype)) continue;    // validity filter
        if (v == 2561 && !gemm256_eligible(g, batch, dtype, 128)) continue;
        g_forced = v;
        for (int i = 0; i < 2 && st == MHIP_OK; i++)
            st = mhip_gemm(stream, a, b, bias, c, M, N, K, batch, stride_a, stride_b, stride_c, trans_a, trans_b, activation, dtype);
        if (st == MHIP_OK) {
            (void)hipEventRecord(e0, s);
            for (int i = 0; i < iters && st == MHIP_OK; i++)
                st = mhip_gemm(stream, a, b, bias, c, M, N, K, batch, stride_a, stride_b, stride_c, trans_a, trans_b, activation, dtype);
            (void)hipEventRecord(e1, s);
        }
        g_forced = 0;
        if (st != MHIP_OK) break;
        float ms = 0.f;
        if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) {
            st = fail(MHIP_ERR_LAUNCH, "mhip_gemm_autotune: timing failed: %s", hipGetErrorString(hipGetLastError()));
            break;
        }
        const float us = ms * 1000.f / (float)iters;
        if (!best || us < best_us) { best = v; best_us = us; }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (st != MHIP_OK) return st;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        g_table[Key(M, N, K, batch, trans_a, trans_b, dtype)] = Entry{best, best_us};
    }
    if (out_variant) *out_variant = best;
    if (out_us) *out_us = best_us;
    return MHIP_OK;
}

extern "C" int mhip_tuning_save(const char* path) {
    if (!path) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_tuning_save: NULL path");
    FILE* f = fopen(path, "w");
    if (!f) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_tuning_save: cannot open %s", path);
    fprintf(f, "# gemm M N K batch trans_a trans_b dtype variant microseconds\n");
    std::lock_guard<std::mutex> lk(g_mu);
    for (auto& kv : g_table) {
        const Key& k = kv.first;
        fprintf(f, "gemm %lld %lld %lld %lld %d %d %d %d %.3f\n", (long long)std::get<0>(k), (long long)std::get<1>(k),
                (long long)std::get<2>(k), (long long)std::get<3>(k), std::get<4>(k), std::get<5>(k), std::get<6>(k),
                kv.second.variant, kv.second.us);
    }
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
}

extern "C" int mhip_tuning_count(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    return (int)g_table.size();
}
