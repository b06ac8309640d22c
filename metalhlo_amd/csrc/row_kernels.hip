// Bandwidth-bound row operators for gfx950: softmax, LayerNorm, RMSNorm, bias+GELU.
//
// Fast path: one 64-lane wavefront owns one row and keeps the whole row in
// VGPRs (NV 128-bit vectors per lane), so HBM sees exactly one read and one
// write per element; reductions are cross-lane only (no LDS, no barrier).
// Four waves per workgroup -> four rows per workgroup, grid = rows / 4.
// Rows that are too long for registers, or whose byte length is not a multiple
// of 16, take a workgroup-per-row multi-pass path.
#include <math.h>

#include "common.h"

namespace mhip {

enum RowOp { kSoftmax = 0, kLayerNorm = 1, kRmsNorm = 2 };

constexpr int kRowsPerBlock = 4;

// Per-column parameters (gamma, beta, bias) are converted to fp32 once per
// workgroup and parked in LDS, split into planes of four floats so that the
// 64 lanes of a wave read 64 consecutive 16-byte slots (no bank conflicts);
// each workgroup then walks many rows, so the parameters cost no HBM or L2
// traffic per row.
template <typename T>
__device__ inline void stage_params(const T* __restrict__ p, f32x4* lds, int nvec) {
    constexpr int E = Elem<T>::kPerVec;
    for (int i = threadIdx.x; i < nvec; i += 256) {
        const Vec16<T> t = load16(p + (int64_t)i * E);
#pragma unroll
        for (int q = 0; q < E / 4; q++) {
            f32x4 w;
#pragma unroll
            for (int e = 0; e < 4; e++) w[e] = Elem<T>::to_f32(t.v[4 * q + e]);
            lds[q * nvec + i] = w;
        }
    }
}

// The same, kept in the storage type (one 16-byte vector per 16 bytes of LDS): half the
// LDS of the fp32 planes for 16-bit types, so more workgroups fit on a CU, and one LDS
// read per vector instead of two; the widening to fp32 happens at the use.
template <typename T>
__device__ inline void stage_params_raw(const T* __restrict__ p, Vec16<T>* lds, int nvec) {
    constexpr int E = Elem<T>::kPerVec;
    for (int i = threadIdx.x; i < nvec; i += 256) lds[i] = load16(p + (int64_t)i * E);
}

template <typename T, int OP, int NV>
__global__ __launch_bounds__(256) void row_wave_kernel(const T* __restrict__ x,
                                                       const T* __restrict__ gamma,
                                                       const T* __restrict__ beta,
                                                       T* __restrict__ y, int64_t rows, int cols,
                                                       float eps) {
    constexpr int E = Elem<T>::kPerVec;
    extern __shared__ __attribute__((aligned(16))) char row_params[];
    const int lane = threadIdx.x & 63;
    const int nvec = cols / E;
    Vec16<T>* gs = reinterpret_cast<Vec16<T>*>(row_params);
    Vec16<T>* bs = gs + (gamma ? nvec : 0);
    if (OP != kSoftmax && (gamma || beta)) {
        if (gamma) stage_params_raw(gamma, gs, nvec);
        if (OP == kLayerNorm && beta) stage_params_raw(beta, bs, nvec);
        __syncthreads();
    }

    for (int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6); row < rows;
         row += (int64_t)gridDim.x * kRowsPerBlock) {
        const T* xr = x + row * cols;
        T* yr = y + row * cols;

        float f[NV][E];
#pragma unroll
        for (int v = 0; v < NV; v++) {
            const int idx = v * 64 + lane;
            if (idx < nvec) {
                Vec16<T> t = load16_stream(xr + (int64_t)idx * E);
#pragma unroll
                for (int e = 0; e < E; e++) f[v][e] = Elem<T>::to_f32(t.v[e]);
            } else {
#pragma unroll
                for (int e = 0; e < E; e++) f[v][e] = (OP == kSoftmax) ? -INFINITY : 0.f;
            }
        }

        float a = 0.f, b = 0.f;  // per-row statistics; meaning depends on OP
        if (OP == kSoftmax) {
            float m = -INFINITY;
#pragma unroll
            for (int v = 0; v < NV; v++)
#pragma unroll
                for (int e = 0; e < E; e++) m = fmaxf(m, f[v][e]);
            m = wave_max(m);
            float s = 0.f;
#pragma unroll
            for (int v = 0; v < NV; v++)
#pragma unroll
                for (int e = 0; e < E; e++) {
                    float ex = (sizeof(T) == 4) ? expf(f[v][e] - m)
                                                : __builtin_amdgcn_exp2f((f[v][e] - m) * 1.4426950408889634f);
                    f[v][e] = ex;
                    s += ex;
                }
            s = wave_sum(s);
            a = 1.f / s;
        } else if (OP == kLayerNorm) {
            float s = 0.f;
#pragma unroll
            for (int v = 0; v < NV; v++)
#pragma unroll
                for (int e = 0; e < E; e++) s += f[v][e];
            const float mean = wave_sum(s) / (float)cols;
            float q = 0.f;
#pragma unroll
            for (int v = 0; v < NV; v++) {
                if (v * 64 + lane < nvec) {
#pragma unroll
                    for (int e = 0; e < E; e++) {
                        const float d = f[v][e] - mean;
                        q += d * d;
                    }
                }
            }
            const float var = wave_sum(q) / (float)cols;
            b = 1.f / sqrtf(var + eps);
            a = -mean * b;
        } else {
            float q = 0.f;
#pragma unroll
            for (int v = 0; v < NV; v++)
#pragma unroll
                for (int e = 0; e < E; e++) q += f[v][e] * f[v][e];
            a = 1.f / sqrtf(wave_sum(q) / (float)cols + eps);
        }

#pragma unroll
        for (int v = 0; v < NV; v++) {
            const int idx = v * 64 + lane;
            if (idx < nvec) {
                Vec16<T> o;
                if (OP == kSoftmax) {
#pragma unroll
                    for (int e = 0; e < E; e++) o.v[e] = Elem<T>::from_f32(f[v][e] * a);
                } else {
                    Vec16<T> gv, bv;
                    if (gamma) gv = gs[idx];
                    if (OP == kLayerNorm && beta) bv = bs[idx];
#pragma unroll
                    for (int e = 0; e < E; e++) {
                        const float g = gamma ? Elem<T>::to_f32(gv.v[e]) : 1.f;
                        const float bt = (OP == kLayerNorm && beta) ? Elem<T>::to_f32(bv.v[e]) : 0.f;
                        const float xv = f[v][e];
                        // LayerNorm: (x - mean) * rstd == x * rstd + (-mean * rstd)
                        const float n = (OP == kLayerNorm) ? fmaf(xv, b, a) : xv * a;
                        o.v[e] = Elem<T>::from_f32(fmaf(n, g, bt));
                    }
                }
                store16_stream(yr + (int64_t)idx * E, o);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// General path: one workgroup per row, scalar accesses, statistics reduced
// through LDS.  Any `cols`, any alignment.
// ---------------------------------------------------------------------------
__device__ inline float block_reduce(float v, bool is_max, float* lds) {
    v = is_max ? wave_max(v) : wave_sum(v);
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) lds[w] = v;
    __syncthreads();
    float r = lds[0];
    for (int i = 1; i < (int)(blockDim.x >> 6); i++) r = is_max ? fmaxf(r, lds[i]) : r + lds[i];
    return r;
}

template <typename T, int OP>
__global__ __launch_bounds__(256) void row_block_kernel(const T* __restrict__ x,
                                                        const T* __restrict__ gamma,
                                                        const T* __restrict__ beta,
                                                        T* __restrict__ y, int64_t cols,
                                                        float eps) {
    __shared__ float lds[4];
    const T* xr = x + (int64_t)blockIdx.x * cols;
    T* yr = y + (int64_t)blockIdx.x * cols;
    const int t = threadIdx.x;
    if (OP == kSoftmax) {
        float m = -INFINITY;
        for (int64_t c = t; c < cols; c += 256) m = fmaxf(m, Elem<T>::to_f32(xr[c]));
        m = block_reduce(m, true, lds);
        float s = 0.f;
        for (int64_t c = t; c < cols; c += 256) s += expf(Elem<T>::to_f32(xr[c]) - m);
        s = block_reduce(s, false, lds);
        const float inv = 1.f / s;
        for (int64_t c = t; c < cols; c += 256)
            yr[c] = Elem<T>::from_f32(expf(Elem<T>::to_f32(xr[c]) - m) * inv);
    } else if (OP == kLayerNorm) {
        float s = 0.f;
        for (int64_t c = t; c < cols; c += 256) s += Elem<T>::to_f32(xr[c]);
        const float mean = block_reduce(s, false, lds) / (float)cols;
        float q = 0.f;
        for (int64_t c = t; c < cols; c += 256) {
            const float d = Elem<T>::to_f32(xr[c]) - mean;
            q += d * d;
        }
        const float inv = 1.f / sqrtf(block_reduce(q, false, lds) / (float)cols + eps);
        for (int64_t c = t; c < cols; c += 256) {
            float v = (Elem<T>::to_f32(xr[c]) - mean) * inv;
            if (gamma) v *= Elem<T>::to_f32(gamma[c]);
            if (beta) v += Elem<T>::to_f32(beta[c]);
            yr[c] = Elem<T>::from_f32(v);
        }
    } else {
        float q = 0.f;
        for (int64_t c = t; c < cols; c += 256) {
            const float v = Elem<T>::to_f32(xr[c]);
            q += v * v;
        }
        const float inv = 1.f / sqrtf(block_reduce(q, false, lds) / (float)cols + eps);
        for (int64_t c = t; c < cols; c += 256) {
            float v = Elem<T>::to_f32(xr[c]) * inv;
            if (gamma) v *= Elem<T>::to_f32(gamma[c]);
            yr[c] = Elem<T>::from_f32(v);
        }
    }
}

// Softmax over a middle axis of [outer, len, inner]: one thread per
// (outer, inner) column; neighbouring threads read neighbouring addresses.
template <typename T>
__global__ __launch_bounds__(256) void softmax_strided_kernel(const T* __restrict__ x,
                                                              T* __restrict__ y, int64_t outer,
                                                              int64_t len, int64_t inner) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= outer * inner) return;
    const int64_t base = (gid / inner) * len * inner + (gid % inner);
    float m = -INFINITY;
    for (int64_t i = 0; i < len; i++) m = fmaxf(m, Elem<T>::to_f32(x[base + i * inner]));
    float s = 0.f;
    for (int64_t i = 0; i < len; i++) s += expf(Elem<T>::to_f32(x[base + i * inner]) - m);
    const float inv = 1.f / s;
    for (int64_t i = 0; i < len; i++)
        y[base + i * inner] = Elem<T>::from_f32(expf(Elem<T>::to_f32(x[base + i * inner]) - m) * inv);
}

// ---------------------------------------------------------------------------
// bias + GELU(tanh): pure streaming; the bias sits in LDS as fp32 planes.
// ---------------------------------------------------------------------------
template <typename T>
__device__ inline float gelu_tanh_f(float v) {
    if (sizeof(T) == 4) {
        const float inner = 0.7978845608028654f * (v + 0.044715f * v * v * v);
        return 0.5f * v * (1.f + tanhf(inner));
    }
    // 0.5 (1 + tanh u) == 1 / (1 + exp(-2u)) == 1 / (1 + 2^(-2 log2(e) u)); ample for
    // a 16-bit result and three VALU + two transcendental operations.
    constexpr float c0 = -2.f * 1.4426950408889634f * 0.7978845608028654f;
    constexpr float c1 = c0 * 0.044715f;
    const float t = v * fmaf(v * v, c1, c0);
    return v * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(t));
}

template <typename T>
__global__ __launch_bounds__(256) void bias_gelu_vec_kernel(const T* __restrict__ x,
                                                            const T* __restrict__ bias,
                                                            T* __restrict__ y, int64_t nvec,
                                                            int nvec_row, int bias_in_lds) {
    constexpr int E = Elem<T>::kPerVec;
    constexpr int P = E / 4;
    extern __shared__ __attribute__((aligned(16))) f32x4 gelu_params[];
    if (bias && bias_in_lds) {
        stage_params(bias, gelu_params, nvec_row);
        __syncthreads();
    }
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i0 = (int64_t)blockIdx.x * 256 + threadIdx.x; i0 < nvec; i0 += 2 * stride) {
        const int64_t i1 = i0 + stride;
        const bool two = i1 < nvec;
        Vec16<T> in0 = load16_stream(x + i0 * E), in1;
        if (two) in1 = load16_stream(x + i1 * E);
#pragma unroll
        for (int u = 0; u < 2; u++) {
            if (u == 1 && !two) break;
            const int64_t i = u ? i1 : i0;
            const Vec16<T>& in = u ? in1 : in0;
            Vec16<T> o;
            const int cv = (int)(i % nvec_row);
#pragma unroll
            for (int q = 0; q < P; q++) {
                f32x4 bv = {0.f, 0.f, 0.f, 0.f};
                if (bias) {
                    if (bias_in_lds) {
                        bv = gelu_params[q * nvec_row + cv];
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++) bv[e] = Elem<T>::to_f32(bias[(int64_t)cv * E + 4 * q + e]);
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; e++)
                    o.v[4 * q + e] = Elem<T>::from_f32(
                        gelu_tanh_f<T>(Elem<T>::to_f32(in.v[4 * q + e]) + bv[e]));
            }
            store16_stream(y + i * E, o);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void bias_gelu_scalar_kernel(const T* __restrict__ x,
                                                               const T* __restrict__ bias,
                                                               T* __restrict__ y, int64_t n,
                                                               int64_t cols) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float v = Elem<T>::to_f32(x[i]);
    if (bias) v += Elem<T>::to_f32(bias[i % cols]);
    y[i] = Elem<T>::from_f32(gelu_tanh_f<T>(v));
}

// ---------------------------------------------------------------------------
// Host-side dispatch
// ---------------------------------------------------------------------------
static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T, int OP>
static int launch_row(hipStream_t s, const void* x, const void* g, const void* b, void* y,
                      int64_t rows, int64_t cols, float eps) {
    constexpr int E = Elem<T>::kPerVec;
    const T* xp = static_cast<const T*>(x);
    const T* gp = static_cast<const T*>(g);
    const T* bp = static_cast<const T*>(b);
    T* yp = static_cast<T*>(y);
    const bool vec_ok = cols % E == 0 && cols <= 64 * 16 * E && aligned16(x) && aligned16(y) &&
                        aligned16(g) && aligned16(b);
    if (vec_ok) {
        const int nvec = (int)(cols / E);
        // Persistent workgroups, exactly as many as the device holds at once for
        // this kernel's register and LDS footprint: every CU stays full, and the
        // LDS staging of the parameters is amortised over many rows.
        const int64_t want = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
        const size_t lds = (OP == kSoftmax) ? 0
                                            : ((gp ? 1 : 0) + ((OP == kLayerNorm && bp) ? 1 : 0)) *
                                                  (size_t)cols * sizeof(T);
#define MHIP_ROW_CASE(NV)                                                                      \
    {                                                                                          \
        auto kern = row_wave_kernel<T, OP, NV>;                                                \
        int per_cu = tune_int("MHIP_ROW_BLOCKS_PER_CU", 0);                                    \
        if (per_cu == 0 &&                                                                     \
            (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 256, lds) !=          \
                 hipSuccess || per_cu <= 0))                                                   \
            per_cu = 4;                                                                        \
        /* the occupancy query counts LDS to the last byte; keep a margin so that */          \
        /* every workgroup of the grid really is resident at once */                          \
        if (lds && per_cu > (int)((160 * 1024 - 4096) / (lds + 512)))                          \
            per_cu = (int)((160 * 1024 - 4096) / (lds + 512));                                 \
        if (per_cu < 1) per_cu = 1;                                                            \
        const int64_t cap = (int64_t)compute_units() * per_cu;                                 \
        const unsigned grid = (unsigned)(want < cap ? want : cap);                             \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, s, xp, gp, bp, yp, rows,          \
                           (int)cols, eps);                                                    \
    }
        if (nvec <= 64) MHIP_ROW_CASE(1)
        else if (nvec <= 128) MHIP_ROW_CASE(2)
        else if (nvec <= 256) MHIP_ROW_CASE(4)
        else if (nvec <= 512) MHIP_ROW_CASE(8)
        else MHIP_ROW_CASE(16)
#undef MHIP_ROW_CASE
    } else {
        hipLaunchKernelGGL((row_block_kernel<T, OP>), dim3((unsigned)rows), dim3(256), 0, s, xp,
                           gp, bp, yp, cols, eps);
    }
    return check_launch("row kernel");
}

template <int OP>
static int row_entry(const char* name, void* stream, const void* x, const void* g, const void* b,
                     void* y, int64_t rows, int64_t cols, float eps, int dtype) {
    if (rows < 0 || cols < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative size", name);
    if (rows == 0 || cols == 0) return MHIP_OK;
    if (!x || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", name);
    if (rows > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "%s: more than 2^31-1 rows", name);
    hipStream_t s = as_stream(stream);
    switch (dtype) {
        case MHIP_F32: return launch_row<float, OP>(s, x, g, b, y, rows, cols, eps);
        case MHIP_BF16: return launch_row<bf16_t, OP>(s, x, g, b, y, rows, cols, eps);
        case MHIP_F16: return launch_row<f16_t, OP>(s, x, g, b, y, rows, cols, eps);
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: dtype %d (need f32, f16 or bf16)", name, dtype);
    }
}

template <typename T>
static int launch_gelu(hipStream_t s, const void* x, const void* bias, void* y, int64_t rows,
                       int64_t cols) {
    constexpr int E = Elem<T>::kPerVec;
    const int64_t n = rows * cols;
    const bool vec_ok = cols % E == 0 && cols <= 0x7FFFFFFF && aligned16(x) && aligned16(y) &&
                        aligned16(bias);
    if (vec_ok) {
        const int64_t nvec = n / E;
        const int64_t want = (nvec + 511) / 512;
        const int64_t cap = (int64_t)compute_units() * tune_int("MHIP_GELU_BLOCKS_PER_CU", 64);
        const unsigned grid = (unsigned)(want < cap ? want : cap);
        const bool in_lds = bias && cols * sizeof(float) <= 48 * 1024;
        hipLaunchKernelGGL((bias_gelu_vec_kernel<T>), dim3(grid), dim3(256),
                           in_lds ? (size_t)cols * sizeof(float) : 0, s, static_cast<const T*>(x),
                           static_cast<const T*>(bias), static_cast<T*>(y), nvec, (int)(cols / E),
                           in_lds ? 1 : 0);
    } else {
        const int64_t grid = (n + 255) / 256;
        if (grid > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "bias_gelu: tensor too large");
        hipLaunchKernelGGL((bias_gelu_scalar_kernel<T>), dim3((unsigned)grid), dim3(256), 0, s,
                           static_cast<const T*>(x), static_cast<const T*>(bias),
                           static_cast<T*>(y), n, cols);
    }
    return check_launch("bias_gelu");
}

}  // namespace mhip

using namespace mhip;

extern "C" int mhip_softmax(void* stream, const void* x, void* y, int64_t rows, int64_t cols,
                            int dtype) {
    return row_entry<kSoftmax>("mhip_softmax", stream, x, nullptr, nullptr, y, rows, cols, 0.f, dtype);
}

extern "C" int mhip_layer_norm(void* stream, const void* x, const void* gamma, const void* beta,
                               void* y, int64_t rows, int64_t cols, float eps, int dtype) {
    return row_entry<kLayerNorm>("mhip_layer_norm", stream, x, gamma, beta, y, rows, cols, eps, dtype);
}

extern "C" int mhip_rms_norm(void* stream, const void* x, const void* gamma, void* y, int64_t rows,
                             int64_t cols, float eps, int dtype) {
    return row_entry<kRmsNorm>("mhip_rms_norm", stream, x, gamma, nullptr, y, rows, cols, eps, dtype);
}

extern "C" int mhip_bias_gelu(void* stream, const void* x, const void* bias, void* y, int64_t rows,
                              int64_t cols, int dtype) {
    if (rows < 0 || cols < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_bias_gelu: negative size");
    if (rows == 0 || cols == 0) return MHIP_OK;
    if (!x || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_bias_gelu: NULL tensor pointer");
    hipStream_t s = as_stream(stream);
    switch (dtype) {
        case MHIP_F32: return launch_gelu<float>(s, x, bias, y, rows, cols);
        case MHIP_BF16: return launch_gelu<bf16_t>(s, x, bias, y, rows, cols);
        case MHIP_F16: return launch_gelu<f16_t>(s, x, bias, y, rows, cols);
        default: return fail(MHIP_ERR_UNSUPPORTED, "mhip_bias_gelu: dtype %d", dtype);
    }
}

extern "C" int mhip_softmax_strided(void* stream, const void* x, void* y, int64_t outer,
                                    int64_t axis_len, int64_t inner, int dtype) {
    if (outer < 0 || axis_len < 0 || inner < 0)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_softmax_strided: negative size");
    if (outer == 0 || axis_len == 0 || inner == 0) return MHIP_OK;
    if (!x || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_softmax_strided: NULL tensor pointer");
    if (inner == 1) return mhip_softmax(stream, x, y, outer, axis_len, dtype);
    const int64_t grid = (outer * inner + 255) / 256;
    if (grid > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "mhip_softmax_strided: too large");
    hipStream_t s = as_stream(stream);
#define MHIP_SS(T)                                                                             \
    hipLaunchKernelGGL((softmax_strided_kernel<T>), dim3((unsigned)grid), dim3(256), 0, s,     \
                       static_cast<const T*>(x), static_cast<T*>(y), outer, axis_len, inner)
    switch (dtype) {
        case MHIP_F32: MHIP_SS(float); break;
        case MHIP_BF16: MHIP_SS(bf16_t); break;
        case MHIP_F16: MHIP_SS(f16_t); break;
        default: return fail(MHIP_ERR_UNSUPPORTED, "mhip_softmax_strided: dtype %d", dtype);
    }
#undef MHIP_SS
    return check_launch("softmax_strided");
}
