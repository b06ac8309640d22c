// Four more of the reference's fused operators, all bound by memory bandwidth:
//
//   batch normalisation with given statistics (CustomCallHandlers.swift:414-452, "fused_batch_norm"):
//       y = (x - mean) / sqrt(variance + eps) * gamma + beta, the four vectors along the last axis;
//   attention over a few stored layer outputs (CustomCallHandlers.swift:1084-1140, "fused_depth_attention"):
//       out = softmax(q K^T scale) V for one query row against `depth` <= 64 key / value rows;
//   rotary position embedding (Compiler/CustomCallHandlers.swift:720-846, target "fused_rope"):
//       x = [x1 | x2] along the last axis (halves of h = D / 2 elements),
//       y = [x1 cos - x2 sin | x1 sin + x2 cos], cos / sin of shape [S, h] spread over the leading axes;
//   a chain of elementwise operations (CustomCallHandlers.swift:927-1079, target "fused_elementwise"):
//       the running value starts as input 0, every binary operation consumes the next input,
//       every unary one transforms the running value.
//
// All read every operand once and write the result once (rope, chains and batch normalisation 16
// bytes per lane where the layout allows); the arithmetic is fp32 whatever the element type,
// rounded once at the store.
#include <math.h>

#include "common.h"

namespace mhip {

namespace {

// MODE 0: `f` is [S, 2h], cos in the first half of each row and sin in the second.
// MODE 1: `f` is [S, h] angles; cos and sin are computed here.
// V = elements per thread along the half (1, or a 16-byte vector's worth).
template <typename T, int MODE, int V>
__global__ __launch_bounds__(256) void rope_kernel(const T* __restrict__ x, const T* __restrict__ f, T* __restrict__ y,
                                                   int64_t rows, int64_t S, int h) {
    const int per_row = h / V;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows * per_row) return;
    const int64_t row = idx / per_row;
    const int i0 = (int)(idx % per_row) * V;
    const int64_t s = row % S;
    const T* xr = x + row * 2 * h;
    T* yr = y + row * 2 * h;
    const T* fr = f + s * (MODE == 0 ? 2 * h : h);
    float x1[V], x2[V], c[V], sn[V];
    if constexpr (V == 1) {
        x1[0] = Elem<T>::to_f32(xr[i0]);
        x2[0] = Elem<T>::to_f32(xr[h + i0]);
        if constexpr (MODE == 0) {
            c[0] = Elem<T>::to_f32(fr[i0]);
            sn[0] = Elem<T>::to_f32(fr[h + i0]);
        } else {
            const float a = Elem<T>::to_f32(fr[i0]);
            c[0] = cosf(a);
            sn[0] = sinf(a);
        }
    } else {
        const Vec16<T> a1 = load16(xr + i0), a2 = load16(xr + h + i0), fc = load16(fr + i0);
        Vec16<T> fs = fc;
        if constexpr (MODE == 0) fs = load16(fr + h + i0);
#pragma unroll
        for (int e = 0; e < V; e++) {
            x1[e] = Elem<T>::to_f32(a1.v[e]);
            x2[e] = Elem<T>::to_f32(a2.v[e]);
            if constexpr (MODE == 0) {
                c[e] = Elem<T>::to_f32(fc.v[e]);
                sn[e] = Elem<T>::to_f32(fs.v[e]);
            } else {
                const float a = Elem<T>::to_f32(fc.v[e]);
                c[e] = cosf(a);
                sn[e] = sinf(a);
            }
        }
    }
    if constexpr (V == 1) {
        yr[i0] = Elem<T>::from_f32(x1[0] * c[0] - x2[0] * sn[0]);
        yr[h + i0] = Elem<T>::from_f32(x1[0] * sn[0] + x2[0] * c[0]);
    } else {
        Vec16<T> o1, o2;
#pragma unroll
        for (int e = 0; e < V; e++) {
            o1.v[e] = Elem<T>::from_f32(x1[e] * c[e] - x2[e] * sn[e]);
            o2.v[e] = Elem<T>::from_f32(x1[e] * sn[e] + x2[e] * c[e]);
        }
        store16(yr + i0, o1);
        store16(yr + h + i0, o2);
    }
}

template <typename T>
int launch_rope(hipStream_t s, const void* x, const void* f, void* y, int64_t rows, int64_t S, int64_t D, int mode) {
    constexpr int E = Elem<T>::kPerVec;
    const int h = (int)(D / 2);
    auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool vec = h % E == 0 && al(x) && al(y) && al(f);
    const int64_t threads = rows * (vec ? h / E : h);
    const int64_t grid = (threads + 255) / 256;
    if (grid > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "mhip_rope: tensor too large for one launch");
    const T* xp = static_cast<const T*>(x);
    const T* fp = static_cast<const T*>(f);
    T* yp = static_cast<T*>(y);
#define MHIP_ROPE(MODE, V) hipLaunchKernelGGL((rope_kernel<T, MODE, V>), dim3((unsigned)grid), dim3(256), 0, s, xp, fp, yp, rows, S, h)
    if (mode == 0) {
        if (vec) MHIP_ROPE(0, E); else MHIP_ROPE(0, 1);
    } else {
        if (vec) MHIP_ROPE(1, E); else MHIP_ROPE(1, 1);
    }
#undef MHIP_ROPE
    return check_launch("mhip_rope");
}

// ---- elementwise chains -----------------------------------------------------------------------
struct ChainArgs {
    const void* in[MHIP_CHAIN_MAX_INPUTS];
    int scalar[MHIP_CHAIN_MAX_INPUTS];        // 1: the input has one element, used for every position
    int ops[MHIP_CHAIN_MAX_OPS];              // unary: the mhip_unary_op code; binary: MHIP_CHAIN_BINARY + mhip_binary_op
    int n_ops;
};

__device__ inline float chain_unary(int op, float v) {
    switch (op) {
        case MHIP_UN_EXP: return expf(v);
        case MHIP_UN_TANH: return tanhf(v);
        case MHIP_UN_RSQRT: return 1.f / sqrtf(v);
        case MHIP_UN_SQRT: return sqrtf(v);
        case MHIP_UN_NEG: return -v;
        case MHIP_UN_LOGISTIC: return 1.f / (1.f + expf(-v));
        case MHIP_UN_ABS: return fabsf(v);
        case MHIP_UN_LOG: return logf(v);
        case MHIP_UN_ERF: return erff(v);
        case MHIP_UN_SIN: return sinf(v);
        case MHIP_UN_COS: return cosf(v);
        case MHIP_UN_FLOOR: return floorf(v);
        case MHIP_UN_CEIL: return ceilf(v);
        default: return v;
    }
}
__device__ inline float chain_binary(int op, float a, float b) {
    switch (op) {
        case MHIP_BIN_ADD: return a + b;
        case MHIP_BIN_SUB: return a - b;
        case MHIP_BIN_MUL: return a * b;
        case MHIP_BIN_DIV: return a / b;
        case MHIP_BIN_MAX: return fmaxf(a, b);
        case MHIP_BIN_MIN: return fminf(a, b);
        case MHIP_BIN_POW: return powf(a, b);
        default: return a;
    }
}

// V elements per thread (1, or a 16-byte vector's worth); the operation list is uniform across
// the grid, so the switches do not diverge.
template <typename T, int V>
__global__ __launch_bounds__(256) void chain_kernel(ChainArgs a, T* __restrict__ y, int64_t n) {
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (i0 >= n) return;
    auto load = [&](int k, float (&dst)[V]) {
        const T* p = static_cast<const T*>(a.in[k]);
        if (a.scalar[k]) {
            const float v = Elem<T>::to_f32(p[0]);
#pragma unroll
            for (int e = 0; e < V; e++) dst[e] = v;
        } else if constexpr (V == 1) {
            dst[0] = Elem<T>::to_f32(p[i0]);
        } else {
            const Vec16<T> v = load16(p + i0);
#pragma unroll
            for (int e = 0; e < V; e++) dst[e] = Elem<T>::to_f32(v.v[e]);
        }
    };
    float cur[V], rhs[V];
    load(0, cur);
    int next = 1;
    for (int o = 0; o < a.n_ops; o++) {
        const int op = a.ops[o];
        if (op >= MHIP_CHAIN_BINARY) {
            load(next++, rhs);
#pragma unroll
            for (int e = 0; e < V; e++) cur[e] = chain_binary(op - MHIP_CHAIN_BINARY, cur[e], rhs[e]);
        } else {
#pragma unroll
            for (int e = 0; e < V; e++) cur[e] = chain_unary(op, cur[e]);
        }
    }
    if constexpr (V == 1) {
        y[i0] = Elem<T>::from_f32(cur[0]);
    } else {
        Vec16<T> o;
#pragma unroll
        for (int e = 0; e < V; e++) o.v[e] = Elem<T>::from_f32(cur[e]);
        store16(y + i0, o);
    }
}

template <typename T>
int launch_chain(hipStream_t s, const ChainArgs& a, int n_inputs, void* y, int64_t n) {
    constexpr int E = Elem<T>::kPerVec;
    bool vec = n % E == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
    for (int k = 0; k < n_inputs; k++) vec = vec && (a.scalar[k] || (reinterpret_cast<uintptr_t>(a.in[k]) & 15) == 0);
    const int64_t threads = vec ? n / E : n;
    const int64_t grid = (threads + 255) / 256;
    if (grid > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "mhip_elementwise_chain: tensor too large for one launch");
    if (vec) hipLaunchKernelGGL((chain_kernel<T, E>), dim3((unsigned)grid), dim3(256), 0, s, a, static_cast<T*>(y), n);
    else hipLaunchKernelGGL((chain_kernel<T, 1>), dim3((unsigned)grid), dim3(256), 0, s, a, static_cast<T*>(y), n);
    return check_launch("mhip_elementwise_chain");
}


// ---- batch normalisation with given statistics -------------------------------------------------
// V elements per thread along the channel axis (1, or a 16-byte vector's worth).
template <typename T, int V>
__global__ __launch_bounds__(256) void batch_norm_kernel(const T* __restrict__ x, const T* __restrict__ gamma,
                                                         const T* __restrict__ beta, const T* __restrict__ mean,
                                                         const T* __restrict__ var, T* __restrict__ y, int64_t n, int C,
                                                         float eps) {
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (i0 >= n) return;
    const int c0 = (int)(i0 % C);
    auto one = [&](float xv, int c) {
        const float inv = 1.f / sqrtf(Elem<T>::to_f32(var[c]) + eps);
        return (xv - Elem<T>::to_f32(mean[c])) * inv * Elem<T>::to_f32(gamma[c]) + Elem<T>::to_f32(beta[c]);
    };
    if constexpr (V == 1) {
        y[i0] = Elem<T>::from_f32(one(Elem<T>::to_f32(x[i0]), c0));
    } else {
        const Vec16<T> v = load16(x + i0);
        Vec16<T> o;
#pragma unroll
        for (int e = 0; e < V; e++) o.v[e] = Elem<T>::from_f32(one(Elem<T>::to_f32(v.v[e]), c0 + e));
        store16(y + i0, o);
    }
}

template <typename T>
int launch_batch_norm(hipStream_t s, const void* x, const void* g, const void* b, const void* m, const void* v, void* y,
                      int64_t rows, int64_t C, float eps) {
    constexpr int E = Elem<T>::kPerVec;
    const int64_t n = rows * C;
    const bool vec = C % E == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
    const int64_t grid = ((vec ? n / E : n) + 255) / 256;
    if (grid > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "mhip_batch_norm: tensor too large for one launch");
#define MHIP_BN(V) hipLaunchKernelGGL((batch_norm_kernel<T, V>), dim3((unsigned)grid), dim3(256), 0, s, static_cast<const T*>(x), \
        static_cast<const T*>(g), static_cast<const T*>(b), static_cast<const T*>(m), static_cast<const T*>(v), static_cast<T*>(y), n, (int)C, eps)
    if (vec) MHIP_BN(E); else MHIP_BN(1);
#undef MHIP_BN
    return check_launch("mhip_batch_norm");
}

// ---- attention over a few rows ------------------------------------------------------------------
// One workgroup of 256 threads per query row.  Scores: thread t sums q[h] K[l][h] over h = t, t + 256, ..
// for every l, the 64 lanes of a wave add up, the four waves meet in LDS; lane l < depth of wave 0
// then holds score l, and the softmax over depth is two wave reductions.  Output: thread t sums
// w[l] V[l][h] over l for its h.
constexpr int kDepthMax = 64;

template <typename T>
__global__ __launch_bounds__(256) void depth_attention_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                              const T* __restrict__ v, T* __restrict__ o, int depth, int H,
                                                              float scale) {
    __shared__ float part[4][kDepthMax];
    __shared__ float w[kDepthMax];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t row = blockIdx.x;
    const T* qr = q + row * H;
    const T* kr = k + row * (int64_t)depth * H;
    const T* vr = v + row * (int64_t)depth * H;
    for (int l = 0; l < depth; l++) {
        float acc = 0.f;
        for (int h = tid; h < H; h += 256) acc += Elem<T>::to_f32(qr[h]) * Elem<T>::to_f32(kr[(int64_t)l * H + h]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if (lane == 0) part[wave][l] = acc;
    }
    __syncthreads();
    if (wave == 0) {
        const bool live = lane < depth;
        const float sc = live ? (part[0][lane] + part[1][lane] + part[2][lane] + part[3][lane]) * scale : -INFINITY;
        float mx = sc;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        const float e = live ? expf(sc - mx) : 0.f;
        float sum = e;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
        if (live) w[lane] = e / sum;
    }
    __syncthreads();
    for (int h = tid; h < H; h += 256) {
        float acc = 0.f;
        for (int l = 0; l < depth; l++) acc += w[l] * Elem<T>::to_f32(vr[(int64_t)l * H + h]);
        o[row * H + h] = Elem<T>::from_f32(acc);
    }
}

template <typename T>
int launch_depth_attention(hipStream_t s, const void* q, const void* k, const void* v, void* o, int64_t rows, int depth, int H,
                           float scale) {
    hipLaunchKernelGGL((depth_attention_kernel<T>), dim3((unsigned)rows), dim3(256), 0, s, static_cast<const T*>(q),
                       static_cast<const T*>(k), static_cast<const T*>(v), static_cast<T*>(o), depth, H, scale);
    return check_launch("mhip_depth_attention");
}

}  // namespace
}  // namespace mhip

using namespace mhip;

extern "C" int mhip_batch_norm(void* stream, const void* x, const void* gamma, const void* beta, const void* mean,
                               const void* variance, void* y, int64_t rows, int64_t channels, float eps, int dtype) {
    if (rows < 0 || channels < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_batch_norm: negative size");
    if (rows == 0 || channels == 0) return MHIP_OK;
    if (!x || !gamma || !beta || !mean || !variance || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_batch_norm: NULL pointer");
    if (channels > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "mhip_batch_norm: too many channels");
    hipStream_t s = as_stream(stream);
    switch (dtype) {
        case MHIP_F32: return launch_batch_norm<float>(s, x, gamma, beta, mean, variance, y, rows, channels, eps);
        case MHIP_BF16: return launch_batch_norm<bf16_t>(s, x, gamma, beta, mean, variance, y, rows, channels, eps);
        case MHIP_F16: return launch_batch_norm<f16_t>(s, x, gamma, beta, mean, variance, y, rows, channels, eps);
        default: return fail(MHIP_ERR_UNSUPPORTED, "mhip_batch_norm: dtype %d (need f32, f16 or bf16)", dtype);
    }
}

extern "C" int mhip_depth_attention(void* stream, const void* q, const void* k, const void* v, void* out, int64_t rows,
                                    int64_t depth, int64_t hidden, float scale, int dtype) {
    if (rows < 0 || depth < 0 || hidden < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_depth_attention: negative size");
    if (rows == 0 || hidden == 0) return MHIP_OK;
    if (!q || !k || !v || !out) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_depth_attention: NULL pointer");
    if (depth < 1 || depth > kDepthMax)
        return fail(MHIP_ERR_UNSUPPORTED, "mhip_depth_attention: depth %lld (1 to %d rows are served)", (long long)depth, kDepthMax);
    if (rows > 0x7FFFFFFFLL || hidden > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "mhip_depth_attention: tensor too large for one launch");
    hipStream_t s = as_stream(stream);
    switch (dtype) {
        case MHIP_F32: return launch_depth_attention<float>(s, q, k, v, out, rows, (int)depth, (int)hidden, scale);
        case MHIP_BF16: return launch_depth_attention<bf16_t>(s, q, k, v, out, rows, (int)depth, (int)hidden, scale);
        case MHIP_F16: return launch_depth_attention<f16_t>(s, q, k, v, out, rows, (int)depth, (int)hidden, scale);
        default: return fail(MHIP_ERR_UNSUPPORTED, "mhip_depth_attention: dtype %d (need f32, f16 or bf16)", dtype);
    }
}

extern "C" int mhip_rope(void* stream, const void* x, const void* freqs, void* y, int64_t rows, int64_t S, int64_t D,
                         int freqs_are_angles, int dtype) {
    if (rows < 0 || S < 0 || D < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_rope: negative size");
    if (rows == 0 || D == 0) return MHIP_OK;
    if (!x || !freqs || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_rope: NULL pointer");
    if (D % 2 != 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_rope: the rotated axis has %lld elements, an odd number", (long long)D);
    if (S <= 0 || rows % S != 0)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_rope: %lld rows are no whole number of sequences of %lld positions", (long long)rows, (long long)S);
    if (D > 0x7FFFFFFELL) return fail(MHIP_ERR_UNSUPPORTED, "mhip_rope: row too long");
    hipStream_t s = as_stream(stream);
    const int mode = freqs_are_angles ? 1 : 0;
    switch (dtype) {
        case MHIP_F32: return launch_rope<float>(s, x, freqs, y, rows, S, D, mode);
        case MHIP_BF16: return launch_rope<bf16_t>(s, x, freqs, y, rows, S, D, mode);
        case MHIP_F16: return launch_rope<f16_t>(s, x, freqs, y, rows, S, D, mode);
        default: return fail(MHIP_ERR_UNSUPPORTED, "mhip_rope: dtype %d (need f32, f16 or bf16)", dtype);
    }
}

extern "C" int mhip_elementwise_chain(void* stream, int n_inputs, const void* const* inputs, const int64_t* input_elements,
                                      int n_ops, const int* ops, void* y, int64_t n, int dtype) {
    const char* what = "mhip_elementwise_chain";
    if (n < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative size", what);
    if (n_inputs < 1 || n_inputs > MHIP_CHAIN_MAX_INPUTS || n_ops < 1 || n_ops > MHIP_CHAIN_MAX_OPS || !inputs || !input_elements || !ops)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: 1..%d inputs and 1..%d operations", what, MHIP_CHAIN_MAX_INPUTS, MHIP_CHAIN_MAX_OPS);
    ChainArgs a{};
    int need = 1;
    for (int o = 0; o < n_ops; o++) {
        const int op = ops[o];
        const bool binary = op >= MHIP_CHAIN_BINARY;
        if (binary ? (op - MHIP_CHAIN_BINARY > MHIP_BIN_POW) : (op < MHIP_UN_EXP || op > MHIP_UN_CEIL))
            return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: unknown operation code %d", what, op);
        need += binary ? 1 : 0;
        a.ops[o] = op;
    }
    a.n_ops = n_ops;
    if (need != n_inputs)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: the chain consumes %d inputs, %d were given", what, need, n_inputs);
    if (n == 0) return MHIP_OK;
    if (!y) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL result", what);
    for (int k = 0; k < n_inputs; k++) {
        if (!inputs[k]) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: input %d is NULL", what, k);
        if (input_elements[k] != n && input_elements[k] != 1)
            return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: input %d has %lld elements (need %lld or 1)", what, k,
                        (long long)input_elements[k], (long long)n);
        a.in[k] = inputs[k];
        a.scalar[k] = input_elements[k] == 1 && n != 1;
    }
    hipStream_t s = as_stream(stream);
    switch (dtype) {
        case MHIP_F32: return launch_chain<float>(s, a, n_inputs, y, n);
        case MHIP_BF16: return launch_chain<bf16_t>(s, a, n_inputs, y, n);
        case MHIP_F16: return launch_chain<f16_t>(s, a, n_inputs, y, n);
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: dtype %d (need f32, f16 or bf16)", what, dtype);
    }
}
