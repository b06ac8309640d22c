// Unfused StableHLO glue for the host executor: unary / binary / compare /
// select elementwise ops, one strided-gather copy that serves broadcast_in_dim,
// transpose and slice, a single-axis reduce, and fill.  These are the ops that sit
// between the fused kernels in a module (the reference generates one MSL kernel
// per such op, Compiler/CodeGenerator.swift:851-3151); none is on the roofline
// path, so they are written for coverage and exactness, not for peak bandwidth.
#include <math.h>

#include <type_traits>

#include "common.h"

namespace mhip {

static int ew_grid(int64_t n, unsigned* out) {
    const int64_t g = (n + 255) / 256;
    if (g > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "tensor too large for one launch");
    *out = (unsigned)g;
    return MHIP_OK;
}

// Compute type of a floating element type: fp32 for the 16- and 32-bit types (one rounding at
// the store), double for f64.
template <typename T> struct Num {
    typedef float F;
    __device__ static float ld(const T* p, int64_t i) { return (float)p[i]; }
    __device__ static void st(T* p, int64_t i, float v) { p[i] = (T)v; }
};
template <> struct Num<double> {
    typedef double F;
    __device__ static double ld(const double* p, int64_t i) { return p[i]; }
    __device__ static void st(double* p, int64_t i, double v) { p[i] = v; }
};

template <typename T>
__global__ __launch_bounds__(256) void unary_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                    int64_t n, int op) {
    typedef typename Num<T>::F F;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const F v = Num<T>::ld(x, i);
    F r;
    switch (op) {
        case MHIP_UN_EXP: r = exp(v); break;
        case MHIP_UN_TANH: r = tanh(v); break;
        case MHIP_UN_RSQRT: r = (F)1 / sqrt(v); break;
        case MHIP_UN_SQRT: r = sqrt(v); break;
        case MHIP_UN_NEG: r = -v; break;
        case MHIP_UN_LOGISTIC: r = (F)1 / ((F)1 + exp(-v)); break;
        case MHIP_UN_ABS: r = fabs(v); break;
        case MHIP_UN_LOG: r = log(v); break;
        case MHIP_UN_ERF: r = erf(v); break;
        case MHIP_UN_SIN: r = sin(v); break;
        case MHIP_UN_COS: r = cos(v); break;
        case MHIP_UN_FLOOR: r = floor(v); break;
        case MHIP_UN_CEIL: r = ceil(v); break;
        default: r = v; break;
    }
    Num<T>::st(y, i, r);
}

// negate wraps around (also for unsigned types); abs of an unsigned value is the value
template <typename T>
__global__ __launch_bounds__(256) void unary_int_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                        int64_t n, int op) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    typedef typename std::make_unsigned<T>::type U;
    const T v = x[i];
    const T neg = (T)((U)0 - (U)v);
    y[i] = op == MHIP_UN_NEG ? neg : (op == MHIP_UN_ABS ? ((std::is_signed<T>::value && v < 0) ? neg : v) : v);
}

// Integer power as StableHLO defines it: repeated wrap-around multiplication for a
// non-negative exponent; for a negative one 1 / x^|e| truncated, i.e. 1 for x = 1,
// (-1)^|e| for x = -1 and 0 otherwise.
template <typename T>
__device__ inline T int_pow(T base, T e) {
    typedef typename std::make_unsigned<T>::type U;
    if (std::is_signed<T>::value && e < 0) {
        if (base == (T)1) return (T)1;
        if (base == (T)-1) return ((U)e & 1) ? (T)-1 : (T)1;
        return (T)0;
    }
    U r = 1, b = (U)base, k = (U)e;
    while (k) {
        if (k & 1) r *= b;
        b *= b;
        k >>= 1;
    }
    return (T)r;
}

// fp32 math for float types (one rounding at the store); exact wrap-around
// arithmetic for integers.
template <typename T>
__global__ __launch_bounds__(256) void binary_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                     T* __restrict__ y, int64_t n, int op) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    if constexpr (std::is_integral<T>::value) {
        const T u = a[i], v = b[i];
        using U = typename std::make_unsigned<T>::type;
        T r;
        switch (op) {
            case MHIP_BIN_ADD: r = (T)((U)u + (U)v); break;
            case MHIP_BIN_SUB: r = (T)((U)u - (U)v); break;
            case MHIP_BIN_MUL: r = (T)((U)u * (U)v); break;
            case MHIP_BIN_DIV: r = v == 0 ? (T)-1 : (T)(u / v); break;
            case MHIP_BIN_MAX: r = u > v ? u : v; break;
            case MHIP_BIN_MIN: r = u < v ? u : v; break;
            case MHIP_BIN_POW: r = int_pow<T>(u, v); break;
            default: r = u; break;
        }
        y[i] = r;
    } else {
        typedef typename Num<T>::F F;
        const F u = Num<T>::ld(a, i), v = Num<T>::ld(b, i);
        F r;
        switch (op) {
            case MHIP_BIN_ADD: r = u + v; break;
            case MHIP_BIN_SUB: r = u - v; break;
            case MHIP_BIN_MUL: r = u * v; break;
            case MHIP_BIN_DIV: r = u / v; break;
            case MHIP_BIN_MAX: r = (u != u || v != v) ? (F)NAN : fmax(u, v); break;
            case MHIP_BIN_MIN: r = (u != u || v != v) ? (F)NAN : fmin(u, v); break;
            case MHIP_BIN_POW: r = pow(u, v); break;
            default: r = u; break;
        }
        Num<T>::st(y, i, r);
    }
}

// booleans (one byte each, 0 / 1): add and maximum are OR, multiply and minimum are AND
__global__ __launch_bounds__(256) void binary_bool_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                                                          uint8_t* __restrict__ y, int64_t n, int op) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const bool u = a[i] != 0, v = b[i] != 0;
    y[i] = (op == MHIP_BIN_ADD || op == MHIP_BIN_MAX) ? (u || v) : (op == MHIP_BIN_MUL || op == MHIP_BIN_MIN) ? (u && v)
         : op == MHIP_BIN_SUB ? (u != v) : u;
}

template <typename T>
__global__ __launch_bounds__(256) void compare_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                      uint8_t* __restrict__ y, int64_t n, int dir) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    bool r;
    if constexpr (std::is_integral<T>::value) {
        const T u = a[i], v = b[i];
        r = dir == MHIP_CMP_EQ ? u == v : dir == MHIP_CMP_NE ? u != v : dir == MHIP_CMP_LT ? u < v
          : dir == MHIP_CMP_LE ? u <= v : dir == MHIP_CMP_GT ? u > v : u >= v;
    } else {
        const typename Num<T>::F u = Num<T>::ld(a, i), v = Num<T>::ld(b, i);
        r = dir == MHIP_CMP_EQ ? u == v : dir == MHIP_CMP_NE ? u != v : dir == MHIP_CMP_LT ? u < v
          : dir == MHIP_CMP_LE ? u <= v : dir == MHIP_CMP_GT ? u > v : u >= v;
    }
    y[i] = r ? 1 : 0;
}

template <typename W>
__global__ __launch_bounds__(256) void select_kernel(const uint8_t* __restrict__ p, const W* __restrict__ a,
                                                     const W* __restrict__ b, W* __restrict__ y,
                                                     int64_t n, int scalar_pred) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = p[scalar_pred ? 0 : i] ? a[i] : b[i];
}

struct StridedArgs {
    int rank;
    int64_t out_shape[8];
    int64_t in_stride[8];   // elements; 0 broadcasts
    int64_t in_offset;
};

template <typename W>
__global__ __launch_bounds__(256) void strided_copy_kernel(const W* __restrict__ x, W* __restrict__ y,
                                                           int64_t n, StridedArgs s) {
    const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= n) return;
    int64_t rem = o, src = s.in_offset;
#pragma unroll
    for (int d = 7; d >= 0; d--) {
        if (d < s.rank) {
            const int64_t idx = rem % s.out_shape[d];
            rem /= s.out_shape[d];
            src += idx * s.in_stride[d];
        }
    }
    y[o] = x[src];
}

// General gather: every output element reads operand[base(o) + sum_c clamp(index_c(o)) * stride_c].
struct GatherArgs {
    int rank, n_comp;
    int64_t out_shape[8];
    int64_t op_stride[8];    // operand elements per step of each result dim (offset and batching dims)
    int64_t idx_stride[8];   // index elements per step of each result dim (batch dims)
    int64_t comp_stride;     // between the components of one index vector
    int64_t comp_op_stride[8], comp_max[8];
};

template <typename W, typename I>
__global__ __launch_bounds__(256) void gather_kernel(const W* __restrict__ x, const I* __restrict__ idx,
                                                     W* __restrict__ y, int64_t n, GatherArgs g) {
    const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= n) return;
    int64_t rem = o, src = 0, ib = 0;
#pragma unroll
    for (int d = 7; d >= 0; d--) {
        if (d < g.rank) {
            const int64_t i = rem % g.out_shape[d];
            rem /= g.out_shape[d];
            src += i * g.op_stride[d];
            ib += i * g.idx_stride[d];
        }
    }
    for (int c = 0; c < g.n_comp; c++) {
        int64_t v = (int64_t)idx[ib + c * g.comp_stride];
        v = v < 0 ? 0 : (v > g.comp_max[c] ? g.comp_max[c] : v);
        src += v * g.comp_op_stride[c];
    }
    y[o] = x[src];
}

// y[o, i] = reduce over l of x[o, l, i]; one thread per output element, sequential
// over the reduced axis in index order (fp32 accumulator for 16-bit floats).
template <typename T>
__global__ __launch_bounds__(256) void reduce_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                     int64_t outer, int64_t len, int64_t inner,
                                                     int op, double init) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= outer * inner) return;
    const int64_t base = (gid / inner) * len * inner + gid % inner;
    if constexpr (std::is_integral<T>::value) {
        using U = typename std::make_unsigned<T>::type;
        T acc = (T)(int64_t)init;
        for (int64_t l = 0; l < len; l++) {
            const T v = x[base + l * inner];
            acc = op == MHIP_RED_SUM ? (T)((U)acc + (U)v) : op == MHIP_RED_MAX ? (v > acc ? v : acc)
                : op == MHIP_RED_MIN ? (v < acc ? v : acc) : (T)((U)acc * (U)v);
        }
        y[gid] = acc;
    } else {
        float acc = (float)init;
        for (int64_t l = 0; l < len; l++) {
            const float v = Num<T>::ld(x, base + l * inner);
            acc = op == MHIP_RED_SUM ? acc + v : op == MHIP_RED_MAX ? ((v != v || acc != acc) ? NAN : fmaxf(acc, v))
                : op == MHIP_RED_MIN ? ((v != v || acc != acc) ? NAN : fminf(acc, v)) : acc * v;
        }
        Num<T>::st(y, gid, acc);
    }
}

template <typename W>
__global__ __launch_bounds__(256) void fill_kernel(W* y, int64_t n, W v) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = v;
}

}  // namespace mhip

using namespace mhip;

#define MHIP_FLOAT_DISPATCH(DT, CALL)                 \
    switch (DT) {                                     \
        case MHIP_F32: { using T = float; CALL; } break;   \
        case MHIP_BF16: { using T = bf16_t; CALL; } break; \
        case MHIP_F16: { using T = f16_t; CALL; } break;   \
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: dtype %d", what, DT); \
    }

extern "C" int mhip_unary(void* stream, int op, const void* x, void* y, int64_t n, int dtype) {
    const char* what = "mhip_unary";
    if (n < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative size", what);
    if (n == 0) return MHIP_OK;
    if (!x || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL pointer", what);
    if (op < MHIP_UN_EXP || op > MHIP_UN_CEIL) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: unknown op %d", what, op);
    unsigned grid;
    if (ew_grid(n, &grid)) return MHIP_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
#define MHIP_UN_INT(T) hipLaunchKernelGGL((unary_int_kernel<T>), dim3(grid), dim3(256), 0, s, (const T*)x, (T*)y, n, op)
    if (dtype >= MHIP_I8 && dtype <= MHIP_UI64) {
        if (op != MHIP_UN_NEG && op != MHIP_UN_ABS)
            return fail(MHIP_ERR_UNSUPPORTED, "%s: op %d on an integer type", what, op);
        switch (dtype) {
            case MHIP_I8: MHIP_UN_INT(int8_t); break;
            case MHIP_I16: MHIP_UN_INT(int16_t); break;
            case MHIP_I32: MHIP_UN_INT(int32_t); break;
            case MHIP_I64: MHIP_UN_INT(int64_t); break;
            case MHIP_UI8: MHIP_UN_INT(uint8_t); break;
            case MHIP_UI16: MHIP_UN_INT(uint16_t); break;
            case MHIP_UI32: MHIP_UN_INT(uint32_t); break;
            default: MHIP_UN_INT(uint64_t); break;
        }
        return check_launch(what);
    }
#undef MHIP_UN_INT
    if (dtype == MHIP_F64) {
        hipLaunchKernelGGL((unary_kernel<double>), dim3(grid), dim3(256), 0, s, (const double*)x, (double*)y, n, op);
        return check_launch(what);
    }
    MHIP_FLOAT_DISPATCH(dtype, hipLaunchKernelGGL((unary_kernel<T>), dim3(grid), dim3(256), 0, s, (const T*)x, (T*)y, n, op))
    return check_launch(what);
}

extern "C" int mhip_binary(void* stream, int op, const void* a, const void* b, void* y, int64_t n,
                           int dtype) {
    const char* what = "mhip_binary";
    if (n < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative size", what);
    if (n == 0) return MHIP_OK;
    if (!a || !b || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL pointer", what);
    if (op < MHIP_BIN_ADD || op > MHIP_BIN_POW) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: unknown op %d", what, op);
    unsigned grid;
    if (ew_grid(n, &grid)) return MHIP_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
#define MHIP_BIN(T) hipLaunchKernelGGL((binary_kernel<T>), dim3(grid), dim3(256), 0, s, (const T*)a, (const T*)b, (T*)y, n, op)
    switch (dtype) {
        case MHIP_F32: MHIP_BIN(float); break;
        case MHIP_BF16: MHIP_BIN(bf16_t); break;
        case MHIP_F16: MHIP_BIN(f16_t); break;
        case MHIP_I32: MHIP_BIN(int32_t); break;
        case MHIP_I64: MHIP_BIN(int64_t); break;
        case MHIP_UI32: MHIP_BIN(uint32_t); break;
        case MHIP_UI64: MHIP_BIN(uint64_t); break;
        case MHIP_I8: MHIP_BIN(int8_t); break;
        case MHIP_UI8: MHIP_BIN(uint8_t); break;
        case MHIP_I16: MHIP_BIN(int16_t); break;
        case MHIP_UI16: MHIP_BIN(uint16_t); break;
        case MHIP_F64: MHIP_BIN(double); break;
        case MHIP_I1:
            if (op == MHIP_BIN_DIV || op == MHIP_BIN_POW) return fail(MHIP_ERR_UNSUPPORTED, "%s: op %d on booleans", what, op);
            hipLaunchKernelGGL(binary_bool_kernel, dim3(grid), dim3(256), 0, s, (const uint8_t*)a, (const uint8_t*)b, (uint8_t*)y, n, op);
            break;
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: dtype %d", what, dtype);
    }
#undef MHIP_BIN
    return check_launch(what);
}

extern "C" int mhip_compare(void* stream, int direction, const void* a, const void* b, void* y,
                            int64_t n, int dtype) {
    const char* what = "mhip_compare";
    if (n < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative size", what);
    if (n == 0) return MHIP_OK;
    if (!a || !b || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL pointer", what);
    if (direction < MHIP_CMP_EQ || direction > MHIP_CMP_GE)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: unknown direction %d", what, direction);
    unsigned grid;
    if (ew_grid(n, &grid)) return MHIP_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
#define MHIP_CMP(T) hipLaunchKernelGGL((compare_kernel<T>), dim3(grid), dim3(256), 0, s, (const T*)a, (const T*)b, (uint8_t*)y, n, direction)
    switch (dtype) {
        case MHIP_F32: MHIP_CMP(float); break;
        case MHIP_BF16: MHIP_CMP(bf16_t); break;
        case MHIP_F16: MHIP_CMP(f16_t); break;
        case MHIP_I32: MHIP_CMP(int32_t); break;
        case MHIP_I64: MHIP_CMP(int64_t); break;
        case MHIP_UI32: MHIP_CMP(uint32_t); break;
        case MHIP_UI64: MHIP_CMP(uint64_t); break;
        case MHIP_I8: MHIP_CMP(int8_t); break;
        case MHIP_UI8: case MHIP_I1: MHIP_CMP(uint8_t); break;
        case MHIP_I16: MHIP_CMP(int16_t); break;
        case MHIP_UI16: MHIP_CMP(uint16_t); break;
        case MHIP_F64: MHIP_CMP(double); break;
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: dtype %d", what, dtype);
    }
#undef MHIP_CMP
    return check_launch(what);
}

extern "C" int mhip_select(void* stream, const void* pred, const void* a, const void* b, void* y,
                           int64_t n, int elem_size, int scalar_pred) {
    const char* what = "mhip_select";
    if (n < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative size", what);
    if (n == 0) return MHIP_OK;
    if (!pred || !a || !b || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL pointer", what);
    unsigned grid;
    if (ew_grid(n, &grid)) return MHIP_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
#define MHIP_SEL(W) hipLaunchKernelGGL((select_kernel<W>), dim3(grid), dim3(256), 0, s, (const uint8_t*)pred, (const W*)a, (const W*)b, (W*)y, n, scalar_pred)
    switch (elem_size) {
        case 1: MHIP_SEL(uint8_t); break;
        case 2: MHIP_SEL(uint16_t); break;
        case 4: MHIP_SEL(uint32_t); break;
        case 8: MHIP_SEL(uint64_t); break;
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: element size %d", what, elem_size);
    }
#undef MHIP_SEL
    return check_launch(what);
}

extern "C" int mhip_strided_copy(void* stream, const void* x, void* y, int rank,
                                 const int64_t* out_shape, const int64_t* in_strides,
                                 int64_t in_offset, int elem_size) {
    const char* what = "mhip_strided_copy";
    if (rank < 0 || rank > 8) return fail(MHIP_ERR_UNSUPPORTED, "%s: rank %d (max 8)", what, rank);
    if (rank > 0 && (!out_shape || !in_strides)) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL shape", what);
    StridedArgs a;
    a.rank = rank;
    a.in_offset = in_offset;
    int64_t n = 1;
    for (int d = 0; d < 8; d++) {
        a.out_shape[d] = d < rank ? out_shape[d] : 1;
        a.in_stride[d] = d < rank ? in_strides[d] : 0;
        if (d < rank) {
            if (out_shape[d] < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative dimension", what);
            n *= out_shape[d];
        }
    }
    if (n == 0) return MHIP_OK;
    if (!x || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL pointer", what);
    hipStream_t s = as_stream(stream);
    // Whole 16-byte groups: when the innermost axis is contiguous in the source and everything
    // else (its length, the other strides, the offset, both pointers) is a multiple of V = 16 /
    // elem_size elements, the copy is the same copy of 16-byte elements with that axis V times
    // shorter -- a broadcast, a slice of rows or a transpose of outer axes then moves 16 bytes per
    // lane and does its index arithmetic once per group ([8,1024,768] f32 broadcast: 20 -> 7 us).
    if (rank >= 1 && (elem_size == 1 || elem_size == 2 || elem_size == 4 || elem_size == 8)) {
        const int64_t V = 16 / elem_size;
        bool ok = in_strides[rank - 1] == 1 && out_shape[rank - 1] % V == 0 && in_offset % V == 0 &&
                  ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
        for (int d = 0; ok && d < rank - 1; d++) ok = in_strides[d] % V == 0;
        if (ok) {
            StridedArgs v = a;
            v.out_shape[rank - 1] /= V;
            for (int d = 0; d < rank - 1; d++) v.in_stride[d] /= V;
            v.in_offset /= V;
            const int64_t nv = n / V;
            unsigned gridv;
            if (ew_grid(nv, &gridv)) return MHIP_ERR_UNSUPPORTED;
            hipLaunchKernelGGL((strided_copy_kernel<u32x4>), dim3(gridv), dim3(256), 0, s, (const u32x4*)x, (u32x4*)y, nv, v);
            return check_launch(what);
        }
    }
    unsigned grid;
    if (ew_grid(n, &grid)) return MHIP_ERR_UNSUPPORTED;
#define MHIP_SC(W) hipLaunchKernelGGL((strided_copy_kernel<W>), dim3(grid), dim3(256), 0, s, (const W*)x, (W*)y, n, a)
    switch (elem_size) {
        case 1: MHIP_SC(uint8_t); break;
        case 2: MHIP_SC(uint16_t); break;
        case 4: MHIP_SC(uint32_t); break;
        case 8: MHIP_SC(uint64_t); break;
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: element size %d", what, elem_size);
    }
#undef MHIP_SC
    return check_launch(what);
}

extern "C" int mhip_gather(void* stream, const void* operand, const void* indices, void* out, int rank,
                           const int64_t* out_shape, const int64_t* out_operand_strides,
                           const int64_t* out_index_strides, int n_components, int64_t component_stride,
                           const int64_t* component_operand_strides, const int64_t* component_max,
                           int elem_size, int idx_dtype) {
    const char* what = "mhip_gather";
    if (rank < 0 || rank > 8 || n_components < 0 || n_components > 8)
        return fail(MHIP_ERR_UNSUPPORTED, "%s: rank %d / %d index components (max 8)", what, rank, n_components);
    if ((rank > 0 && (!out_shape || !out_operand_strides || !out_index_strides)) ||
        (n_components > 0 && (!component_operand_strides || !component_max)))
        return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL descriptor", what);
    GatherArgs g;
    g.rank = rank;
    g.n_comp = n_components;
    g.comp_stride = component_stride;
    int64_t n = 1;
    for (int d = 0; d < 8; d++) {
        g.out_shape[d] = d < rank ? out_shape[d] : 1;
        g.op_stride[d] = d < rank ? out_operand_strides[d] : 0;
        g.idx_stride[d] = d < rank ? out_index_strides[d] : 0;
        g.comp_op_stride[d] = d < n_components ? component_operand_strides[d] : 0;
        g.comp_max[d] = d < n_components ? component_max[d] : 0;
        if (d < rank) {
            if (out_shape[d] < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative dimension", what);
            n *= out_shape[d];
        }
        if (d < n_components && component_max[d] < 0)
            return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: a slice is larger than the operand", what);
    }
    if (n == 0) return MHIP_OK;
    if (!operand || !out || (n_components > 0 && !indices)) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL pointer", what);
    if (idx_dtype != MHIP_I32 && idx_dtype != MHIP_I64)
        return fail(MHIP_ERR_UNSUPPORTED, "%s: index dtype %d (need i32 or i64)", what, idx_dtype);
    unsigned grid;
    if (ew_grid(n, &grid)) return MHIP_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
#define MHIP_GA(W)                                                                                                      \
    do {                                                                                                                \
        if (idx_dtype == MHIP_I32)                                                                                      \
            hipLaunchKernelGGL((gather_kernel<W, int32_t>), dim3(grid), dim3(256), 0, s, (const W*)operand,             \
                               (const int32_t*)indices, (W*)out, n, g);                                                 \
        else                                                                                                            \
            hipLaunchKernelGGL((gather_kernel<W, int64_t>), dim3(grid), dim3(256), 0, s, (const W*)operand,             \
                               (const int64_t*)indices, (W*)out, n, g);                                                 \
    } while (0)
    switch (elem_size) {
        case 1: MHIP_GA(uint8_t); break;
        case 2: MHIP_GA(uint16_t); break;
        case 4: MHIP_GA(uint32_t); break;
        case 8: MHIP_GA(uint64_t); break;
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: element size %d", what, elem_size);
    }
#undef MHIP_GA
    return check_launch(what);
}

extern "C" int mhip_reduce(void* stream, int op, const void* x, void* y, int64_t outer, int64_t len,
                           int64_t inner, double init, int dtype) {
    const char* what = "mhip_reduce";
    if (outer < 0 || len < 0 || inner < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative size", what);
    if (op < MHIP_RED_SUM || op > MHIP_RED_PROD) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: unknown op %d", what, op);
    if (outer * inner == 0) return MHIP_OK;
    if (!y || (len > 0 && !x)) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL pointer", what);
    unsigned grid;
    if (ew_grid(outer * inner, &grid)) return MHIP_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
#define MHIP_RED(T) hipLaunchKernelGGL((reduce_kernel<T>), dim3(grid), dim3(256), 0, s, (const T*)x, (T*)y, outer, len, inner, op, init)
    switch (dtype) {
        case MHIP_F32: MHIP_RED(float); break;
        case MHIP_BF16: MHIP_RED(bf16_t); break;
        case MHIP_F16: MHIP_RED(f16_t); break;
        case MHIP_I32: MHIP_RED(int32_t); break;
        case MHIP_I64: MHIP_RED(int64_t); break;
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: dtype %d", what, dtype);
    }
#undef MHIP_RED
    return check_launch(what);
}

extern "C" int mhip_fill(void* stream, void* y, int64_t n, uint64_t pattern, int elem_size) {
    const char* what = "mhip_fill";
    if (n < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative size", what);
    if (n == 0) return MHIP_OK;
    if (!y) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL pointer", what);
    unsigned grid;
    if (ew_grid(n, &grid)) return MHIP_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
    switch (elem_size) {
        case 1: hipLaunchKernelGGL((fill_kernel<uint8_t>), dim3(grid), dim3(256), 0, s, (uint8_t*)y, n, (uint8_t)pattern); break;
        case 2: hipLaunchKernelGGL((fill_kernel<uint16_t>), dim3(grid), dim3(256), 0, s, (uint16_t*)y, n, (uint16_t)pattern); break;
        case 4: hipLaunchKernelGGL((fill_kernel<uint32_t>), dim3(grid), dim3(256), 0, s, (uint32_t*)y, n, (uint32_t)pattern); break;
        case 8: hipLaunchKernelGGL((fill_kernel<uint64_t>), dim3(grid), dim3(256), 0, s, (uint64_t*)y, n, (uint64_t)pattern); break;
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: element size %d", what, elem_size);
    }
    return check_launch(what);
}
