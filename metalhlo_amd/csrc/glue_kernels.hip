// Glue operators between the fused kernels: gather / embedding, add, convert,
// head transposes, iota, argmax.  All are streaming or index kernels; integer
// results are bit-exact by construction (pure copies and integer arithmetic).
#include <math.h>

#include <type_traits>

#include "common.h"

namespace mhip {

static int dtype_size(int dt) {
    switch (dt) {
        case MHIP_F16: case MHIP_BF16: case MHIP_I16: case MHIP_UI16: return 2;
        case MHIP_F32: case MHIP_I32: case MHIP_UI32: return 4;
        case MHIP_F64: case MHIP_I64: case MHIP_UI64: return 8;
        case MHIP_I1: case MHIP_I8: case MHIP_UI8: return 1;
        default: return 0;
    }
}

static int grid_for(int64_t n, int per_block, unsigned* out) {
    const int64_t g = (n + per_block - 1) / per_block;
    if (g > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "tensor too large for one launch");
    *out = (unsigned)g;
    return MHIP_OK;
}

// ---- gather of whole rows (byte copy) --------------------------------------
template <typename I>
__global__ __launch_bounds__(256) void gather_rows_kernel(const char* __restrict__ table,
                                                          const I* __restrict__ idx,
                                                          char* __restrict__ out, int64_t n_idx,
                                                          int64_t n_rows, int64_t row_bytes,
                                                          int vec) {
    // One workgroup per output row; `vec` = bytes moved per thread per step.
    const int64_t i = blockIdx.x;
    int64_t r = (int64_t)idx[i];
    r = r < 0 ? 0 : (r > n_rows - 1 ? n_rows - 1 : r);
    const char* src = table + r * row_bytes;
    char* dst = out + i * row_bytes;
    if (vec == 16) {
        for (int64_t o = (int64_t)threadIdx.x * 16; o < row_bytes; o += 256 * 16)
            *reinterpret_cast<u32x4*>(dst + o) = *reinterpret_cast<const u32x4*>(src + o);
    } else {
        for (int64_t o = threadIdx.x; o < row_bytes; o += 256) dst[o] = src[o];
    }
}

// ---- plain device copy (16 bytes per lane, streaming) --------------------------
__global__ __launch_bounds__(256) void copy_kernel(const u32x4* __restrict__ src,
                                                   u32x4* __restrict__ dst, int64_t nvec) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < nvec) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}
__global__ __launch_bounds__(256) void copy_bytes_kernel(const char* __restrict__ src,
                                                         char* __restrict__ dst, int64_t start,
                                                         int64_t n) {
    const int64_t i = start + (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

// ---- token + position embedding --------------------------------------------
template <typename P, typename O>
__global__ __launch_bounds__(256) void embed_kernel(const int32_t* __restrict__ ids,
                                                    const P* __restrict__ wte,
                                                    const P* __restrict__ wpe,
                                                    O* __restrict__ out, int64_t S, int64_t d,
                                                    int64_t vocab, int vec4) {
    // over B*S; with a grid that is a multiple of 8, XCD x (workgroup ids x, x + 8, ...) takes the
    // x-th eighth of the tokens: the rows a following row kernel or GEMM handles on that XCD
    const int64_t tok = gridDim.x % 8 == 0 ? (int64_t)(blockIdx.x % 8u) * (gridDim.x / 8u) + blockIdx.x / 8u : blockIdx.x;
    int64_t id = ids[tok];
    id = id < 0 ? 0 : (id > vocab - 1 ? vocab - 1 : id);
    const P* te = wte + id * d;
    const P* pe = wpe + (tok % S) * d;
    O* o = out + tok * d;
    if (vec4) {       // rows of all three tensors start on 16-byte (params) / 8-byte (result) boundaries
        struct alignas(4 * sizeof(P)) P4 { P v[4]; };
        struct alignas(4 * sizeof(O)) O4 { O v[4]; };
        for (int64_t c = (int64_t)threadIdx.x * 4; c < d; c += 1024) {
            const P4 t = *reinterpret_cast<const P4*>(te + c), q = *reinterpret_cast<const P4*>(pe + c);
            O4 r;
#pragma unroll
            for (int e = 0; e < 4; e++) r.v[e] = Elem<O>::from_f32(Elem<P>::to_f32(t.v[e]) + Elem<P>::to_f32(q.v[e]));
            *reinterpret_cast<O4*>(o + c) = r;
        }
        return;
    }
    for (int64_t c = threadIdx.x; c < d; c += 256)
        o[c] = Elem<O>::from_f32(Elem<P>::to_f32(te[c]) + Elem<P>::to_f32(pe[c]));
}

// ---- elementwise add ---------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void add_vec_kernel(const T* __restrict__ a,
                                                      const T* __restrict__ b, T* __restrict__ y,
                                                      int64_t nvec) {
    constexpr int E = Elem<T>::kPerVec;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nvec) return;
    Vec16<T> va = load16(a + i * E), vb = load16(b + i * E), o;
#pragma unroll
    for (int e = 0; e < E; e++)
        o.v[e] = Elem<T>::from_f32(Elem<T>::to_f32(va.v[e]) + Elem<T>::to_f32(vb.v[e]));
    store16(y + i * E, o);
}
template <typename T>
__global__ __launch_bounds__(256) void add_float_kernel(const T* a, const T* b, T* y, int64_t n,
                                                        int64_t start) {
    const int64_t i = start + (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = Elem<T>::from_f32(Elem<T>::to_f32(a[i]) + Elem<T>::to_f32(b[i]));
}
template <typename T>
__global__ __launch_bounds__(256) void add_int_kernel(const T* a, const T* b, T* y, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = (T)(a[i] + b[i]);
}

// ---- convert -------------------------------------------------------------------
template <typename T> struct Cvt {
    __device__ static double ld(const T* p, int64_t i) { return (double)p[i]; }
    __device__ static void st(T* p, int64_t i, double v) { p[i] = (T)v; }
};
template <> struct Cvt<bf16_t> {
    __device__ static double ld(const bf16_t* p, int64_t i) { return (double)(float)p[i]; }
    __device__ static void st(bf16_t* p, int64_t i, double v) { p[i] = (bf16_t)(float)v; }
};
template <> struct Cvt<f16_t> {
    __device__ static double ld(const f16_t* p, int64_t i) { return (double)(float)p[i]; }
    __device__ static void st(f16_t* p, int64_t i, double v) { p[i] = (f16_t)(float)v; }
};

// Float -> float goes through fp32 when the source is not f64 so that exactly
// one rounding happens; integer sources of up to 32 bits are exact in double.
template <typename S, typename D>
__global__ __launch_bounds__(256) void convert_kernel(const S* __restrict__ x, D* __restrict__ y,
                                                      int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    if constexpr (std::is_integral<S>::value && std::is_integral<D>::value) {
        y[i] = (D)x[i];  // integer -> integer keeps all 64 bits
    } else if constexpr (std::is_integral<S>::value && sizeof(S) == 8 && std::is_same<D, double>::value) {
        y[i] = (double)x[i];                        // 64-bit integer -> f64: one rounding
    } else if constexpr (std::is_same<S, double>::value && std::is_integral<D>::value && sizeof(D) == 8) {
        y[i] = (D)x[i];
    } else {
        Cvt<D>::st(y, i, Cvt<S>::ld(x, i));
    }
}

// anything -> boolean: x != 0 (one byte per element)
template <typename S>
__global__ __launch_bounds__(256) void to_bool_kernel(const S* __restrict__ x, uint8_t* __restrict__ y, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    if constexpr (std::is_integral<S>::value) y[i] = x[i] != 0;
    else y[i] = Cvt<S>::ld(x, i) != 0.0;
}

// fp32 -> 16-bit float.  A workgroup narrows 2048 consecutive elements as two rows of 256
// four-element groups: every load instruction of a wave reads 1 KB that is contiguous across its
// lanes (16 bytes each) and every store writes 512 contiguous bytes, the access form of the plain
// copy above.  Source and result are both streamed past the caches (non-temporal): the typical
// call narrows a model's parameters, far more than the L2 holds, long before most of them are
// read (measured on 124 M parameters: 133 -> 115 us against ordinary stores).
template <typename D> struct alignas(8) Narrow4 { D v[4]; };

template <typename D>
__device__ __forceinline__ void narrow_group(const float* __restrict__ x, D* __restrict__ y) {
    const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x));
    Narrow4<D> o;
#pragma unroll
    for (int e = 0; e < 4; e++) o.v[e] = Elem<D>::from_f32(a[e]);
    __builtin_nontemporal_store(__builtin_bit_cast(u32x2, o), reinterpret_cast<u32x2*>(y));
}

template <typename D>
__global__ __launch_bounds__(256) void narrow_vec_kernel(const float* __restrict__ x,
                                                         D* __restrict__ y, int64_t ngroups) {
    const int64_t g0 = (int64_t)blockIdx.x * 512 + threadIdx.x, g1 = g0 + 256;
    // both loads are issued before either is converted
    f32x4 a = {0.f, 0.f, 0.f, 0.f}, b = a;
    if (g0 < ngroups) a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x + g0 * 4));
    if (g1 < ngroups) b = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x + g1 * 4));
    Narrow4<D> oa, ob;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        oa.v[e] = Elem<D>::from_f32(a[e]);
        ob.v[e] = Elem<D>::from_f32(b[e]);
    }
    if (g0 < ngroups) __builtin_nontemporal_store(__builtin_bit_cast(u32x2, oa), reinterpret_cast<u32x2*>(y + g0 * 4));
    if (g1 < ngroups) __builtin_nontemporal_store(__builtin_bit_cast(u32x2, ob), reinterpret_cast<u32x2*>(y + g1 * 4));
}

// fp32 -> 16-bit float for up to kBatchMax tensors in one launch (a model's parameters: many
// of them small).  The table travels in the kernel arguments; a workgroup handles 2048
// consecutive elements of one tensor (in the access form of narrow_vec_kernel), which it finds
// by bisecting the running block counts.
constexpr int kBatchMax = 96;
struct ConvertBatch {
    const float* x[kBatchMax];
    void* y[kBatchMax];
    int64_t n[kBatchMax];
    uint32_t first_block[kBatchMax + 1];
    int count;
};
static_assert(sizeof(ConvertBatch) <= 4000, "the table must fit the kernel argument space");

template <typename D>
__global__ __launch_bounds__(256) void narrow_batch_kernel(ConvertBatch b) {
    int lo = 0, hi = b.count - 1;                  // largest t with first_block[t] <= blockIdx.x
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (b.first_block[mid] <= blockIdx.x) lo = mid; else hi = mid - 1;
    }
    const float* x = b.x[lo];
    D* y = static_cast<D*>(b.y[lo]);
    const int64_t n = b.n[lo];
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    const int64_t base = (int64_t)(blockIdx.x - b.first_block[lo]) * 2048;
#pragma unroll
    for (int h = 0; h < 2; h++) {                  // (the two loads are independent: both in flight)
        const int64_t i = base + (int64_t)(h * 256 + threadIdx.x) * 4;
        if (i >= n) continue;
        if (aligned && i + 4 <= n) narrow_group<D>(x + i, y + i);
        else
            for (int64_t e = i; e < n && e < i + 4; e++) y[e] = Elem<D>::from_f32(x[e]);
    }
}

// ---- [d0,d1,d2,d3] -> [d0,d2,d1,d3] ------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void transpose_0213_kernel(const T* __restrict__ x,
                                                             T* __restrict__ y, int64_t d1,
                                                             int64_t d2, int64_t d3, int64_t n) {
    const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;  // output linear index
    if (o >= n) return;
    const int64_t c = o % d3;
    int64_t t = o / d3;
    const int64_t i1 = t % d1;
    t /= d1;
    const int64_t i2 = t % d2;
    const int64_t i0 = t / d2;
    y[o] = x[((i0 * d1 + i1) * d2 + i2) * d3 + c];
}

// qkv [B,S,3,H,D] -> q,k,v [B,H,S,D], 16 bytes per thread.
__global__ __launch_bounds__(256) void split_qkv_kernel(const u32x4* __restrict__ qkv,
                                                        u32x4* __restrict__ q,
                                                        u32x4* __restrict__ k,
                                                        u32x4* __restrict__ v, int64_t S,
                                                        int64_t H, int64_t dv, int64_t n) {
    // dv = D in 16-byte vectors; input index i runs over [B,S,3,H,dv]
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t c = i % dv;
    int64_t t = i / dv;
    const int64_t h = t % H;
    t /= H;
    const int64_t which = t % 3;
    t /= 3;
    const int64_t s = t % S;
    const int64_t b = t / S;
    u32x4* dst = which == 0 ? q : (which == 1 ? k : v);
    dst[((b * H + h) * S + s) * dv + c] = qkv[i];
}

// ---- iota -----------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void iota_kernel(T* y, int64_t n, int64_t inner, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int64_t v = (i / inner) % n;
    if constexpr (std::is_same<T, bf16_t>::value || std::is_same<T, f16_t>::value) y[i] = (T)(float)v;
    else y[i] = (T)v;
}

// ---- argmax over the last axis: one wave per row -----------------------------------
// Order: NaN beats everything; otherwise larger value; ties -> lower index.
__device__ inline bool better(float v, int64_t i, float bv, int64_t bi) {
    const bool vn = v != v, bn = bv != bv;
    if (vn || bn) return vn && (!bn || i < bi);
    return v > bv || (v == bv && i < bi);
}
template <typename T, typename I>
__global__ __launch_bounds__(256) void argmax_kernel(const T* __restrict__ x, I* __restrict__ oi,
                                                     T* __restrict__ ov, int64_t rows,
                                                     int64_t cols) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + row * cols;
    float bv = -INFINITY;
    int64_t bi = 0x7FFFFFFFFFFFFFFFLL;
    for (int64_t c = lane; c < cols; c += 64) {
        const float v = Elem<T>::to_f32(xr[c]);
        if (bi == 0x7FFFFFFFFFFFFFFFLL || better(v, c, bv, bi)) { bv = v; bi = c; }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const float ovv = __shfl_xor(bv, o, 64);
        const int lo = __shfl_xor((int)(bi & 0xFFFFFFFF), o, 64);
        const int hi = __shfl_xor((int)(bi >> 32), o, 64);
        const int64_t oii = ((int64_t)hi << 32) | (uint32_t)lo;
        if (oii != 0x7FFFFFFFFFFFFFFFLL && (bi == 0x7FFFFFFFFFFFFFFFLL || better(ovv, oii, bv, bi))) {
            bv = ovv;
            bi = oii;
        }
    }
    if (lane == 0) {
        oi[row] = (I)(bi == 0x7FFFFFFFFFFFFFFFLL ? 0 : bi);
        if (ov) ov[row] = xr[bi == 0x7FFFFFFFFFFFFFFFLL ? 0 : bi];
    }
}

}  // namespace mhip

using namespace mhip;

extern "C" int mhip_gather_rows(void* stream, const void* table, const void* indices, void* out,
                                int64_t n_idx, int64_t n_rows, int64_t row_elems, int table_dtype,
                                int idx_dtype) {
    if (!table || !indices || !out) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_gather_rows: NULL pointer");
    if (n_idx < 0 || n_rows <= 0 || row_elems < 0)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_gather_rows: bad size");
    const int es = dtype_size(table_dtype);
    if (!es) return fail(MHIP_ERR_UNSUPPORTED, "mhip_gather_rows: dtype %d", table_dtype);
    if (n_idx == 0 || row_elems == 0) return MHIP_OK;
    if (n_idx > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "mhip_gather_rows: too many indices");
    const int64_t row_bytes = row_elems * es;
    const bool v16 = row_bytes % 16 == 0 && (reinterpret_cast<uintptr_t>(table) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(out) & 15) == 0;
    hipStream_t s = as_stream(stream);
    if (idx_dtype == MHIP_I32)
        hipLaunchKernelGGL((gather_rows_kernel<int32_t>), dim3((unsigned)n_idx), dim3(256), 0, s,
                           (const char*)table, (const int32_t*)indices, (char*)out, n_idx, n_rows,
                           row_bytes, v16 ? 16 : 1);
    else if (idx_dtype == MHIP_I64)
        hipLaunchKernelGGL((gather_rows_kernel<int64_t>), dim3((unsigned)n_idx), dim3(256), 0, s,
                           (const char*)table, (const int64_t*)indices, (char*)out, n_idx, n_rows,
                           row_bytes, v16 ? 16 : 1);
    else
        return fail(MHIP_ERR_UNSUPPORTED, "mhip_gather_rows: index dtype %d (need i32 or i64)", idx_dtype);
    return check_launch("gather_rows");
}

extern "C" int mhip_copy(void* stream, const void* src, void* dst, int64_t bytes) {
    if (bytes < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_copy: negative size");
    if (bytes == 0) return MHIP_OK;
    if (!src || !dst) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_copy: NULL pointer");
    hipStream_t s = as_stream(stream);
    const bool al = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
    const int64_t nvec = al ? bytes / 16 : 0;
    unsigned grid;
    if (nvec) {
        if (grid_for(nvec, 256, &grid)) return MHIP_ERR_UNSUPPORTED;
        hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(256), 0, s, (const u32x4*)src, (u32x4*)dst, nvec);
    }
    if (bytes - nvec * 16) {
        if (grid_for(bytes - nvec * 16, 256, &grid)) return MHIP_ERR_UNSUPPORTED;
        hipLaunchKernelGGL(copy_bytes_kernel, dim3(grid), dim3(256), 0, s, (const char*)src, (char*)dst,
                           nvec * 16, bytes);
    }
    return check_launch("copy");
}

extern "C" int mhip_embed_tokens(void* stream, const void* ids, const void* wte, const void* wpe,
                                 void* out, int64_t B, int64_t S, int64_t d_model, int64_t vocab,
                                 int param_dtype, int out_dtype) {
    if (!ids || !wte || !wpe || !out) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_embed_tokens: NULL pointer");
    if (B < 0 || S < 0 || d_model < 0 || vocab <= 0)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_embed_tokens: bad size");
    if (B * S == 0 || d_model == 0) return MHIP_OK;
    if (B * S > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "mhip_embed_tokens: too many tokens");
    hipStream_t s = as_stream(stream);
    const dim3 grid((unsigned)(B * S)), blk(256);
    // four elements per lane when every row starts on a 16-byte boundary (in either element size)
    const int vec4 = d_model % 4 == 0 && ((reinterpret_cast<uintptr_t>(wte) | reinterpret_cast<uintptr_t>(wpe) |
                                            reinterpret_cast<uintptr_t>(out)) & 15) == 0;
#define MHIP_EMB(P, O)                                                                      \
    hipLaunchKernelGGL((embed_kernel<P, O>), grid, blk, 0, s, (const int32_t*)ids,          \
                       (const P*)wte, (const P*)wpe, (O*)out, S, d_model, vocab, vec4)
    if (param_dtype == MHIP_F32 && out_dtype == MHIP_BF16) MHIP_EMB(float, bf16_t);
    else if (param_dtype == MHIP_F32 && out_dtype == MHIP_F16) MHIP_EMB(float, f16_t);
    else if (param_dtype == MHIP_F32 && out_dtype == MHIP_F32) MHIP_EMB(float, float);
    else if (param_dtype == MHIP_BF16 && out_dtype == MHIP_BF16) MHIP_EMB(bf16_t, bf16_t);
    else if (param_dtype == MHIP_F16 && out_dtype == MHIP_F16) MHIP_EMB(f16_t, f16_t);
    else return fail(MHIP_ERR_UNSUPPORTED, "mhip_embed_tokens: dtype pair %d -> %d", param_dtype, out_dtype);
#undef MHIP_EMB
    return check_launch("embed_tokens");
}

extern "C" int mhip_add(void* stream, const void* a, const void* b, void* y, int64_t n, int dtype) {
    if (!a || !b || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_add: NULL pointer");
    if (n < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_add: negative size");
    if (n == 0) return MHIP_OK;
    hipStream_t s = as_stream(stream);
    unsigned grid;
    const bool al = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
                      reinterpret_cast<uintptr_t>(y)) & 15) == 0;
#define MHIP_ADD_F(T)                                                                          \
    {                                                                                          \
        constexpr int E = Elem<T>::kPerVec;                                                    \
        const int64_t nvec = al ? n / E : 0;                                                   \
        if (nvec) {                                                                            \
            if (grid_for(nvec, 256, &grid)) return MHIP_ERR_UNSUPPORTED;                       \
            hipLaunchKernelGGL((add_vec_kernel<T>), dim3(grid), dim3(256), 0, s, (const T*)a,  \
                               (const T*)b, (T*)y, nvec);                                      \
        }                                                                                      \
        const int64_t rest = n - nvec * E;                                                     \
        if (rest) {                                                                            \
            if (grid_for(rest, 256, &grid)) return MHIP_ERR_UNSUPPORTED;                       \
            hipLaunchKernelGGL((add_float_kernel<T>), dim3(grid), dim3(256), 0, s,             \
                               (const T*)a, (const T*)b, (T*)y, n, nvec * E);                  \
        }                                                                                      \
    }
#define MHIP_ADD_I(T)                                                                          \
    {                                                                                          \
        if (grid_for(n, 256, &grid)) return MHIP_ERR_UNSUPPORTED;                              \
        hipLaunchKernelGGL((add_int_kernel<T>), dim3(grid), dim3(256), 0, s, (const T*)a,      \
                           (const T*)b, (T*)y, n);                                             \
    }
    switch (dtype) {
        case MHIP_F32: MHIP_ADD_F(float) break;
        case MHIP_BF16: MHIP_ADD_F(bf16_t) break;
        case MHIP_F16: MHIP_ADD_F(f16_t) break;
        case MHIP_I32: case MHIP_UI32: MHIP_ADD_I(uint32_t) break;
        case MHIP_I64: case MHIP_UI64: MHIP_ADD_I(uint64_t) break;
        default: return fail(MHIP_ERR_UNSUPPORTED, "mhip_add: dtype %d", dtype);
    }
#undef MHIP_ADD_F
#undef MHIP_ADD_I
    return check_launch("add");
}

namespace mhip {
template <typename S>
static int convert_from(hipStream_t s, const void* x, void* y, int64_t n, int dst) {
    unsigned grid;
    if (grid_for(n, 256, &grid)) return MHIP_ERR_UNSUPPORTED;
#define MHIP_CV(D)                                                                           \
    hipLaunchKernelGGL((convert_kernel<S, D>), dim3(grid), dim3(256), 0, s, (const S*)x, (D*)y, n)
    switch (dst) {
        case MHIP_F32: MHIP_CV(float); break;
        case MHIP_F64: MHIP_CV(double); break;
        case MHIP_BF16: MHIP_CV(bf16_t); break;
        case MHIP_F16: MHIP_CV(f16_t); break;
        case MHIP_I32: MHIP_CV(int32_t); break;
        case MHIP_I64: MHIP_CV(int64_t); break;
        case MHIP_UI32: MHIP_CV(uint32_t); break;
        case MHIP_UI8: MHIP_CV(uint8_t); break;
        case MHIP_I8: MHIP_CV(int8_t); break;
        case MHIP_I16: MHIP_CV(int16_t); break;
        case MHIP_UI16: MHIP_CV(uint16_t); break;
        case MHIP_UI64: MHIP_CV(uint64_t); break;
        case MHIP_I1: hipLaunchKernelGGL((to_bool_kernel<S>), dim3(grid), dim3(256), 0, s, (const S*)x, (uint8_t*)y, n); break;
        default: return fail(MHIP_ERR_UNSUPPORTED, "mhip_convert: destination dtype %d", dst);
    }
#undef MHIP_CV
    return check_launch("convert");
}
}  // namespace mhip

extern "C" int mhip_convert(void* stream, const void* x, void* y, int64_t n, int src_dtype,
                            int dst_dtype) {
    if (!x || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_convert: NULL pointer");
    if (n < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_convert: negative size");
    if (n == 0) return MHIP_OK;
    hipStream_t s = as_stream(stream);
    if (src_dtype == MHIP_F32 && (dst_dtype == MHIP_BF16 || dst_dtype == MHIP_F16) && n >= 8 &&
        ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0) {
        const int64_t ngroups = n / 4;
        unsigned grid;
        if (grid_for(ngroups, 512, &grid)) return MHIP_ERR_UNSUPPORTED;
        if (dst_dtype == MHIP_BF16)
            hipLaunchKernelGGL((narrow_vec_kernel<bf16_t>), dim3(grid), dim3(256), 0, s, (const float*)x, (bf16_t*)y, ngroups);
        else
            hipLaunchKernelGGL((narrow_vec_kernel<f16_t>), dim3(grid), dim3(256), 0, s, (const float*)x, (f16_t*)y, ngroups);
        const int64_t done = ngroups * 4;
        if (done == n) return check_launch("convert");
        const int es = 2;
        return mhip_convert(stream, (const char*)x + done * 4, (char*)y + done * es, n - done, src_dtype, dst_dtype);
    }
    switch (src_dtype) {
        case MHIP_F32: return convert_from<float>(s, x, y, n, dst_dtype);
        case MHIP_F64: return convert_from<double>(s, x, y, n, dst_dtype);
        case MHIP_BF16: return convert_from<bf16_t>(s, x, y, n, dst_dtype);
        case MHIP_F16: return convert_from<f16_t>(s, x, y, n, dst_dtype);
        case MHIP_I32: return convert_from<int32_t>(s, x, y, n, dst_dtype);
        case MHIP_I64: return convert_from<int64_t>(s, x, y, n, dst_dtype);
        case MHIP_UI32: return convert_from<uint32_t>(s, x, y, n, dst_dtype);
        case MHIP_UI8: case MHIP_I1: return convert_from<uint8_t>(s, x, y, n, dst_dtype);
        case MHIP_I8: return convert_from<int8_t>(s, x, y, n, dst_dtype);
        case MHIP_I16: return convert_from<int16_t>(s, x, y, n, dst_dtype);
        case MHIP_UI16: return convert_from<uint16_t>(s, x, y, n, dst_dtype);
        case MHIP_UI64: return convert_from<uint64_t>(s, x, y, n, dst_dtype);
        default: return fail(MHIP_ERR_UNSUPPORTED, "mhip_convert: source dtype %d", src_dtype);
    }
}

extern "C" int mhip_convert_batch(void* stream, int count, const void* const* xs, void* const* ys,
                                  const int64_t* ns, int src_dtype, int dst_dtype) {
    const char* what = "mhip_convert_batch";
    if (count < 0 || (count > 0 && (!xs || !ys || !ns))) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: bad table", what);
    if (src_dtype != MHIP_F32 || (dst_dtype != MHIP_BF16 && dst_dtype != MHIP_F16))
        return fail(MHIP_ERR_UNSUPPORTED, "%s: f32 -> bf16 / f16 only (got %d -> %d)", what, src_dtype, dst_dtype);
    hipStream_t s = as_stream(stream);
    for (int done = 0; done < count;) {
        ConvertBatch b;
        b.count = 0;
        uint64_t blocks = 0;
        for (; done < count && b.count < kBatchMax; done++) {
            if (ns[done] < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative size", what);
            if (ns[done] == 0) continue;
            if (!xs[done] || !ys[done]) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL pointer", what);
            const uint64_t nb = (uint64_t)((ns[done] + 2047) / 2048);
            if (blocks + nb > 0x7FFFFFFFull) break;           // the rest goes into another launch
            b.x[b.count] = static_cast<const float*>(xs[done]);
            b.y[b.count] = ys[done];
            b.n[b.count] = ns[done];
            b.first_block[b.count] = (uint32_t)blocks;
            blocks += nb;
            b.count++;
        }
        if (b.count == 0) {
            if (done < count) return fail(MHIP_ERR_UNSUPPORTED, "%s: tensor too large for one launch", what);
            break;
        }
        b.first_block[b.count] = (uint32_t)blocks;
        if (dst_dtype == MHIP_BF16) hipLaunchKernelGGL((narrow_batch_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, s, b);
        else hipLaunchKernelGGL((narrow_batch_kernel<f16_t>), dim3((unsigned)blocks), dim3(256), 0, s, b);
        const int st = check_launch(what);
        if (st != MHIP_OK) return st;
    }
    return MHIP_OK;
}

extern "C" int mhip_transpose_0213(void* stream, const void* x, void* y, int64_t d0, int64_t d1,
                                   int64_t d2, int64_t d3, int dtype) {
    if (!x || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_transpose_0213: NULL pointer");
    if (d0 < 0 || d1 < 0 || d2 < 0 || d3 < 0)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_transpose_0213: negative size");
    const int64_t n = d0 * d1 * d2 * d3;
    if (n == 0) return MHIP_OK;
    unsigned grid;
    if (grid_for(n, 256, &grid)) return MHIP_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
    const int es = dtype_size(dtype);
    // output is [d0][d2][d1][d3]: the kernel walks output indices with (d1, d2) swapped roles
    if (es == 2)
        hipLaunchKernelGGL((transpose_0213_kernel<uint16_t>), dim3(grid), dim3(256), 0, s,
                           (const uint16_t*)x, (uint16_t*)y, d1, d2, d3, n);
    else if (es == 4)
        hipLaunchKernelGGL((transpose_0213_kernel<uint32_t>), dim3(grid), dim3(256), 0, s,
                           (const uint32_t*)x, (uint32_t*)y, d1, d2, d3, n);
    else
        return fail(MHIP_ERR_UNSUPPORTED, "mhip_transpose_0213: dtype %d", dtype);
    return check_launch("transpose_0213");
}

extern "C" int mhip_split_qkv_heads(void* stream, const void* qkv, void* q, void* k, void* v,
                                    int64_t B, int64_t S, int64_t H, int64_t D, int dtype) {
    if (!qkv || !q || !k || !v) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_split_qkv_heads: NULL pointer");
    if (B < 0 || S < 0 || H < 0 || D < 0)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_split_qkv_heads: negative size");
    const int es = dtype_size(dtype);
    if (es != 2 && es != 4) return fail(MHIP_ERR_UNSUPPORTED, "mhip_split_qkv_heads: dtype %d", dtype);
    if ((D * es) % 16 != 0) return fail(MHIP_ERR_UNSUPPORTED, "mhip_split_qkv_heads: head_dim bytes %% 16 != 0");
    if (((reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(q) |
          reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v)) & 15) != 0)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_split_qkv_heads: buffers must be 16-byte aligned");
    const int64_t dv = D * es / 16, n = B * S * 3 * H * dv;
    if (n == 0) return MHIP_OK;
    unsigned grid;
    if (grid_for(n, 256, &grid)) return MHIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(split_qkv_kernel, dim3(grid), dim3(256), 0, as_stream(stream),
                       (const u32x4*)qkv, (u32x4*)q, (u32x4*)k, (u32x4*)v, S, H, dv, n);
    return check_launch("split_qkv_heads");
}

extern "C" int mhip_iota(void* stream, void* y, int64_t outer, int64_t n, int64_t inner, int dtype) {
    if (!y) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_iota: NULL pointer");
    if (outer < 0 || n < 0 || inner < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_iota: negative size");
    const int64_t total = outer * n * inner;
    if (total == 0) return MHIP_OK;
    unsigned grid;
    if (grid_for(total, 256, &grid)) return MHIP_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
#define MHIP_IOTA(T) \
    hipLaunchKernelGGL((iota_kernel<T>), dim3(grid), dim3(256), 0, s, (T*)y, n, inner, total)
    switch (dtype) {
        case MHIP_I32: MHIP_IOTA(int32_t); break;
        case MHIP_I64: MHIP_IOTA(int64_t); break;
        case MHIP_UI32: MHIP_IOTA(uint32_t); break;
        case MHIP_UI64: MHIP_IOTA(uint64_t); break;
        case MHIP_I16: MHIP_IOTA(int16_t); break;
        case MHIP_UI16: MHIP_IOTA(uint16_t); break;
        case MHIP_I8: MHIP_IOTA(int8_t); break;
        case MHIP_UI8: MHIP_IOTA(uint8_t); break;
        case MHIP_F32: MHIP_IOTA(float); break;
        case MHIP_F64: MHIP_IOTA(double); break;
        case MHIP_BF16: MHIP_IOTA(bf16_t); break;
        case MHIP_F16: MHIP_IOTA(f16_t); break;
        default: return fail(MHIP_ERR_UNSUPPORTED, "mhip_iota: dtype %d", dtype);
    }
#undef MHIP_IOTA
    return check_launch("iota");
}

extern "C" int mhip_argmax(void* stream, const void* x, void* out_idx, void* out_val, int64_t rows,
                           int64_t cols, int dtype, int idx_dtype) {
    if (!x || !out_idx) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_argmax: NULL pointer");
    if (rows < 0 || cols <= 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_argmax: bad size");
    if (rows == 0) return MHIP_OK;
    unsigned grid;
    if (grid_for(rows, 4, &grid)) return MHIP_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
#define MHIP_AM(T, I)                                                                         \
    hipLaunchKernelGGL((argmax_kernel<T, I>), dim3(grid), dim3(256), 0, s, (const T*)x,       \
                       (I*)out_idx, (T*)out_val, rows, cols)
    if (idx_dtype == MHIP_I32) {
        if (dtype == MHIP_F32) MHIP_AM(float, int32_t);
        else if (dtype == MHIP_BF16) MHIP_AM(bf16_t, int32_t);
        else if (dtype == MHIP_F16) MHIP_AM(f16_t, int32_t);
        else return fail(MHIP_ERR_UNSUPPORTED, "mhip_argmax: dtype %d", dtype);
    } else if (idx_dtype == MHIP_I64) {
        if (dtype == MHIP_F32) MHIP_AM(float, int64_t);
        else if (dtype == MHIP_BF16) MHIP_AM(bf16_t, int64_t);
        else if (dtype == MHIP_F16) MHIP_AM(f16_t, int64_t);
        else return fail(MHIP_ERR_UNSUPPORTED, "mhip_argmax: dtype %d", dtype);
    } else {
        return fail(MHIP_ERR_UNSUPPORTED, "mhip_argmax: index dtype %d", idx_dtype);
    }
#undef MHIP_AM
    return check_launch("argmax");
}
