// Definitions shared by the GEMM kernels.
#pragma once
#include <math.h>

#include <type_traits>

#include "common.h"

namespace mhip {

constexpr int kBK = 64;              // k extent of one LDS stage
constexpr int kRowBytes = kBK * 2;   // bytes per LDS tile row (16-bit elements)
constexpr uint32_t kOob = 0x80000000u;  // byte offset beyond any buffer: load returns 0

struct GemmArgs {
    const void* a;
    const void* b;
    const void* bias;
    void* c;
    int M, N, K;
    int lda, ldb;           // leading dimensions in elements of the stored matrices
    int64_t sa, sb, sc;     // batch strides in elements
    int act;
    int tiles_m, tiles_n;
    const void* residual = nullptr;   // C's layout and batch stride; added after the activation (may alias c)
    int ldc = 0;                      // row stride of C and the residual in elements; 0 = N (gemm256.hip only: a column slice of a wider C)
    int stream_c = 0;                 // gemm256.hip: C is far larger than the L2s, store it with the streaming hint
};

template <typename T> struct Mfma32;
template <> struct Mfma32<bf16_t> {
    __device__ static f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mfma32<f16_t> {
    __device__ static f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};

template <typename T> struct alignas(8) Pack4 { T v[4]; };

__device__ inline float apply_act(float v, int act) {
    switch (act) {
        case MHIP_ACT_RELU: return fmaxf(v, 0.f);
        case MHIP_ACT_GELU: {
            const float inner = 0.7978845608028654f * (v + 0.044715f * v * v * v);
            return 0.5f * v * (1.f + tanhf(inner));
        }
        case MHIP_ACT_SILU: return v / (1.f + expf(-v));
        case MHIP_ACT_TANH: return tanhf(v);
        case MHIP_ACT_SIGMOID: return 1.f / (1.f + expf(-v));
        case MHIP_ACT_GELU_ERF: return 0.5f * v * (1.f + erff(v * 0.7071067811865476f));
        default: return v;
    }
}

// Activation known at compile time (the switch folds away), and a dispatcher that
// turns the runtime code into such a constant ONCE per kernel: an epilogue that
// tests the code per element unrolls into hundreds of branchy copies, far larger
// than the instruction cache.
// The same functions for results that are rounded to 16 bits (the MFMA kernels): exp2 and the
// hardware reciprocal (about 1 ulp each) instead of the library's tanhf / expf, which cost
// an epilogue of 256 accumulators per lane more than the K loop of a short GEMM.
//   0.5 (1 + tanh u) = 1 / (1 + 2^(-2 log2(e) u)),  tanh u = 1 - 2 / (1 + 2^(2 log2(e) u))
template <int ACT>
__device__ inline float apply_act_c(float v) {
    constexpr float kLog2e = 1.4426950408889634f;
    if (ACT == MHIP_ACT_NONE) return v;
    if (ACT == MHIP_ACT_RELU) return fmaxf(v, 0.f);
    float r = v;
    if (ACT == MHIP_ACT_GELU) {
        constexpr float c0 = -2.f * kLog2e * 0.7978845608028654f;
        constexpr float c1 = c0 * 0.044715f;
        const float t = v * fmaf(v * v, c1, c0);
        r = v * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(t));
    }
    if (ACT == MHIP_ACT_SILU) r = v * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-kLog2e * v));
    if (ACT == MHIP_ACT_SIGMOID) r = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-kLog2e * v));
    if (ACT == MHIP_ACT_TANH) r = 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(2.f * kLog2e * v));
    if (ACT == MHIP_ACT_GELU_ERF) r = 0.5f * v * (1.f + erff(v * 0.7071067811865476f));
    // The fp32 result is final here.  Without this the compiler may merge the last multiply with
    // the conversion to f16 that follows (one rounding instead of two) in some kernels and not in
    // others, and the same problem would round differently depending on the tile choice.
    asm("" : "+v"(r));
    return r;
}
// eight stored elements (one 16-byte chunk of a C row) plus eight residual elements: each sum
// is rounded once more, exactly what a separate add kernel over the stored C would produce
template <typename T>
__device__ inline u32x4 add_chunk(u32x4 w, u32x4 r) {
    Pack4<T> a0 = __builtin_bit_cast(Pack4<T>, u32x2{w.x, w.y}), a1 = __builtin_bit_cast(Pack4<T>, u32x2{w.z, w.w});
    const Pack4<T> r0 = __builtin_bit_cast(Pack4<T>, u32x2{r.x, r.y}), r1 = __builtin_bit_cast(Pack4<T>, u32x2{r.z, r.w});
#pragma unroll
    for (int e = 0; e < 4; e++) {
        a0.v[e] = Elem<T>::from_f32(Elem<T>::to_f32(a0.v[e]) + Elem<T>::to_f32(r0.v[e]));
        a1.v[e] = Elem<T>::from_f32(Elem<T>::to_f32(a1.v[e]) + Elem<T>::to_f32(r1.v[e]));
    }
    const u32x2 lo = __builtin_bit_cast(u32x2, a0), hi = __builtin_bit_cast(u32x2, a1);
    return u32x4{lo.x, lo.y, hi.x, hi.y};
}

template <typename F>
__device__ inline void dispatch_act(int act, F&& f) {
    switch (act) {
        case MHIP_ACT_RELU: f(std::integral_constant<int, MHIP_ACT_RELU>{}); break;
        case MHIP_ACT_GELU: f(std::integral_constant<int, MHIP_ACT_GELU>{}); break;
        case MHIP_ACT_SILU: f(std::integral_constant<int, MHIP_ACT_SILU>{}); break;
        case MHIP_ACT_TANH: f(std::integral_constant<int, MHIP_ACT_TANH>{}); break;
        case MHIP_ACT_SIGMOID: f(std::integral_constant<int, MHIP_ACT_SIGMOID>{}); break;
        case MHIP_ACT_GELU_ERF: f(std::integral_constant<int, MHIP_ACT_GELU_ERF>{}); break;
        default: f(std::integral_constant<int, MHIP_ACT_NONE>{}); break;
    }
}

// Maps the linear workgroup id to a C tile.  Consecutive ids go to different
// XCDs (round-robin dispatch), so ids are first regrouped so that each XCD's
// share is a contiguous range, then walked in bands of kGroupM tile rows:
// the workgroups resident on one XCD then share A row panels and B column
// panels through that XCD's L2.
constexpr int kXcds = 8;
constexpr int kGroupM = 4;
__device__ inline void tile_of(int pid, int grid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int per = (grid + kXcds - 1) / kXcds;
    const int tall = (grid % kXcds == 0) ? kXcds : grid % kXcds;
    const int xcd = pid % kXcds, local = pid / kXcds;
    const int lpid = (xcd < tall) ? xcd * per + local
                                  : tall * per + (xcd - tall) * (per - 1) + local;
    const int band = kGroupM * tiles_n;
    const int g = lpid / band, first = g * kGroupM;
    const int gsz = min(tiles_m - first, kGroupM);
    tm = first + (lpid % band) % gsz;
    tn = (lpid % band) / gsz;
}

}  // namespace mhip
