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

template <typename T>
__device__ inline Vec16<T> opaque(const Vec16<T>& v) {
    u32x4 t = __builtin_bit_cast(u32x4, v);
    asm volatile("" : "+v"(t));
    return __builtin_bit_cast(Vec16<T>, t);
}

// Sums over the elements of one 16-byte vector without widening them first: for 16-bit types
// the two-element dot product instruction adds a pair per issue (against the pair itself for a
// sum of squares, against (1, 1) for a plain sum).
template <typename T> struct VecSum;
template <> struct VecSum<float> {
    __device__ static float sum(const Vec16<float>& v, float acc) { return acc + ((v.v[0] + v.v[1]) + (v.v[2] + v.v[3])); }
    __device__ static float sumsq(const Vec16<float>& v, float acc) {
#pragma unroll
        for (int e = 0; e < 4; e++) acc = fmaf(v.v[e], v.v[e], acc);
        return acc;
    }
};
template <> struct VecSum<bf16_t> {
    typedef __bf16 pair_t __attribute__((ext_vector_type(2)));
    struct Pairs { pair_t p[4]; };
    __device__ static float sum(const Vec16<bf16_t>& v, float acc) {
        const Pairs q = __builtin_bit_cast(Pairs, v);
        const pair_t ones = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
        for (int i = 0; i < 4; i++) acc = __builtin_amdgcn_fdot2_f32_bf16(q.p[i], ones, acc, false);
        return acc;
    }
    __device__ static float sumsq(const Vec16<bf16_t>& v, float acc) {
        const Pairs q = __builtin_bit_cast(Pairs, v);
#pragma unroll
        for (int i = 0; i < 4; i++) acc = __builtin_amdgcn_fdot2_f32_bf16(q.p[i], q.p[i], acc, false);
        return acc;
    }
};
template <> struct VecSum<f16_t> {
    typedef _Float16 pair_t __attribute__((ext_vector_type(2)));
    struct Pairs { pair_t p[4]; };
    __device__ static float sum(const Vec16<f16_t>& v, float acc) {
        const Pairs q = __builtin_bit_cast(Pairs, v);
        const pair_t ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
        for (int i = 0; i < 4; i++) acc = __builtin_amdgcn_fdot2(q.p[i], ones, acc, false);
        return acc;
    }
    __device__ static float sumsq(const Vec16<f16_t>& v, float acc) {
        const Pairs q = __builtin_bit_cast(Pairs, v);
#pragma unroll
        for (int i = 0; i < 4; i++) acc = __builtin_amdgcn_fdot2(q.p[i], q.p[i], acc, false);
        return acc;
    }
};

// A row shared by WPR waves of the workgroup (WPR = 2 or 4), R rows per wave group at a time
// (4 / WPR * R rows per workgroup): each lane holds only NV vectors of each row and of the
// parameters, so the kernel needs few registers and the CU holds its full complement of waves,
// each with a small contiguous piece of memory in flight.  Statistics: DPP reduction inside
// each wave, then one LDS slot per wave and a workgroup barrier (two slot sets, used
// alternately, so a set is never rewritten before every wave has read it).  Vectors beyond
// the row hold zeros (softmax skips them).  The kernel is as fast as its instruction count is
// low -- it measures a few percent per instruction and element -- hence the pair sums above
// and no per-element selects.  R = 2 halves the parameter reads per row: with gamma AND beta
// (16 KB at 4096 columns) those reads no longer stay in the CU's vector cache.
//
// chunk > 0: the workgroup takes `chunk` consecutive iterations' worth of rows and the grid
// covers all rows once -- workgroups start in address order as CUs free up, so the rows in
// flight on the chip form one contiguous window of memory (measured 10 % faster than a
// persistent grid whose workgroups drift apart); chunk == 0: a persistent grid, workgroup b
// takes rows b, b + grid, ...
template <typename T, int OP, int NV, int WPR, int R>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(NV * R <= 2 ? 8 : NV * R <= 4 ? 4 : 2)))
void row_split_kernel(const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta,
                      T* __restrict__ y, int64_t rows, int cols, float eps, int chunk) {
    constexpr int E = Elem<T>::kPerVec;
    constexpr int RPB = 4 / WPR * R;             // rows per workgroup and iteration
    constexpr bool k16 = sizeof(T) == 2;
    __shared__ float red[2][4][R];
    // the wave number is uniform: as a scalar it keeps the row addresses in scalar registers
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int sub = wave % WPR;                  // which part of the row this wave holds
    const int grp = wave / WPR;                  // which rows of the workgroup's RPB rows
    const int nvec = cols / E;
    const float inv_cols = 1.f / (float)cols;
    const bool has_g = OP != kSoftmax && gamma != nullptr;
    const bool has_b = OP == kLayerNorm && beta != nullptr;
    // vector v of this lane: index (v * WPR + sub) * 64 + lane  (consecutive waves, consecutive KB)
    bool in[NV];
    unsigned off[NV];                            // element offset of the vector inside its row
    Vec16<T> gv[NV], bv[NV];
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int idx = (v * WPR + sub) * 64 + lane;
        in[v] = idx < nvec;
        off[v] = (unsigned)idx * E;
        if (OP != kSoftmax) {
            if (has_g && in[v]) gv[v] = load16(gamma + off[v]);
            if (has_b && in[v]) bv[v] = load16(beta + off[v]);
        }
    }
    // each of the R values summed (or maximised) over the waves of the row
    auto group_reduce = [&](float (&v)[R], bool is_max, int set) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            v[r] = is_max ? wave_max(v[r]) : wave_sum(v[r]);
            if (lane == 0) red[set][wave][r] = v[r];
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; r++) {
            float t = red[set][grp * WPR][r];
#pragma unroll
            for (int i = 1; i < WPR; i++) t = is_max ? fmaxf(t, red[set][grp * WPR + i][r]) : t + red[set][grp * WPR + i][r];
            v[r] = t;
        }
    };
    // chunk < 0: one iteration per workgroup, and the workgroups of XCD x (ids x, x + 8, ...: the
    // dispatcher deals ids round-robin over the eight XCDs) take the x-th eighth of the rows -- the
    // rows whose tiles a GEMM on [rows, cols] has just written from that XCD, and whose tiles the
    // next GEMM reads on it, so a tensor that fits the L2s is found there (grid a multiple of 8).
    const unsigned bid = chunk < 0 ? (blockIdx.x % 8u) * (gridDim.x / 8u) + blockIdx.x / 8u : blockIdx.x;
    if (chunk < 0) chunk = 1;
    const int64_t first = chunk > 0 ? (int64_t)bid * chunk * RPB : (int64_t)bid * RPB;
    const int64_t stop = chunk > 0 ? (first + (int64_t)chunk * RPB < rows ? first + (int64_t)chunk * RPB : rows) : rows;
    const int64_t step = chunk > 0 ? RPB : (int64_t)gridDim.x * RPB;
    for (int64_t base = first; base < stop; base += step) {
        const int64_t row0 = base + grp * R;
        bool live[R];
        Vec16<T> cur[R][NV];
#pragma unroll
        for (int r = 0; r < R; r++) {
            live[r] = row0 + r < rows;
            const T* xr = x + (row0 + r) * cols;
#pragma unroll
            for (int v = 0; v < NV; v++) {
                cur[r][v] = __builtin_bit_cast(Vec16<T>, u32x4{0, 0, 0, 0});
                if (live[r] && in[v]) cur[r][v] = load16_stream(xr + off[v]);
            }
        }
        float f[R][NV][E];
        float a[R];
        if (OP == kSoftmax) {
            float m[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                m[r] = -INFINITY;
#pragma unroll
                for (int v = 0; v < NV; v++) {
                    float mv = -INFINITY;
#pragma unroll
                    for (int e = 0; e < E; e++) {
                        f[r][v][e] = Elem<T>::to_f32(cur[r][v].v[e]);
                        mv = fmaxf(mv, f[r][v][e]);
                    }
                    m[r] = (live[r] && in[v]) ? fmaxf(m[r], mv) : m[r];
                }
            }
            group_reduce(m, true, 0);
            constexpr float kLog2e = 1.4426950408889634f;
            float s[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float ms = m[r] * kLog2e;
                s[r] = 0.f;
#pragma unroll
                for (int v = 0; v < NV; v++) {
                    float sv = 0.f;
#pragma unroll
                    for (int e = 0; e < E; e++) {
                        f[r][v][e] = k16 ? __builtin_amdgcn_exp2f(fmaf(f[r][v][e], kLog2e, -ms)) : expf(f[r][v][e] - m[r]);
                        sv += f[r][v][e];
                    }
                    s[r] += (live[r] && in[v]) ? sv : 0.f;
                }
            }
            group_reduce(s, false, 1);
#pragma unroll
            for (int r = 0; r < R; r++) a[r] = 1.f / s[r];
        } else if (OP == kLayerNorm) {
            float s[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                s[r] = 0.f;
#pragma unroll
                for (int v = 0; v < NV; v++) s[r] = VecSum<T>::sum(cur[r][v], s[r]);
            }
            group_reduce(s, false, 0);
            float q[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float mean = s[r] * inv_cols;
                q[r] = 0.f;
#pragma unroll
                for (int v = 0; v < NV; v++) {
                    const float mv = (live[r] && in[v]) ? mean : 0.f;       // vectors beyond the row stay 0
#pragma unroll
                    for (int e = 0; e < E; e++) {
                        f[r][v][e] = Elem<T>::to_f32(cur[r][v].v[e]) - mv;
                        q[r] = fmaf(f[r][v][e], f[r][v][e], q[r]);
                    }
                }
            }
            group_reduce(q, false, 1);
#pragma unroll
            for (int r = 0; r < R; r++) a[r] = 1.f / sqrtf(q[r] * inv_cols + eps);
        } else {
            float q[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                q[r] = 0.f;
#pragma unroll
                for (int v = 0; v < NV; v++) q[r] = VecSum<T>::sumsq(cur[r][v], q[r]);
            }
            group_reduce(q, false, 0);
            __syncthreads();      // one reduction per row: the barrier that frees the slot set
#pragma unroll
            for (int r = 0; r < R; r++) {
                a[r] = 1.f / sqrtf(q[r] * inv_cols + eps);
#pragma unroll
                for (int v = 0; v < NV; v++)
#pragma unroll
                    for (int e = 0; e < E; e++) f[r][v][e] = Elem<T>::to_f32(cur[r][v].v[e]);
            }
        }
#pragma unroll
        for (int v = 0; v < NV; v++) {
            Vec16<T> gq, bq;
            if (OP != kSoftmax) {          // widened here, not earlier (registers)
                gq = opaque(gv[v]);
                bq = opaque(bv[v]);
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                if (live[r] && in[v]) {
                    Vec16<T> o;
#pragma unroll
                    for (int e = 0; e < E; e++) {
                        float t = f[r][v][e] * a[r];     // softmax: exp / sum; norms: (x - mean) * rstd, x * rstd
                        if (OP != kSoftmax) {
                            const float g = has_g ? Elem<T>::to_f32(gq.v[e]) : 1.f;
                            const float bt = has_b ? Elem<T>::to_f32(bq.v[e]) : 0.f;
                            t = fmaf(t, g, bt);
                        }
                        o.v[e] = Elem<T>::from_f32(t);
                    }
                    store16_stream(y + (row0 + r) * cols + off[v], o);
                }
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
// EXACT: 0.5 v (1 + erf(v / sqrt 2)) with the library's erff; otherwise the tanh approximation.
template <typename T, bool EXACT = false>
__device__ inline float gelu_tanh_f(float v) {
    if (EXACT) return 0.5f * v * (1.f + erff(v * 0.7071067811865476f));
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

template <typename T, bool EXACT>
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
                        gelu_tanh_f<T, EXACT>(Elem<T>::to_f32(in.v[4 * q + e]) + bv[e]));
            }
            store16_stream(y + i * E, o);
        }
    }
}

// Tiles of R rows x 256 vectors, one workgroup each, workgroups in address order (the grid is
// one-dimensional: row tile major, column block minor).  A thread keeps one column of the tile:
// its bias vector is read once, the R loads are issued together, no index arithmetic per vector.
template <typename T, int R, bool EXACT>
__global__ __launch_bounds__(256) void bias_gelu_tile_kernel(const T* __restrict__ x,
                                                             const T* __restrict__ bias,
                                                             T* __restrict__ y, int64_t rows,
                                                             int nvec_row, unsigned blocks_per_row) {
    constexpr int E = Elem<T>::kPerVec;
    const unsigned by = blockIdx.x / blocks_per_row, bx = blockIdx.x - by * blocks_per_row;
    const int c = (int)(bx * 256 + threadIdx.x);
    if (c >= nvec_row) return;
    Vec16<T> bv;
#pragma unroll
    for (int e = 0; e < E; e++) bv.v[e] = Elem<T>::from_f32(0.f);
    if (bias) bv = load16(bias + (int64_t)c * E);
    const int64_t r0 = (int64_t)by * R;
    Vec16<T> in[R];
#pragma unroll
    for (int r = 0; r < R; r++)
        if (r0 + r < rows) in[r] = load16_stream(x + ((r0 + r) * nvec_row + c) * E);
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (r0 + r < rows) {
            Vec16<T> o;
#pragma unroll
            for (int e = 0; e < E; e++)
                o.v[e] = Elem<T>::from_f32(gelu_tanh_f<T, EXACT>(Elem<T>::to_f32(in[r].v[e]) + Elem<T>::to_f32(bv.v[e])));
            store16_stream(y + ((r0 + r) * nvec_row + c) * E, o);
        }
    }
}

template <typename T, bool EXACT>
__global__ __launch_bounds__(256) void bias_gelu_scalar_kernel(const T* __restrict__ x,
                                                               const T* __restrict__ bias,
                                                               T* __restrict__ y, int64_t n,
                                                               int64_t cols) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float v = Elem<T>::to_f32(x[i]);
    if (bias) v += Elem<T>::to_f32(bias[i % cols]);
    y[i] = Elem<T>::from_f32(gelu_tanh_f<T, EXACT>(v));
}

// ---------------------------------------------------------------------------
// Host-side dispatch
// ---------------------------------------------------------------------------
static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename K, typename... Args>
static void launch_persistent(K kern, size_t lds, int per_cu, int64_t want, hipStream_t s, Args... args) {
    if (per_cu <= 0 &&
        (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 256, lds) != hipSuccess || per_cu <= 0))
        per_cu = 4;
    // the occupancy query counts LDS to the last byte; keep a margin so that every workgroup of
    // the grid really is resident at once
    if (lds && per_cu > (int)((160 * 1024 - 4096) / (lds + 512))) per_cu = (int)((160 * 1024 - 4096) / (lds + 512));
    if (per_cu < 1) per_cu = 1;
    const int64_t cap = (int64_t)compute_units() * per_cu;
    hipLaunchKernelGGL(kern, dim3((unsigned)(want < cap ? want : cap)), dim3(256), lds, s, args...);
}

template <typename T, int OP, int NVS, int WPR>
static void launch_split(const RowLaunch& c, hipStream_t s, const T* xp, const T* gp, const T* bp, T* yp, int64_t rows,
                         int cols, float eps) {
    const int rpb = 4 / WPR * (c.r == 2 ? 2 : 1);
    const int64_t units = (rows + rpb - 1) / rpb;
    if (c.ordered) {
        // a tensor small enough to sit in the L2s between two kernels: rows by XCD (see the kernel).
        // Not for large ones: eight separate windows of memory in flight instead of one cost the
        // [32768, 4096] benchmarks 4 to 17 % (softmax 0.80 -> 0.71 of the HBM peak, RMSNorm 0.79 -> 0.65).
        const bool by_xcd = units % 8 == 0 && (int64_t)rows * cols * (int64_t)sizeof(T) <= (16 << 20);
        const int chunk = by_xcd ? -1 : 1;
        if (c.r == 2)
            hipLaunchKernelGGL((row_split_kernel<T, OP, NVS, WPR, 2>), dim3((unsigned)units), dim3(256), 0, s, xp, gp, bp, yp,
                               rows, cols, eps, chunk);
        else
            hipLaunchKernelGGL((row_split_kernel<T, OP, NVS, WPR, 1>), dim3((unsigned)units), dim3(256), 0, s, xp, gp, bp, yp,
                               rows, cols, eps, chunk);
    } else if (c.r == 2) {
        launch_persistent(row_split_kernel<T, OP, NVS, WPR, 2>, 0, c.per_cu, units, s, xp, gp, bp, yp, rows, cols, eps, 0);
    } else {
        launch_persistent(row_split_kernel<T, OP, NVS, WPR, 1>, 0, c.per_cu, units, s, xp, gp, bp, yp, rows, cols, eps, 0);
    }
}

template <typename T, int OP>
static int launch_row(hipStream_t s, const void* x, const void* g, const void* b, void* y,
                      int64_t rows, int64_t cols, float eps, const RowLaunch* forced, int dtype) {
    constexpr int E = Elem<T>::kPerVec;
    const T* xp = static_cast<const T*>(x);
    const T* gp = static_cast<const T*>(g);
    const T* bp = static_cast<const T*>(b);
    T* yp = static_cast<T*>(y);
    const bool vec_ok = cols % E == 0 && cols <= 64 * 16 * E && aligned16(x) && aligned16(y) &&
                        aligned16(g) && aligned16(b);
    if (vec_ok) {
        const int nvec = (int)(cols / E);
        RowLaunch c;
        if (forced) c = *forced;
        else if (!tuned_row_launch(OP, dtype, rows, cols, gp != nullptr, OP == kLayerNorm && bp != nullptr, &c)) c = RowLaunch();
        // defaults (measured on [32768, 4096] bf16: ordered split launches run at the rate of a plain
        // copy; with both gamma and beta two rows per wave group keep the parameters' 16 KB per row
        // from falling out of the CU's vector cache; rows of up to 256 vectors are faster two at a
        // time for every operator)
        if (c.kind != 1 && c.kind != 2) c.kind = nvec > 64 ? 2 : 1;
        if (c.kind == 2 && nvec <= 64) c.kind = 1;
        if (c.r != 1 && c.r != 2) c.r = (nvec <= 256 || (OP == kLayerNorm && gp && bp)) ? 2 : 1;
        if (c.ordered < 0) c.ordered = 1;
        if (c.kind == 2) {
            if (nvec <= 128) launch_split<T, OP, 1, 2>(c, s, xp, gp, bp, yp, rows, (int)cols, eps);
            else if (nvec <= 256) launch_split<T, OP, 1, 4>(c, s, xp, gp, bp, yp, rows, (int)cols, eps);
            else if (nvec <= 512) launch_split<T, OP, 2, 4>(c, s, xp, gp, bp, yp, rows, (int)cols, eps);
            else launch_split<T, OP, 4, 4>(c, s, xp, gp, bp, yp, rows, (int)cols, eps);
        } else {
            // persistent workgroups of four waves, one row per wave, as many as the device holds at
            // once for the kernel's register and LDS footprint; the parameters are staged once
            const int64_t want = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
            const size_t lds = (OP == kSoftmax) ? 0 : ((gp ? 1 : 0) + ((OP == kLayerNorm && bp) ? 1 : 0)) * (size_t)cols * sizeof(T);
#define MHIP_ROW_CASE(NV) launch_persistent(row_wave_kernel<T, OP, NV>, lds, c.per_cu, want, s, xp, gp, bp, yp, rows, (int)cols, eps)
            if (nvec <= 64) MHIP_ROW_CASE(1);
            else if (nvec <= 128) MHIP_ROW_CASE(2);
            else if (nvec <= 256) MHIP_ROW_CASE(4);
            else if (nvec <= 512) MHIP_ROW_CASE(8);
            else MHIP_ROW_CASE(16);
#undef MHIP_ROW_CASE
        }
    } else {
        hipLaunchKernelGGL((row_block_kernel<T, OP>), dim3((unsigned)rows), dim3(256), 0, s, xp,
                           gp, bp, yp, cols, eps);
    }
    return check_launch("row kernel");
}

template <int OP>
static int row_entry(const char* name, void* stream, const void* x, const void* g, const void* b,
                     void* y, int64_t rows, int64_t cols, float eps, int dtype, const RowLaunch* forced = nullptr) {
    if (rows < 0 || cols < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative size", name);
    if (rows == 0 || cols == 0) return MHIP_OK;
    if (!x || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", name);
    if (rows > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "%s: more than 2^31-1 rows", name);
    hipStream_t s = as_stream(stream);
    switch (dtype) {
        case MHIP_F32: return launch_row<float, OP>(s, x, g, b, y, rows, cols, eps, forced, dtype);
        case MHIP_BF16: return launch_row<bf16_t, OP>(s, x, g, b, y, rows, cols, eps, forced, dtype);
        case MHIP_F16: return launch_row<f16_t, OP>(s, x, g, b, y, rows, cols, eps, forced, dtype);
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: dtype %d (need f32, f16 or bf16)", name, dtype);
    }
}

template <typename T, bool EXACT>
static int launch_gelu(hipStream_t s, const void* x, const void* bias, void* y, int64_t rows,
                       int64_t cols) {
    constexpr int E = Elem<T>::kPerVec;
    const int64_t n = rows * cols;
    const bool vec_ok = cols % E == 0 && cols <= 0x7FFFFFFF && aligned16(x) && aligned16(y) &&
                        aligned16(bias);
    if (vec_ok) {
        const int64_t nvec = n / E;
        const int64_t nvec_row = cols / E;
        // tiles of `tile_rows` rows x 256 vectors in address order (two rows measured fastest on
        // [32768, 4096]: 0.775 of the HBM peak against 0.70 for one row and 0.755 for four)
        const int64_t bpr = (nvec_row + 255) / 256;
        constexpr int tile_rows = 2;
        const int64_t tiles = bpr * ((rows + tile_rows - 1) / tile_rows);
        if (tiles <= 0x7FFFFFFFLL) {
#define MHIP_GELU_TILE(R)                                                                              \
    hipLaunchKernelGGL((bias_gelu_tile_kernel<T, R, EXACT>), dim3((unsigned)tiles), dim3(256), 0, s, static_cast<const T*>(x), \
                       static_cast<const T*>(bias), static_cast<T*>(y), rows, (int)nvec_row, (unsigned)bpr)
            MHIP_GELU_TILE(2);
#undef MHIP_GELU_TILE
        } else {      // more tiles than a grid holds: the grid-stride kernel
            const int64_t want = (nvec + 511) / 512;
            const int64_t cap = (int64_t)compute_units() * 64;
            const bool in_lds = bias && cols * sizeof(float) <= 48 * 1024;
            hipLaunchKernelGGL((bias_gelu_vec_kernel<T, EXACT>), dim3((unsigned)(want < cap ? want : cap)), dim3(256),
                               in_lds ? (size_t)cols * sizeof(float) : 0, s, static_cast<const T*>(x),
                               static_cast<const T*>(bias), static_cast<T*>(y), nvec, (int)nvec_row,
                               in_lds ? 1 : 0);
        }
    } else {
        const int64_t grid = (n + 255) / 256;
        if (grid > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "bias_gelu: tensor too large");
        hipLaunchKernelGGL((bias_gelu_scalar_kernel<T, EXACT>), dim3((unsigned)grid), dim3(256), 0, s,
                           static_cast<const T*>(x), static_cast<const T*>(bias),
                           static_cast<T*>(y), n, cols);
    }
    return check_launch("bias_gelu");
}

// One launch of row operator `op` (0 softmax, 1 LayerNorm, 2 RMSNorm) carried out as `how` says:
// what the autotuner times.
int row_launch_as(int op, const RowLaunch& how, void* stream, const void* x, const void* g, const void* b, void* y,
                  int64_t rows, int64_t cols, float eps, int dtype) {
    switch (op) {
        case kSoftmax: return row_entry<kSoftmax>("row_launch_as", stream, x, nullptr, nullptr, y, rows, cols, 0.f, dtype, &how);
        case kLayerNorm: return row_entry<kLayerNorm>("row_launch_as", stream, x, g, b, y, rows, cols, eps, dtype, &how);
        case kRmsNorm: return row_entry<kRmsNorm>("row_launch_as", stream, x, g, nullptr, y, rows, cols, eps, dtype, &how);
        default: return fail(MHIP_ERR_INVALID_ARGUMENT, "row_launch_as: unknown operator %d", op);
    }
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

template <bool EXACT>
static int gelu_entry(const char* name, void* stream, const void* x, const void* bias, void* y, int64_t rows, int64_t cols,
                      int dtype) {
    if (rows < 0 || cols < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative size", name);
    if (rows == 0 || cols == 0) return MHIP_OK;
    if (!x || !y) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", name);
    hipStream_t s = as_stream(stream);
    switch (dtype) {
        case MHIP_F32: return launch_gelu<float, EXACT>(s, x, bias, y, rows, cols);
        case MHIP_BF16: return launch_gelu<bf16_t, EXACT>(s, x, bias, y, rows, cols);
        case MHIP_F16: return launch_gelu<f16_t, EXACT>(s, x, bias, y, rows, cols);
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: dtype %d", name, dtype);
    }
}

extern "C" int mhip_bias_gelu(void* stream, const void* x, const void* bias, void* y, int64_t rows,
                              int64_t cols, int dtype) {
    return gelu_entry<false>("mhip_bias_gelu", stream, x, bias, y, rows, cols, dtype);
}

extern "C" int mhip_bias_gelu_erf(void* stream, const void* x, const void* bias, void* y, int64_t rows,
                                  int64_t cols, int dtype) {
    return gelu_entry<true>("mhip_bias_gelu_erf", stream, x, bias, y, rows, cols, dtype);
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
