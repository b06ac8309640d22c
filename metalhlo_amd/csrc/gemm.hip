// dot_general GEMM for gfx950: C[b] = act(op(A[b]) . op(B[b]) + bias).
//
// 16-bit types run on v_mfma_f32_32x32x16_{bf16,f16}: a workgroup owns a
// BM x BN tile of C, walks K in steps of 64 with both operand tiles staged in
// LDS (double-buffered, XOR-swizzled 16-byte chunks so that every 128-bit LDS
// access is conflict free), and each wave accumulates a (BM/WGM) x (BN/WGN)
// sub-tile in fp32 registers.  Operand tiles always sit in LDS "k-major"
// ([row][64 k]) because the MFMA wants eight consecutive k per lane; an operand
// whose memory layout has k as the slow axis is transposed in registers on the
// way in (16-byte global loads either way).
// Everything else (fp32, shapes that are not 16-byte friendly) goes through a
// plain LDS-tiled kernel.
#include <mutex>

#include "gemm_common.h"

namespace mhip {

// Swizzle of the 16-byte chunk index inside a 128-byte LDS row.  Rows r..r+15
// (r % 16 == 0) map one chunk column onto 16 distinct bank groups.
__device__ inline int swz(int row) { return ((row >> 1) ^ (row >> 4)) & 7; }

__device__ inline uint32_t lds_off(int row, int chunk) {
    return (uint32_t)(row * kRowBytes + ((chunk ^ swz(row)) << 4));
}

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// ---- operand with k contiguous in memory: [rows_total][ld] ----------------
template <int ROWS, int NT>
struct KMajorLoader {
    static constexpr int kIters = ROWS * 8 / NT;
    u32x4 regs[kIters];
    __device__ void load(__amdgpu_buffer_rsrc_t rsrc, int row0, int k0, int rows_total, int K,
                         int ld) {
        const int c = threadIdx.x & 7;
#pragma unroll
        for (int i = 0; i < kIters; i++) {
            const int r = (threadIdx.x >> 3) + i * (NT / 8);
            const int grow = row0 + r, gk = k0 + c * 8;
            const uint32_t off =
                (grow < rows_total && gk < K) ? (uint32_t)(((int64_t)grow * ld + gk) * 2) : kOob;
            regs[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
        }
    }
    __device__ void store(char* tile) const {
        const int c = threadIdx.x & 7;
#pragma unroll
        for (int i = 0; i < kIters; i++) {
            const int r = (threadIdx.x >> 3) + i * (NT / 8);
            *reinterpret_cast<u32x4*>(tile + lds_off(r, c)) = regs[i];
        }
    }
};

// ---- operand with k as the slow axis in memory: [K][ld] -------------------
// The tile keeps the memory orientation in LDS, [64 k][ROWS mn] (16-byte global
// loads, 16-byte LDS stores), and the MFMA operand is formed on the way OUT of
// LDS with ds_read_b64_tr_b16, which transposes a 4(k) x 16(mn) block across
// 16 lanes: lane i of a 16-lane group supplies the address of k-row i/4,
// mn-columns 4*(i%4)..+3 and receives column i for the four k-rows.
// Chunk swizzle: chunk' = chunk ^ (4 * (k % 4)) puts the four k-rows that one
// transposing read touches on disjoint banks.
template <int ROWS>
__device__ inline uint32_t mn_off(int k, int chunk) {
    return (uint32_t)(k * (ROWS * 2) + ((chunk ^ ((k & 3) << 2)) << 4));
}

template <int ROWS, int NT>
struct MnMajorLoader {
    static constexpr int kCpr = ROWS / 8;               // 16-byte chunks per k-row
    static constexpr int kIters = kBK * kCpr / NT;
    static_assert((kBK * kCpr) % NT == 0, "tile does not split evenly over the workgroup");
    u32x4 regs[kIters];
    __device__ void load(__amdgpu_buffer_rsrc_t rsrc, int col0, int k0, int cols_total, int K,
                         int ld) {
        const int c = threadIdx.x % kCpr;
#pragma unroll
        for (int i = 0; i < kIters; i++) {
            const int k = threadIdx.x / kCpr + i * (NT / kCpr);
            const int gk = k0 + k, gcol = col0 + c * 8;
            const uint32_t off = (gk < K && gcol < cols_total)
                                     ? (uint32_t)(((int64_t)gk * ld + gcol) * 2)
                                     : kOob;
            regs[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
        }
    }
    __device__ void store(char* tile) const {
        const int c = threadIdx.x % kCpr;
#pragma unroll
        for (int i = 0; i < kIters; i++) {
            const int k = threadIdx.x / kCpr + i * (NT / kCpr);
            *reinterpret_cast<u32x4*>(tile + mn_off<ROWS>(k, c)) = regs[i];
        }
    }
};

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// MFMA operand (32 mn x 16 k) for k-step `s` out of a k-major tile.
__device__ inline u32x4 frag_kmajor(const char* tile, int row0, int s, int lane) {
    return *reinterpret_cast<const u32x4*>(tile + lds_off(row0 + (lane & 31), 2 * s + (lane >> 5)));
}
// Same operand out of an mn-major tile via two transposing reads.
template <int ROWS>
__device__ inline u32x4 frag_mnmajor(const char* tile, int mn0, int s, int lane) {
    const int i = lane & 15, g = lane >> 4;
    const int mn = mn0 + 16 * (g & 1) + 4 * (i & 3);
    const int k = 16 * s + 8 * (g >> 1) + (i >> 2);
    const char* p0 = tile + mn_off<ROWS>(k, mn >> 3) + (mn & 7) * 2;
    const char* p1 = tile + mn_off<ROWS>(k + 4, mn >> 3) + (mn & 7) * 2;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p0);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p1);
    u32x4 r;
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    r.x = l2.x; r.y = l2.y; r.z = h2.x; r.w = h2.y;
    return r;
}

template <int ROWS, int NT, bool KMAJOR> struct LoaderSel { using type = KMajorLoader<ROWS, NT>; };
template <int ROWS, int NT> struct LoaderSel<ROWS, NT, false> { using type = MnMajorLoader<ROWS, NT>; };

template <typename T, int BM, int BN, int WGM, int WGN, bool TA, bool TB>
__global__ __launch_bounds__(WGM* WGN * 64) void gemm_mfma_kernel(GemmArgs g) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int kATile = BM * kRowBytes, kBTile = BN * kRowBytes;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    auto a_tile = [&](int buf) { return smem + buf * kATile; };
    auto b_tile = [&](int buf) { return smem + 2 * kATile + buf * kBTile; };

    int tm, tn;
    tile_of(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int64_t batch = blockIdx.y;
    const T* a = static_cast<const T*>(g.a) + batch * g.sa;
    const T* b = static_cast<const T*>(g.b) + batch * g.sb;
    T* c = static_cast<T*>(g.c) + batch * g.sc;
    const T* res = g.residual ? static_cast<const T*>(g.residual) + batch * g.sc : nullptr;

    // A is stored [M][K] (k contiguous) unless TA ([K][M]); B is stored [K][N]
    // (k slow) unless TB ([N][K]).
    const uint32_t a_bytes = (uint32_t)((int64_t)(TA ? g.K : g.M) * g.lda * 2);
    const uint32_t b_bytes = (uint32_t)((int64_t)(TB ? g.N : g.K) * g.ldb * 2);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(a, a_bytes), rb = make_rsrc(b, b_bytes);

    typename LoaderSel<BM, NT, !TA>::type la;
    typename LoaderSel<BN, NT, TB>::type lb;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int lrow = lane & 31, lhalf = lane >> 5;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    auto read_frags = [&](int buf, int s, u32x4(&af)[TM], u32x4(&bf)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; i++)
            af[i] = TA ? frag_mnmajor<BM>(a_tile(buf), wm * WTM + i * 32, s, lane)
                       : frag_kmajor(a_tile(buf), wm * WTM + i * 32, s, lane);
#pragma unroll
        for (int j = 0; j < TN; j++)
            bf[j] = TB ? frag_kmajor(b_tile(buf), wn * WTN + j * 32, s, lane)
                       : frag_mnmajor<BN>(b_tile(buf), wn * WTN + j * 32, s, lane);
    };

    const int KT = (g.K + kBK - 1) / kBK;
    la.load(ra, m0, 0, g.M, g.K, g.lda);
    lb.load(rb, n0, 0, g.N, g.K, g.ldb);
    la.store(a_tile(0));
    lb.store(b_tile(0));
    __syncthreads();

    for (int kt = 0; kt < KT; kt++) {
        const int cur = kt & 1;
        if (kt + 1 < KT) {
            la.load(ra, m0, (kt + 1) * kBK, g.M, g.K, g.lda);
            lb.load(rb, n0, (kt + 1) * kBK, g.N, g.K, g.ldb);
        }
        // Fragments for k-step s+1 are fetched from LDS while the MFMAs of step
        // s run (register double buffer).
        u32x4 af[2][TM], bf[2][TN];
        read_frags(cur, 0, af[0], bf[0]);
#pragma unroll
        for (int s = 0; s < kBK / 16; s++) {
            if (s + 1 < kBK / 16) read_frags(cur, s + 1, af[(s + 1) & 1], bf[(s + 1) & 1]);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = Mfma32<T>::run(bf[s & 1][j], af[s & 1][i], acc[i][j]);
        }
        if (kt + 1 < KT) {
            la.store(a_tile(cur ^ 1));
            lb.store(b_tile(cur ^ 1));
        }
        __syncthreads();
    }

    // Epilogue.  The MFMAs were issued as (B-fragment, A-fragment), so each
    // 32x32 accumulator tile is held transposed: a lane owns row m = lrow and,
    // in register group q = r/4, the four consecutive columns 8q + 4*lhalf + r%4.
    const T* bias = static_cast<const T*>(g.bias);
    const bool vec_store = (g.N % 8 == 0) && ((reinterpret_cast<uintptr_t>(c) & 15) == 0);
    // Stage the wave's sub-tile in LDS as rounded 16-bit rows (padded by 16 bytes
    // against bank conflicts); the rows then go out with lanes running along n, so
    // every store instruction writes whole contiguous row segments.
    constexpr int kRowPad = WTN * 2 + 16;
    char* stage = smem + wave * (WTM * kRowPad);
    dispatch_act(g.act, [&](auto act_tag) {
    constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int nl = j * 32 + 8 * q + 4 * lhalf;          // column inside the wave tile
            const int n = n0 + wn * WTN + nl;
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias) {
                if (vec_store && n < g.N) {
                    const Pack4<T> t = __builtin_bit_cast(Pack4<T>, *reinterpret_cast<const u32x2*>(bias + n));
#pragma unroll
                    for (int e = 0; e < 4; e++) bv[e] = Elem<T>::to_f32(t.v[e]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < g.N) bv[e] = Elem<T>::to_f32(bias[n + e]);
                }
            }
#pragma unroll
            for (int i = 0; i < TM; i++) {
                Pack4<T> o;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float v = acc[i][j][4 * q + e] + bv[e];
                    v = apply_act_c<ACT>(v);
                    o.v[e] = Elem<T>::from_f32(v);
                }
                *reinterpret_cast<u32x2*>(stage + (i * 32 + lrow) * kRowPad + nl * 2) =
                    __builtin_bit_cast(u32x2, o);
            }
        }
    }
    });
    // each wave only re-reads what it wrote itself
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (vec_store) {
        constexpr int kCpr = WTN / 8;                // 16-byte chunks per row
        constexpr int kRowsPerPass = 64 / kCpr;
        const int cc = lane % kCpr, rr = lane / kCpr;
#pragma unroll
        for (int p = 0; p < WTM / kRowsPerPass; p++) {
            const int ml = p * kRowsPerPass + rr;
            const int m = m0 + wm * WTM + ml;
            const int n = n0 + wn * WTN + cc * 8;
            if (m < g.M && n < g.N) {
                u32x4 w = *reinterpret_cast<const u32x4*>(stage + ml * kRowPad + cc * 16);
                if (res) w = add_chunk<T>(w, *reinterpret_cast<const u32x4*>(res + (int64_t)m * g.N + n));
                *reinterpret_cast<u32x4*>(c + (int64_t)m * g.N + n) = w;
            }
        }
    } else {
        // rows of C are not 16-byte aligned (odd N): one element per lane, 64
        // consecutive columns per store instruction
        const uint16_t* st16 = reinterpret_cast<const uint16_t*>(stage);
        uint16_t* c16 = reinterpret_cast<uint16_t*>(c);
#pragma unroll 4
        for (int ml = 0; ml < WTM; ml++) {
            const int m = m0 + wm * WTM + ml;
            if (m >= g.M) break;
#pragma unroll
            for (int cb = 0; cb < WTN / 64; cb++) {
                const int nl = cb * 64 + lane;
                const int n = n0 + wn * WTN + nl;
                if (n < g.N) {
                    T val = __builtin_bit_cast(T, st16[ml * (kRowPad / 2) + nl]);
                    if (res) val = Elem<T>::from_f32(Elem<T>::to_f32(val) + Elem<T>::to_f32(res[(int64_t)m * g.N + n]));
                    c16[(int64_t)m * g.N + n] = __builtin_bit_cast(uint16_t, val);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Plain tiled kernel: any type, any shape.  16x16 threads, one output each.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gemm_simple_kernel(GemmArgs g, int trans_a, int trans_b) {
    __shared__ float As[16][17];
    __shared__ float Bs[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int64_t batch = blockIdx.z;
    const T* a = static_cast<const T*>(g.a) + batch * g.sa;
    const T* b = static_cast<const T*>(g.b) + batch * g.sb;
    T* c = static_cast<T*>(g.c) + batch * g.sc;
    const int m = blockIdx.y * 16 + ty, n = blockIdx.x * 16 + tx;
    float acc = 0.f;
    for (int k0 = 0; k0 < g.K; k0 += 16) {
        const int ka = k0 + tx, kb = k0 + ty;
        float av = 0.f, bv = 0.f;
        if (m < g.M && ka < g.K)
            av = Elem<T>::to_f32(trans_a ? a[(int64_t)ka * g.lda + m] : a[(int64_t)m * g.lda + ka]);
        if (n < g.N && kb < g.K)
            bv = Elem<T>::to_f32(trans_b ? b[(int64_t)n * g.ldb + kb] : b[(int64_t)kb * g.ldb + n]);
        As[ty][tx] = av;
        Bs[ty][tx] = bv;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; k++) acc = fmaf(As[ty][k], Bs[k][tx], acc);
        __syncthreads();
    }
    if (m < g.M && n < g.N) {
        if (g.bias) acc += Elem<T>::to_f32(static_cast<const T*>(g.bias)[n]);
        if (g.act != MHIP_ACT_NONE) acc = apply_act(acc, g.act);
        T val = Elem<T>::from_f32(acc);
        if (g.residual)    // second rounding on purpose: the same result as a separate add over the stored C
            val = Elem<T>::from_f32(Elem<T>::to_f32(val) +
                                    Elem<T>::to_f32((static_cast<const T*>(g.residual) + batch * g.sc)[(int64_t)m * g.N + n]));
        c[(int64_t)m * g.N + n] = val;
    }
}

// ---------------------------------------------------------------------------
// Exact kernel for i32 / i64 (wrap-around arithmetic) and f64: accumulates in the element
// type itself, k ascending.  Bias and residual are plain adds; no activation.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gemm_exact_kernel(GemmArgs g, int trans_a, int trans_b) {
    typedef typename std::conditional<std::is_integral<T>::value, typename std::make_unsigned<
        typename std::conditional<std::is_integral<T>::value, T, int>::type>::type, T>::type A;   // wraps without UB
    __shared__ A As[16][17];
    __shared__ A Bs[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int64_t batch = blockIdx.z;
    const T* a = static_cast<const T*>(g.a) + batch * g.sa;
    const T* b = static_cast<const T*>(g.b) + batch * g.sb;
    T* c = static_cast<T*>(g.c) + batch * g.sc;
    const int m = blockIdx.y * 16 + ty, n = blockIdx.x * 16 + tx;
    A acc = 0;
    for (int k0 = 0; k0 < g.K; k0 += 16) {
        const int ka = k0 + tx, kb = k0 + ty;
        A av = 0, bv = 0;
        if (m < g.M && ka < g.K) av = (A)(trans_a ? a[(int64_t)ka * g.lda + m] : a[(int64_t)m * g.lda + ka]);
        if (n < g.N && kb < g.K) bv = (A)(trans_b ? b[(int64_t)n * g.ldb + kb] : b[(int64_t)kb * g.ldb + n]);
        As[ty][tx] = av;
        Bs[ty][tx] = bv;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; k++) acc += As[ty][k] * Bs[k][tx];
        __syncthreads();
    }
    if (m < g.M && n < g.N) {
        if (g.bias) acc += (A) static_cast<const T*>(g.bias)[n];
        if (g.residual) acc += (A)(static_cast<const T*>(g.residual) + batch * g.sc)[(int64_t)m * g.N + n];
        c[(int64_t)m * g.N + n] = (T)acc;
    }
}

// ---------------------------------------------------------------------------
// Host dispatch
// ---------------------------------------------------------------------------
template <typename T, int BM, int BN, int WGM, int WGN, bool TA, bool TB>
static int launch_mfma(hipStream_t s, GemmArgs g, int64_t batch) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int kWaves = WGM * WGN;
    constexpr int kStage = kWaves * (BM / WGM) * ((BN / WGN) * 2 + 16);   // epilogue staging
    constexpr int kLoop = 2 * (BM + BN) * kRowBytes;
    constexpr int kSmem = kLoop > kStage ? kLoop : kStage;
    auto kern = gemm_mfma_kernel<T, BM, BN, WGM, WGN, TA, TB>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
    });
    if (attr_err != hipSuccess)
        return fail(MHIP_ERR_LAUNCH, "gemm: cannot reserve %d bytes of LDS: %s", kSmem,
                    hipGetErrorString(attr_err));
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
    if (tiles > 0x7FFFFFFFLL || batch > 65535) return fail(MHIP_ERR_UNSUPPORTED, "gemm: grid too large");
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles, (unsigned)batch), dim3(NT), kSmem, s, g);
    return check_launch("gemm_mfma");
}

// gemm256.hip: 4-wave 256x256 kernel with a hand-scheduled main loop.
bool gemm256_eligible(const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype, int bw = 256, bool any_tile_count = false);
int launch_gemm256(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype, int bw = 256, int ring = 5);
bool gemm384_activation_ok(int act);
bool gemm_stream_eligible(const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype);
int launch_gemm_stream(hipStream_t s, const GemmArgs& g, int trans_b, int dtype);
// gemm_f32.hip: fp32 operands on the fp32 matrix instruction, 128x128 tiles.
bool gemm_f32_mfma_wanted(const GemmArgs& g);
int launch_gemm_f32_mfma(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b);
// tuning.hip: variant prescribed by the tuning table for this problem, 0 = none.
int tuned_gemm_variant(const GemmArgs& g, int64_t batch, int ta, int tb, int dtype);

// A problem whose wide (256x256) tiles fill whole rounds of the device except for a narrow band
// of columns is run as two launches: wide tiles on the first `n_wide` columns, 256x128 tiles on
// the rest (one round at most) -- [8192,2304] x K 768: 256 wide + 64 narrow tiles instead of two
// and a quarter rounds of narrow ones.  The slices are plain pointer offsets: B[:, n_wide:] (or B[n_wide:, :] when it is
// stored [N, K]), bias, residual and C at column n_wide with the full row stride.
// Returns -1 when the problem does not have that shape (the caller goes on to the other kernels).
// The columns that go to wide tiles: the largest multiple of 256 whose tiles make whole rounds of
// the device, leaving a band of at most one round of narrow tiles.  False: no such split.
bool gemm_split_shape(const GemmArgs& g, int64_t batch, int* n_wide_out) {
    constexpr int cus = 256;
    if (batch != 1 || g.ldc != 0 || g.M % 256 != 0 || g.N % 8 != 0) return false;
    const int64_t tiles_m = g.M / 256;
    int64_t c = g.N / 256;
    while (c > 0 && (tiles_m * c) % cus != 0) c--;
    if (c == 0) return false;
    const int64_t rest = g.N - c * 256;
    if (rest <= 0 || tiles_m * ((rest + 127) / 128) > cus) return false;
    if (n_wide_out) *n_wide_out = (int)(c * 256);
    return true;
}

template <typename T, bool TA, bool TB>
static int launch_column_split(hipStream_t s, const GemmArgs& g, int64_t batch, int dt, bool forced) {
    constexpr int cus = 256;
    int n_wide = 0;
    if (!gemm_split_shape(g, batch, &n_wide)) return -1;
    const int64_t tiles_m = g.M / 256;
    const int rest = g.N - n_wide;
    if (!forced) {
        // Worth it from a third round of narrow tiles on.  Measured inside a GPT-2 forward pass
        // (operands from memory, K 768; a round of wide tiles takes 31 us there, a streamed narrow
        // tile 14-17): [8192,2304], whose third narrow round holds 64 tiles, 48.6 -> 45.8 us;
        // [8192,3072], three full rounds, 2 us better than streamed or plain narrow tiles (the
        // whole pass 3.385 -> 3.362 ms).
        const int64_t narrow = tiles_m * ((g.N + 127) / 128);
        if (narrow <= 2 * cus) return -1;
    }
    GemmArgs w = g, r = g;
    w.N = n_wide; w.ldc = g.N;
    r.N = rest; r.ldc = g.N;
    const int64_t boff = TB ? (int64_t)n_wide * g.ldb : (int64_t)n_wide;
    r.b = static_cast<const T*>(g.b) + boff;
    if (g.bias) r.bias = static_cast<const T*>(g.bias) + n_wide;
    if (g.residual) r.residual = static_cast<const T*>(g.residual) + n_wide;
    r.c = static_cast<T*>(g.c) + n_wide;
    if (!gemm256_eligible(w, 1, TA, TB, dt) || !gemm256_eligible(r, 1, TA, TB, dt, 128, /*any_tile_count=*/true)) return -1;
    // The band first: what the wide tiles store at their common end is
    // then the freshest content of the L2s when the next kernel starts at column 0.
    const int st = launch_gemm256(s, r, 1, TA, TB, dt, 128);
    if (st != MHIP_OK) return st;
    return launch_gemm256(s, w, 1, TA, TB, dt);
}

// Which kernel serves a 16-bit problem (MHIP_GEMM_TILE = 128 | 256 | 2560 ... 2570 forces one; 2570 = the 256x288 tile; 2564 / 2565 = the
// 256x128 tile with a ring of six / four stages, 2566 = the 256x256 tile with four, 2568 = the 256x128
// tile as two workgroups per compute unit: members of the generated family that only a forced choice
// or the tuning table selects; 2567 = the 256x384 tile):
//   * the four-wave ring kernel (gemm256.hip) on 256x256 tiles (2560) or 256x128 tiles
//     (2561) when K >= 512 and the problem is eligible: one workgroup per CU, so its time is
//     rounds x (stages x per-stage time + prologue and epilogue), rounds = ceil(tiles / 256 CUs);
//     the cheaper of the two by that count is taken.  In units of one MFMA issue slot per wave
//     a K stage costs 32 on the wide tile and 18 on the narrow one (16 MFMAs, but three
//     fragment reads for every four MFMAs instead of two), prologue + epilogue about 700 and
//     500 -- figures fitted to seven measured shapes (4096^3: wide; [8192,768] x K 3072
//     or 768, [8192,2304..3072] x K 768: narrow);
//   * the same 256x128 kernel as persistent workgroups that store a tile inside the loop of the
//     next one (2562; gemm_stream_kernel): forced or recorded by the tuner (see below why it is
//     not a default);
//   * wide tiles on the columns that fill whole rounds and narrow tiles on the rest (2563;
//     launch_column_split) where the problem has that shape;
//   * 256x384 tiles (2567; no activation, relu or tanh-GELU) where one round of them replaces two
//     or three of the others;
//   * 128x192 tiles (2569) where 256-row tiles would leave compute units idle (few columns);
//   * the eight-wave 256x256 kernel for large problems the ring kernel cannot take whose
//     rows of C are not 16-byte aligned (odd N): its eight waves hide the narrow stores;
//   * otherwise 128x128 tiles, two workgroups per CU (short K, few tiles).
// An entry of the tuning table (mhip_gemm_autotune) for the problem overrides the heuristic.
// The kernel the last mhip_gemm / mhip_gemm_residual call of this thread chose (mhip_gemm_last_variant).
static thread_local int g_last_variant = 0;
static inline int chose(int variant, int status) { g_last_variant = variant; return status; }

template <typename T, bool TA, bool TB>
static int pick_tile(hipStream_t s, const GemmArgs& g, int64_t batch) {
    const int64_t tiles_m = (g.M + 255) / 256;
    const int64_t big = tiles_m * ((g.N + 255) / 256) * batch;
    constexpr int dt = std::is_same<T, bf16_t>::value ? MHIP_BF16 : MHIP_F16;
    int force = tune_int("MHIP_GEMM_TILE", 0);
    if (force == 0) force = tuned_gemm_variant(g, batch, TA, TB, dt);   // tuning table / running tuner
    if (force == 2562) {
        if (gemm_stream_eligible(g, batch, TA, TB, dt)) return chose(2562, launch_gemm_stream(s, g, TB, dt));
    }
    if (force == 2561) {
        if (gemm256_eligible(g, batch, TA, TB, dt, 128)) return chose(2561, launch_gemm256(s, g, batch, TA, TB, dt, 128));
    }
    if (force == 2560) {
        if (gemm256_eligible(g, batch, TA, TB, dt)) return chose(2560, launch_gemm256(s, g, batch, TA, TB, dt));
    }
    // the other members of the generated tile family: ring depth 6 or 4 on the narrow tile, 4 on the wide one
    if (force == 2564 || force == 2565) {
        if (gemm256_eligible(g, batch, TA, TB, dt, 128))
            return chose(force, launch_gemm256(s, g, batch, TA, TB, dt, 128, force == 2564 ? 6 : 4));
    }
    if (force == 2566) {
        if (gemm256_eligible(g, batch, TA, TB, dt)) return chose(2566, launch_gemm256(s, g, batch, TA, TB, dt, 256, 4));
    }
    // the 256x288 tile (ring of four)
    if (force == 2570) {
        if (gemm256_eligible(g, batch, TA, TB, dt, 288) && gemm384_activation_ok(g.act)) return chose(2570, launch_gemm256(s, g, batch, TA, TB, dt, 288, 4));
    }
    // the 128x192 tile (ring of six)
    if (force == 2569) {
        if (gemm256_eligible(g, batch, TA, TB, dt, 192)) return chose(2569, launch_gemm256(s, g, batch, TA, TB, dt, 192, 6));
    }
    // the 256x128 tile with two workgroups per compute unit (ring of three)
    if (force == 2568) {
        if (gemm256_eligible(g, batch, TA, TB, dt, 128)) return chose(2568, launch_gemm256(s, g, batch, TA, TB, dt, 128, 3));
    }
    // the 256x384 tile (ring of four)
    if (force == 2567) {
        if (gemm256_eligible(g, batch, TA, TB, dt, 384) && gemm384_activation_ok(g.act)) return chose(2567, launch_gemm256(s, g, batch, TA, TB, dt, 384, 4));
    }
    constexpr int cus = 256;                           // compute units of the device this is written for
    const int64_t narrow = tiles_m * ((g.N + 127) / 128) * batch, stages = g.K / 32;
    const int64_t wide_cost = ((big + cus - 1) / cus) * (stages * 32 + 700);
    const int64_t narrow_cost = ((narrow + cus - 1) / cus) * (stages * 18 + 500);
    // (wide tiles on the columns that make whole rounds + one round of a narrow band, where the default takes that form)
    int n_split = 0;
    const bool split_ok = gemm_split_shape(g, batch, &n_split) && narrow > 2 * cus;
    const int64_t split_cost = split_ok ? (tiles_m * (n_split / 256) / cus) * (stages * 32 + 700) + (stages * 18 + 500) : ((int64_t)1 << 62);
    const bool wider_ok = gemm256_eligible(g, batch, TA, TB, dt, 384) && gemm384_activation_ok(g.act);
    const int64_t wider_cost = ((tiles_m * ((g.N + 383) / 384) * batch + cus - 1) / cus) * (stages * 53 + 1050);
    if (force == 0 && g.K >= 512 && gemm256_eligible(g, batch, TA, TB, dt, 192)) {
        // The 128x192 tile where 256-row tiles leave compute units idle: its stage moves 20 KB
        // from the L2s against the narrow tile's 24 and costs 14 slots, the ends 500 -- fitted to
        // [8192,3072] x [3072,768] (256 tiles of it against 192 narrow ones: 46.4 us against 53.5
        // in a loop of its own, 40.6 against 48.2 with the caches emptied before each launch) and
        // K 768 (24.5 against 25.7); inside a GPT-2 pass the two GEMMs with 768 columns take
        // 72 us less in all (3.313 -> 3.241 ms on one box).
        const int64_t small = ((g.M + 127) / 128) * ((g.N + 191) / 192) * batch;
        const int64_t small_cost = ((small + cus - 1) / cus) * (stages * 14 + 500);
        int64_t other = (int64_t)1 << 62;
        if (gemm256_eligible(g, batch, TA, TB, dt) && wide_cost < other) other = wide_cost;
        if (gemm256_eligible(g, batch, TA, TB, dt, 128) && narrow_cost < other) other = narrow_cost;
        if (wider_ok && wider_cost < other) other = wider_cost;
        if (split_cost < other) other = split_cost;
        if (small_cost < other) return chose(2569, launch_gemm256(s, g, batch, TA, TB, dt, 192, 6));
    }
    if (force == 0 && g.K >= 512 && wider_ok) {
        // The 256x384 tile where it saves a round: its stage costs 53 slots (48 MFMAs, and only
        // one k-step of fragments read ahead), its prologue and epilogue 1050 (half as many
        // accumulators again to convert and store) -- fitted to [8192,2304..12288] x K 768..6144:
        // one round of it beats two of wide or three of narrow tiles ([8192,3072] x K 768 44 us
        // against 49; inside a GPT-2 pass 50.3 against 55, and [8192,2304] 41.8 against 45.8 for
        // the column split), while from two rounds on the wide tile's shorter epilogue wins
        // ([8192,12288] x K 768: 170 us against 159).
        int64_t other = wide_cost < narrow_cost ? wide_cost : narrow_cost;
        if (split_ok) other = split_cost;
        if (wider_cost < other) return chose(2567, launch_gemm256(s, g, batch, TA, TB, dt, 384, 4));
    }
    if (force == 2563 || (force == 0 && g.K >= 512)) {
        const int st = launch_column_split<T, TA, TB>(s, g, batch, dt, force == 2563);
        if (st >= 0) return chose(2563, st);
    }
    if (force == 0 && g.K >= 512) {
        const bool wide_ok = gemm256_eligible(g, batch, TA, TB, dt), narrow_ok = gemm256_eligible(g, batch, TA, TB, dt, 128);
        // (The streamed form of the narrow tile, 2562, is not chosen here: it is 5 % ahead of wide tiles
        // on a few shapes when the operands sit in the L2 -- [4096,8320] x K 1024 77 against 81 us,
        // [8192,4608] x K 768 67 against 71 -- and 10 to 15 % behind on the same shapes when they come
        // from memory, 92 against 84 and 83 against 72, which is how a GEMM inside a model finds
        // them.  The tuner times it and the table selects it where it wins.)
        if (narrow_ok && (!wide_ok || narrow_cost < wide_cost)) return chose(2561, launch_gemm256(s, g, batch, TA, TB, dt, 128));
        if (wide_ok) return chose(2560, launch_gemm256(s, g, batch, TA, TB, dt));
    }
    const bool want256 = force == 256 || (force != 128 && big >= 192 && (g.K >= 1024 || g.N % 8 != 0));
    if (want256) return chose(256, launch_mfma<T, 256, 256, 2, 4, TA, TB>(s, g, batch));
    return chose(128, launch_mfma<T, 128, 128, 2, 2, TA, TB>(s, g, batch));
}

template <typename T>
static int pick_layout(hipStream_t s, const GemmArgs& g, int64_t batch, int ta, int tb) {
    if (!ta && !tb) return pick_tile<T, false, false>(s, g, batch);
    if (!ta && tb) return pick_tile<T, false, true>(s, g, batch);
    if (ta && !tb) return pick_tile<T, true, false>(s, g, batch);
    return pick_tile<T, true, true>(s, g, batch);
}

template <typename T>
static int launch_simple(hipStream_t s, const GemmArgs& g, int64_t batch, int ta, int tb) {
    const int64_t gx = (g.N + 15) / 16, gy = (g.M + 15) / 16;
    if (gy > 65535 || batch > 65535) return fail(MHIP_ERR_UNSUPPORTED, "gemm: grid too large");
    hipLaunchKernelGGL((gemm_simple_kernel<T>), dim3((unsigned)gx, (unsigned)gy, (unsigned)batch),
                       dim3(256), 0, s, g, ta, tb);
    return check_launch("gemm_simple");
}

template <typename T>
static int launch_exact(hipStream_t s, const GemmArgs& g, int64_t batch, int ta, int tb) {
    if (g.act != MHIP_ACT_NONE) return fail(MHIP_ERR_UNSUPPORTED, "gemm: no activation on i32 / i64 / f64");
    const int64_t gx = (g.N + 15) / 16, gy = (g.M + 15) / 16;
    if (gy > 65535 || batch > 65535) return fail(MHIP_ERR_UNSUPPORTED, "gemm: grid too large");
    hipLaunchKernelGGL((gemm_exact_kernel<T>), dim3((unsigned)gx, (unsigned)gy, (unsigned)batch),
                       dim3(256), 0, s, g, ta, tb);
    return check_launch("gemm_exact");
}

}  // namespace mhip

using namespace mhip;

static int gemm_entry(void* stream, const void* a, const void* b, const void* bias, const void* residual, void* c,
                      int64_t M, int64_t N, int64_t K, int64_t batch, int64_t stride_a,
                      int64_t stride_b, int64_t stride_c, int trans_a, int trans_b,
                      int activation, int dtype) {
    if (M < 0 || N < 0 || K < 0 || batch < 0)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_gemm: negative size");
    if (activation < MHIP_ACT_NONE || activation > MHIP_ACT_GELU_ERF)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_gemm: unknown activation %d", activation);
    if (M == 0 || N == 0 || batch == 0) return MHIP_OK;
    if (!a || !b || !c) return fail(MHIP_ERR_INVALID_ARGUMENT, "mhip_gemm: NULL matrix pointer");
    if (M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF)
        return fail(MHIP_ERR_UNSUPPORTED, "mhip_gemm: dimension exceeds 2^31-1");
    hipStream_t s = as_stream(stream);
    g_last_variant = 0;
    GemmArgs g;
    g.a = a; g.b = b; g.bias = bias; g.c = c;
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.lda = trans_a ? (int)M : (int)K;
    g.ldb = trans_b ? (int)K : (int)N;
    g.sa = stride_a; g.sb = stride_b; g.sc = stride_c;
    g.act = activation;
    g.residual = residual;
    g.tiles_m = g.tiles_n = 0;

    const bool is16 = dtype == MHIP_BF16 || dtype == MHIP_F16;
    // 16-byte global loads need every row start and every 8-element chunk aligned.
    const bool vec_ok = is16 && K > 0 && g.lda % 8 == 0 && g.ldb % 8 == 0 &&
                        (reinterpret_cast<uintptr_t>(a) & 15) == 0 &&
                        (reinterpret_cast<uintptr_t>(b) & 15) == 0 && stride_a % 8 == 0 &&
                        stride_b % 8 == 0 && (int64_t)M * K * 2 < 0x7FFFFFFFLL &&
                        (int64_t)N * K * 2 < 0x7FFFFFFFLL;
    if (vec_ok) {
        if (dtype == MHIP_BF16) return pick_layout<bf16_t>(s, g, batch, trans_a, trans_b);
        return pick_layout<f16_t>(s, g, batch, trans_a, trans_b);
    }
    switch (dtype) {
        case MHIP_F32:
            if (gemm_f32_mfma_wanted(g)) return launch_gemm_f32_mfma(s, g, batch, trans_a, trans_b);
            return launch_simple<float>(s, g, batch, trans_a, trans_b);
        case MHIP_BF16: return launch_simple<bf16_t>(s, g, batch, trans_a, trans_b);
        case MHIP_F16: return launch_simple<f16_t>(s, g, batch, trans_a, trans_b);
        case MHIP_I32: return launch_exact<int32_t>(s, g, batch, trans_a, trans_b);
        case MHIP_I64: return launch_exact<int64_t>(s, g, batch, trans_a, trans_b);
        case MHIP_F64: return launch_exact<double>(s, g, batch, trans_a, trans_b);
        default: return fail(MHIP_ERR_UNSUPPORTED, "mhip_gemm: dtype %d (need f32, f16, bf16, f64, i32 or i64)", dtype);
    }
}

extern "C" int mhip_gemm(void* stream, const void* a, const void* b, const void* bias, void* c,
                         int64_t M, int64_t N, int64_t K, int64_t batch, int64_t stride_a,
                         int64_t stride_b, int64_t stride_c, int trans_a, int trans_b,
                         int activation, int dtype) {
    return gemm_entry(stream, a, b, bias, nullptr, c, M, N, K, batch, stride_a, stride_b, stride_c, trans_a, trans_b,
                      activation, dtype);
}

extern "C" int mhip_gemm_last_variant(void) { return g_last_variant; }

extern "C" int mhip_gemm_residual(void* stream, const void* a, const void* b, const void* bias,
                                  const void* residual, void* c, int64_t M, int64_t N, int64_t K,
                                  int64_t batch, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                                  int trans_a, int trans_b, int activation, int dtype) {
    return gemm_entry(stream, a, b, bias, residual, c, M, N, K, batch, stride_a, stride_b, stride_c, trans_a, trans_b,
                      activation, dtype);
}
