// The members of the ring-kernel family that run on two fragment sets (gen_gemm256_loop.py, second part ->
// gemm_twoset_loop.inc): the 256x384 and the 256x288 tile, whose accumulators do not fit the accumulation
// registers, the 128x192 tile for problems with few columns, and the 256x128 tile in 256 registers a wave
// for two workgroups per compute unit.  Operand layouts and the epilogue of the narrow tile are those of
// gemm256.hip (gemm_ring.h).
#include "gemm_ring.h"

namespace mhip {

#include "gemm_twoset_loop.inc"

namespace {

// ---- the 256x384 tile ------------------------------------------------------------------------------
// The widest member of the family (gemm256x384_loop_* of the generated file): each wave 128 x 192,
// 24 accumulator blocks, sixteen of them in the accumulation registers and eight in v[128:255].  B is
// held as the wide kernel's 256-column tile followed by the narrow kernel's 128-column tile (columns
// 256..383 of the workgroup's 384); wave (wm, wn) owns rows 128 wm .. + 127 and the columns
// 128 wn .. + 127 (blocks j = 0..3) and 256 + 64 wn .. + 63 (j = 4, 5) of the workgroup's tile.
constexpr int k384Stage = 40 * 1024;
constexpr int k384Smem = 4 * k384Stage;

template <typename T, bool TA, bool TB>
__device__ __forceinline__ void main_loop384(f32x16 (&acc)[24], u32x4 ra, u32x4 rb, u32x2 rb2, u32x4& goff,
                                    __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb, uint32_t pa,
                                    uint32_t pb, uint32_t ta, uint32_t tb, uint32_t m0b, uint32_t kt) {
    constexpr bool bf = std::is_same<T, bf16_t>::value;
#define MHIP_LOOP(cond, name) \
    if constexpr (cond) gemm256x384_loop_##name(acc, ra, rb, rb2, goff, rsa, rsb, pa, pb, ta, tb, m0b, kt);
    MHIP_LOOP(bf && !TA && !TB, nn_bf16)
    MHIP_LOOP(bf && !TA && TB, nt_bf16)
    MHIP_LOOP(bf && TA && !TB, tn_bf16)
    MHIP_LOOP(bf && TA && TB, tt_bf16)
    MHIP_LOOP(!bf && !TA && !TB, nn_f16)
    MHIP_LOOP(!bf && !TA && TB, nt_f16)
    MHIP_LOOP(!bf && TA && !TB, tn_f16)
    MHIP_LOOP(!bf && TA && TB, tt_f16)
#undef MHIP_LOOP
}

// Epilogue of the 256x384 tile.  A wave's 128 x 192 sub-tile passes through LDS one 32-row block at
// a time (32 rows of 384 + 16 bytes per wave, in the ring, which is free behind the loop's last
// barrier); a row of the staging area holds the wave's 128 columns of B, then its 64 of B2.  A block
// is written back by twelve instructions of 64 lanes x 16 bytes: lane slot u * 64 + lane = row
// (slot / 24) of the block's rows 8 (u / 3) .., chunk slot % 24.
template <typename T>
__device__ __forceinline__ void store_tile384(f32x16 (&acc)[24], char* smem, const GemmArgs& g, T* c, const T* res,
                                              int m0, int n0) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, lhalf = lane >> 5;
    const T* bias = static_cast<const T*>(g.bias);
    constexpr int kRowPad = 192 * 2 + 16;
    char* stage = smem + wave * (32 * kRowPad);
    const int ldc = g.ldc ? g.ldc : g.N;
    // A workgroup whose 384 columns lie inside C loads its bias without per-element conditions; a
    // wave whose sub-tile lies inside C, with rows of C on 16-byte boundaries, stores without any.
    const bool full_cols = __builtin_amdgcn_readfirstlane(n0 + 384 <= g.N);
    const bool interior = __builtin_amdgcn_readfirstlane(full_cols && m0 + wm * 128 + 128 <= g.M && ldc % 8 == 0);
    const bool stream = __builtin_amdgcn_readfirstlane(g.stream_c != 0);
    // first column of the wave's block j
    auto col_of = [&](int j) { return j < 4 ? n0 + wn * 128 + 32 * j : n0 + 256 + wn * 64 + 32 * (j - 4); };
    // The bias of all the lane's columns (zero without a bias and for columns past N), asked for in
    // one go: a load inside each group of four values would be waited for 96 times.
    Pack4<T> bq[24];
    static_for<24>([&](auto jq_tag) {
        constexpr int jq = decltype(jq_tag)::value;
        bq[jq] = __builtin_bit_cast(Pack4<T>, u32x2{0u, 0u});
    });
    if (bias) {
        if (full_cols) {
            static_for<24>([&](auto jq_tag) {
                constexpr int jq = decltype(jq_tag)::value;
                bq[jq] = __builtin_bit_cast(Pack4<T>, *reinterpret_cast<const u32x2*>(bias + col_of(jq >> 2) + 8 * (jq & 3) + 4 * lhalf));
            });
        } else {
            static_for<24>([&](auto jq_tag) {
                constexpr int jq = decltype(jq_tag)::value;
                const int n = col_of(jq >> 2) + 8 * (jq & 3) + 4 * lhalf;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < g.N) bq[jq].v[e] = bias[n + e];
            });
        }
    }
    // The activation is a uniform branch around each group of four values, not a compile-time
    // constant chosen once around the whole epilogue as in store_tile: with the eight register-resident
    // accumulator blocks live into every copy of the epilogue the compiler fails to assign registers.
    // Served here: none, relu, tanh-GELU (gemm384_activation_ok).
    const int act = __builtin_amdgcn_readfirstlane(g.act);
    static_for<4>([&](auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
        static_for<24>([&](auto jq_tag) {
            constexpr int j = decltype(jq_tag)::value >> 2, q = decltype(jq_tag)::value & 3;
            constexpr int b = 6 * i + j;
            Pack4<T> o;
            float v4[4];
            static_for<4>([&](auto e_tag) {
                constexpr int e = decltype(e_tag)::value;
                if constexpr (b < 16) v4[e] = acc_value(acc[b][4 * q + e]);
                else v4[e] = acc[b][4 * q + e];
                v4[e] += Elem<T>::to_f32(bq[j * 4 + q].v[e]);
            });
            if (act == MHIP_ACT_GELU) {
#pragma unroll
                for (int e = 0; e < 4; e++) v4[e] = apply_act_c<MHIP_ACT_GELU>(v4[e]);
            } else if (act == MHIP_ACT_RELU) {
#pragma unroll
                for (int e = 0; e < 4; e++) v4[e] = apply_act_c<MHIP_ACT_RELU>(v4[e]);
            }
#pragma unroll
            for (int e = 0; e < 4; e++) o.v[e] = Elem<T>::from_f32(v4[e]);
            *reinterpret_cast<u32x2*>(stage + lrow * kRowPad + (j * 32 + 8 * q + 4 * lhalf) * 2) =
                __builtin_bit_cast(u32x2, o);
            __builtin_amdgcn_sched_barrier(0);
        });
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // a wave re-reads only its own rows
        if (interior) {
            // two groups of six chunks: the residual chunks of a group are asked for together
#pragma unroll
            for (int h = 0; h < 2; h++) {
                u32x4 w[6], r[6];
                int64_t off[6];
#pragma unroll
                for (int u = 0; u < 6; u++) {
                    // slot (6 h + u) * 64 + lane: 64 = 2 * 24 + 16 slots further on per instruction
                    const int slot = ((6 * h + u) % 3) * 64 + lane;
                    const int rl = 8 * ((6 * h + u) / 3) + slot / 24, ch = slot % 24;
                    const int n = ch < 16 ? n0 + wn * 128 + 8 * ch : n0 + 256 + wn * 64 + 8 * (ch - 16);
                    off[u] = (int64_t)(m0 + wm * 128 + i * 32 + rl) * ldc + n;
                    if (res) r[u] = *reinterpret_cast<const u32x4*>(res + off[u]);
                    w[u] = *reinterpret_cast<const u32x4*>(stage + rl * kRowPad + ch * 16);
                }
#pragma unroll
                for (int u = 0; u < 6; u++) {
                    if (res) w[u] = add_chunk<T>(w[u], r[u]);
                    if (stream) __builtin_nontemporal_store(w[u], reinterpret_cast<u32x4*>(c + off[u]));
                    else *reinterpret_cast<u32x4*>(c + off[u]) = w[u];
                }
            }
        } else {
#pragma unroll 1
            for (int u = 0; u < 12; u++) {
                const int slot = (u % 3) * 64 + lane;
                const int rl = 8 * (u / 3) + slot / 24, ch = slot % 24;
                const int m = m0 + wm * 128 + i * 32 + rl;
                const int n = ch < 16 ? n0 + wn * 128 + 8 * ch : n0 + 256 + wn * 64 + 8 * (ch - 16);
                T* cp = c + (int64_t)m * ldc + n;
                const T* rp = res + (int64_t)m * ldc + n;
                if (m < g.M && n + 8 <= g.N) {
                    // (rows of C at any even byte: the device takes 16-byte accesses there)
                    u32x4 w = *reinterpret_cast<const u32x4*>(stage + rl * kRowPad + ch * 16);
                    if (res) w = add_chunk<T>(w, *reinterpret_cast<const u32x4_unaligned*>(rp));
                    *reinterpret_cast<u32x4_unaligned*>(cp) = w;
                } else if (m < g.M && n < g.N) {                 // the last, partial chunk of a row
                    const T* sv = reinterpret_cast<const T*>(stage + rl * kRowPad + ch * 16);
                    for (int e = 0; e < g.N - n; e++) {
                        T val = sv[e];
                        if (res) val = Elem<T>::from_f32(Elem<T>::to_f32(val) + Elem<T>::to_f32(rp[e]));
                        cp[e] = val;
                    }
                }
            }
        }
        // the next block overwrites the rows just read
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    });
}

template <typename T, bool TA, bool TB>
__global__ __launch_bounds__(256) void gemm384_kernel(GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    using LA = typename std::conditional<TA, MnMajor<256>, KMajor>::type;
    using LB = typename std::conditional<TB, KMajor, MnMajor<256>>::type;
    using LB2 = typename std::conditional<TB, KMajor, MnMajor<128>>::type;

    int tm, tn;
    tile_of(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tm, tn);
    const int m0 = tm * 256, n0 = tn * 384;
    const int64_t batch = blockIdx.y;
    const char* a = reinterpret_cast<const char*>(static_cast<const T*>(g.a) + batch * g.sa);
    const char* b = reinterpret_cast<const char*>(static_cast<const T*>(g.b) + batch * g.sb);
    T* c = static_cast<T*>(g.c) + batch * g.sc;
    const T* res = g.residual ? static_cast<const T*>(g.residual) + batch * g.sc : nullptr;
    const uint32_t a_bytes = (uint32_t)(((int64_t)((TA ? g.K : g.M) - 1) * g.lda + (TA ? g.M : g.K)) * 2);
    const uint32_t b_bytes = (uint32_t)(((int64_t)((TB ? g.N : g.K) - 1) * g.ldb + (TB ? g.K : g.N)) * 2);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;

    const u32x4 ra = LA::raddr(lane, wm * 128, lds0);
    const u32x4 rb = LB::raddr(lane, wn * 128, lds0 + kOperBytes);
    const u32x4 rb2w = LB2::raddr(lane, wn * 64, lds0 + 2 * kOperBytes);
    u32x2 rb2;
    rb2.x = rb2w.x; rb2.y = rb2w.y;
    u32x4 goff;
    goff.x = LA::goff(lane, wave, m0, g.lda, g.M);
    goff.y = LB::goff(lane, wave, n0, g.ldb, g.N);
    goff.z = LB2::goff(lane, wave, n0 + 256, g.ldb, g.N);
    goff.w = 0;
    const uint32_t m0b = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)wave * 1024u);
    const __amdgpu_buffer_rsrc_t rsa =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a), 0, a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsb =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(b), 0, b_bytes, 0x00020000);

    f32x16 acc[24];
    main_loop384<T, TA, TB>(acc, ra, rb, rb2, goff, rsa, rsb, LA::pass_stride(g.lda), LB::pass_stride(g.ldb),
                            LA::stage_stride(g.lda), LB::stage_stride(g.ldb), m0b, (uint32_t)(g.K / 32));

    store_tile384<T>(acc, smem, g, c, res, m0, n0);
}

template <typename T, bool TA, bool TB>
int launch384(hipStream_t s, GemmArgs g, int64_t batch) {
    auto kern = gemm384_kernel<T, TA, TB>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, k384Smem);
    });
    if (attr_err != hipSuccess)
        return fail(MHIP_ERR_LAUNCH, "gemm384: cannot reserve %d bytes of LDS: %s", k384Smem,
                    hipGetErrorString(attr_err));
    g.tiles_m = (g.M + 255) / 256;
    g.tiles_n = (g.N + 383) / 384;
    g.stream_c = (int64_t)g.M * g.N * batch * 2 > (256ll << 20) && (g.ldc ? g.ldc : g.N) % 8 == 0;
    hipLaunchKernelGGL(kern, dim3((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch), dim3(256),
                       k384Smem, s, g);
    return check_launch("gemm384");
}

template <typename T>
int layout384(hipStream_t s, const GemmArgs& g, int64_t batch, int ta, int tb) {
    if (!ta && !tb) return launch384<T, false, false>(s, g, batch);
    if (!ta && tb) return launch384<T, false, true>(s, g, batch);
    if (ta && !tb) return launch384<T, true, false>(s, g, batch);
    return launch384<T, true, true>(s, g, batch);
}

// ---- the 256x128 tile, two workgroups per compute unit ------------------------------------------------
// gemm_pair_loop_* of the generated file: the narrow tile on two fragment sets, every register
// below v64 and a[0:127] (256 registers a wave) and a ring of three 24 KB stages (72 KB), so that
// two workgroups share a compute unit: one's prologue, epilogue and load latency run under the
// other's MFMAs.  Accumulators and epilogue are those of the one-workgroup kernel.
constexpr int kPairSmem = 3 * 24 * 1024;

template <typename T, bool TA, bool TB>
__device__ __forceinline__ void main_loop_pair(f32x16 (&acc)[8], u32x4 ra, u32x2 rb, u32x2& goff,
                                               __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb, uint32_t pa,
                                               uint32_t pb, uint32_t ta, uint32_t tb, uint32_t m0b, uint32_t kt) {
    constexpr bool bf = std::is_same<T, bf16_t>::value;
#define MHIP_LOOP(cond, name) \
    if constexpr (cond) gemm_pair_loop_##name(acc, ra, rb, goff, rsa, rsb, pa, pb, ta, tb, m0b, kt);
    MHIP_LOOP(bf && !TA && !TB, nn_bf16)
    MHIP_LOOP(bf && !TA && TB, nt_bf16)
    MHIP_LOOP(bf && TA && !TB, tn_bf16)
    MHIP_LOOP(bf && TA && TB, tt_bf16)
    MHIP_LOOP(!bf && !TA && !TB, nn_f16)
    MHIP_LOOP(!bf && !TA && TB, nt_f16)
    MHIP_LOOP(!bf && TA && !TB, tn_f16)
    MHIP_LOOP(!bf && TA && TB, tt_f16)
#undef MHIP_LOOP
}

template <typename T, bool TA, bool TB>
__global__ __launch_bounds__(256, 2) void gemm_pair_kernel(GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    using LA = typename std::conditional<TA, MnMajor<256>, KMajor>::type;
    using LB = typename std::conditional<TB, KMajor, MnMajor<128>>::type;

    int tm, tn;
    tile_of(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tm, tn);
    const int m0 = tm * 256, n0 = tn * 128;
    const int64_t batch = blockIdx.y;
    const char* a = reinterpret_cast<const char*>(static_cast<const T*>(g.a) + batch * g.sa);
    const char* b = reinterpret_cast<const char*>(static_cast<const T*>(g.b) + batch * g.sb);
    T* c = static_cast<T*>(g.c) + batch * g.sc;
    const T* res = g.residual ? static_cast<const T*>(g.residual) + batch * g.sc : nullptr;
    const uint32_t a_bytes = (uint32_t)(((int64_t)((TA ? g.K : g.M) - 1) * g.lda + (TA ? g.M : g.K)) * 2);
    const uint32_t b_bytes = (uint32_t)(((int64_t)((TB ? g.N : g.K) - 1) * g.ldb + (TB ? g.K : g.N)) * 2);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    const u32x4 ra = LA::raddr(lane, wm * 128, lds0);
    const u32x4 rbw = LB::raddr(lane, wn * 64, lds0 + kOperBytes);
    u32x2 rb;
    rb.x = rbw.x; rb.y = rbw.y;
    u32x2 goff;
    goff.x = LA::goff(lane, wave, m0, g.lda, g.M);
    goff.y = LB::goff(lane, wave, n0, g.ldb, g.N);
    const uint32_t m0b = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)wave * 1024u);
    const __amdgpu_buffer_rsrc_t rsa =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a), 0, a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsb =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(b), 0, b_bytes, 0x00020000);

    f32x16 acc[8];
    main_loop_pair<T, TA, TB>(acc, ra, rb, goff, rsa, rsb, LA::pass_stride(g.lda), LB::pass_stride(g.ldb),
                              LA::stage_stride(g.lda), LB::stage_stride(g.ldb), m0b, (uint32_t)(g.K / 32));
    if (g.stream_c) store_tile<T, 128, true, 1>(acc, smem, g, c, res, m0, n0);
    else store_tile<T, 128, false, 1>(acc, smem, g, c, res, m0, n0);
}

template <typename T, bool TA, bool TB>
int launch_pair(hipStream_t s, GemmArgs g, int64_t batch) {
    auto kern = gemm_pair_kernel<T, TA, TB>;
    static_assert(kPairSmem >= 4 * 128 * (128 + 16), "the epilogue's staging area reuses the ring");
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kPairSmem);
    });
    if (attr_err != hipSuccess)
        return fail(MHIP_ERR_LAUNCH, "gemm_pair: cannot reserve %d bytes of LDS: %s", kPairSmem,
                    hipGetErrorString(attr_err));
    g.tiles_m = (g.M + 255) / 256;
    g.tiles_n = (g.N + 127) / 128;
    g.stream_c = (int64_t)g.M * g.N * batch * 2 > (256ll << 20) && (g.ldc ? g.ldc : g.N) % 8 == 0;
    hipLaunchKernelGGL(kern, dim3((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch), dim3(256),
                       kPairSmem, s, g);
    return check_launch("gemm_pair");
}

template <typename T>
int layout_pair(hipStream_t s, const GemmArgs& g, int64_t batch, int ta, int tb) {
    if (!ta && !tb) return launch_pair<T, false, false>(s, g, batch);
    if (!ta && tb) return launch_pair<T, false, true>(s, g, batch);
    if (ta && !tb) return launch_pair<T, true, false>(s, g, batch);
    return launch_pair<T, true, true>(s, g, batch);
}

// ---- the 128x192 tile --------------------------------------------------------------------------------
// gemm128x192_loop_* of the generated file: a tile for problems with so few columns that 256-row
// tiles leave compute units idle ([8192, 768] has 192 tiles of 256x128 and 256 of 128x192; the sum of
// rows and columns, which is what a stage moves from the L2s, is the smallest for that area).  Each
// wave 64 x 96 = 2 x 3 accumulator blocks; A is 128 rows; B's 192 columns lie in the 256-column layout
// of the wide kernel (loads of the last quarter carry an out-of-range offset and move nothing); a
// stage is 24 KB, the ring six deep.
constexpr int k192Stage = 24 * 1024;
constexpr int k192Smem = 6 * k192Stage;
constexpr uint32_t k192BOffset = 8 * 1024;   // B tile behind the 8 KB A tile of a stage

template <typename T, bool TA, bool TB>
__device__ __forceinline__ void main_loop192(f32x16 (&acc)[6], u32x2 ra, u32x4 rb, u32x2& goff,
                                             __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb, uint32_t pa,
                                             uint32_t pb, uint32_t ta, uint32_t tb, uint32_t m0b, uint32_t kt) {
    constexpr bool bf = std::is_same<T, bf16_t>::value;
#define MHIP_LOOP(cond, name) \
    if constexpr (cond) gemm128x192_loop_##name(acc, ra, rb, goff, rsa, rsb, pa, pb, ta, tb, m0b, kt);
    MHIP_LOOP(bf && !TA && !TB, nn_bf16)
    MHIP_LOOP(bf && !TA && TB, nt_bf16)
    MHIP_LOOP(bf && TA && !TB, tn_bf16)
    MHIP_LOOP(bf && TA && TB, tt_bf16)
    MHIP_LOOP(!bf && !TA && !TB, nn_f16)
    MHIP_LOOP(!bf && !TA && TB, nt_f16)
    MHIP_LOOP(!bf && TA && !TB, tn_f16)
    MHIP_LOOP(!bf && TA && TB, tt_f16)
#undef MHIP_LOOP
}

// Epilogue: a wave's 64 x 96 sub-tile through LDS one 32-row block at a time (32 rows of 192 + 16
// bytes per wave); a block goes out as six instructions of 64 lanes x 16 bytes: lane slot
// (u % 3) * 64 + lane = row 16 (u / 3) + slot / 12 of the block, chunk slot % 12.
template <typename T>
__device__ __forceinline__ void store_tile192(f32x16 (&acc)[6], char* smem, const GemmArgs& g, T* c, const T* res,
                                              int m0, int n0) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, lhalf = lane >> 5;
    const T* bias = static_cast<const T*>(g.bias);
    constexpr int kRowPad = 96 * 2 + 16;
    char* stage = smem + wave * (32 * kRowPad);
    const int ldc = g.ldc ? g.ldc : g.N;
    const int nw = n0 + wn * 96;                         // the wave's first column
    const bool full_cols = __builtin_amdgcn_readfirstlane(n0 + 192 <= g.N);
    const bool interior = __builtin_amdgcn_readfirstlane(full_cols && m0 + wm * 64 + 64 <= g.M && ldc % 8 == 0);
    Pack4<T> bq[12];
    static_for<12>([&](auto jq_tag) {
        constexpr int jq = decltype(jq_tag)::value;
        bq[jq] = __builtin_bit_cast(Pack4<T>, u32x2{0u, 0u});
    });
    if (bias) {
        if (full_cols) {
            static_for<12>([&](auto jq_tag) {
                constexpr int jq = decltype(jq_tag)::value;
                bq[jq] = __builtin_bit_cast(Pack4<T>, *reinterpret_cast<const u32x2*>(bias + nw + 8 * jq + 4 * lhalf));
            });
        } else {
            static_for<12>([&](auto jq_tag) {
                constexpr int jq = decltype(jq_tag)::value;
                const int n = nw + 8 * jq + 4 * lhalf;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < g.N) bq[jq].v[e] = bias[n + e];
            });
        }
    }
    dispatch_act(g.act, [&](auto act_tag) __attribute__((always_inline)) {
    constexpr int ACT = decltype(act_tag)::value;
    static_for<2>([&](auto i_tag) __attribute__((always_inline)) {
        constexpr int i = decltype(i_tag)::value;
        static_for<12>([&](auto jq_tag) __attribute__((always_inline)) {
            constexpr int j = decltype(jq_tag)::value >> 2, q = decltype(jq_tag)::value & 3;
            Pack4<T> o;
            static_for<4>([&](auto e_tag) {
                constexpr int e = decltype(e_tag)::value;
                float v = acc_value(acc[3 * i + j][4 * q + e]) + Elem<T>::to_f32(bq[j * 4 + q].v[e]);
                v = apply_act_c<ACT>(v);
                o.v[e] = Elem<T>::from_f32(v);
            });
            *reinterpret_cast<u32x2*>(stage + lrow * kRowPad + (j * 32 + 8 * q + 4 * lhalf) * 2) =
                __builtin_bit_cast(u32x2, o);
            __builtin_amdgcn_sched_barrier(0);
        });
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // a wave re-reads only its own rows
        if (interior) {
            u32x4 w[6], r[6];
            int64_t off[6];
#pragma unroll
            for (int u = 0; u < 6; u++) {
                const int slot = (u % 3) * 64 + lane;
                const int rl = 16 * (u / 3) + slot / 12, ch = slot % 12;
                off[u] = (int64_t)(m0 + wm * 64 + i * 32 + rl) * ldc + nw + 8 * ch;
                if (res) r[u] = *reinterpret_cast<const u32x4*>(res + off[u]);
                w[u] = *reinterpret_cast<const u32x4*>(stage + rl * kRowPad + ch * 16);
            }
#pragma unroll
            for (int u = 0; u < 6; u++) {
                if (res) w[u] = add_chunk<T>(w[u], r[u]);
                *reinterpret_cast<u32x4*>(c + off[u]) = w[u];
            }
        } else {
#pragma unroll 1
            for (int u = 0; u < 6; u++) {
                const int slot = (u % 3) * 64 + lane;
                const int rl = 16 * (u / 3) + slot / 12, ch = slot % 12;
                const int m = m0 + wm * 64 + i * 32 + rl;
                const int n = nw + 8 * ch;
                T* cp = c + (int64_t)m * ldc + n;
                const T* rp = res + (int64_t)m * ldc + n;
                if (m < g.M && n + 8 <= g.N) {
                    u32x4 w = *reinterpret_cast<const u32x4*>(stage + rl * kRowPad + ch * 16);
                    if (res) w = add_chunk<T>(w, *reinterpret_cast<const u32x4_unaligned*>(rp));
                    *reinterpret_cast<u32x4_unaligned*>(cp) = w;
                } else if (m < g.M && n < g.N) {                 // the last, partial chunk of a row
                    const T* sv = reinterpret_cast<const T*>(stage + rl * kRowPad + ch * 16);
                    for (int e = 0; e < g.N - n; e++) {
                        T val = sv[e];
                        if (res) val = Elem<T>::from_f32(Elem<T>::to_f32(val) + Elem<T>::to_f32(rp[e]));
                        cp[e] = val;
                    }
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the next block overwrites the rows just read
        __builtin_amdgcn_sched_barrier(0);
    });
    });
}

template <typename T, bool TA, bool TB>
__global__ __launch_bounds__(256) void gemm192_kernel(GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    using LA = typename std::conditional<TA, MnMajor<128>, KMajor>::type;
    using LB = typename std::conditional<TB, KMajor, MnMajor<256>>::type;

    int tm, tn;
    tile_of(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tm, tn);
    const int m0 = tm * 128, n0 = tn * 192;
    const int64_t batch = blockIdx.y;
    const char* a = reinterpret_cast<const char*>(static_cast<const T*>(g.a) + batch * g.sa);
    const char* b = reinterpret_cast<const char*>(static_cast<const T*>(g.b) + batch * g.sb);
    T* c = static_cast<T*>(g.c) + batch * g.sc;
    const T* res = g.residual ? static_cast<const T*>(g.residual) + batch * g.sc : nullptr;
    const uint32_t a_bytes = (uint32_t)(((int64_t)((TA ? g.K : g.M) - 1) * g.lda + (TA ? g.M : g.K)) * 2);
    const uint32_t b_bytes = (uint32_t)(((int64_t)((TB ? g.N : g.K) - 1) * g.ldb + (TB ? g.K : g.N)) * 2);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    const u32x4 raw = LA::raddr(lane, wm * 64, lds0);
    u32x2 ra;
    ra.x = raw.x; ra.y = raw.y;
    const u32x4 rb = LB::raddr(lane, wn * 96, lds0 + k192BOffset);
    u32x2 goff;
    goff.x = LA::goff(lane, wave, m0, g.lda, g.M);
    // (columns past the tile's 192 are not asked for: the layout is 256 wide)
    goff.y = LB::goff(lane, wave, n0, g.ldb, min(g.N, n0 + 192));
    const uint32_t m0b = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)wave * 1024u);
    const __amdgpu_buffer_rsrc_t rsa =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a), 0, a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsb =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(b), 0, b_bytes, 0x00020000);

    f32x16 acc[6];
    main_loop192<T, TA, TB>(acc, ra, rb, goff, rsa, rsb, LA::pass_stride(g.lda), LB::pass_stride(g.ldb),
                            LA::stage_stride(g.lda), LB::stage_stride(g.ldb), m0b, (uint32_t)(g.K / 32));
    store_tile192<T>(acc, smem, g, c, res, m0, n0);
}

template <typename T, bool TA, bool TB>
int launch192(hipStream_t s, GemmArgs g, int64_t batch) {
    auto kern = gemm192_kernel<T, TA, TB>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, k192Smem);
    });
    if (attr_err != hipSuccess)
        return fail(MHIP_ERR_LAUNCH, "gemm192: cannot reserve %d bytes of LDS: %s", k192Smem,
                    hipGetErrorString(attr_err));
    g.tiles_m = (g.M + 127) / 128;
    g.tiles_n = (g.N + 191) / 192;
    hipLaunchKernelGGL(kern, dim3((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch), dim3(256),
                       k192Smem, s, g);
    return check_launch("gemm192");
}

template <typename T>
int layout192(hipStream_t s, const GemmArgs& g, int64_t batch, int ta, int tb) {
    if (!ta && !tb) return launch192<T, false, false>(s, g, batch);
    if (!ta && tb) return launch192<T, false, true>(s, g, batch);
    if (ta && !tb) return launch192<T, true, false>(s, g, batch);
    return launch192<T, true, true>(s, g, batch);
}

// ---- the 256x288 tile --------------------------------------------------------------------------------
// gemm256x288_loop_* of the generated file: for problems whose 256x384 tiling leaves a quarter of the
// compute units idle ([8192, 2304]: 192 tiles of 256x384, 256 of 256x288).  Four waves one above the
// other, each 64 x 288 = 2 x 9 accumulator blocks (sixteen in the accumulation registers, two in
// v[128:159]); every wave reads all of B, which lies as in the 256x384 kernel -- the 256-column tile,
// then the 128-column tile, of which only the first 32 columns are ever loaded.
template <typename T, bool TA, bool TB>
__device__ __forceinline__ void main_loop288(f32x16 (&acc)[18], u32x2 ra, u32x4 rb, u32x2 rb2, u32x4& goff,
                                             __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb, uint32_t pa,
                                             uint32_t pb, uint32_t ta, uint32_t tb, uint32_t m0b, uint32_t kt) {
    constexpr bool bf = std::is_same<T, bf16_t>::value;
#define MHIP_LOOP(cond, name) \
    if constexpr (cond) gemm256x288_loop_##name(acc, ra, rb, rb2, goff, rsa, rsb, pa, pb, ta, tb, m0b, kt);
    MHIP_LOOP(bf && !TA && !TB, nn_bf16)
    MHIP_LOOP(bf && !TA && TB, nt_bf16)
    MHIP_LOOP(bf && TA && !TB, tn_bf16)
    MHIP_LOOP(bf && TA && TB, tt_bf16)
    MHIP_LOOP(!bf && !TA && !TB, nn_f16)
    MHIP_LOOP(!bf && !TA && TB, nt_f16)
    MHIP_LOOP(!bf && TA && !TB, tn_f16)
    MHIP_LOOP(!bf && TA && TB, tt_f16)
#undef MHIP_LOOP
}

// Epilogue: a wave's 64 x 288 sub-tile through LDS one 32-row block at a time (32 rows of 576 + 16
// bytes per wave); a block goes out as eighteen instructions of 64 lanes x 16 bytes: lane slot
// (u % 9) * 64 + lane = row 16 (u / 9) + slot / 36 of the block, chunk slot % 36.  The activation
// is a uniform branch around each group of four values, as in store_tile384 and for its reason.
template <typename T>
__device__ __forceinline__ void store_tile288(f32x16 (&acc)[18], char* smem, const GemmArgs& g, T* c, const T* res,
                                              int m0, int n0) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lrow = lane & 31, lhalf = lane >> 5;
    const T* bias = static_cast<const T*>(g.bias);
    constexpr int kRowPad = 288 * 2 + 16;
    char* stage = smem + wave * (32 * kRowPad);
    const int ldc = g.ldc ? g.ldc : g.N;
    const bool full_cols = __builtin_amdgcn_readfirstlane(n0 + 288 <= g.N);
    const bool interior = __builtin_amdgcn_readfirstlane(full_cols && m0 + wave * 64 + 64 <= g.M && ldc % 8 == 0);
    const bool stream = __builtin_amdgcn_readfirstlane(g.stream_c != 0);
    Pack4<T> bq[36];
    static_for<36>([&](auto jq_tag) {
        constexpr int jq = decltype(jq_tag)::value;
        bq[jq] = __builtin_bit_cast(Pack4<T>, u32x2{0u, 0u});
    });
    if (bias) {
        if (full_cols) {
            static_for<36>([&](auto jq_tag) {
                constexpr int jq = decltype(jq_tag)::value;
                bq[jq] = __builtin_bit_cast(Pack4<T>, *reinterpret_cast<const u32x2*>(bias + n0 + 8 * jq + 4 * lhalf));
            });
        } else {
            static_for<36>([&](auto jq_tag) {
                constexpr int jq = decltype(jq_tag)::value;
                const int n = n0 + 8 * jq + 4 * lhalf;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < g.N) bq[jq].v[e] = bias[n + e];
            });
        }
    }
    const int act = __builtin_amdgcn_readfirstlane(g.act);
    static_for<2>([&](auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
        static_for<36>([&](auto jq_tag) {
            constexpr int j = decltype(jq_tag)::value >> 2, q = decltype(jq_tag)::value & 3;
            constexpr int b = 9 * i + j;
            Pack4<T> o;
            float v4[4];
            static_for<4>([&](auto e_tag) {
                constexpr int e = decltype(e_tag)::value;
                if constexpr (b < 16) v4[e] = acc_value(acc[b][4 * q + e]);
                else v4[e] = acc[b][4 * q + e];
                v4[e] += Elem<T>::to_f32(bq[j * 4 + q].v[e]);
            });
            if (act == MHIP_ACT_GELU) {
#pragma unroll
                for (int e = 0; e < 4; e++) v4[e] = apply_act_c<MHIP_ACT_GELU>(v4[e]);
            } else if (act == MHIP_ACT_RELU) {
#pragma unroll
                for (int e = 0; e < 4; e++) v4[e] = apply_act_c<MHIP_ACT_RELU>(v4[e]);
            }
#pragma unroll
            for (int e = 0; e < 4; e++) o.v[e] = Elem<T>::from_f32(v4[e]);
            *reinterpret_cast<u32x2*>(stage + lrow * kRowPad + (j * 32 + 8 * q + 4 * lhalf) * 2) =
                __builtin_bit_cast(u32x2, o);
            __builtin_amdgcn_sched_barrier(0);
        });
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // a wave re-reads only its own rows
        if (interior) {
#pragma unroll
            for (int h = 0; h < 3; h++) {
                u32x4 w[6], r[6];
                int64_t off[6];
#pragma unroll
                for (int u = 0; u < 6; u++) {
                    const int U = 6 * h + u;
                    const int slot = (U % 9) * 64 + lane;
                    const int rl = 16 * (U / 9) + slot / 36, ch = slot % 36;
                    off[u] = (int64_t)(m0 + wave * 64 + i * 32 + rl) * ldc + n0 + 8 * ch;
                    if (res) r[u] = *reinterpret_cast<const u32x4*>(res + off[u]);
                    w[u] = *reinterpret_cast<const u32x4*>(stage + rl * kRowPad + ch * 16);
                }
#pragma unroll
                for (int u = 0; u < 6; u++) {
                    if (res) w[u] = add_chunk<T>(w[u], r[u]);
                    if (stream) __builtin_nontemporal_store(w[u], reinterpret_cast<u32x4*>(c + off[u]));
                    else *reinterpret_cast<u32x4*>(c + off[u]) = w[u];
                }
            }
        } else {
#pragma unroll 1
            for (int u = 0; u < 18; u++) {
                const int slot = (u % 9) * 64 + lane;
                const int rl = 16 * (u / 9) + slot / 36, ch = slot % 36;
                const int m = m0 + wave * 64 + i * 32 + rl;
                const int n = n0 + 8 * ch;
                T* cp = c + (int64_t)m * ldc + n;
                const T* rp = res + (int64_t)m * ldc + n;
                if (m < g.M && n + 8 <= g.N) {
                    u32x4 w = *reinterpret_cast<const u32x4*>(stage + rl * kRowPad + ch * 16);
                    if (res) w = add_chunk<T>(w, *reinterpret_cast<const u32x4_unaligned*>(rp));
                    *reinterpret_cast<u32x4_unaligned*>(cp) = w;
                } else if (m < g.M && n < g.N) {                 // the last, partial chunk of a row
                    const T* sv = reinterpret_cast<const T*>(stage + rl * kRowPad + ch * 16);
                    for (int e = 0; e < g.N - n; e++) {
                        T val = sv[e];
                        if (res) val = Elem<T>::from_f32(Elem<T>::to_f32(val) + Elem<T>::to_f32(rp[e]));
                        cp[e] = val;
                    }
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the next block overwrites the rows just read
        __builtin_amdgcn_sched_barrier(0);
    });
}

template <typename T, bool TA, bool TB>
__global__ __launch_bounds__(256) void gemm288_kernel(GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    using LA = typename std::conditional<TA, MnMajor<256>, KMajor>::type;
    using LB = typename std::conditional<TB, KMajor, MnMajor<256>>::type;
    using LB2 = typename std::conditional<TB, KMajor, MnMajor<128>>::type;

    int tm, tn;
    tile_of(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tm, tn);
    const int m0 = tm * 256, n0 = tn * 288;
    const int64_t batch = blockIdx.y;
    const char* a = reinterpret_cast<const char*>(static_cast<const T*>(g.a) + batch * g.sa);
    const char* b = reinterpret_cast<const char*>(static_cast<const T*>(g.b) + batch * g.sb);
    T* c = static_cast<T*>(g.c) + batch * g.sc;
    const T* res = g.residual ? static_cast<const T*>(g.residual) + batch * g.sc : nullptr;
    const uint32_t a_bytes = (uint32_t)(((int64_t)((TA ? g.K : g.M) - 1) * g.lda + (TA ? g.M : g.K)) * 2);
    const uint32_t b_bytes = (uint32_t)(((int64_t)((TB ? g.N : g.K) - 1) * g.ldb + (TB ? g.K : g.N)) * 2);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    const u32x4 raw = LA::raddr(lane, wave * 64, lds0);
    u32x2 ra;
    ra.x = raw.x; ra.y = raw.y;
    const u32x4 rb = LB::raddr(lane, 0, lds0 + kOperBytes);
    const u32x4 rb2w = LB2::raddr(lane, 0, lds0 + 2 * kOperBytes);
    u32x2 rb2;
    rb2.x = rb2w.x; rb2.y = rb2w.y;
    const int n_end = min(g.N, n0 + 288);                    // nothing past the tile's 288 columns is asked for
    u32x4 goff;
    goff.x = LA::goff(lane, wave, m0, g.lda, g.M);
    goff.y = LB::goff(lane, wave, n0, g.ldb, n_end);
    goff.z = LB2::goff(lane, wave, n0 + 256, g.ldb, n_end);
    if (TB && n0 + 256 + 16 * wave + (lane >> 2) >= n_end) goff.z = kOob;     // (a k-contiguous tile is bounded by rows)
    goff.w = 0;
    const uint32_t m0b = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)wave * 1024u);
    const __amdgpu_buffer_rsrc_t rsa =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a), 0, a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsb =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(b), 0, b_bytes, 0x00020000);

    f32x16 acc[18];
    main_loop288<T, TA, TB>(acc, ra, rb, rb2, goff, rsa, rsb, LA::pass_stride(g.lda), LB::pass_stride(g.ldb),
                            LA::stage_stride(g.lda), LB::stage_stride(g.ldb), m0b, (uint32_t)(g.K / 32));
    store_tile288<T>(acc, smem, g, c, res, m0, n0);
}

template <typename T, bool TA, bool TB>
int launch288(hipStream_t s, GemmArgs g, int64_t batch) {
    auto kern = gemm288_kernel<T, TA, TB>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, k384Smem);
    });
    if (attr_err != hipSuccess)
        return fail(MHIP_ERR_LAUNCH, "gemm288: cannot reserve %d bytes of LDS: %s", k384Smem,
                    hipGetErrorString(attr_err));
    g.tiles_m = (g.M + 255) / 256;
    g.tiles_n = (g.N + 287) / 288;
    g.stream_c = (int64_t)g.M * g.N * batch * 2 > (256ll << 20) && (g.ldc ? g.ldc : g.N) % 8 == 0;
    hipLaunchKernelGGL(kern, dim3((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch), dim3(256),
                       k384Smem, s, g);
    return check_launch("gemm288");
}

template <typename T>
int layout288(hipStream_t s, const GemmArgs& g, int64_t batch, int ta, int tb) {
    if (!ta && !tb) return launch288<T, false, false>(s, g, batch);
    if (!ta && tb) return launch288<T, false, true>(s, g, batch);
    if (ta && !tb) return launch288<T, true, false>(s, g, batch);
    return launch288<T, true, true>(s, g, batch);
}

}  // namespace

// The activations the epilogues of the 256x384 and the 256x288 kernel serve.
bool gemm384_activation_ok(int act) { return act == MHIP_ACT_NONE || act == MHIP_ACT_RELU || act == MHIP_ACT_GELU; }

int launch_gemm384(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype) {
    return dtype == MHIP_BF16 ? layout384<bf16_t>(s, g, batch, trans_a, trans_b) : layout384<f16_t>(s, g, batch, trans_a, trans_b);
}

int launch_gemm288(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype) {
    return dtype == MHIP_BF16 ? layout288<bf16_t>(s, g, batch, trans_a, trans_b) : layout288<f16_t>(s, g, batch, trans_a, trans_b);
}

int launch_gemm192(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype) {
    return dtype == MHIP_BF16 ? layout192<bf16_t>(s, g, batch, trans_a, trans_b) : layout192<f16_t>(s, g, batch, trans_a, trans_b);
}

int launch_gemm_pair(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype) {
    return dtype == MHIP_BF16 ? layout_pair<bf16_t>(s, g, batch, trans_a, trans_b) : layout_pair<f16_t>(s, g, batch, trans_a, trans_b);
}

}  // namespace mhip
