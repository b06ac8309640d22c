// Large-problem GEMM for gfx950: 256x256 C tile, four waves (one per SIMD), each
// wave a 128x128 sub-tile = 4x4 v_mfma_f32_32x32x16 accumulators that fill the
// AGPR file; and the same kernel on a 256x128 tile (each wave 128x64, B tile 128 wide).  The main loop is generated, hand-scheduled inline assembly
// (gen_gemm256_loop.py -> gemm256_loop.inc: schedule and register map are
// documented there); this file computes the per-thread addresses it consumes and
// holds the epilogue.
//
// K is consumed in stages of 32 through a ring of five 32 KB LDS buffers
// ([A tile 16 KB][B tile 16 KB]) filled by buffer loads that write LDS directly:
// a wave's load instruction deposits 64 x 16 bytes contiguously, so the LDS
// layout is fixed by which 16-byte chunk of global memory each lane asks for.
// An operand whose k axis is contiguous in memory is stored [256 rows][32 k]
// (64-byte rows, chunk c of row r at position c ^ ((r >> 2) & 3)) and read with
// ds_read_b128; an operand whose k axis is the slow one is stored as it lies,
// [32 k][256 mn] (chunk c of k-row k at position c ^ ((k & 3) << 2)), and
// transposed on the way out with ds_read_b64_tr_b16.  The loads are
// bounds-checked buffer loads: rows or columns beyond the matrix read as zero, so
// ragged M and N need no special path.
#include "gemm_ring.h"

namespace mhip {

#include "gemm256_loop.inc"

// gemm_twoset.hip: the 256x384 tile and the 256x128 tile for two workgroups per compute unit
int launch_gemm384(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype);
int launch_gemm_pair(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype);
int launch_gemm192(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype);
int launch_gemm288(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype);

namespace {

template <typename T, bool TA, bool TB, int BW, int RING>
__device__ inline void main_loop(f32x16 (&acc)[BW / 16], u32x4 ra, u32x4 rb, u32x2& misc,
                                 __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb, uint32_t pa,
                                 uint32_t pb, uint32_t ta, uint32_t tb, uint32_t m0b, uint32_t kt) {
    constexpr bool bf = std::is_same<T, bf16_t>::value;
    // the member of the generated tile family: B width x ring depth
#define MHIP_LOOP(cond, name)                                                                        \
    if constexpr (cond) {                                                                            \
        if constexpr (BW == 256 && RING == 5) gemm256_loop_##name(acc, ra, rb, misc, rsa, rsb, pa, pb, ta, tb, m0b, kt); \
        else if constexpr (BW == 256 && RING == 4) gemm256r4_loop_##name(acc, ra, rb, misc, rsa, rsb, pa, pb, ta, tb, m0b, kt); \
        else if constexpr (BW == 128 && RING == 5) gemm256x128_loop_##name(acc, ra, rb, misc, rsa, rsb, pa, pb, ta, tb, m0b, kt); \
        else if constexpr (BW == 128 && RING == 4) gemm256x128r4_loop_##name(acc, ra, rb, misc, rsa, rsb, pa, pb, ta, tb, m0b, kt); \
        else gemm256x128r6_loop_##name(acc, ra, rb, misc, rsa, rsb, pa, pb, ta, tb, m0b, kt);          \
    }
    static_assert((BW == 256 && (RING == 4 || RING == 5)) || (BW == 128 && RING >= 4 && RING <= 6),
                  "not a member of the generated tile family");
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

// BW = 256: the 256x256 tile (each wave 128x128).  BW = 128: a 256x128 tile (each wave
// 128x64, half the accumulators, a 24 KB stage) for problems whose 256x256 tiling would
// leave compute units idle or a last round nearly empty.
// RING: stage buffers in the LDS ring (4, 5 or 6; loads run that many stages ahead).
template <typename T, bool TA, bool TB, int BW, int RING>
__global__ __launch_bounds__(256) void gemm256_kernel(GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    using LA = typename std::conditional<TA, MnMajor<256>, KMajor>::type;
    using LB = typename std::conditional<TB, KMajor, MnMajor<BW>>::type;
    constexpr int WN = BW / 2;            // columns per wave
    constexpr int NBF = BW / 64;          // 32-column accumulator blocks per wave

    int tm, tn;
    tile_of(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tm, tn);
    const int m0 = tm * 256, n0 = tn * BW;
    const int64_t batch = blockIdx.y;
    const char* a = reinterpret_cast<const char*>(static_cast<const T*>(g.a) + batch * g.sa);
    const char* b = reinterpret_cast<const char*>(static_cast<const T*>(g.b) + batch * g.sb);
    T* c = static_cast<T*>(g.c) + batch * g.sc;
    const T* res = g.residual ? static_cast<const T*>(g.residual) + batch * g.sc : nullptr;
    // (extents to the last element: the matrices may be column slices of wider ones)
    const uint32_t a_bytes = (uint32_t)(((int64_t)((TA ? g.K : g.M) - 1) * g.lda + (TA ? g.M : g.K)) * 2);
    const uint32_t b_bytes = (uint32_t)(((int64_t)((TB ? g.N : g.K) - 1) * g.ldb + (TB ? g.K : g.N)) * 2);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, lhalf = lane >> 5;
    // LDS byte address of the dynamic segment
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;

    const u32x4 ra = LA::raddr(lane, wm * 128, lds0);
    const u32x4 rb = LB::raddr(lane, wn * WN, lds0 + kOperBytes);
    u32x2 misc;
    misc.x = LA::goff(lane, wave, m0, g.lda, g.M);
    misc.y = LB::goff(lane, wave, n0, g.ldb, g.N);
    // LDS address of this wave's 1 KB slot in pass 0 of buffer 0 (wave-uniform)
    const uint32_t m0b = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)wave * 1024u);
    const __amdgpu_buffer_rsrc_t rsa =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a), 0, a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsb =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(b), 0, b_bytes, 0x00020000);

    f32x16 acc[4 * NBF];
    main_loop<T, TA, TB, BW, RING>(acc, ra, rb, misc, rsa, rsb, LA::pass_stride(g.lda), LB::pass_stride(g.ldb),
                                   LA::stage_stride(g.lda), LB::stage_stride(g.ldb), m0b, (uint32_t)(g.K / 32));

    // (a compile-time variant: the same branch inside the epilogue upsets the compiler)
    if (g.stream_c) store_tile<T, BW, true>(acc, smem, g, c, res, m0, n0);
    else store_tile<T, BW, false>(acc, smem, g, c, res, m0, n0);
}

// ---- streamed tiles ------------------------------------------------------------------------------
// The 256x128 kernel as a persistent workgroup: one workgroup per compute unit runs tile after tile,
// and the stores of a tile travel inside the main loop of the NEXT one (gemm_stream_loop_* of the
// generated file), so that the matrix pipes do not idle through a burst of C stores at the end of
// every round, nor through the load latency at the start of one: the loads of the next tile's first
// stages are issued before the finished accumulators are converted.  Between two tiles only that
// conversion (bias, activation, rounding to 16 bits: 64 registers of packed results) is exposed.
// LDS: the ring of five 24 KB stage buffers, a 4 KB transposition area per wave, two 256-byte
// buffers for the bias values of the current and the previous tile.
// Served: A with k contiguous, M a multiple of 256, N of 128 (no ragged tiles: the in-loop stores
// carry no bounds checks), no residual, one batch, K >= 640.  Tile 0 of a workgroup runs the
// ordinary loop, the last one the ordinary epilogue; results are those of gemm256_kernel bit for bit.
constexpr int kStreamWorkgroups = 256;          // one per compute unit of the device this is written for
constexpr uint32_t kStreamRing = 5 * 24 * 1024;
constexpr uint32_t kStreamXpose = kStreamRing;                 // 4 waves x 4 KB
constexpr uint32_t kStreamBias = kStreamRing + 4 * 4096;       // 2 x 256 bytes
constexpr uint32_t kStreamSmem = kStreamBias + 512;

template <typename T, bool TB>
__device__ __forceinline__ void stream_prologue(u32x2& misc, __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb,
                                       uint32_t pa, uint32_t pb, uint32_t ta, uint32_t tb, uint32_t m0b,
                                       __amdgpu_buffer_rsrc_t rsbias, uint32_t m0bias, uint32_t vbias) {
    constexpr bool bf = std::is_same<T, bf16_t>::value;
    if constexpr (bf && !TB) gemm_stream_loop_nn_bf16_prologue(misc, rsa, rsb, pa, pb, ta, tb, m0b, rsbias, m0bias, vbias);
    if constexpr (bf && TB) gemm_stream_loop_nt_bf16_prologue(misc, rsa, rsb, pa, pb, ta, tb, m0b, rsbias, m0bias, vbias);
    if constexpr (!bf && !TB) gemm_stream_loop_nn_f16_prologue(misc, rsa, rsb, pa, pb, ta, tb, m0b, rsbias, m0bias, vbias);
    if constexpr (!bf && TB) gemm_stream_loop_nt_f16_prologue(misc, rsa, rsb, pa, pb, ta, tb, m0b, rsbias, m0bias, vbias);
}

template <typename T, bool TB>
__device__ __forceinline__ void stream_loop(f32x16 (&acc)[8], u32x4 ra, u32x4 rb, u32x2& misc, __amdgpu_buffer_rsrc_t rsa,
                                   __amdgpu_buffer_rsrc_t rsb, uint32_t pa, uint32_t pb, uint32_t ta, uint32_t tb,
                                   uint32_t m0b, uint32_t kt, const u32x16 (&pk)[4], u32x4 xaddr, uint64_t cptr,
                                   uint32_t srow) {
    constexpr bool bf = std::is_same<T, bf16_t>::value;
    if constexpr (bf && !TB) gemm_stream_loop_nn_bf16(acc, ra, rb, misc, rsa, rsb, pa, pb, ta, tb, m0b, kt, pk, xaddr, cptr, srow);
    if constexpr (bf && TB) gemm_stream_loop_nt_bf16(acc, ra, rb, misc, rsa, rsb, pa, pb, ta, tb, m0b, kt, pk, xaddr, cptr, srow);
    if constexpr (!bf && !TB) gemm_stream_loop_nn_f16(acc, ra, rb, misc, rsa, rsb, pa, pb, ta, tb, m0b, kt, pk, xaddr, cptr, srow);
    if constexpr (!bf && TB) gemm_stream_loop_nt_f16(acc, ra, rb, misc, rsa, rsb, pa, pb, ta, tb, m0b, kt, pk, xaddr, cptr, srow);
}

// Bias, activation and rounding of a finished tile, in the arithmetic of store_tile; the bias values
// come from the LDS buffer the tile's prologue filled.  pk[i][2 c], pk[i][2 c + 1]: accumulator block
// i (32 rows), columns 8 c + 4 (lane >> 5) .. + 3 of the wave's 64.
template <typename T>
__device__ __forceinline__ void pack_tile(const f32x16 (&acc)[8], const char* bias_lds, int act, int wn, int lhalf,
                                 u32x16 (&pk)[4]) {
    dispatch_act(act, [&](auto act_tag) {
    constexpr int ACT = decltype(act_tag)::value;
    static_for<8>([&](auto c_tag) {
        constexpr int cidx = decltype(c_tag)::value, j = cidx >> 2, q = cidx & 3;
        const Pack4<T> t = __builtin_bit_cast(
            Pack4<T>, *reinterpret_cast<const u32x2*>(bias_lds + (wn * 64 + 8 * cidx + 4 * lhalf) * 2));
        float bv[4];
#pragma unroll
        for (int e = 0; e < 4; e++) bv[e] = Elem<T>::to_f32(t.v[e]);
        static_for<4>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            Pack4<T> o;
            static_for<4>([&](auto e_tag) {
                constexpr int e = decltype(e_tag)::value;
                float v = acc_value(acc[i * 2 + j][4 * q + e]) + bv[e];
                v = apply_act_c<ACT>(v);
                o.v[e] = Elem<T>::from_f32(v);
            });
            const u32x2 w = __builtin_bit_cast(u32x2, o);
            pk[i][2 * cidx] = w.x;
            pk[i][2 * cidx + 1] = w.y;
        });
        __builtin_amdgcn_sched_barrier(0);
    });
    });
}

template <typename T, bool TB>
__global__ __launch_bounds__(256) void gemm_stream_kernel(GemmArgs g, int total) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    using LA = KMajor;
    using LB = typename std::conditional<TB, KMajor, MnMajor<128>>::type;
    const char* a = reinterpret_cast<const char*>(g.a);
    const char* b = reinterpret_cast<const char*>(g.b);
    T* c = static_cast<T*>(g.c);
    const T* bias = static_cast<const T*>(g.bias);
    const uint32_t a_bytes = (uint32_t)((int64_t)g.M * g.lda * 2);
    const uint32_t b_bytes = (uint32_t)((int64_t)(TB ? g.N : g.K) * g.ldb * 2);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, lhalf = lane >> 5;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    const u32x4 ra = LA::raddr(lane, wm * 128, lds0);
    const u32x4 rb = LB::raddr(lane, wn * 64, lds0 + kOperBytes);
    const uint32_t m0b = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)wave * 1024u);
    const __amdgpu_buffer_rsrc_t rsa =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a), 0, a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsb =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(b), 0, b_bytes, 0x00020000);
    // without a bias: an empty buffer, whose loads put zeros into LDS
    const __amdgpu_buffer_rsrc_t rsbias = __builtin_amdgcn_make_buffer_rsrc(
        bias ? const_cast<T*>(bias) : c, 0, bias ? (uint32_t)g.N * 2u : 0u, 0x00020000);
    const uint32_t pa = LA::pass_stride(g.lda), pb = LB::pass_stride(g.ldb);
    const uint32_t ta = LA::stage_stride(g.lda), tb = LB::stage_stride(g.ldb);
    const uint32_t kt = (uint32_t)(g.K / 32);
    // transposition area of this wave: write address of this lane's row (chunk 0), read address
    const uint32_t xbase = lds0 + kStreamXpose + (uint32_t)wave * 4096u;
    u32x4 xaddr;
    xaddr.x = xbase + (uint32_t)(lrow * 128 + 8 * lhalf + (((lrow >> 1) & 7) << 4));
    xaddr.y = xbase + (uint32_t)lane * 16u;
    const uint32_t srow = (uint32_t)g.N * 16u;            // eight rows of C, in bytes
    const int chunk_even = (lane & 7) ^ ((lane >> 4) & 3);

    f32x16 acc[8];
    u32x16 pk[4];
    int m0 = 0, n0 = 0, it = 0;
    for (int vp = blockIdx.x; vp < total; vp += gridDim.x, it++) {
        const int pm0 = m0, pn0 = n0;
        int tm, tn;
        tile_of(vp, total, g.tiles_m, g.tiles_n, tm, tn);
        m0 = tm * 256; n0 = tn * 128;
        u32x2 misc;
        misc.x = LA::goff(lane, wave, m0, g.lda, g.M);
        misc.y = LB::goff(lane, wave, n0, g.ldb, g.N);
        if (it == 0) {
            if (wave == 0)
                *reinterpret_cast<uint32_t*>(smem + kStreamBias + lane * 4) =
                    bias ? *reinterpret_cast<const uint32_t*>(bias + n0 + 2 * lane) : 0u;
            main_loop<T, false, TB, 128, 5>(acc, ra, rb, misc, rsa, rsb, pa, pb, ta, tb, m0b, kt);
        } else {
            const uint32_t m0bias = __builtin_amdgcn_readfirstlane(lds0 + kStreamBias + (uint32_t)(it & 1) * 256u);
            stream_prologue<T, TB>(misc, rsa, rsb, pa, pb, ta, tb, m0b, rsbias, m0bias,
                                   (uint32_t)(n0 * 2 + lane * 4));
            pack_tile<T>(acc, smem + kStreamBias + ((it - 1) & 1) * 256, g.act, wn, lhalf, pk);
            // where the previous tile's rows go: this lane's chunk of row (lane / 8) of each 8-row group
            const uint32_t off_even =
                (uint32_t)((((int64_t)(pm0 + wm * 128 + (lane >> 3)) * g.N) + pn0 + wn * 64 + chunk_even * 8) * 2);
            xaddr.z = off_even;
            xaddr.w = off_even ^ 64u;
            stream_loop<T, TB>(acc, ra, rb, misc, rsa, rsb, pa, pb, ta, tb, m0b, kt, pk, xaddr,
                               (uint64_t)reinterpret_cast<uintptr_t>(c), srow);
        }
    }
    store_tile<T, 128>(acc, smem, g, c, static_cast<const T*>(nullptr), m0, n0);
}

template <typename T, bool TB>
int launch_stream(hipStream_t s, GemmArgs g) {
    auto kern = gemm_stream_kernel<T, TB>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kStreamSmem);
    });
    if (attr_err != hipSuccess)
        return fail(MHIP_ERR_LAUNCH, "gemm_stream: cannot reserve %u bytes of LDS: %s", kStreamSmem,
                    hipGetErrorString(attr_err));
    g.tiles_m = g.M / 256;
    g.tiles_n = g.N / 128;
    const int total = g.tiles_m * g.tiles_n;
    const int grid = total < kStreamWorkgroups ? total : kStreamWorkgroups;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), kStreamSmem, s, g, total);
    return check_launch("gemm_stream");
}

template <typename T, bool TA, bool TB, int BW, int RING>
int launch256(hipStream_t s, GemmArgs g, int64_t batch) {
    // the ring of stage buffers; the epilogue's staging (four waves x 128 rows of WN 16-bit values + 16
    // bytes of padding) reuses it and is the larger of the two for a short ring of wide tiles
    constexpr int kRing = RING * (16 + BW / 16) * 1024, kStaging = 4 * 128 * (BW + 16);
    constexpr int kSmem = kRing > kStaging ? kRing : kStaging;
    static_assert(kSmem <= 160 * 1024, "ring or staging exceeds the LDS of a compute unit");
    auto kern = gemm256_kernel<T, TA, TB, BW, RING>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
    });
    if (attr_err != hipSuccess)
        return fail(MHIP_ERR_LAUNCH, "gemm256: cannot reserve %d bytes of LDS: %s", kSmem,
                    hipGetErrorString(attr_err));
    g.tiles_m = (g.M + 255) / 256;
    g.tiles_n = (g.N + BW - 1) / BW;
    // A result of more than 256 MB passes through the L2s (32 MB) and the memory-side cache once and
    // is gone before anything reads it; stored the ordinary way it evicts the operands on its way.
    const int stream_mode = tune_int("MHIP_GEMM_STREAM_C", 1);                     // 2 = never, 3 = always
    // (only rows on 16-byte boundaries: with N = 50257 the hint cost 55 us where with 50304 it gains 50)
    g.stream_c = stream_mode == 3 || ((int64_t)g.M * g.N * batch * 2 > (256ll << 20) && stream_mode != 2 &&
                                      (g.ldc ? g.ldc : g.N) % 8 == 0);
    hipLaunchKernelGGL(kern, dim3((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch), dim3(256),
                       kSmem, s, g);
    return check_launch("gemm256");
}

template <typename T, int BW, int RING>
int layout256(hipStream_t s, const GemmArgs& g, int64_t batch, int ta, int tb) {
    if (!ta && !tb) return launch256<T, false, false, BW, RING>(s, g, batch);
    if (!ta && tb) return launch256<T, false, true, BW, RING>(s, g, batch);
    if (ta && !tb) return launch256<T, true, false, BW, RING>(s, g, batch);
    return launch256<T, true, true, BW, RING>(s, g, batch);
}

template <typename T>
int family256(hipStream_t s, const GemmArgs& g, int64_t batch, int ta, int tb, int bw, int ring) {
    if (bw == 256) {
        if (ring == 4) return layout256<T, 256, 4>(s, g, batch, ta, tb);
        return layout256<T, 256, 5>(s, g, batch, ta, tb);
    }
    if (ring == 4) return layout256<T, 128, 4>(s, g, batch, ta, tb);
    if (ring == 6) return layout256<T, 128, 6>(s, g, batch, ta, tb);
    return layout256<T, 128, 5>(s, g, batch, ta, tb);
}

}  // namespace

// The kernels need whole K stages, 16-byte-aligned operand rows (checked by the
// caller), a 16-byte-aligned output (its rows may start anywhere when N is no multiple of 8:
// they are then stored with unaligned 16-byte accesses), operands small enough for
// 32-bit byte offsets including the prefetch overrun of five K stages, and enough
// tiles (256 x `bw`) to occupy the device.
bool gemm256_eligible(const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype, int bw, bool any_tile_count) {
    if (dtype != MHIP_BF16 && dtype != MHIP_F16) return false;
    if (g.K % 32 != 0 || g.K < 32) return false;
    if ((reinterpret_cast<uintptr_t>(g.c) & 15) != 0 || (batch > 1 && g.sc % 8 != 0)) return false;
    if (g.residual && (reinterpret_cast<uintptr_t>(g.residual) & 15) != 0) return false;
    if (g.bias && (reinterpret_cast<uintptr_t>(g.bias) & 7) != 0) return false;
    // (the extents the kernel puts into its buffer descriptors: the last stored row ends the operand;
    // a column slice keeps the row stride of the whole matrix)
    const int64_t a_bytes = ((int64_t)((trans_a ? g.K : g.M) - 1) * g.lda + (trans_a ? g.M : g.K)) * 2;
    const int64_t b_bytes = ((int64_t)((trans_b ? g.N : g.K) - 1) * g.ldb + (trans_b ? g.K : g.N)) * 2;
    if (a_bytes >= 0x70000000LL || b_bytes >= 0x70000000LL) return false;
    const int tile_rows = bw == 192 ? 128 : 256;
    const int64_t tiles = (int64_t)((g.M + tile_rows - 1) / tile_rows) * ((g.N + bw - 1) / bw) * batch;
    return (tiles >= 192 || any_tile_count) && tiles <= 0x7FFFFFFF && batch <= 65535;
}

// `bw` x `ring`: the member of the tile family (384 x 4, 256 x {4, 5}, 128 x {4, 5, 6}; anything else runs
// depth 5).
int launch_gemm256(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b,
                   int dtype, int bw, int ring) {
    if (bw == 384) return launch_gemm384(s, g, batch, trans_a, trans_b, dtype);
    if (bw == 192) return launch_gemm192(s, g, batch, trans_a, trans_b, dtype);                     // 128-row tiles
    if (bw == 288) return launch_gemm288(s, g, batch, trans_a, trans_b, dtype);
    if (bw == 128 && ring == 3) return launch_gemm_pair(s, g, batch, trans_a, trans_b, dtype);      // two workgroups per compute unit
    if (dtype == MHIP_BF16) return family256<bf16_t>(s, g, batch, trans_a, trans_b, bw, ring);
    return family256<f16_t>(s, g, batch, trans_a, trans_b, bw, ring);
}

// Streamed tiles (persistent workgroups, stores inside the next tile's loop): see gemm_stream_kernel.
// Worth it from the second round on, i.e. with more tiles than compute units.
bool gemm_stream_eligible(const GemmArgs& g, int64_t batch, int trans_a, int trans_b, int dtype) {
    if (!gemm256_eligible(g, batch, trans_a, trans_b, dtype, 128, false)) return false;
    if (trans_a || batch != 1 || g.residual) return false;
    if (g.M % 256 != 0 || g.N % 128 != 0 || g.K < 640 || g.ldc != 0) return false;
    if ((int64_t)g.M * g.N * 2 >= 0xFFFFFFFFLL) return false;          // 32-bit byte offsets into C
    return (int64_t)(g.M / 256) * (g.N / 128) > kStreamWorkgroups;
}

int launch_gemm_stream(hipStream_t s, const GemmArgs& g, int trans_b, int dtype) {
    if (dtype == MHIP_BF16) return trans_b ? launch_stream<bf16_t, true>(s, g) : launch_stream<bf16_t, false>(s, g);
    return trans_b ? launch_stream<f16_t, true>(s, g) : launch_stream<f16_t, false>(s, g);
}

}  // namespace mhip
