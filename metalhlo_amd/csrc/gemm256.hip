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
#include <mutex>
#include <type_traits>
#include <utility>

#include "gemm_common.h"

namespace mhip {

typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));

#include "gemm256_loop.inc"

namespace {

constexpr uint32_t kOperBytes = 16 * 1024;   // B tile offset inside a 32 KB stage buffer
typedef u32x4 u32x4_unaligned __attribute__((aligned(2)));

template <typename F, int... I>
__device__ inline void static_for_impl(F& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ inline void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// ---- operand with k contiguous in memory --------------------------------------
// One load instruction of wave w in pass p fills rows 64p + 16w .. +15 (64 bytes
// each): lane -> row (lane >> 2), position (lane & 3).
struct KMajor {
    __device__ static uint32_t goff(int lane, int wave, int row0, int ld, int cols_total) {
        (void)cols_total;
        const int row = row0 + 16 * wave + (lane >> 2);
        const int c = (lane & 3) ^ ((lane >> 4) & 3);
        return (uint32_t)(((int64_t)row * ld + c * 8) * 2);
    }
    __device__ static uint32_t pass_stride(int ld) { return (uint32_t)(64 * ld * 2); }
    __device__ static uint32_t stage_stride(int ld) { (void)ld; return 64u; }
    // read addresses of ring buffers 0 and 1: element s = k-step s of row block 0
    // (+ 2048 per row block of 32, + 32768 for buffer 1); the loop derives the other
    // buffers' addresses
    __device__ static u32x4 raddr(int lane, int row_block0, uint32_t base) {
        const int lrow = lane & 31, lhalf = lane >> 5;
        const uint32_t b = base + (uint32_t)((row_block0 + lrow) * 64 + ((lhalf ^ ((lrow >> 2) & 3)) << 4));
        u32x4 r;
        r.x = b; r.y = b ^ 32u; r.z = 0; r.w = 0;
        return r;
    }
};

// ---- operand with k as the slow memory axis -------------------------------------
// Tile of W mn-columns: k-rows of 2W bytes.  One load instruction of a wave fills 1 KB =
// 1024 / 2W consecutive k-rows (W = 256: k rows 8p + 2w, 8p + 2w + 1 of pass p, lane -> k row
// lane >> 5, position lane & 31; W = 128: k rows 16p + 4w .. + 3, lane -> lane >> 4, lane & 15).
template <int W>
struct MnMajor {
    static constexpr int kLanesPerRow = W / 8;           // 16-byte chunks per k-row
    static constexpr int kRowsPerSlot = 64 / kLanesPerRow;
    __device__ static uint32_t goff(int lane, int wave, int col0, int ld, int cols_total) {
        const int k = kRowsPerSlot * wave + lane / kLanesPerRow;
        const int c = (lane % kLanesPerRow) ^ ((k & 3) << 2);
        const int col = col0 + c * 8;
        return col < cols_total ? (uint32_t)(((int64_t)k * ld + col) * 2) : kOob;
    }
    __device__ static uint32_t pass_stride(int ld) { return (uint32_t)(4 * kRowsPerSlot * ld * 2); }
    __device__ static uint32_t stage_stride(int ld) { return (uint32_t)(32 * ld * 2); }
    // read addresses of ring buffers 0 and 1: element j = this wave's mn block j (32 columns)
    // at k-step 0 (+ 16 k-rows per k-step, + 4 k-rows for the upper four k of a fragment,
    // + one stage buffer for buffer 1); the loop derives the other buffers' addresses.
    // The 64-byte position of a block in its k-row is (block ^ (k & 3)): the chunk swizzle above.
    __device__ static u32x4 raddr(int lane, int mn_block0, uint32_t base) {
        const int i = lane & 15, gq = lane >> 4;
        const int xr = (i >> 2) & 3;
        const int blk0 = mn_block0 >> 5;
        const uint32_t b = base + (uint32_t)((8 * (gq >> 1) + (i >> 2)) * (2 * W) + (16 * (gq & 1) + 4 * (i & 3)) * 2);
        u32x4 r;
        r.x = b + (uint32_t)(((blk0 + 0) ^ xr) << 6); r.y = b + (uint32_t)(((blk0 + 1) ^ xr) << 6);
        r.z = b + (uint32_t)(((blk0 + 2) ^ xr) << 6); r.w = b + (uint32_t)(((blk0 + 3) ^ xr) << 6);
        return r;
    }
};

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

// One accumulator value, moved out of the accumulation registers where it is used.  Left to
// itself the compiler copies all 256 of them into ordinary registers right behind the loop
// (the copies are common to every activation's branch), which leaves no register for
// anything else: addresses then sit in scratch memory and every register group waits for a
// reload.
__device__ __forceinline__ float acc_value(float in_agpr) {
    float v;
    asm("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(in_agpr));
    return v;
}

// Epilogue of one tile: bias, activation, conversion, then through LDS (the ring, free after the
// loop's last barrier) so that every store instruction writes whole 16-byte chunks of C rows.
template <typename T, int BW, bool STREAM_C = false, int AHEAD = (BW == 256 ? 2 : 4)>
__device__ __forceinline__ void store_tile(f32x16 (&acc)[BW / 16], char* smem, const GemmArgs& g, T* c, const T* res,
                                  int m0, int n0) {
    constexpr int WN = BW / 2;            // columns per wave
    constexpr int NBF = BW / 64;          // 32-column accumulator blocks per wave
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, lhalf = lane >> 5;
    // The loop ends with every wave's outstanding loads landed and a barrier, so the
    // ring may be reused as the staging area below.  Waves may still have (unused)
    // fragment reads of a stage past the end in flight; overwriting those is harmless.
    //
    // Accumulator tiles are transposed: lane = row m (lrow), register group
    // q = r / 4 holds columns 8q + 4*lhalf + r % 4 of the 32-column block.
    const T* bias = static_cast<const T*>(g.bias);
    constexpr int kRowPad = WN * 2 + 16;
    char* stage = smem + wave * (128 * kRowPad);
    constexpr int kChunks = WN / 8;                      // 16-byte chunks per row of the wave's sub-tile
    constexpr int kRowsPerPass = 64 / kChunks;
    constexpr int kPasses = 128 / kRowsPerPass;
    const int cc = lane % kChunks, rr = lane / kChunks;
    const int ldc = g.ldc ? g.ldc : g.N;                 // (a column slice of a wider C: its row stride)
    const bool rows_aligned = ldc % 8 == 0;
    // A wave whose 128 x WN sub-tile lies inside C stores it without per-row conditions (below).
    const bool interior = __builtin_amdgcn_readfirstlane(m0 + wm * 128 + 128 <= g.M && n0 + wn * WN + WN <= g.N);
    const int64_t first = (int64_t)(m0 + wm * 128 + rr) * ldc + (n0 + wn * WN + cc * 8);   // the lane's chunk of pass 0
    const int64_t step = (int64_t)kRowsPerPass * ldc;
    // Its residual chunks are asked for now: they come from memory (the tensor was written
    // several kernels ago), and a load in front of each store would be waited for pass by pass.
    // (The wide tile has registers for half of them, the kernel that runs two workgroups per compute
    // unit for a quarter; the rest is fetched block by block.)
    constexpr int kPB = kPasses / 4;                     // passes per 32-row block
    constexpr int kAheadBlocks = AHEAD;
    u32x4 rv[kAheadBlocks * kPB];
    if (interior && res) {
        const T* rp = res + first;
#pragma unroll
        for (int p = 0; p < kAheadBlocks * kPB; p++) {
            rv[p] = rows_aligned ? *reinterpret_cast<const u32x4*>(rp) : *reinterpret_cast<const u32x4_unaligned*>(rp);
            rp += step;
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // The bias of all the lane's columns, fetched before the first register group needs it (a
    // load inside each group would be waited for sixteen times); zero without a bias and for
    // columns past N.
    Pack4<T> bq[4 * NBF];
    static_for<4 * NBF>([&](auto jq_tag) {
        constexpr int jq = decltype(jq_tag)::value;
        bq[jq] = __builtin_bit_cast(Pack4<T>, u32x2{0u, 0u});
    });
    if (bias) {
        const int nw = n0 + wn * WN + 4 * lhalf;
        if (__builtin_amdgcn_readfirstlane(n0 + wn * WN + WN <= g.N)) {
            static_for<4 * NBF>([&](auto jq_tag) {
                constexpr int jq = decltype(jq_tag)::value;
                bq[jq] = __builtin_bit_cast(Pack4<T>, *reinterpret_cast<const u32x2*>(bias + nw + (jq >> 2) * 32 + 8 * (jq & 3)));
            });
        } else {
            static_for<4 * NBF>([&](auto jq_tag) {
                constexpr int jq = decltype(jq_tag)::value;
                const int n = nw + (jq >> 2) * 32 + 8 * (jq & 3);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < g.N) bq[jq].v[e] = bias[n + e];
            });
        }
    }
    // The sub-tile goes through LDS one 32-row block at a time.  For an interior sub-tile the
    // stores of a block are issued behind the conversion of the next one (its chunks were read
    // back from LDS in front of it), so the store traffic overlaps the arithmetic instead of
    // following it: same values, same addresses as the general loop below.
    T* cw = c + first;
    const T* rw = res + first;
    const char* sp = stage + rr * kRowPad + cc * 16;
    u32x4 w[kPB];
    auto store_block = [&](auto i_tag) __attribute__((always_inline)) {
        constexpr int i = decltype(i_tag)::value;
        if (res) {
#pragma unroll
            for (int u = 0; u < kPB; u++) {
                u32x4 r;
                if constexpr (i < kAheadBlocks) r = rv[i * kPB + u];
                else r = rows_aligned ? *reinterpret_cast<const u32x4*>(rw + (i * kPB + u) * step)
                                      : *reinterpret_cast<const u32x4_unaligned*>(rw + (i * kPB + u) * step);
                w[u] = add_chunk<T>(w[u], r);
            }
        }
#pragma unroll
        for (int u = 0; u < kPB; u++) {
            // (rows at any even byte when N is no multiple of 8: see below)
            if constexpr (STREAM_C) {
                if (rows_aligned) __builtin_nontemporal_store(w[u], reinterpret_cast<u32x4*>(cw));
                else __builtin_nontemporal_store(w[u], reinterpret_cast<u32x4_unaligned*>(cw));
            } else {
                if (rows_aligned) *reinterpret_cast<u32x4*>(cw) = w[u];
                else *reinterpret_cast<u32x4_unaligned*>(cw) = w[u];
            }
            cw += step;
        }
    };
    dispatch_act(g.act, [&](auto act_tag) {
    constexpr int ACT = decltype(act_tag)::value;
    static_for<4>([&](auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
        static_for<4 * NBF>([&](auto jq_tag) {
            constexpr int j = decltype(jq_tag)::value >> 2, q = decltype(jq_tag)::value & 3;
            const int nl = j * 32 + 8 * q + 4 * lhalf;
            Pack4<T> o;
            static_for<4>([&](auto e_tag) {
                constexpr int e = decltype(e_tag)::value;
                float v = acc_value(acc[i * NBF + j][4 * q + e]) + Elem<T>::to_f32(bq[j * 4 + q].v[e]);
                v = apply_act_c<ACT>(v);
                o.v[e] = Elem<T>::from_f32(v);
            });
            *reinterpret_cast<u32x2*>(stage + (i * 32 + lrow) * kRowPad + nl * 2) =
                __builtin_bit_cast(u32x2, o);
            // one register group at a time: do not let all the accumulator reads pile up
            __builtin_amdgcn_sched_barrier(0);
        });
        if (interior) {
            if constexpr (i > 0) store_block(std::integral_constant<int, i - 1>{});
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // a wave re-reads only its own rows
#pragma unroll
            for (int u = 0; u < kPB; u++)
                w[u] = *reinterpret_cast<const u32x4*>(sp + (i * kPB + u) * kRowsPerPass * kRowPad);
            __builtin_amdgcn_sched_barrier(0);
        }
    });
    });
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (interior) {
        store_block(std::integral_constant<int, 3>{});
    } else {
#pragma unroll 4
        for (int p = 0; p < 128 / kRowsPerPass; p++) {
            const int ml = p * kRowsPerPass + rr;
            const int m = m0 + wm * 128 + ml;
            const int n = n0 + wn * WN + cc * 8;
            if (m < g.M && n + 8 <= g.N) {
                u32x4 w = *reinterpret_cast<const u32x4*>(stage + ml * kRowPad + cc * 16);
                if (rows_aligned) {
                    if (res) w = add_chunk<T>(w, *reinterpret_cast<const u32x4*>(res + (int64_t)m * ldc + n));
                    *reinterpret_cast<u32x4*>(c + (int64_t)m * ldc + n) = w;
                } else {
                    // N is no multiple of 8: rows of C start at any even byte.  The device takes 16-byte
                    // accesses at such addresses (alignment is not enforced for global memory); the type
                    // says so, so the compiler assumes nothing more.
                    if (res) w = add_chunk<T>(w, *reinterpret_cast<const u32x4_unaligned*>(res + (int64_t)m * ldc + n));
                    *reinterpret_cast<u32x4_unaligned*>(c + (int64_t)m * ldc + n) = w;
                }
            } else if (m < g.M && n < g.N) {         // the last, partial chunk of a row
                const T* sv = reinterpret_cast<const T*>(stage + ml * kRowPad + cc * 16);
                for (int e = 0; e < g.N - n; e++) {
                    T val = sv[e];
                    if (res) val = Elem<T>::from_f32(Elem<T>::to_f32(val) + Elem<T>::to_f32(res[(int64_t)m * ldc + n + e]));
                    c[(int64_t)m * ldc + n + e] = val;
                }
            }
        }
    }
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
    const int64_t tiles = (int64_t)((g.M + 255) / 256) * ((g.N + bw - 1) / bw) * batch;
    return (tiles >= 192 || any_tile_count) && tiles <= 0x7FFFFFFF && batch <= 65535;
}

// The activations the 256x384 kernel's epilogue serves.
bool gemm384_activation_ok(int act) { return act == MHIP_ACT_NONE || act == MHIP_ACT_RELU || act == MHIP_ACT_GELU; }

// `bw` x `ring`: the member of the tile family (384 x 4, 256 x {4, 5}, 128 x {4, 5, 6}; anything else runs
// depth 5).
int launch_gemm256(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b,
                   int dtype, int bw, int ring) {
    if (bw == 384)
        return dtype == MHIP_BF16 ? layout384<bf16_t>(s, g, batch, trans_a, trans_b)
                                  : layout384<f16_t>(s, g, batch, trans_a, trans_b);
    if (bw == 128 && ring == 3)       // two workgroups per compute unit
        return dtype == MHIP_BF16 ? layout_pair<bf16_t>(s, g, batch, trans_a, trans_b)
                                  : layout_pair<f16_t>(s, g, batch, trans_a, trans_b);
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
