// Shared by the four-wave LDS-ring GEMM kernels (gemm256.hip, gemm_twoset.hip): how an operand tile lies in
// LDS and which bytes of global memory each lane asks for, and the epilogue of a 256-row tile whose
// accumulators live in the accumulation registers.
#pragma once
#include <mutex>
#include <type_traits>
#include <utility>

#include "gemm_common.h"

namespace mhip {

typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));

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

}  // namespace
}  // namespace mhip
