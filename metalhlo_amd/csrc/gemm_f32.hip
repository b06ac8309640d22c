// fp32 GEMM on the matrix cores of gfx950: v_mfma_f32_32x32x2_f32 (fp32 operands, fp32
// accumulate -- the products are exact fp32 products, so the 1e-5 bar of fp32 programs holds).
//
// One workgroup = a 64x64 tile of C, four waves (2 x 2), one 32x32 accumulator each (or a
// 128x128 tile, 2 x 2 accumulators per wave).  K advances in steps of 16 through two LDS stage buffers: while a
// step is multiplied, the next step's operands travel global -> registers, and are written to
// the other buffer after the step (one barrier per step).  Both operands lie in LDS as
// [rows or columns][16 k] with rows padded to 20 floats, whatever their layout in memory:
// an operand whose k axis is contiguous in memory is copied with 16-byte accesses, the other
// one is transposed on the way in (16-byte global reads along m / n, scalar LDS writes).
//
// The instruction sums two k per issue: lanes 0..31 supply k = 0, lanes 32..63 k = 1.  Which
// two of the step's sixteen k a given issue takes is free as long as both operands agree, so
// issue p takes k = p (lower half) and k = 8 + p (upper half): a lane then needs eight
// CONSECUTIVE k of its row -- two 16-byte LDS reads per fragment and step.
//
// The product is issued as (B, A), so an accumulator comes out transposed: a lane holds one
// row m of the block and, per register group of four, four consecutive columns -- rows of C
// are written with 16-byte stores.
#include <type_traits>

#include "gemm_common.h"

namespace mhip {
namespace {

constexpr int kStep = 16;       // k per stage
constexpr int kPad = 20;        // floats per LDS row (16 + 4: rows stay 16-byte aligned, banks spread)
// Start of row r of a stage: 20 floats per row and four more after every sixteenth row.  The
// transposing store below has the lanes of a wave sixteen row groups apart in steps of four
// rows: 4 x 20 floats are 16 banks, so without the extra step lanes i and i + 4 (rows 16 apart
// = 320 floats = five times around the 64 banks) would land on the same bank, four deep.
__device__ __forceinline__ constexpr int lds_row(int r) { return r * kPad + 4 * (r >> 4); }
constexpr int lds_floats(int rows) { return rows * kPad + 4 * (rows / 16); }

// Copies this thread's share (NF = TILE / 16 floats) of one operand's [TILE x 16] stage into
// registers.  K_CONTIG: element (row, k) at p[row * ld + k]; otherwise at p[k * ld + row].
// Out-of-range rows / k read as zero.  `vec` = rows and k offsets are 16-byte aligned.
template <bool K_CONTIG, int NF>
__device__ inline void stage_load(const float* __restrict__ p, int ld, int row0, int rows, int k0, int K, bool vec, float (&r)[NF]) {
    const int t = threadIdx.x;
    constexpr int TPR = 16 / NF;           // threads per row of a k-contiguous stage
    if (K_CONTIG) {
        const int row = row0 + t / TPR, k = k0 + (t % TPR) * NF;
#pragma unroll
        for (int h = 0; h < NF / 4; h++) {
            const int kk = k + 4 * h;
            if (vec && row < rows && kk + 4 <= K) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(p + (int64_t)row * ld + kk);
                r[4 * h + 0] = v[0]; r[4 * h + 1] = v[1]; r[4 * h + 2] = v[2]; r[4 * h + 3] = v[3];
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) r[4 * h + e] = (row < rows && kk + e < K) ? p[(int64_t)row * ld + kk + e] : 0.f;
            }
        }
    } else {
        const int k = k0 + (t >> 4), row = row0 + (t & 15) * NF;
#pragma unroll
        for (int h = 0; h < NF / 4; h++) {
            const int rr = row + 4 * h;
            if (vec && k < K && rr + 4 <= rows) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(p + (int64_t)k * ld + rr);
                r[4 * h + 0] = v[0]; r[4 * h + 1] = v[1]; r[4 * h + 2] = v[2]; r[4 * h + 3] = v[3];
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) r[4 * h + e] = (k < K && rr + e < rows) ? p[(int64_t)k * ld + rr + e] : 0.f;
            }
        }
    }
}

template <bool K_CONTIG, int NF>
__device__ inline void stage_store(float* lds, const float (&r)[NF]) {
    const int t = threadIdx.x;
    constexpr int TPR = 16 / NF;
    if (K_CONTIG) {
        float* d = lds + lds_row(t / TPR) + (t % TPR) * NF;
#pragma unroll
        for (int h = 0; h < NF / 4; h++) *reinterpret_cast<f32x4*>(d + 4 * h) = f32x4{r[4 * h], r[4 * h + 1], r[4 * h + 2], r[4 * h + 3]};
    } else {
        const int k = t >> 4, row = (t & 15) * NF;
#pragma unroll
        for (int e = 0; e < NF; e++) lds[lds_row(row + e) + k] = r[e];
    }
}

// WB = 32x32 accumulator blocks per wave and side: tile = (64 WB) x (64 WB)
template <bool TA, bool TB, int WB>
__global__ __launch_bounds__(256, 2) void gemm_f32_mfma_kernel(GemmArgs g, int vec_a, int vec_b) {
    constexpr int kTile = 64 * WB, NF = kTile / 16;
    __shared__ __attribute__((aligned(16))) float lds[2][2][lds_floats(kTile)];   // [stage][A | B]
    int tm, tn;
    tile_of(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tm, tn);
    const int m0 = tm * kTile, n0 = tn * kTile;
    const int64_t batch = blockIdx.y;
    const float* a = static_cast<const float*>(g.a) + batch * g.sa;
    const float* b = static_cast<const float*>(g.b) + batch * g.sb;
    float* c = static_cast<float*>(g.c) + batch * g.sc;
    const float* res = g.residual ? static_cast<const float*>(g.residual) + batch * g.sc : nullptr;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, lhalf = lane >> 5;

    f32x16 acc[WB][WB];
#pragma unroll
    for (int i = 0; i < WB; i++)
#pragma unroll
        for (int j = 0; j < WB; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    float ra[NF], rb[NF];
    // A in memory: [M, K] (k contiguous) unless TA; B in memory: [K, N] (n contiguous) unless TB
    stage_load<!TA, NF>(a, g.lda, m0, g.M, 0, g.K, vec_a, ra);
    stage_load<TB, NF>(b, g.ldb, n0, g.N, 0, g.K, vec_b, rb);
    stage_store<!TA, NF>(lds[0][0], ra);
    stage_store<TB, NF>(lds[0][1], rb);
    __syncthreads();
    const int steps = (g.K + kStep - 1) / kStep;
    for (int t = 0; t < steps; t++) {
        const int cur = t & 1;
        if (t + 1 < steps) {
            stage_load<!TA, NF>(a, g.lda, m0, g.M, (t + 1) * kStep, g.K, vec_a, ra);
            stage_load<TB, NF>(b, g.ldb, n0, g.N, (t + 1) * kStep, g.K, vec_b, rb);
        }
        f32x4 fa[WB][2], fb[WB][2];
#pragma unroll
        for (int i = 0; i < WB; i++) {
            const float* pa = lds[cur][0] + lds_row(wm * 32 * WB + i * 32 + lrow) + lhalf * 8;
            const float* pb = lds[cur][1] + lds_row(wn * 32 * WB + i * 32 + lrow) + lhalf * 8;
            fa[i][0] = *reinterpret_cast<const f32x4*>(pa);
            fa[i][1] = *reinterpret_cast<const f32x4*>(pa + 4);
            fb[i][0] = *reinterpret_cast<const f32x4*>(pb);
            fb[i][1] = *reinterpret_cast<const f32x4*>(pb + 4);
        }
#pragma unroll
        for (int p = 0; p < 8; p++)
#pragma unroll
            for (int i = 0; i < WB; i++)
#pragma unroll
                for (int j = 0; j < WB; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j][p >> 2][p & 3], fa[i][p >> 2][p & 3], acc[i][j], 0, 0, 0);
        if (t + 1 < steps) {
            stage_store<!TA, NF>(lds[cur ^ 1][0], ra);
            stage_store<TB, NF>(lds[cur ^ 1][1], rb);
        }
        __syncthreads();
    }

    // lane = row m of the block; register 4q + e = column 8q + 4 * lhalf + e
    const float* bias = static_cast<const float*>(g.bias);
    const bool rows_vec = g.N % 4 == 0 && (reinterpret_cast<uintptr_t>(c) & 15) == 0 &&
                          (!res || (reinterpret_cast<uintptr_t>(res) & 15) == 0);
#pragma unroll
    for (int i = 0; i < WB; i++) {
        const int m = m0 + wm * 32 * WB + i * 32 + lrow;
#pragma unroll
        for (int j = 0; j < WB; j++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int n = n0 + wn * 32 * WB + j * 32 + 8 * q + 4 * lhalf;
                if (m >= g.M || n >= g.N) continue;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float x = acc[i][j][4 * q + e];
                    if (bias && n + e < g.N) x += bias[n + e];
                    if (g.act != MHIP_ACT_NONE) x = apply_act(x, g.act);
                    v[e] = x;
                }
                float* dst = c + (int64_t)m * g.N + n;
                if (rows_vec && n + 4 <= g.N) {
                    f32x4 o = {v[0], v[1], v[2], v[3]};
                    if (res) {
                        const f32x4 r = *reinterpret_cast<const f32x4*>(res + (int64_t)m * g.N + n);
                        o += r;
                    }
                    *reinterpret_cast<f32x4*>(dst) = o;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < g.N) dst[e] = res ? v[e] + res[(int64_t)m * g.N + n + e] : v[e];
                }
            }
    }
}

template <bool TA, bool TB, int WB>
int launch_tile(hipStream_t s, GemmArgs g, int64_t batch) {
    constexpr int kTile = 64 * WB;
    g.tiles_m = (g.M + kTile - 1) / kTile;
    g.tiles_n = (g.N + kTile - 1) / kTile;
    const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
    if (tiles > 0x7FFFFFFFLL || batch > 65535) return fail(MHIP_ERR_UNSUPPORTED, "gemm: grid too large");
    auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const int vec_a = al(g.a) && g.lda % 4 == 0 && g.sa % 4 == 0;
    const int vec_b = al(g.b) && g.ldb % 4 == 0 && g.sb % 4 == 0;
    hipLaunchKernelGGL((gemm_f32_mfma_kernel<TA, TB, WB>), dim3((unsigned)tiles, (unsigned)batch), dim3(256), 0, s, g, vec_a, vec_b);
    return check_launch("gemm_f32_mfma");
}

// 128x128 tiles (three workgroups resident per CU: 768 on the device) once there are enough of
// them for a round and a quarter, 64x64 tiles (eight per CU) below that.  Measured (TFLOP/s,
// 64 | 128): 4096^3 101 | 116, [8192,3072] x K 768 (1536 large tiles) 100 | 113; [3000,3000] x K 1000
// (576) 89 | 73, [2048,2048] x K 2048 (256) 99 | 91, [8192,768] x K 3072 (384) 100 | 87, 1024^3 (64)
// 62 | 23.
template <bool TA, bool TB>
int launch(hipStream_t s, const GemmArgs& g, int64_t batch) {
    const int64_t large_tiles = (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128) * batch;
    if (large_tiles >= 960) return launch_tile<TA, TB, 2>(s, g, batch);
    return launch_tile<TA, TB, 1>(s, g, batch);
}

}  // namespace

// fp32 problems with enough work for a 64x64 tile to pay (smaller ones keep the plain kernel:
// it wastes nothing on a 20x24 product).  MHIP_GEMM_F32_MFMA = 2 turns the kernel off, = 3
// takes it for every fp32 problem.
bool gemm_f32_mfma_wanted(const GemmArgs& g) {
    const int mode = tune_int("MHIP_GEMM_F32_MFMA", 1);
    if (mode == 2 || g.K < 1) return false;
    return mode == 3 || ((int64_t)g.M * g.N >= 48 * 48 && g.K >= 16);
}

int launch_gemm_f32_mfma(hipStream_t s, const GemmArgs& g, int64_t batch, int trans_a, int trans_b) {
    if (!trans_a && !trans_b) return launch<false, false>(s, g, batch);
    if (!trans_a && trans_b) return launch<false, true>(s, g, batch);
    if (trans_a && !trans_b) return launch<true, false>(s, g, batch);
    return launch<true, true>(s, g, batch);
}

}  // namespace mhip
