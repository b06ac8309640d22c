// Flash-attention forward for gfx950: O = softmax(scale * Q K^T + mask, causal) V.
//
// MFMA path (16-bit types, D in {64, 128}).  A workgroup of four waves owns 128
// query rows of one (batch, head); each wave owns 32 of them.  Keys/values are
// walked in blocks of 64, staged in LDS and double-buffered.
//
// The scores are computed TRANSPOSED, S^T = K . Q^T, with v_mfma_f32_32x32x16:
// in the accumulator layout every lane then holds 16 keys of ONE query column,
// so the online-softmax row statistics are plain per-lane loops plus a single
// exchange between the two 32-lane halves, and the probabilities can be fed
// straight back as the B operand of O^T += V^T . P^T without any cross-lane
// movement.  V is transposed (and its keys put in the order that B operand
// needs) in registers on the way into LDS.  Softmax state and both
// accumulations are fp32; the output is rounded once.
//
// Everything else (fp32, other head sizes) takes a wave-per-query scalar path.
#include "attention_common.h"

namespace mhip {

// NB: depth of the K and of the V ring in LDS.  Two everywhere: with head size 64 a ring of three or
// four measured 8 to 13 % slower (B8 H12 S1024: 38.5 / 40.5 against 35.7 us) -- it costs the third
// resident workgroup per CU, which hides more latency than the deeper prefetch does.

template <typename T, int D, bool CAUSAL, bool HAS_MASK, int NB>
__global__ __launch_bounds__(256, 2) void fa_fwd_kernel(FaArgs a) {
    constexpr int CPR = D / 8;                  // 16-byte chunks per row
    constexpr int kTile = kBKV * D * 2;         // bytes of one K (or V) tile
    constexpr int kRowsPerInst = 64 / CPR;      // tile rows one wave-wide LDS-DMA load fills
    constexpr int kInst = kBKV / kRowsPerInst / 4;   // such loads per wave per tile
    constexpr int ND = D / 32, NS = D / 16;
    constexpr int kLoadsPerTile = 2 * kInst;    // per wave
    __shared__ __attribute__((aligned(1024))) char smem[2 * NB * kTile];   // K ring, then V ring

    // ---- which (batch*head, query block): see tile_of_workgroup
    int bh, qb;
    tile_of_workgroup<CAUSAL>(a, blockIdx.x, bh, qb);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lrow = lane & 31, lhalf = lane >> 5;
    const int qblk0 = qb * kBQ;
    const int qw = qblk0 + wave * 32;          // first query row of this wave
    const int qpos = qw + lrow;

    const int b_i = bh / a.H, h_i = bh % a.H;
    const T* qp = static_cast<const T*>(a.q) + b_i * a.qs[0] + h_i * a.qs[1];
    const T* kp = static_cast<const T*>(a.k) + b_i * a.ks[0] + h_i * a.ks[1];
    const T* vp = static_cast<const T*>(a.v) + b_i * a.vs[0] + h_i * a.vs[1];
    T* op = static_cast<T*>(a.o) + b_i * a.os[0] + h_i * a.os[1];
    const int q_rs = (int)a.qs[2], k_rs = (int)a.ks[2], v_rs = (int)a.vs[2];      // row pitches in elements
    const __amdgpu_buffer_rsrc_t rq = fa_rsrc(qp, (uint32_t)((((int64_t)a.Sq - 1) * q_rs + D) * 2));
    const __amdgpu_buffer_rsrc_t rk = fa_rsrc(kp, (uint32_t)((((int64_t)a.Skv - 1) * k_rs + D) * 2));
    const __amdgpu_buffer_rsrc_t rv = fa_rsrc(vp, (uint32_t)((((int64_t)a.Skv - 1) * v_rs + D) * 2));

    // ---- Q^T operand: lane = query column, 8 consecutive d per k-step ------
    u32x4 qf[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const uint32_t off = qpos < a.Sq ? (uint32_t)((qpos * q_rs + 16 * s + 8 * lhalf) * 2) : kOobA;
        qf[s] = __builtin_amdgcn_raw_buffer_load_b128(rq, off, 0, 0);
        if (a.negate_q) {
            qf[s].x ^= 0x80008000u; qf[s].y ^= 0x80008000u;
            qf[s].z ^= 0x80008000u; qf[s].w ^= 0x80008000u;
        }
    }

    int nkv = (a.Skv + kBKV - 1) / kBKV;
    if (CAUSAL) {
        const int last_q = min(qblk0 + kBQ, a.Sq) - 1;
        nkv = min(nkv, last_q / kBKV + 1);
    }

    // ---- global -> LDS without a register stop: every wave-wide load fills 1 KB
    // of a tile (lane l lands at byte 16*l of that KB); the swizzle is applied by
    // choosing which global chunk each lane fetches.  Keys past the end read 0.
    const int ld_row = lane / CPR, ld_pos = lane % CPR;
    // (a block past the last one this workgroup needs is loaded all the same: the waits below
    // count loads, so every step issues the same number.)  Each lane's offsets inside block 0
    // are computed once; a step adds the block's offset.  Keys past the end need no test: their
    // offsets lie beyond the extent of the buffer descriptors above, and such loads put zeros
    // into LDS (V rows of zeros, so that a probability of zero times them stays zero).
    // (The swizzles repeat every sixteen rows and a wave's loads of a tile are 4 * kRowsPerInst
    // = 16 or 32 rows apart, so load i differs from load 0 by a constant.)
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const int ld_row0 = wave_s * kRowsPerInst + ld_row;
    const uint32_t koff0 = (uint32_t)((ld_row0 * k_rs + ((ld_pos ^ k_swz<D>(ld_row0)) << 3)) * 2);
    const uint32_t voff0 = (uint32_t)((ld_row0 * v_rs + ((ld_pos ^ v_swz<D>(ld_row0)) << 3)) * 2);
    auto load_tile = [&](int kv0, int buf) {
#pragma unroll
        for (int i = 0; i < kInst; i++) {
            const int blk = i * 4 + wave_s;               // which KB of the tile
            const int row = kv0 + i * 4 * kRowsPerInst;   // (scalar)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (fa_lds_void*)(smem + buf * kTile + blk * 1024), 16,
                                                     koff0 + (uint32_t)(row * k_rs * 2), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (fa_lds_void*)(smem + (NB + buf) * kTile + blk * 1024), 16,
                                                     voff0 + (uint32_t)(row * v_rs * 2), 0, 0, 0);
        }
    };
    // loads land in program order: the next block has landed when only the NB - 2 blocks issued
    // behind it are still in flight
    auto tiles_ready = [&]() {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NB - 2) * kLoadsPerTile) : "memory");
        __builtin_amdgcn_s_barrier();
    };

    // V^T fragment addresses: lane i of a 16-lane group supplies key row i/4 and
    // d columns 4*(i%4)..+3 of its group's 16-column block.
    const int ti = lane & 15, tg = lane >> 4;
    const int v_row0 = 4 * (tg >> 1) + (ti >> 2);                   // + 16u (+ 8)
    const int v_d0 = 16 * (tg & 1) + 4 * (ti & 3);                  // + 32 dt

    f32x16 oacc[ND];
#pragma unroll
    for (int i = 0; i < ND; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[i][r] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;   // reference maximum in the log2 domain (see moved_reference), running sum

#pragma unroll
    for (int p = 0; p < NB - 1; p++) load_tile(p * kBKV, p);
    tiles_ready();

    for (int it = 0; it < nkv; it++) {
        const int cur = it % NB, kv0 = it * kBKV;
        load_tile(kv0 + (NB - 1) * kBKV, (it + NB - 1) % NB);

        const bool wave_active = !CAUSAL || kv0 <= qw + 31;
        if (wave_active) {
            const char* kt = smem + cur * kTile;
            const char* vt = smem + (NB + cur) * kTile;
            // ---- S^T = K . Q^T ---------------------------------------------
            f32x16 sacc[2];
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) sacc[t][r] = 0.f;
            // two workgroups share a SIMD: let a wave in a matrix phase issue ahead of
            // the other wave's softmax arithmetic
            __builtin_amdgcn_s_setprio(2);
#pragma unroll
            for (int s = 0; s < NS; s++) {
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const u32x4 kf = *reinterpret_cast<const u32x4*>(kt + k_off<D>(32 * t + lrow, 2 * s + lhalf));
                    sacc[t] = Mfma32A<T>::run(kf, qf[s], sacc[t]);
                }
            }
            __builtin_amdgcn_s_setprio(0);
            float sv[32];
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) sv[t * 16 + r] = sacc[t][r];
            // Register i of the pair (t = i/16, r = i%16) is key
            // kv0 + 32t + 8(r/4) + 4*lhalf + r%4 of query column qpos.
            const bool boundary = (CAUSAL && kv0 + kBKV - 1 > qw) || kv0 + kBKV > a.Skv;
            float m_new;
            if (HAS_MASK || boundary) {
                // general form: scores to the log2 domain first, then mask
#pragma unroll
                for (int i = 0; i < 32; i++) sv[i] *= a.c;
                if (HAS_MASK) {
                    const T* mp = static_cast<const T*>(a.mask) + (int64_t)(bh / a.H) * a.mask_sb +
                                  (int64_t)(bh % a.H) * a.mask_sh;
#pragma unroll
                    for (int i = 0; i < 32; i++) {
                        const int key = kv0 + 32 * (i >> 4) + 8 * ((i & 15) >> 2) + 4 * lhalf + (i & 3);
                        if (qpos < a.Sq && key < a.Skv)
                            sv[i] += Elem<T>::to_f32(mp[(int64_t)qpos * a.Skv + key]) * kLog2e;
                    }
                }
                if (boundary) {
#pragma unroll
                    for (int i = 0; i < 32; i++) {
                        const int key = kv0 + 32 * (i >> 4) + 8 * ((i & 15) >> 2) + 4 * lhalf + (i & 3);
                        if ((CAUSAL && key > qpos) || key >= a.Skv) sv[i] = -INFINITY;
                    }
                }
                float mloc = sv[0];
#pragma unroll
                for (int i = 1; i < 32; i++) mloc = fmaxf(mloc, sv[i]);
                mloc = half_max(mloc);
                m_new = moved_reference(m_run, mloc);
                const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
#pragma unroll
                for (int i = 0; i < 32; i++) sv[i] = __builtin_amdgcn_exp2f(sv[i] - m_use);
            } else {
                // interior block: max over raw scores (the scale is positive), and
                // scale + shift folded into one fma in front of the exp2
                float mloc = sv[0];
#pragma unroll
                for (int i = 1; i < 32; i++) mloc = fmaxf(mloc, sv[i]);
                mloc = half_max(mloc);
                m_new = moved_reference(m_run, mloc * a.c);
                const float neg_m = -m_new;     // finite: an interior block has no masked score
#pragma unroll
                for (int i = 0; i < 32; i++) sv[i] = __builtin_amdgcn_exp2f(fmaf(sv[i], a.c, neg_m));
            }
            const float m_use2 = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_use2);
            m_run = m_new;
            float lsum = 0.f;
#pragma unroll
            for (int i = 0; i < 32; i++) lsum += sv[i];
            l_run = l_run * alpha + lsum;
            // the accumulator only needs rescaling when some row's maximum moved
            if (__any(alpha != 1.f)) {
#pragma unroll
                for (int i = 0; i < ND; i++)
#pragma unroll
                    for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;
            }
            // ---- P^T as B operand: slot j of step u is register 8u + j ------
            u32x4 pb[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                pb[u].x = Mfma32A<T>::pack2(sv[8 * u + 0], sv[8 * u + 1]);
                pb[u].y = Mfma32A<T>::pack2(sv[8 * u + 2], sv[8 * u + 3]);
                pb[u].z = Mfma32A<T>::pack2(sv[8 * u + 4], sv[8 * u + 5]);
                pb[u].w = Mfma32A<T>::pack2(sv[8 * u + 6], sv[8 * u + 7]);
            }
            __builtin_amdgcn_s_setprio(2);
            // ---- O^T += V^T . P^T: A operand slot j of step u is key
            // 16u + 8(j/4) + 4*lhalf + j%4, i.e. two transposing reads 8 keys apart
#pragma unroll
            for (int u = 0; u < 4; u++) {
#pragma unroll
                for (int dt = 0; dt < ND; dt++) {
                    const int row = 16 * u + v_row0;
                    const int d0 = 32 * dt + v_d0;
                    const char* p0 = vt + v_off<D>(row, d0 >> 3) + (d0 & 7) * 2;
                    const char* p1 = vt + v_off<D>(row + 8, d0 >> 3) + (d0 & 7) * 2;
                    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((fa_lds_s16x4*)p0));
                    const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((fa_lds_s16x4*)p1));
                    u32x4 vf;
                    vf.x = lo.x; vf.y = lo.y; vf.z = hi.x; vf.w = hi.y;
                    oacc[dt] = Mfma32A<T>::run(vf, pb[u], oacc[dt]);
                }
            }
            __builtin_amdgcn_s_setprio(0);
        }
        if (it + 1 < nkv) tiles_ready();
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // nothing may land in LDS after the workgroup ends

    // ---- normalise and store: lane holds 4 consecutive d per register group -
    const float l_tot = half_sum(l_run);
    const float inv = l_tot > 1e-10f ? 1.f / l_tot : 0.f;
    if (qpos < a.Sq) {
        T* orow = op + (int64_t)qpos * a.os[2];
#pragma unroll
        for (int dt = 0; dt < ND; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                u32x2 w;
                w.x = Mfma32A<T>::pack2(oacc[dt][4 * g + 0] * inv, oacc[dt][4 * g + 1] * inv);
                w.y = Mfma32A<T>::pack2(oacc[dt][4 * g + 2] * inv, oacc[dt][4 * g + 3] * inv);
                *reinterpret_cast<u32x2*>(orow + 32 * dt + 8 * g + 4 * lhalf) = w;
            }
    }
}

// ---------------------------------------------------------------------------
// Scalar path: one wave per query row, any type, D <= 256.
// Per block of 64 keys: lanes own keys for the scores, then own head-dim
// columns for the weighted sum.  The recurrence is the reference's
// (FlashAttentionKernel.swift:589-598) applied per block of keys.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void fa_scalar_kernel(FaArgs a, int D, float scale) {
    __shared__ float qs[4][256];
    __shared__ float ps[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;      // over B*H*Sq
    const int64_t nrows = (int64_t)a.B * a.H * a.Sq;
    const bool live = row < nrows;
    const int64_t bh = live ? row / a.Sq : 0;
    const int qpos = live ? (int)(row % a.Sq) : 0;
    const T* qp = static_cast<const T*>(a.q) + (bh * a.Sq + qpos) * D;
    const T* kp = static_cast<const T*>(a.k) + bh * a.Skv * D;
    const T* vp = static_cast<const T*>(a.v) + bh * a.Skv * D;
    const T* mp = a.mask ? static_cast<const T*>(a.mask) + (bh / a.H) * a.mask_sb +
                               (bh % a.H) * a.mask_sh + (int64_t)qpos * a.Skv
                         : nullptr;
    for (int d = lane; d < D; d += 64) qs[wave][d] = live ? Elem<T>::to_f32(qp[d]) : 0.f;
    __syncthreads();
    float oacc[4] = {0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    const int kv_end = live ? (a.is_causal ? min(a.Skv, qpos + 1) : a.Skv) : 0;
    for (int kv0 = 0; kv0 < kv_end; kv0 += 64) {
        const int key = kv0 + lane;
        float s = -INFINITY;
        if (key < kv_end) {
            float acc = 0.f;
            const T* kr = kp + (int64_t)key * D;
            for (int d = 0; d < D; d++) acc = fmaf(qs[wave][d], Elem<T>::to_f32(kr[d]), acc);
            s = acc * scale;
            if (mp) s += Elem<T>::to_f32(mp[key]);
        }
        const float m_new = fmaxf(m_run, wave_max(s));
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = expf(m_run - m_use);
        const float p = expf(s - m_use);
        m_run = m_new;
        l_run = l_run * alpha + wave_sum(p);
        ps[wave][lane] = p;
        __builtin_amdgcn_wave_barrier();
        const int nk = min(64, kv_end - kv0);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int d = lane + 64 * j;
            if (d < D) {
                float acc = oacc[j] * alpha;
                for (int t = 0; t < nk; t++)
                    acc = fmaf(ps[wave][t], Elem<T>::to_f32(vp[(int64_t)(kv0 + t) * D + d]), acc);
                oacc[j] = acc;
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
    if (live) {
        const float inv = l_run > 1e-10f ? 1.f / l_run : 0.f;
        T* orow = static_cast<T*>(a.o) + (bh * a.Sq + qpos) * D;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int d = lane + 64 * j;
            if (d < D) orow[d] = Elem<T>::from_f32(oacc[j] * inv);
        }
    }
}

template <typename T, int D>
static int launch_fa(hipStream_t s, FaArgs a, bool causal, bool has_mask) {
    a.nqb = (a.Sq + kBQ - 1) / kBQ;
    const int64_t bh = (int64_t)a.B * a.H;
    set_tile_order(a);
    const int64_t grid = bh * a.nqb;
    if (grid > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "flash_attention: grid too large");
    constexpr int NB = 2;
#define MHIP_FA(C, M)                                                                       \
    hipLaunchKernelGGL((fa_fwd_kernel<T, D, C, M, NB>), dim3((unsigned)grid), dim3(256), 0, s, a)
    if (causal && has_mask) MHIP_FA(true, true);
    else if (causal) MHIP_FA(true, false);
    else if (has_mask) MHIP_FA(false, true);
    else MHIP_FA(false, false);
#undef MHIP_FA
    return check_launch("flash_attention");
}

template <typename T>
static int launch_fa_scalar(hipStream_t s, FaArgs a, int D, float scale) {
    const int64_t rows = (int64_t)a.B * a.H * a.Sq;
    const int64_t grid = (rows + 3) / 4;
    if (grid > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "flash_attention: grid too large");
    hipLaunchKernelGGL((fa_scalar_kernel<T>), dim3((unsigned)grid), dim3(256), 0, s, a, D, scale);
    return check_launch("flash_attention_scalar");
}

}  // namespace mhip

namespace mhip {
// attention_pipe.hip: head size 128, four waves x 64 query rows, matrix / softmax overlap in one wave.
bool fa_pipe_eligible(const FaArgs& a, int64_t D, int dtype, bool has_mask, int variant);
int launch_fa_pipe(hipStream_t s, const FaArgs& a, int dtype, bool causal, int pair);
// attention_f32.hip: fp32 tensors on the fp32 matrix instruction.
bool fa_f32_mfma_eligible(const FaArgs& a, int64_t D);
int launch_fa_f32_mfma(hipStream_t s, const FaArgs& a, int64_t D, float scale);
}  // namespace mhip

using namespace mhip;

// `strides`: NULL (packed [B,H,S,D]) or twelve element strides {batch, head, row} x {q, k, v, o}.
static int fa_entry(const char* name, void* stream, const void* q, const void* k, const void* v, const void* mask, void* o,
                    int64_t B, int64_t H, int64_t Sq, int64_t Skv, int64_t D, float scale, int is_causal,
                    int64_t mask_stride_b, int64_t mask_stride_h, int dtype, const int64_t* strides) {
    if (B < 0 || H < 0 || Sq < 0 || Skv < 0 || D <= 0)
        return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: bad size", name);
    if (D > 256) return fail(MHIP_ERR_UNSUPPORTED, "%s: head_dim %lld > 256", name, (long long)D);
    if (B == 0 || H == 0 || Sq == 0) return MHIP_OK;
    if (!q || !o || (Skv > 0 && (!k || !v)))
        return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", name);
    if (Sq > 0x7FFFFFFF || Skv > 0x7FFFFFFF || B * H > 0x7FFFFFFF)
        return fail(MHIP_ERR_UNSUPPORTED, "%s: dimension exceeds 2^31-1", name);
    hipStream_t s = as_stream(stream);
    FaArgs a;
    a.q = q; a.k = k; a.v = v; a.mask = mask; a.o = o;
    a.B = (int)B; a.H = (int)H; a.Sq = (int)Sq; a.Skv = (int)Skv;
    a.c = fabsf(scale) * kLog2e;
    a.negate_q = scale < 0.f;
    a.is_causal = is_causal ? 1 : 0;
    a.mask_sb = mask_stride_b; a.mask_sh = mask_stride_h;
    a.nqb = 0; a.xcd_map = 0; a.pair_tiles = 0; a.cu_group = 1;
    const int64_t packed[12] = {H * Sq * D, Sq * D, D, H * Skv * D, Skv * D, D, H * Skv * D, Skv * D, D, H * Sq * D, Sq * D, D};
    bool is_packed = true;
    int64_t max_row = D, max_span = 0;
    for (int i = 0; i < 12; i++) {
        const int64_t st = strides ? strides[i] : packed[i];
        if (st < 0) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: negative stride", name);
        (i < 3 ? a.qs : i < 6 ? a.ks : i < 9 ? a.vs : a.os)[i % 3] = st;
        is_packed = is_packed && st == packed[i];
    }
    const int64_t* rows[4] = {a.qs, a.ks, a.vs, a.os};
    bool strides_aligned = true;
    for (int t = 0; t < 4; t++) {
        if (rows[t][2] < D) return fail(MHIP_ERR_INVALID_ARGUMENT, "%s: row stride smaller than head_dim", name);
        strides_aligned = strides_aligned && rows[t][0] % 8 == 0 && rows[t][1] % 8 == 0 && rows[t][2] % 8 == 0;
        max_row = rows[t][2] > max_row ? rows[t][2] : max_row;
        const int64_t n = (t == 0 || t == 3) ? Sq : Skv;
        const int64_t span = (n > 0 ? (n - 1) * rows[t][2] : 0) + D;
        max_span = span > max_span ? span : max_span;
    }
    const bool is16 = dtype == MHIP_BF16 || dtype == MHIP_F16;
    const bool aligned = ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) |
                           reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(o)) & 15) == 0;
    const bool fits = max_span * 2 < 0x7FFFFFFFLL;
    if (is16 && aligned && strides_aligned && fits && Skv > 0 && (D == 64 || D == 128)) {
        const bool hm = mask != nullptr;
        // 0 = no tuned choice; 1 = 128-row kernel; 2 / 3 = 256-row pipelined kernel, causal tiles unpaired / paired
        const int variant = is_packed ? tuned_attention_variant(dtype, B * H, Sq, Skv, D, is_causal != 0) : 0;
        if (is_packed && fa_pipe_eligible(a, D, dtype, hm, variant))
            return launch_fa_pipe(s, a, dtype, is_causal != 0, variant == 2 ? 0 : variant == 3 ? 1 : -1);
        if (dtype == MHIP_BF16)
            return D == 128 ? launch_fa<bf16_t, 128>(s, a, is_causal, hm)
                            : launch_fa<bf16_t, 64>(s, a, is_causal, hm);
        return D == 128 ? launch_fa<f16_t, 128>(s, a, is_causal, hm)
                        : launch_fa<f16_t, 64>(s, a, is_causal, hm);
    }
    if (!is_packed)
        return fail(MHIP_ERR_UNSUPPORTED, "%s: strided layouts need bf16 / f16, head_dim 64 or 128, 16-byte aligned pointers and "
                                          "strides that are multiples of 8 elements", name);
    switch (dtype) {
        case MHIP_F32:
            if (fa_f32_mfma_eligible(a, D)) return launch_fa_f32_mfma(s, a, D, scale);
            return launch_fa_scalar<float>(s, a, (int)D, scale);
        case MHIP_BF16: return launch_fa_scalar<bf16_t>(s, a, (int)D, scale);
        case MHIP_F16: return launch_fa_scalar<f16_t>(s, a, (int)D, scale);
        default: return fail(MHIP_ERR_UNSUPPORTED, "%s: dtype %d", name, dtype);
    }
}

extern "C" int mhip_flash_attention(void* stream, const void* q, const void* k, const void* v,
                                    const void* mask, void* o, int64_t B, int64_t H, int64_t Sq,
                                    int64_t Skv, int64_t D, float scale, int is_causal,
                                    int64_t mask_stride_b, int64_t mask_stride_h, int dtype) {
    return fa_entry("mhip_flash_attention", stream, q, k, v, mask, o, B, H, Sq, Skv, D, scale, is_causal, mask_stride_b,
                    mask_stride_h, dtype, nullptr);
}

extern "C" int mhip_flash_attention_strided(void* stream, const void* q, const void* k, const void* v,
                                            const void* mask, void* o, int64_t B, int64_t H, int64_t Sq,
                                            int64_t Skv, int64_t D, float scale, int is_causal,
                                            int64_t mask_stride_b, int64_t mask_stride_h, int dtype,
                                            const int64_t* strides) {
    return fa_entry("mhip_flash_attention_strided", stream, q, k, v, mask, o, B, H, Sq, Skv, D, scale, is_causal,
                    mask_stride_b, mask_stride_h, dtype, strides);
}
