// Flash-attention forward for fp32 tensors on the fp32 matrix instruction
// (v_mfma_f32_32x32x2_f32): both products and the softmax in fp32, so the result keeps the
// 1e-5 bar of the scalar kernel it replaces for head sizes 32, 64, 96 and 128 (the reference's
// flagship kernel is fp32: Metal/Kernels/FlashAttentionKernel.swift:489-613).
//
// One workgroup = four waves = 128 query rows of one (batch, head); a wave owns 32 of them
// and walks blocks of 32 keys that the workgroup stages in LDS.  Scores are computed
// transposed, S^T = K . Q^T, so that a lane holds 16 keys of ONE query column per
// accumulator: the row statistics are per-lane loops plus one exchange between the two
// 32-lane halves, and the probabilities are already laid out as the B operand of the second
// product O^T += V^T . P^T (k-step i of that product pairs key 8 (i / 4) + 4 (lane / 32) + i % 4
// of the block with the lane's own register i), so P never moves between lanes.
#include <math.h>

#include "attention_common.h"

namespace mhip {
namespace {

typedef float f32x2 __attribute__((ext_vector_type(2)));
constexpr int kFBQ = 128;     // query rows per workgroup
constexpr int kFBK = 32;      // keys per block

// key (within a block) of accumulator register i in the 32-lane half h
__device__ __forceinline__ int f32_key(int i, int h) { return 8 * (i >> 2) + 4 * h + (i & 3); }

template <int D, bool CAUSAL, bool HAS_MASK>
__global__ __launch_bounds__(256, 2) void fa_f32_mfma_kernel(FaArgs a, float scale) {
    // K rows padded to D + 2 floats (lane = key reads fall on distinct banks), V rows to D + 8
    // (the two halves of a wave read rows four apart)
    constexpr int KS = D + 2, VS = D + 8;
    constexpr int NS = D / 2;            // k-steps of the first product
    constexpr int ND = D / 32;           // 32-column blocks of the output
    constexpr int F4 = kFBK * D / 4 / 256;   // 16-byte pieces of a K (or V) block per thread
    __shared__ __attribute__((aligned(16))) float ks[kFBK * KS];
    __shared__ __attribute__((aligned(16))) float vs[kFBK * VS];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ln = lane & 31, h = lane >> 5;
    int bh, qb;
    tile_of_workgroup<CAUSAL>(a, blockIdx.x, bh, qb);
    const int q0 = qb * kFBQ + wave * 32;
    const int qpos = q0 + ln;                       // this lane's query row
    const bool q_live = qpos < a.Sq;
    const float* qp = static_cast<const float*>(a.q) + (int64_t)bh * a.Sq * D;
    const float* kp = static_cast<const float*>(a.k) + (int64_t)bh * a.Skv * D;
    const float* vp = static_cast<const float*>(a.v) + (int64_t)bh * a.Skv * D;
    float* op = static_cast<float*>(a.o) + (int64_t)bh * a.Sq * D;
    const float* mp = HAS_MASK ? static_cast<const float*>(a.mask) + (int64_t)(bh / a.H) * a.mask_sb +
                                     (int64_t)(bh % a.H) * a.mask_sh + (int64_t)qpos * a.Skv
                               : nullptr;

    // Q^T fragments: k-step s holds Q[qpos][2 s + h]
    float qf[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) qf[s] = q_live ? qp[(int64_t)qpos * D + 2 * s + h] : 0.f;

    int nkv = (a.Skv + kFBK - 1) / kFBK;
    if (CAUSAL) {
        const int last_q = min(qb * kFBQ + kFBQ, a.Sq) - 1;
        nkv = min(nkv, last_q / kFBK + 1);
    }
    const int last_wave_q = min(q0 + 32, a.Sq) - 1;   // causal: blocks past it add nothing for this wave

    f32x16 o[ND];
#pragma unroll
    for (int d = 0; d < ND; d++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[d][i] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;            // l_run: this lane's 16 keys of every block

    // this thread's pieces of a block: piece p covers floats 4 p .. 4 p + 3 of the [32][D] block
    f32x4 kr[F4], vr[F4];
    auto fetch = [&](int blk) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < F4; j++) {
            const int p = j * 256 + tid, row = p / (D / 4), col = (p % (D / 4)) * 4;
            const int key = blk * kFBK + row;
            if (key < a.Skv) {
                kr[j] = *reinterpret_cast<const f32x4*>(kp + (int64_t)key * D + col);
                vr[j] = *reinterpret_cast<const f32x4*>(vp + (int64_t)key * D + col);
            } else {
                kr[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                vr[j] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
    };
    auto stage = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < F4; j++) {
            const int p = j * 256 + tid, row = p / (D / 4), col = (p % (D / 4)) * 4;
            float* kd = ks + row * KS + col;           // 8-byte aligned: two stores
            *reinterpret_cast<f32x2*>(kd) = f32x2{kr[j].x, kr[j].y};
            *reinterpret_cast<f32x2*>(kd + 2) = f32x2{kr[j].z, kr[j].w};
            *reinterpret_cast<f32x4*>(vs + row * VS + col) = vr[j];
        }
    };

    if (nkv > 0) fetch(0);
    for (int blk = 0; blk < nkv; blk++) {
        __syncthreads();                               // the previous block has been read by every wave
        stage();
        __syncthreads();
        if (blk + 1 < nkv) fetch(blk + 1);             // in flight while this block is worked on
        const int kb = blk * kFBK;
        if (CAUSAL && kb > last_wave_q) continue;      // (uniform within the wave; the barriers stay in step)

        // ---- S^T = K . Q^T
        f32x16 sacc;
#pragma unroll
        for (int i = 0; i < 16; i++) sacc[i] = 0.f;
#pragma unroll
        for (int s = 0; s < NS; s++)
            sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ks[ln * KS + 2 * s + h], qf[s], sacc, 0, 0, 0);

        // ---- scale, mask, block maximum (log2 domain)
        float t[16];
        float m_blk = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int key = kb + f32_key(i, h);
            float sv = sacc[i] * scale;
            bool keep = key < a.Skv && q_live;
            if (CAUSAL) keep = keep && key <= qpos;
            if (HAS_MASK) { if (keep) sv += mp[key]; }
            t[i] = keep ? sv * kLog2e : -INFINITY;
            m_blk = fmaxf(m_blk, t[i]);
        }
        m_blk = half_max(m_blk);
        // (a reference maximum that moves only when the block exceeds it by 2^8: see moved_reference)
        const float m_new = moved_reference(m_run, m_blk);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        // (v_exp_f32 itself, about 1 ulp: the library exp2f wraps it in five more instructions that
        // only serve results below 2^-126, which are zeros here either way)
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            t[i] = __builtin_amdgcn_exp2f(t[i] - m_use);
            psum += t[i];
        }
        l_run = l_run * alpha + psum;
        if (__any(alpha != 1.f)) {                     // rare once the reference has settled
#pragma unroll
            for (int d = 0; d < ND; d++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[d][i] *= alpha;
        }

        // ---- O^T += V^T . P^T
#pragma unroll
        for (int d = 0; d < ND; d++)
#pragma unroll
            for (int i = 0; i < 16; i++)
                o[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(vs[f32_key(i, h) * VS + 32 * d + ln], t[i], o[d], 0, 0, 0);
    }

    // ---- normalise and store: register group i / 4 of block d holds columns
    // 32 d + 8 (i / 4) + 4 h .. + 3 of row qpos
    const float l_tot = half_sum(l_run);
    const float inv = l_tot > 1e-10f ? 1.f / l_tot : 0.f;
    if (q_live) {
        float* orow = op + (int64_t)qpos * D;
#pragma unroll
        for (int d = 0; d < ND; d++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const f32x4 w = {o[d][4 * g] * inv, o[d][4 * g + 1] * inv, o[d][4 * g + 2] * inv, o[d][4 * g + 3] * inv};
                *reinterpret_cast<f32x4*>(orow + 32 * d + 8 * g + 4 * h) = w;
            }
    }
}

template <int D>
int launch_f32(hipStream_t s, FaArgs a, float scale, bool causal, bool has_mask) {
    a.nqb = (a.Sq + kFBQ - 1) / kFBQ;
    set_tile_order(a);
    const int64_t grid = (int64_t)a.B * a.H * a.nqb;
    if (grid > 0x7FFFFFFFLL) return fail(MHIP_ERR_UNSUPPORTED, "flash_attention: grid too large");
#define MHIP_FA32(C, M) \
    hipLaunchKernelGGL((fa_f32_mfma_kernel<D, C, M>), dim3((unsigned)grid), dim3(256), 0, s, a, scale)
    if (causal && has_mask) MHIP_FA32(true, true);
    else if (causal) MHIP_FA32(true, false);
    else if (has_mask) MHIP_FA32(false, true);
    else MHIP_FA32(false, false);
#undef MHIP_FA32
    return check_launch("flash_attention_f32");
}

}  // namespace

// fp32, packed [B,H,S,D], head size a multiple of 32 up to 128, 16-byte aligned tensors.
// MHIP_FA_F32_MFMA=2 keeps the scalar kernel.
bool fa_f32_mfma_eligible(const FaArgs& a, int64_t D) {
    if (tune_int("MHIP_FA_F32_MFMA", 1) == 2) return false;
    if (D % 32 != 0 || D > 128 || a.Skv < 1) return false;
    const uintptr_t all = reinterpret_cast<uintptr_t>(a.q) | reinterpret_cast<uintptr_t>(a.k) |
                          reinterpret_cast<uintptr_t>(a.v) | reinterpret_cast<uintptr_t>(a.o);
    return (all & 15) == 0;
}

int launch_fa_f32_mfma(hipStream_t s, const FaArgs& a, int64_t D, float scale) {
    const bool causal = a.is_causal != 0, has_mask = a.mask != nullptr;
    switch (D) {
        case 32: return launch_f32<32>(s, a, scale, causal, has_mask);
        case 64: return launch_f32<64>(s, a, scale, causal, has_mask);
        case 96: return launch_f32<96>(s, a, scale, causal, has_mask);
        default: return launch_f32<128>(s, a, scale, causal, has_mask);
    }
}

}  // namespace mhip
