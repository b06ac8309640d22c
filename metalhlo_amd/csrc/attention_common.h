// Definitions shared by the flash-attention kernels.
#pragma once
#include <math.h>

#include "common.h"

namespace mhip {

constexpr uint32_t kOobA = 0x80000000u;
constexpr int kBQ = 128;   // query rows per workgroup (two-workgroups-per-CU kernel)
constexpr int kBKV = 64;   // keys per LDS stage
constexpr float kLog2e = 1.4426950408889634f;

struct FaArgs {
    const void* q;
    const void* k;
    const void* v;
    const void* mask;
    void* o;
    int B, H, Sq, Skv;
    float c;          // |scale| * log2(e)
    int negate_q;     // scale < 0: flip the sign of Q instead
    int is_causal;    // read by the scalar path (the MFMA path is templated on it)
    int64_t mask_sb, mask_sh;
    int nqb;          // query blocks per (batch, head)
    int xcd_map;      // (batch*head) % 8 == 0: the XCD-aware block order, 1 = an XCD takes a contiguous eighth of the heads, 2 = every eighth head
    int pair_tiles;   // pipelined kernel, causal: a workgroup takes two query tiles (first + last, ...)
    int cu_group;     // 128-row kernel: CUs a run of consecutive workgroup ids is dealt over (per XCD, or all)
    // Element strides {batch, head, row} of q, k, v, o (the last axis is contiguous).  Only
    // fa_fwd_kernel reads them; every other kernel is given the packed [B,H,S,D] layout.
    int64_t qs[3], ks[3], vs[3], os[3];
};

// Which (batch * head, query tile) a workgroup of the one-tile-per-workgroup kernels takes.
// Workgroup ids go round-robin over the 8 XCDs and, inside an XCD, round-robin over its CUs
// (measured: with three workgroups resident per CU, a CU holds XCD-local indices c, c + 32,
// c + 64).  A causal tile's work grows with its position, so the order decides the balance:
// walking one head's tiles after the other puts the SAME tile position of three heads on a CU
// (a tile count of 8 divides 32) -- three longest tiles here, three shortest there, and the
// launch takes as long as the non-causal one.  Instead: all tiles of the XCD sorted longest
// first and dealt to the CUs in rounds of cu_group, every other round in reverse (a snake
// draft), which balances the resident set and is the longest-first rule for what is
// dispatched later (B8 H12 S1024 D64 causal: 35.4 -> 23.7 us).
// An XCD takes a contiguous eighth of the (batch, head) pairs: with the fused projection of a
// transformer layer in front ([B*S, 3*H*D], whose row tiles a GEMM writes XCD by XCD in eighths
// of the rows) and the output projection behind, a batch's heads then read what its own XCD's
// L2 may still hold and leave their output where the next GEMM looks for it.
template <bool CAUSAL>
__device__ inline void tile_of_workgroup(const FaArgs& a, int id, int& bh, int& qb) {
    const int groups = a.xcd_map ? 8 : 1;
    const int xcd = a.xcd_map ? (id & 7) : 0, local = a.xcd_map ? (id >> 3) : id;
    const int heads = (a.B * a.H) / groups;          // heads of this XCD
    if (CAUSAL) {
        const int total = heads * a.nqb;
        const int round = local / a.cu_group, c = local % a.cu_group;
        const int in_round = min(a.cu_group, total - round * a.cu_group);
        const int e = round * a.cu_group + ((round & 1) ? in_round - 1 - c : c);   // place in the longest-first list
        qb = a.nqb - 1 - e / heads;
        bh = a.xcd_map == 2 ? (e % heads) * groups + xcd : xcd * heads + e % heads;
    } else {
        bh = a.xcd_map == 2 ? (local / a.nqb) * groups + xcd : xcd * heads + local / a.nqb;
        qb = local % a.nqb;
    }
}

// host side: a.nqb set; fills xcd_map and cu_group
inline void set_tile_order(FaArgs& a) {
    // (an XCD takes a contiguous eighth of the (batch, head) pairs)
    a.xcd_map = (((int64_t)a.B * a.H) % 8 == 0) ? 1 : 0;
    a.cu_group = a.xcd_map ? compute_units() / 8 : compute_units();
    if (a.cu_group < 1) a.cu_group = 1;
}

template <typename T> struct Mfma32A;
template <> struct Mfma32A<bf16_t> {
    __device__ static f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    __device__ static uint32_t pack2(float lo, float hi) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        bf16x2 t = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, t);
    }
};
template <> struct Mfma32A<f16_t> {
    __device__ static f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    __device__ static uint32_t pack2(float lo, float hi) {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        f16x2 t = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, t);
    }
};

__device__ inline __amdgpu_buffer_rsrc_t fa_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// The softmax keeps a REFERENCE maximum per row (log2 domain) that moves only when a block's
// maximum exceeds it by more than 8: probabilities are exp2(s - ref) <= 2^8, accumulated in fp32,
// and the final division uses the sum taken with the same reference, so the result is the same
// function.  What it saves is the rescaling of the output accumulators, which a strict running
// maximum triggers in nearly every block when 32 rows share a wave.  (-inf + 8 = -inf: the first
// finite block maximum always moves it; a block of masked scores never does.)
__device__ __forceinline__ float moved_reference(float ref, float block_max) {
    return block_max > ref + 8.f ? block_max : ref;
}

// K and V tiles sit in LDS as they lie in memory, [64 keys][D], 16-byte chunks
// XOR-swizzled inside each row.  K is read as the A operand of S^T = K.Q^T with
// ds_read_b128 (lane = key row, eight consecutive d); V is read as the A operand
// of O^T += V^T.P^T with ds_read_b64_tr_b16, which hands lane i of a 16-lane
// group column d = i of four consecutive key rows.
template <int D>
__device__ inline int k_swz(int row) { return (D == 128) ? (row & 15) : ((row >> 1) & 7); }
template <int D>
__device__ inline uint32_t k_off(int row, int chunk) {
    return (uint32_t)(row * (D * 2) + ((chunk ^ k_swz<D>(row)) << 4));
}
// the four key rows that one transposing read touches must fall on disjoint banks
template <int D>
__device__ inline int v_swz(int row) { return (D == 128) ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); }
template <int D>
__device__ inline uint32_t v_off(int row, int chunk) {
    return (uint32_t)(row * (D * 2) + ((chunk ^ v_swz<D>(row)) << 4));
}

typedef short fa_s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) fa_s16x4 fa_lds_s16x4;
typedef __attribute__((address_space(3))) void fa_lds_void;

// The value held by lane ^ 32, through the register-file lane swap of gfx950 instead
// of a round trip through LDS.  The swap exchanges the upper half of its first
// operand with the lower half of its second; picking the result by the lane's own
// half is right whether or not the two operands share a register.
__device__ inline float other_half(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_bit_cast(float, (threadIdx.x & 32) ? r[0] : r[1]);
}
__device__ inline float half_max(float x) { return fmaxf(x, other_half(x)); }
__device__ inline float half_sum(float x) { return x + other_half(x); }

}  // namespace mhip
