// Shared device/host helpers for the gfx950 kernel library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mhip.h"

namespace mhip {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;

// Records a message for mhip_last_error() and returns `code`.
int fail(int code, const char* fmt, ...);

// Checks the launch that was just issued.
int check_launch(const char* what);

// Compute units of the current device (queried once per device).
int compute_units();

// Integer launch-tuning knob from the environment (read on every call; unset or
// unparsable -> `fallback`).
int tune_int(const char* name, int fallback);

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// How a vectorisable row-operator launch (softmax / LayerNorm / RMSNorm over 16-byte-aligned rows)
// is carried out.  `kind`: 1 = one wave per row, parameters staged in LDS, persistent grid;
// 2 = a row split over the waves of a workgroup.  `r` = rows per wave group (split only),
// `ordered` = the grid covers the rows once in address order (split only; 0 = persistent grid),
// `per_cu` = resident workgroups per CU of a persistent grid (0 = what the occupancy query says).
// Zero / negative fields mean "choose".
struct RowLaunch { int kind = 0, r = 0, ordered = -1, per_cu = 0; };

// The launch a tuning pass recorded for this problem on this device, if any (tuning.hip).
bool tuned_row_launch(int op, int dtype, int64_t rows, int64_t cols, bool has_gamma, bool has_beta, RowLaunch* out);

// The attention kernel a tuning pass recorded (or is timing) for this problem: 0 = none, 1 = the
// 128-row kernel, 2 / 3 = the 256-row pipelined kernel with causal tiles unpaired / paired (tuning.hip).
int tuned_attention_variant(int dtype, int64_t batch_heads, int64_t Sq, int64_t Skv, int64_t D, bool causal);

// One launch of row operator `op` (0 softmax, 1 LayerNorm, 2 RMSNorm) carried out as `how` says.
int row_launch_as(int op, const RowLaunch& how, void* stream, const void* x, const void* g, const void* b, void* y,
                  int64_t rows, int64_t cols, float eps, int dtype);

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int kPerVec = 4;  // elements per 16-byte vector
    __device__ static float to_f32(float v) { return v; }
    __device__ static float from_f32(float v) { return v; }
};
template <> struct Elem<bf16_t> {
    static constexpr int kPerVec = 8;
    __device__ static float to_f32(bf16_t v) { return (float)v; }
    __device__ static bf16_t from_f32(float v) { return (bf16_t)v; }  // v_cvt_pk_bf16_f32, RNE
};
template <> struct Elem<f16_t> {
    static constexpr int kPerVec = 8;
    __device__ static float to_f32(f16_t v) { return (float)v; }
    __device__ static f16_t from_f32(float v) { return (f16_t)v; }
};

// 16-byte vector of T, loaded/stored with one 128-bit access.
template <typename T> struct alignas(16) Vec16 {
    T v[Elem<T>::kPerVec];
};

template <typename T>
__device__ inline Vec16<T> load16(const T* p) {
    return *reinterpret_cast<const Vec16<T>*>(p);
}
template <typename T>
__device__ inline void store16(T* p, const Vec16<T>& v) {
    *reinterpret_cast<Vec16<T>*>(p) = v;
}
// Streaming variants: data that is touched once should not displace the cache.
template <typename T>
__device__ inline Vec16<T> load16_stream(const T* p) {
    const u32x4 r = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return __builtin_bit_cast(Vec16<T>, r);
}
template <typename T>
__device__ inline void store16_stream(T* p, const Vec16<T>& v) {
    __builtin_nontemporal_store(__builtin_bit_cast(u32x4, v), reinterpret_cast<u32x4*>(p));
}

// Wave-wide reductions on the DPP cross-lane network (no LDS traffic): four
// steps inside each row of 16 lanes, two row broadcasts, result read from lane 63.
struct SumOp { __device__ static float id() { return 0.f; } __device__ static float f(float a, float b) { return a + b; } };
struct MaxOp { __device__ static float id() { return -__builtin_inff(); } __device__ static float f(float a, float b) { return fmaxf(a, b); } };

template <int CTRL, int ROW_MASK>
__device__ inline float dpp_move(float identity, float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, identity),
                                                                 __builtin_bit_cast(int, v), CTRL,
                                                                 ROW_MASK, 0xF, false));
}
template <typename Op>
__device__ inline float wave_reduce(float v) {
    v = Op::f(v, dpp_move<0xB1, 0xF>(Op::id(), v));   // quad_perm [1,0,3,2]
    v = Op::f(v, dpp_move<0x4E, 0xF>(Op::id(), v));   // quad_perm [2,3,0,1]
    v = Op::f(v, dpp_move<0x141, 0xF>(Op::id(), v));  // row_half_mirror
    v = Op::f(v, dpp_move<0x140, 0xF>(Op::id(), v));  // row_mirror
    v = Op::f(v, dpp_move<0x142, 0xA>(Op::id(), v));  // row_bcast:15 into rows 1 and 3
    v = Op::f(v, dpp_move<0x143, 0xC>(Op::id(), v));  // row_bcast:31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ inline float wave_sum(float v) { return wave_reduce<SumOp>(v); }
__device__ inline float wave_max(float v) { return wave_reduce<MaxOp>(v); }

}  // namespace mhip
