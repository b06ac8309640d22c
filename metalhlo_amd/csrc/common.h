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

constexpr int kWave = 64;

// Records a message for mhip_last_error() and returns `code`.
int fail(int code, const char* fmt, ...);

// Checks the launch that was just issued.
int check_launch(const char* what);

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

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

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

}  // namespace mhip
