// Shared helpers of the gfx950 kernels: element types, wave reductions, launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#define TUFF_EXPORT extern "C" __attribute__((visibility("default")))

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int WAVE = 64;

// Element type codes shared with the Python side.
enum : int { DT_F32 = 0, DT_BF16 = 1 };

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

// Sum over the 64 lanes of a wave; every lane receives the total.  The order of
// the butterfly is fixed, so the result does not depend on anything but the inputs.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = WAVE / 2; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, WAVE));
    return v;
}

// Sum over a workgroup of NWAVES waves; `scratch` holds NWAVES floats of LDS.
// Wave partials are added in wave order.  Ends with the total in every thread.
template <int NWAVES>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int wave = threadIdx.x / WAVE;
    __syncthreads();
    if ((threadIdx.x % WAVE) == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NWAVES; ++i) t += scratch[i];
    return t;
}

// f(std::integral_constant<int, 0>()), ..., f(std::integral_constant<int, N - 1>()): a loop whose
// index is a compile-time constant inside the body (register arrays stay registers).
template <int N, typename F, int I = 0>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>());
        static_for<N, F, I + 1>(static_cast<F&&>(f));
    }
}

static inline int launch_status() { return (int)hipGetLastError(); }

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
static inline long long ceil_div_ll(long long a, long long b) { return (a + b - 1) / b; }
