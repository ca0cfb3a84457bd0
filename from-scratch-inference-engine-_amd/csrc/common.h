// Shared device helpers for the gfx950 kernels: element types, wave reductions, error reporting.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define FSIE_WAVE 64

// ---- element types ---------------------------------------------------------------------
// bfloat16 is carried as its 16 bits; conversions are explicit (round to nearest even).
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
    return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) {  // NaN stays NaN
        return static_cast<uint16_t>((u >> 16) | 0x0040u);
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

// Two floats to two bfloat16 in one register (low half first), round to nearest even: one
// v_cvt_pk_bf16_f32 on gfx950.
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float floatx2_t __attribute__((ext_vector_type(2)));
    const floatx2_t v = {lo, hi};
    const bf16x2_t b = __builtin_convertvector(v, bf16x2_t);
    return *reinterpret_cast<const uint32_t*>(&b);
}

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return bf16_bits_to_float(v.bits); }

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) {
    return v;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) {
    bf16_t r;
    r.bits = float_to_bf16_bits(v);
    return r;
}

// ---- reductions over a 64-lane wave ------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = FSIE_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, FSIE_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = FSIE_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, FSIE_WAVE));
    return v;
}

// This lane's value combined with that of lane ^ 16 or lane ^ 32, through the lane swaps of
// gfx950 (v_permlane16_swap, v_permlane32_swap): two register moves, no trip through LDS as
// a general shuffle takes.
typedef unsigned fsie_u2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float max_xor16(float v) {
    const fsie_u2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float max_xor32(float v) {
    const fsie_u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_xor16(float v) {
    const fsie_u2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float sum_xor32(float v) {
    const fsie_u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `scratch` holds at
// least 16 floats of LDS and may be reused after the call returns.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (FSIE_WAVE - 1);
    const int wave = threadIdx.x / FSIE_WAVE;
    const int n_waves = (blockDim.x + FSIE_WAVE - 1) / FSIE_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < n_waves; ++w) total += scratch[w];
    return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & (FSIE_WAVE - 1);
    const int wave = threadIdx.x / FSIE_WAVE;
    const int n_waves = (blockDim.x + FSIE_WAVE - 1) / FSIE_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = scratch[0];
    for (int w = 1; w < n_waves; ++w) total = fmaxf(total, scratch[w]);
    return total;
}

// ---- host side: errors -------------------------------------------------------------------
// Every entry point returns 0 on success.  On failure it returns nonzero and leaves a message
// that fsie_last_error() hands out (per host thread).
void fsie_set_error(const char* fmt, ...);

// compute units of the current device (0 if it cannot be asked); asked once per device
int fsie_compute_units();

#define FSIE_REQUIRE(cond, ...)          \
    do {                                 \
        if (!(cond)) {                   \
            fsie_set_error(__VA_ARGS__); \
            return 1;                    \
        }                                \
    } while (0)

#define FSIE_CHECK_LAUNCH(name)                                                    \
    do {                                                                           \
        hipError_t e_ = hipGetLastError();                                         \
        if (e_ != hipSuccess) {                                                    \
            fsie_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));  \
            return 2;                                                              \
        }                                                                          \
    } while (0)

enum FsieDtype { FSIE_F32 = 0, FSIE_BF16 = 1 };

static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }
