// Shared device helpers for the gfx950 kernels: storage types, conversions, wave and
// block reductions, and the error channel of the C entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#define MV_WAVE 64

// ---------------------------------------------------------------------------------------
// Storage types. Arithmetic is always done on float; bf16 is storage only.
// ---------------------------------------------------------------------------------------
struct bf16 {
    uint16_t bits;
};

enum MvDtype { MV_F32 = 0, MV_BF16 = 1 };

__device__ __forceinline__ float to_f(float v) { return v; }
__device__ __forceinline__ float to_f(bf16 v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

// float -> bf16, round to nearest even: gfx950 has the conversion in hardware (v_cvt_pk_bf16_f32,
// two values an instruction), which is what these casts compile to. A wave issues about one
// instruction every four cycles, so a rounding written out in integer instructions (five or six
// per value) is what small kernels spend their time on.
typedef __bf16 mv_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float mv_floatx2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    const __bf16 h = (__bf16)f;
    return __builtin_bit_cast(uint16_t, h);
}

// two values in one 32-bit word: a in the low half, b in the high half
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float a, float b) {
    const mv_bf16x2_t h = __builtin_convertvector(mv_floatx2_t{a, b}, mv_bf16x2_t);
    return __builtin_bit_cast(uint32_t, h);
}

template <typename T> __device__ __forceinline__ T from_f(float f);
template <> __device__ __forceinline__ float from_f<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16 from_f<bf16>(float f) {
    bf16 r;
    r.bits = f32_to_bf16_bits(f);
    return r;
}

// A weight tensor whose element type is known only at run time (it is kept as stored:
// bf16 or float). The branch is uniform over a launch.
struct WeightPtr {
    const void* p;
    int dtype;
    __device__ __forceinline__ float at(size_t i) const {
        if (dtype == MV_F32) return ((const float*)p)[i];
        return to_f(((const bf16*)p)[i]);
    }
    // E (2 or 4) consecutive elements from i (i a multiple of E, the tensor 16-byte aligned): one load
    template <int E> __device__ __forceinline__ void at_few(size_t i, float (&out)[E]) const {
        static_assert(E == 2 || E == 4, "at_few: two or four elements");
        if (dtype == MV_F32) {
            if constexpr (E == 4) {
                const float4 a = *reinterpret_cast<const float4*>((const float*)p + i);
                out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
            } else {
                const float2 a = *reinterpret_cast<const float2*>((const float*)p + i);
                out[0] = a.x; out[1] = a.y;
            }
        } else {
            uint32_t w[E / 2];
            if constexpr (E == 4) {
                const uint2 u = *reinterpret_cast<const uint2*>((const bf16*)p + i);
                w[0] = u.x; w[1] = u.y;
            } else {
                w[0] = *reinterpret_cast<const uint32_t*>((const bf16*)p + i);
            }
#pragma unroll
            for (int e = 0; e < E / 2; ++e) {
                out[2 * e] = __uint_as_float(w[e] << 16);
                out[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
            }
        }
    }
    // eight consecutive elements from i (i a multiple of 8, the tensor 16-byte aligned)
    __device__ __forceinline__ void at8(size_t i, float (&out)[8]) const {
        if (dtype == MV_F32) {
            const float4 a = *reinterpret_cast<const float4*>((const float*)p + i);
            const float4 b = *reinterpret_cast<const float4*>((const float*)p + i + 4);
            out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
            out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
        } else {
            const uint4 u = *reinterpret_cast<const uint4*>((const bf16*)p + i);
            const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                out[2 * e] = __uint_as_float(w[e] << 16);
                out[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
            }
        }
    }
};

// ---------------------------------------------------------------------------------------
// Reductions
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = MV_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, MV_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = MV_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, MV_WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds at least 17 floats of LDS.
// Every thread gets the result. The order of additions depends only on the block size.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (MV_WAVE - 1);
    const int wave = threadIdx.x / MV_WAVE;
    const int nwaves = (blockDim.x + MV_WAVE - 1) / MV_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
        for (int i = 0; i < nwaves; ++i) t += scratch[i];
        scratch[16] = t;
    }
    __syncthreads();
    return scratch[16];
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & (MV_WAVE - 1);
    const int wave = threadIdx.x / MV_WAVE;
    const int nwaves = (blockDim.x + MV_WAVE - 1) / MV_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = scratch[0];
        for (int i = 1; i < nwaves; ++i) t = fmaxf(t, scratch[i]);
        scratch[16] = t;
    }
    __syncthreads();
    return scratch[16];
}

// ---------------------------------------------------------------------------------------
// Host side: error reporting of the extern "C" entry points. Each returns 0 on success;
// otherwise mv_last_error() holds the reason.
// ---------------------------------------------------------------------------------------
extern "C" const char* mv_last_error();
int mv_fail(const char* fmt, ...);
int mv_check_launch(const char* what);
int mv_compute_units();     // of the current device (runtime.hip)

#define MV_REQUIRE(cond, ...)                      \
    do {                                           \
        if (!(cond)) return mv_fail(__VA_ARGS__);  \
    } while (0)
