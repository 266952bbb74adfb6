// Shared device helpers for the gfx950 kernels: element types, vector loads,
// wave64 reductions. Every kernel file exports plain C entry points that take raw
// device pointers, sizes and a HIP stream and return a hipError_t as int.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define SOC_EXPORT extern "C" __attribute__((visibility("default")))
#define SOC_WAVE 64

// bfloat16 as its 16 raw bits; conversions are explicit so that every rounding in a
// kernel is visible in its source.
struct bf16 { uint16_t bits; };

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16 v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

// Round to nearest even; gfx950 converts in hardware (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    return __builtin_bit_cast(uint16_t, (__bf16)f);
}

// Two floats to two bfloat16 in one word, `lo` in the low half.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef float soc_f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 soc_bf16x2 __attribute__((ext_vector_type(2)));
    const soc_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, soc_bf16x2));
}

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_float<bf16>(float v) { bf16 r; r.bits = f32_to_bf16_bits(v); return r; }

// Load N consecutive elements as floats; p is aligned to N * sizeof(T) bytes when that
// is a power of two, else to the largest power of two that divides it.
template <typename T, int N> struct VecLoad;

template <int N> struct VecLoad<float, N> {
    __device__ static __forceinline__ void load(const float* p, float (&x)[N]) {
        if constexpr (N % 4 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 4) {
                float4 v = *reinterpret_cast<const float4*>(p + i);
                x[i] = v.x; x[i + 1] = v.y; x[i + 2] = v.z; x[i + 3] = v.w;
            }
        } else if constexpr (N % 2 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 2) {
                float2 v = *reinterpret_cast<const float2*>(p + i);
                x[i] = v.x; x[i + 1] = v.y;
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) x[i] = p[i];
        }
    }
};

template <int N> struct VecLoad<bf16, N> {
    __device__ static __forceinline__ void load(const bf16* p, float (&x)[N]) {
        const uint16_t* q = reinterpret_cast<const uint16_t*>(p);
        if constexpr (N % 8 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 8) {
                uint4 v = *reinterpret_cast<const uint4*>(q + i);
                x[i] = __uint_as_float(v.x << 16); x[i + 1] = __uint_as_float(v.x & 0xffff0000u);
                x[i + 2] = __uint_as_float(v.y << 16); x[i + 3] = __uint_as_float(v.y & 0xffff0000u);
                x[i + 4] = __uint_as_float(v.z << 16); x[i + 5] = __uint_as_float(v.z & 0xffff0000u);
                x[i + 6] = __uint_as_float(v.w << 16); x[i + 7] = __uint_as_float(v.w & 0xffff0000u);
            }
        } else if constexpr (N % 4 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 4) {
                uint2 v = *reinterpret_cast<const uint2*>(q + i);
                x[i] = __uint_as_float(v.x << 16); x[i + 1] = __uint_as_float(v.x & 0xffff0000u);
                x[i + 2] = __uint_as_float(v.y << 16); x[i + 3] = __uint_as_float(v.y & 0xffff0000u);
            }
        } else if constexpr (N % 2 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 2) {
                uint32_t v = *reinterpret_cast<const uint32_t*>(q + i);
                x[i] = __uint_as_float(v << 16); x[i + 1] = __uint_as_float(v & 0xffff0000u);
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) x[i] = __uint_as_float(((uint32_t)q[i]) << 16);
        }
    }
};

// Cross-lane steps of a wave reduction without a trip through LDS: within a row of 16
// lanes DPP operands (lane ^ 1, lane ^ 2, then the mirror images of a half row and of a
// row, which pair groups whose lanes already agree), across rows the gfx950 lane-swap
// instructions. Every step combines a pair symmetrically, so all lanes end with the same bits.
template <int CTRL> __device__ __forceinline__ float soc_dpp(float v) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, true));
}
constexpr int SOC_DPP_XOR1 = 0xB1, SOC_DPP_XOR2 = 0x4E, SOC_DPP_HALF_MIRROR = 0x141, SOC_DPP_ROW_MIRROR = 0x140;

typedef uint32_t soc_u32x2 __attribute__((ext_vector_type(2)));
// this lane's value and that of lane ^ 16 (in some order)
__device__ __forceinline__ soc_u32x2 soc_pair_xor16(float v) {
    return __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
}
__device__ __forceinline__ soc_u32x2 soc_pair_xor32(float v) {
    return __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
}
__device__ __forceinline__ float sum_xor16(float v) { const soc_u32x2 p = soc_pair_xor16(v); return __uint_as_float(p.x) + __uint_as_float(p.y); }
__device__ __forceinline__ float sum_xor32(float v) { const soc_u32x2 p = soc_pair_xor32(v); return __uint_as_float(p.x) + __uint_as_float(p.y); }
__device__ __forceinline__ float max_xor16(float v) { const soc_u32x2 p = soc_pair_xor16(v); return fmaxf(__uint_as_float(p.x), __uint_as_float(p.y)); }
__device__ __forceinline__ float max_xor32(float v) { const soc_u32x2 p = soc_pair_xor32(v); return fmaxf(__uint_as_float(p.x), __uint_as_float(p.y)); }

__device__ __forceinline__ float wave_sum(float v) {
    v += soc_dpp<SOC_DPP_XOR1>(v);
    v += soc_dpp<SOC_DPP_XOR2>(v);
    v += soc_dpp<SOC_DPP_HALF_MIRROR>(v);
    v += soc_dpp<SOC_DPP_ROW_MIRROR>(v);
    return sum_xor32(sum_xor16(v));
}

__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, soc_dpp<SOC_DPP_XOR1>(v));
    v = fmaxf(v, soc_dpp<SOC_DPP_XOR2>(v));
    v = fmaxf(v, soc_dpp<SOC_DPP_HALF_MIRROR>(v));
    v = fmaxf(v, soc_dpp<SOC_DPP_ROW_MIRROR>(v));
    return max_xor32(max_xor16(v));
}

// Sum over the whole workgroup (blockDim.x a multiple of 64, at most 1024); every
// thread receives the result. `scratch` holds at least 16 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int wave = threadIdx.x / SOC_WAVE, lane = threadIdx.x % SOC_WAVE;
    const int n_waves = blockDim.x / SOC_WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < n_waves; ++i) t += scratch[i];
    return t;
}

static inline int soc_last_error() { return (int)hipGetLastError(); }
