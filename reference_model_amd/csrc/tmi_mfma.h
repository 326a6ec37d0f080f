// Matrix-core plumbing shared by the MFMA kernels: vector types, the per-type 32x32 matrix instruction, and
// the small conversions their prologues and epilogues use.
#pragma once
#include "tmi_kernels.h"

namespace tmi
{

typedef int v2i __attribute__((ext_vector_type(2)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8b __attribute__((ext_vector_type(8)));

// One 32x32 MFMA step: 16 bytes of K per lane and operand (32 int8 or 16 half-precision values per row), lane
// half h = lane / 32 holding the K bytes [16h, 16h + 16) of row lane % 32.
template <typename T>
struct Mma;

template <>
struct Mma<int8_t>
{
    using acc_t                  = v16i;
    static constexpr bool is_int = true;
    __device__ static v16i mma(v4i a, v4i b, v16i c)
    {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
    }
};
template <>
struct Mma<_Float16>
{
    using acc_t                  = v16f;
    static constexpr bool is_int = false;
    __device__ static v16f mma(v4i a, v4i b, v16f c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0,
                                                      0, 0);
    }
};
template <>
struct Mma<bf16_t>
{
    using acc_t                  = v16f;
    static constexpr bool is_int = false;
    __device__ static v16f mma(v4i a, v4i b, v16f c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8b, a), __builtin_bit_cast(v8b, b), c, 0,
                                                       0, 0);
    }
};

// min(max(v, lo), hi) as one instruction; lo <= hi
__device__ __forceinline__ int32_t clamp_med3(int32_t v, int32_t lo, int32_t hi)
{
    int32_t r;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "v"(lo), "v"(hi));
    return r;
}

__device__ __forceinline__ int dot4_ones(v4i v)
{
    int s = __builtin_amdgcn_sdot4(v.x, 0x01010101, 0, false);
    s     = __builtin_amdgcn_sdot4(v.y, 0x01010101, s, false);
    s     = __builtin_amdgcn_sdot4(v.z, 0x01010101, s, false);
    return __builtin_amdgcn_sdot4(v.w, 0x01010101, s, false);
}


template <typename T>
__device__ __forceinline__ float load_as_float(const void* p, int i);
template <>
__device__ __forceinline__ float load_as_float<_Float16>(const void* p, int i)
{
    return (float)reinterpret_cast<const _Float16*>(p)[i];
}
template <>
__device__ __forceinline__ float load_as_float<bf16_t>(const void* p, int i)
{
    return bf16_to_float(reinterpret_cast<const bf16_t*>(p)[i]);
}
template <>
__device__ __forceinline__ float load_as_float<int8_t>(const void*, int)
{
    return 0.0f;
}

__device__ __forceinline__ void store_from_float(_Float16* p, float v)
{
    *p = (_Float16)v;
}
__device__ __forceinline__ void store_from_float(bf16_t* p, float v)
{
    *p = float_to_bf16(v);
}
__device__ __forceinline__ void store_from_float(int8_t*, float)
{}

}    // namespace tmi
