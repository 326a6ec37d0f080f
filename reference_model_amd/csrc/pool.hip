// AVG_POOL2D and MAX_POOL2D (reference_model/src/ops/tensor_ops.cpp:542-660, 1546-1640), NHWC.
//
// Bandwidth work: a lane owns VEC consecutive channels of one output pixel (16 bytes of input per tap when the
// channel count and the pointers allow it, one element otherwise), so consecutive lanes read consecutive
// pieces of one input pixel.  The taps inside the image are a rectangle of the window, worked out once per
// pixel; nothing is read outside it, which is what the reference's padding amounts to (a padded tap is
// skipped by AVG_POOL2D and holds the lowest value / NaN for MAX_POOL2D).
//
// AVG_POOL2D, integers: the int32 sum of (in - input_zp) over the window is scaled by the reciprocal of the
// number of taps inside the image - QuantUtil::reciprocal_scale (quant_util.h:32-43) followed by
// apply_scale_32 with a single rounding - then output_zp is added and the value clipped to the type.  The
// REQUIREs of apply_scale_32 go to the context's flag word like RESCALE's, although no int8 / int16 window
// of fewer than 2^13 taps can raise them.  Floating point: an fp32 accumulator over the taps in (ky, kx)
// order, one division, narrowed to the output type: the same roundings as the reference's loop nest.
#include "tmi_kernels.h"

namespace tmi
{

typedef int pl_v4i __attribute__((ext_vector_type(4)));

struct PoolArgs
{
    const uint8_t* in;
    uint8_t* out;
    uint32_t* flag_word;
    int64_t total;    // N * OH * OW * groups
    int32_t IH, IW, C, OH, OW;
    int32_t ky, kx, sy, sx, pad_top, pad_left;
    int32_t in_zp, out_zp, qmin, qmax;
    int32_t nan_mode;    // MAX_POOL2D, floating point: 1 = PROPAGATE, 2 = IGNORE
    int32_t groups;      // channel groups of VEC elements per pixel
    int32_t full_mult, full_k;    // AVG_POOL2D: reciprocal_scale of a whole window (ky * kx taps), worked out on the host
    int32_t xcd_remap;            // the grid is a multiple of 8 workgroups: give each XCD a contiguous range of pixels
};

template <typename T>
struct PoolType;
template <>
struct PoolType<int8_t>
{
    using acc_t                  = int32_t;
    static constexpr bool is_int = true;
    __device__ static int32_t widen(int8_t v) { return v; }
    __device__ static int8_t narrow(int32_t v) { return (int8_t)v; }
};
template <>
struct PoolType<int16_t>
{
    using acc_t                  = int32_t;
    static constexpr bool is_int = true;
    __device__ static int32_t widen(int16_t v) { return v; }
    __device__ static int16_t narrow(int32_t v) { return (int16_t)v; }
};
template <>
struct PoolType<_Float16>
{
    using acc_t                  = float;
    static constexpr bool is_int = false;
    __device__ static float widen(_Float16 v) { return (float)v; }
    __device__ static _Float16 narrow(float v) { return (_Float16)v; }
};
template <>
struct PoolType<bf16_t>
{
    using acc_t                  = float;
    static constexpr bool is_int = false;
    __device__ static float widen(bf16_t v) { return bf16_to_float(v); }
    __device__ static bf16_t narrow(float v) { return float_to_bf16(v); }
};
template <>
struct PoolType<float>
{
    using acc_t                  = float;
    static constexpr bool is_int = false;
    __device__ static float widen(float v) { return v; }
    __device__ static float narrow(float v) { return v; }
};

// applyMax (reference_model/src/arith_util.h:341-373)
__device__ __forceinline__ float pool_max(float a, float b, int nan_mode)
{
    if (a != a || b != b)
        return nan_mode == 1 ? __builtin_nanf("") : (a != a ? b : a);
    return a >= b ? a : b;
}

template <typename T, bool AVG, int VEC>
__global__ __launch_bounds__(256) void pool_kernel(PoolArgs a)
{
    using P                  = PoolType<T>;
    using acc_t              = typename P::acc_t;
    constexpr int kVecBytes  = VEC * (int)sizeof(T);
    uint32_t flags           = 0;
    // Consecutive workgroups go to the 8 XCDs in turn, each with its own L2.  Windows that overlap (stride < kernel)
    // share input rows with the next output row: XCD x takes workgroups [x * per, x * per + per) of the pixel order, so
    // that neighbouring output rows meet in one L2 instead of fetching the shared rows from HBM twice.
    uint32_t bid = blockIdx.x;
    if (a.xcd_remap)
        bid = (bid & 7) * (gridDim.x >> 3) + (bid >> 3);
    {
        const int64_t i = (int64_t)bid * blockDim.x + threadIdx.x;
        if (i >= a.total)
            return;
        // (pixel, channel group); totals below 2^32 are checked on the host
        const uint32_t pix = (uint32_t)i / (uint32_t)a.groups;
        const int grp      = (int)((uint32_t)i - pix * (uint32_t)a.groups);
        const uint32_t row = pix / (uint32_t)a.OW;
        const int ow       = (int)(pix - row * (uint32_t)a.OW);
        const uint32_t n   = row / (uint32_t)a.OH;
        const int oh       = (int)(row - n * (uint32_t)a.OH);
        // taps inside the image: rows [y0, y1) x columns [x0, x1)
        const int iy = oh * a.sy - a.pad_top, ix = ow * a.sx - a.pad_left;
        const int y0 = iy > 0 ? iy : 0, y1 = iy + a.ky < a.IH ? iy + a.ky : a.IH;
        const int x0 = ix > 0 ? ix : 0, x1 = ix + a.kx < a.IW ? ix + a.kx : a.IW;

        acc_t acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++)
        {
            if constexpr (AVG)
                acc[e] = 0;
            else if constexpr (P::is_int)
                acc[e] = a.qmin;    // lowest value of the type
            else
                acc[e] = a.nan_mode == 2 ? __builtin_nanf("") : -__builtin_inff();
        }
        const uint8_t* base = a.in + ((size_t)n * a.IH * a.IW * a.C + (size_t)grp * VEC) * sizeof(T);
        for (int y = y0; y < y1; y++)
            for (int x = x0; x < x1; x++)
            {
                const uint8_t* src = base + ((size_t)y * a.IW + x) * a.C * sizeof(T);
                alignas(16) T v[VEC];
                if constexpr (kVecBytes == 16)
                    *reinterpret_cast<pl_v4i*>(v) = *reinterpret_cast<const pl_v4i*>(src);
                else
                    v[0] = *reinterpret_cast<const T*>(src);
#pragma unroll
                for (int e = 0; e < VEC; e++)
                {
                    const acc_t w = P::widen(v[e]);
                    if constexpr (AVG && P::is_int)
                        acc[e] += w - a.in_zp;
                    else if constexpr (AVG)
                        acc[e] = acc[e] + w;
                    else if constexpr (P::is_int)
                        acc[e] = acc[e] >= w ? acc[e] : w;
                    else
                        acc[e] = pool_max(acc[e], w, a.nan_mode);
                }
            }

        alignas(16) T r[VEC];
        if constexpr (AVG && P::is_int)
        {
            // QuantUtil::reciprocal_scale: (1 << k) / 2 < count <= (1 << k)
            const int count = (y1 - y0) * (x1 - x0);
            int k           = a.full_k;
            int32_t mult    = a.full_mult;
            if (count != a.ky * a.kx)    // a window cut by the border: the 64-bit division is worth avoiding elsewhere
            {
                k    = 32 - __clz(count - 1);    // __clz(0) = 32
                mult = (int32_t)((((uint64_t(1) << 30) + 1) << k) / (uint32_t)count);
            }
            if (a.ky * a.kx <= 8192)
            {
                // |acc| <= taps * 2^16 <= 2^(k + 16) stays below 2^(29 + k), the range apply_scale_32 asks of a value for
                // the shift 30 + k (quant_util.h:59-67), and the scaled value stays below 2^30: neither REQUIRE can
                // fire, so the plain formula is the whole function
                const int shift   = 30 + k;
                const int64_t rnd = int64_t(1) << (shift - 1);
#pragma unroll
                for (int e = 0; e < VEC; e++)
                {
                    int32_t v = (int32_t)(((int64_t)acc[e] * mult + rnd) >> shift) + a.out_zp;
                    v         = v > a.qmin ? v : a.qmin;
                    r[e]      = P::narrow(v < a.qmax ? v : a.qmax);
                }
            }
            else
            {
#pragma unroll
                for (int e = 0; e < VEC; e++)
                {
                    int32_t v = apply_scale_32(acc[e], mult, 30 + k, false, flags) + a.out_zp;
                    v         = v > a.qmin ? v : a.qmin;
                    r[e]      = P::narrow(v < a.qmax ? v : a.qmax);
                }
            }
        }
        else if constexpr (AVG)
        {
            const float count = (float)((y1 - y0) * (x1 - x0));
#pragma unroll
            for (int e = 0; e < VEC; e++)
                r[e] = P::narrow(acc[e] / count);
        }
        else
        {
#pragma unroll
            for (int e = 0; e < VEC; e++)
                r[e] = P::narrow(acc[e]);
        }
        uint8_t* dst = a.out + ((size_t)pix * a.C + (size_t)grp * VEC) * sizeof(T);
        if constexpr (kVecBytes == 16)
            *reinterpret_cast<pl_v4i*>(dst) = *reinterpret_cast<const pl_v4i*>(r);
        else
            *reinterpret_cast<T*>(dst) = r[0];
    }
    if constexpr (AVG && P::is_int)
        raise_flags(a.flag_word, flags);
}

template <typename T, bool AVG>
static const char* launch_pool_t(hipStream_t st, PoolArgs& a, int32_t N, const char* vec_label, const char* label)
{
    constexpr int VEC = 16 / (int)sizeof(T);
    const bool vec    = a.C % VEC == 0 && (((uintptr_t)a.in | (uintptr_t)a.out) & 15) == 0;
    a.groups          = vec ? a.C / VEC : a.C;
    a.total           = (int64_t)N * a.OH * a.OW * a.groups;
    if (a.total >= (int64_t(1) << 32))
        return nullptr;
    const int64_t blocks = ((a.total + 255) / 256 + 7) & ~int64_t(7);    // whole groups of 8 for the XCD order
    a.xcd_remap          = 1;
    if (vec)
        hipLaunchKernelGGL((pool_kernel<T, AVG, VEC>), dim3((int)blocks), dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL((pool_kernel<T, AVG, 1>), dim3((int)blocks), dim3(256), 0, st, a);
    return vec ? vec_label : label;
}

// nullptr for a dtype this file has no kernel for, or a tensor of 2^32 work items or more.
const char* launch_pool(hipStream_t st, bool avg, int32_t dtype, int32_t N, int32_t IH, int32_t IW, int32_t C,
                        int32_t OH, int32_t OW, int32_t kernel_y, int32_t kernel_x, int32_t stride_y, int32_t stride_x,
                        int32_t pad_top, int32_t pad_left, int32_t in_zp, int32_t out_zp, int32_t nan_mode,
                        const void* in, void* out, uint32_t* flag_word)
{
    PoolArgs a{};
    a.in = (const uint8_t*)in, a.out = (uint8_t*)out, a.flag_word = flag_word;
    a.IH = IH, a.IW = IW, a.C = C, a.OH = OH, a.OW = OW;
    a.ky = kernel_y, a.kx = kernel_x, a.sy = stride_y, a.sx = stride_x, a.pad_top = pad_top, a.pad_left = pad_left;
    a.in_zp = in_zp, a.out_zp = out_zp, a.nan_mode = nan_mode;
    {
        // QuantUtil::reciprocal_scale (quant_util.h:32-43) for a window that lies inside the image
        const uint32_t count = (uint32_t)kernel_y * (uint32_t)kernel_x;
        int k                = 0;
        while (k < 32 && (uint64_t(1) << k) < count)
            k++;
        a.full_k    = k;
        a.full_mult = count ? (int32_t)((((uint64_t(1) << 30) + 1) << k) / count) : 0;
    }
    switch (dtype)
    {
        case TMI_INT8:
            a.qmin = -128, a.qmax = 127;
            return avg ? launch_pool_t<int8_t, true>(st, a, N, "avg_pool2d_vec_i8", "avg_pool2d_i8")
                       : launch_pool_t<int8_t, false>(st, a, N, "max_pool2d_vec_i8", "max_pool2d_i8");
        case TMI_INT16:
            a.qmin = -32768, a.qmax = 32767;
            return avg ? launch_pool_t<int16_t, true>(st, a, N, "avg_pool2d_vec_i16", "avg_pool2d_i16")
                       : launch_pool_t<int16_t, false>(st, a, N, "max_pool2d_vec_i16", "max_pool2d_i16");
        case TMI_FP16:
            return avg ? launch_pool_t<_Float16, true>(st, a, N, "avg_pool2d_vec_f16", "avg_pool2d_f16")
                       : launch_pool_t<_Float16, false>(st, a, N, "max_pool2d_vec_f16", "max_pool2d_f16");
        case TMI_BF16:
            return avg ? launch_pool_t<bf16_t, true>(st, a, N, "avg_pool2d_vec_bf16", "avg_pool2d_bf16")
                       : launch_pool_t<bf16_t, false>(st, a, N, "max_pool2d_vec_bf16", "max_pool2d_bf16");
        case TMI_FP32:
            return avg ? launch_pool_t<float, true>(st, a, N, "avg_pool2d_vec_f32", "avg_pool2d_f32")
                       : launch_pool_t<float, false>(st, a, N, "max_pool2d_vec_f32", "max_pool2d_f32");
        default: return nullptr;
    }
}

}    // namespace tmi
