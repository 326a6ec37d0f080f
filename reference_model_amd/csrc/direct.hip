// Direct kernels: one output element per lane, loops in the reference's order.  They accept every legal
// shape (any channel count, stride, dilation, padding, bias length) and are the fall-back behind the
// MFMA and vectorised kernels.  The floating-point variants accumulate in fp32 in the reference's
// ky -> kx -> ic order with separate multiply and add (built with -ffp-contract=off), which makes them
// reproduce the reference's fp32 accumulation exactly.
#include <type_traits>

#include "tmi_kernels.h"

namespace tmi
{

template <typename T>
struct Elem;

template <>
struct Elem<int8_t>
{
    using acc_t = int32_t;
    __device__ static acc_t load(const int8_t* p, int64_t i)
    {
        return (int32_t)p[i];
    }
};
template <>
struct Elem<_Float16>
{
    using acc_t = float;
    __device__ static acc_t load(const _Float16* p, int64_t i)
    {
        return (float)p[i];
    }
};
template <>
struct Elem<float>
{
    using acc_t = float;
    __device__ static acc_t load(const float* p, int64_t i)
    {
        return p[i];
    }
};
template <>
struct Elem<bf16_t>
{
    using acc_t = float;
    __device__ static acc_t load(const bf16_t* p, int64_t i)
    {
        return bf16_to_float(p[i]);
    }
};

__device__ __forceinline__ void store_fp(_Float16* p, int64_t i, float v)
{
    p[i] = (_Float16)v;
}
__device__ __forceinline__ void store_fp(bf16_t* p, int64_t i, float v)
{
    p[i] = float_to_bf16(v);
}
__device__ __forceinline__ void store_fp(float* p, int64_t i, float v)
{
    p[i] = v;
}

template <typename T, typename OutT>
__global__ __launch_bounds__(256) void conv2d_direct_kernel(ConvGeom g, const T* __restrict__ in,
                                                            const T* __restrict__ w, const void* __restrict__ bias,
                                                            int32_t in_zp, int32_t w_zp, RescaleParams rp,
                                                            OutT* __restrict__ out, uint32_t* flag_word)
{
    using acc_t          = typename Elem<T>::acc_t;
    const int64_t total  = (int64_t)g.N * g.OH * g.OW * g.OC;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    uint32_t flags       = 0;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride)
    {
        const int oc = (int)(idx % g.OC);
        int64_t t    = idx / g.OC;
        const int ox = (int)(t % g.OW);
        t /= g.OW;
        const int oy = (int)(t % g.OH);
        const int n  = (int)(t / g.OH);
        acc_t acc    = 0;
        for (int ky = 0; ky < g.KH; ky++)
        {
            const int y = oy * g.stride_y + ky * g.dil_y - g.pad_top;
            if (y < 0 || y >= g.IH)
                continue;
            for (int kx = 0; kx < g.KW; kx++)
            {
                const int x = ox * g.stride_x + kx * g.dil_x - g.pad_left;
                if (x < 0 || x >= g.IW)
                    continue;
                const int64_t ib = (((int64_t)n * g.IH + y) * g.IW + x) * g.IC;
                const int64_t wb = (((int64_t)oc * g.KH + ky) * g.KW + kx) * g.IC;
                for (int ic = 0; ic < g.IC; ic++)
                    acc += (Elem<T>::load(in, ib + ic) - (acc_t)in_zp) * (Elem<T>::load(w, wb + ic) - (acc_t)w_zp);
            }
        }
        const int bi = g.bias_len == 1 ? 0 : oc;
        if constexpr (std::is_same<acc_t, int32_t>::value)
        {
            const int32_t v = reinterpret_cast<const int32_t*>(bias)[bi] + acc;
            if (rp.enabled)
                out[idx] = (OutT)rescale_value(rp, v, load_multiplier(rp, oc), load_shift(rp, oc), flags);
            else
                out[idx] = (OutT)v;
        }
        else
        {
            const float b = Elem<T>::load(reinterpret_cast<const T*>(bias), bi);
            store_fp(out, idx, b + acc);
        }
    }
    raise_flags(flag_word, flags);
}

template <typename T, typename OutT>
__global__ __launch_bounds__(256) void depthwise_direct_kernel(ConvGeom g, const T* __restrict__ in,
                                                               const T* __restrict__ w,
                                                               const void* __restrict__ bias, int32_t in_zp,
                                                               int32_t w_zp, RescaleParams rp, OutT* __restrict__ out,
                                                               uint32_t* flag_word)
{
    using acc_t          = typename Elem<T>::acc_t;
    const int64_t total  = (int64_t)g.N * g.OH * g.OW * g.OC;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    uint32_t flags       = 0;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride)
    {
        const int oc = (int)(idx % g.OC);
        int64_t t    = idx / g.OC;
        const int ox = (int)(t % g.OW);
        t /= g.OW;
        const int oy = (int)(t % g.OH);
        const int n  = (int)(t / g.OH);
        const int ic = oc / g.M, km = oc % g.M;
        acc_t acc    = 0;
        for (int ky = 0; ky < g.KH; ky++)
        {
            const int y = oy * g.stride_y + ky * g.dil_y - g.pad_top;
            if (y < 0 || y >= g.IH)
                continue;
            for (int kx = 0; kx < g.KW; kx++)
            {
                const int x = ox * g.stride_x + kx * g.dil_x - g.pad_left;
                if (x < 0 || x >= g.IW)
                    continue;
                const acc_t a = Elem<T>::load(in, (((int64_t)n * g.IH + y) * g.IW + x) * g.IC + ic) - (acc_t)in_zp;
                const acc_t b = Elem<T>::load(w, (((int64_t)ky * g.KW + kx) * g.IC + ic) * g.M + km) - (acc_t)w_zp;
                acc += a * b;
            }
        }
        const int bi = g.bias_len == 1 ? 0 : oc;
        if constexpr (std::is_same<acc_t, int32_t>::value)
        {
            const int32_t v = reinterpret_cast<const int32_t*>(bias)[bi] + acc;
            if (rp.enabled)
                out[idx] = (OutT)rescale_value(rp, v, load_multiplier(rp, oc), load_shift(rp, oc), flags);
            else
                out[idx] = (OutT)v;
        }
        else
        {
            const float b = Elem<T>::load(reinterpret_cast<const T*>(bias), bi);
            store_fp(out, idx, b + acc);
        }
    }
    raise_flags(flag_word, flags);
}

template <typename T, typename OutT>
__global__ __launch_bounds__(256) void matmul_direct_kernel(int32_t N, int32_t H, int32_t C, int32_t W,
                                                            const T* __restrict__ a, const T* __restrict__ b,
                                                            int32_t a_zp, int32_t b_zp, OutT* __restrict__ out)
{
    using acc_t          = typename Elem<T>::acc_t;
    const int64_t total  = (int64_t)N * H * W;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride)
    {
        const int x = (int)(idx % W);
        int64_t t   = idx / W;
        const int h = (int)(t % H);
        const int n = (int)(t / H);
        acc_t acc   = 0;
        for (int c = 0; c < C; c++)
            acc += (Elem<T>::load(a, ((int64_t)n * H + h) * C + c) - (acc_t)a_zp) *
                   (Elem<T>::load(b, ((int64_t)n * C + c) * W + x) - (acc_t)b_zp);
        out[idx] = (OutT)acc;
    }
}

// INT16 x INT8 -> INT48 convolutions and INT16 x INT16 -> INT48 MATMUL (tensor_ops.cpp:2225, 2247, 2257): accumulator,
// bias and result are int64, the reference's storage of INT48, and the result is clipped to 48 bits at the end
// (tensor_ops.cpp:875-879, 1325-1329, 1485-1489).  The input zero point is zero by rule (only INT8 tensors have one);
// the INT8 weights' need not be.  One output element per lane, loops in the reference's order.
__device__ __forceinline__ int64_t clip_int48(int64_t v)
{
    const int64_t lo = -(int64_t(1) << 47), hi = (int64_t(1) << 47) - 1;
    return v < lo ? lo : (v > hi ? hi : v);
}

template <bool DEPTHWISE>
__global__ __launch_bounds__(256) void conv_i16_direct_kernel(ConvGeom g, const int16_t* __restrict__ in,
                                                              const int8_t* __restrict__ w,
                                                              const int64_t* __restrict__ bias, int32_t w_zp,
                                                              int64_t* __restrict__ out)
{
    const int64_t total  = (int64_t)g.N * g.OH * g.OW * g.OC;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride)
    {
        const int oc = (int)(idx % g.OC);
        int64_t t    = idx / g.OC;
        const int ox = (int)(t % g.OW);
        t /= g.OW;
        const int oy = (int)(t % g.OH);
        const int n  = (int)(t / g.OH);
        int64_t acc  = 0;
        for (int ky = 0; ky < g.KH; ky++)
        {
            const int y = oy * g.stride_y + ky * g.dil_y - g.pad_top;
            if (y < 0 || y >= g.IH)
                continue;
            for (int kx = 0; kx < g.KW; kx++)
            {
                const int x = ox * g.stride_x + kx * g.dil_x - g.pad_left;
                if (x < 0 || x >= g.IW)
                    continue;
                const int64_t ib = (((int64_t)n * g.IH + y) * g.IW + x) * g.IC;
                if constexpr (DEPTHWISE)
                {
                    const int ic = oc / g.M, km = oc % g.M;
                    acc += (int64_t)in[ib + ic] * (int64_t)((int32_t)w[(((int64_t)ky * g.KW + kx) * g.IC + ic) * g.M + km] - w_zp);
                }
                else
                {
                    const int64_t wb = (((int64_t)oc * g.KH + ky) * g.KW + kx) * g.IC;
                    for (int ic = 0; ic < g.IC; ic++)
                        acc += (int64_t)in[ib + ic] * (int64_t)((int32_t)w[wb + ic] - w_zp);
                }
            }
        }
        out[idx] = clip_int48(bias[g.bias_len == 1 ? 0 : oc] + acc);
    }
}

__global__ __launch_bounds__(256) void matmul_i16_direct_kernel(int32_t N, int32_t H, int32_t C, int32_t W,
                                                                const int16_t* __restrict__ a,
                                                                const int16_t* __restrict__ b, int64_t* __restrict__ out)
{
    const int64_t total  = (int64_t)N * H * W;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride)
    {
        const int x = (int)(idx % W);
        int64_t t   = idx / W;
        const int h = (int)(t % H);
        const int n = (int)(t / H);
        int64_t acc = 0;
        for (int c = 0; c < C; c++)
            acc += (int64_t)a[((int64_t)n * H + h) * C + c] * (int64_t)b[((int64_t)n * C + c) * W + x];
        out[idx] = clip_int48(acc);
    }
}

static int grid_for(int64_t work_items)
{
    int64_t blocks = (work_items + 255) / 256;
    if (blocks < 1)
        blocks = 1;
    if (blocks > 256 * 16)
        blocks = 256 * 16;
    return (int)blocks;
}

#define TMI_LAUNCH_CONV(KERNEL, T, OT)                                                                              \
    hipLaunchKernelGGL((KERNEL<T, OT>), dim3(grid_for(total)), dim3(256), 0, st, g, (const T*)in, (const T*)w, bias, \
                       in_zp, w_zp, rp, (OT*)out, flag_word)

#define TMI_DEFINE_CONV_LAUNCH(FUNC, KERNEL, LABEL)                                                                 \
    const char* FUNC(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,        \
                     const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,         \
                     void* out, uint32_t* flag_word)                                                                \
    {                                                                                                               \
        const int64_t total = (int64_t)g.N * g.OH * g.OW * g.OC;                                                    \
        if (total == 0)                                                                                             \
            return LABEL "_empty";                                                                                  \
        if (in_dtype == TMI_INT8)                                                                                   \
        {                                                                                                           \
            if (out_dtype == TMI_INT32)                                                                             \
                TMI_LAUNCH_CONV(KERNEL, int8_t, int32_t);                                                           \
            else if (out_dtype == TMI_INT16 && rp.enabled)                                                          \
                TMI_LAUNCH_CONV(KERNEL, int8_t, int16_t);                                                           \
            else if (out_dtype == TMI_INT8 && rp.enabled)                                                           \
                TMI_LAUNCH_CONV(KERNEL, int8_t, int8_t);                                                            \
            else                                                                                                    \
                return nullptr;                                                                                     \
            return rp.enabled ? LABEL "_i8_rescale" : LABEL "_i8";                                                  \
        }                                                                                                           \
        if (in_dtype == TMI_FP16 && out_dtype == TMI_FP16)                                                          \
        {                                                                                                           \
            TMI_LAUNCH_CONV(KERNEL, _Float16, _Float16);                                                            \
            return LABEL "_f16";                                                                                    \
        }                                                                                                           \
        if (in_dtype == TMI_BF16 && out_dtype == TMI_BF16)                                                          \
        {                                                                                                           \
            TMI_LAUNCH_CONV(KERNEL, bf16_t, bf16_t);                                                                \
            return LABEL "_bf16";                                                                                   \
        }                                                                                                           \
        if (in_dtype == TMI_FP32 && out_dtype == TMI_FP32)                                                          \
        {                                                                                                           \
            TMI_LAUNCH_CONV(KERNEL, float, float);                                                                  \
            return LABEL "_f32";                                                                                    \
        }                                                                                                           \
        return nullptr;                                                                                             \
    }

TMI_DEFINE_CONV_LAUNCH(launch_conv2d_direct, conv2d_direct_kernel, "conv2d_direct")
TMI_DEFINE_CONV_LAUNCH(launch_depthwise_direct, depthwise_direct_kernel, "depthwise_direct")

const char* launch_matmul_direct(hipStream_t st, int32_t in_dtype, int32_t N, int32_t H, int32_t C, int32_t W,
                                 const void* a, const void* b, int32_t a_zp, int32_t b_zp, void* out)
{
    const int64_t total = (int64_t)N * H * W;
    if (total == 0)
        return "matmul_direct_empty";
    if (in_dtype == TMI_INT8)
    {
        hipLaunchKernelGGL((matmul_direct_kernel<int8_t, int32_t>), dim3(grid_for(total)), dim3(256), 0, st, N, H, C,
                           W, (const int8_t*)a, (const int8_t*)b, a_zp, b_zp, (int32_t*)out);
        return "matmul_direct_i8";
    }
    if (in_dtype == TMI_FP16)
    {
        hipLaunchKernelGGL((matmul_direct_kernel<_Float16, float>), dim3(grid_for(total)), dim3(256), 0, st, N, H, C,
                           W, (const _Float16*)a, (const _Float16*)b, 0, 0, (float*)out);
        return "matmul_direct_f16";
    }
    if (in_dtype == TMI_BF16)
    {
        hipLaunchKernelGGL((matmul_direct_kernel<bf16_t, float>), dim3(grid_for(total)), dim3(256), 0, st, N, H, C,
                           W, (const bf16_t*)a, (const bf16_t*)b, 0, 0, (float*)out);
        return "matmul_direct_bf16";
    }
    if (in_dtype == TMI_FP32)
    {
        hipLaunchKernelGGL((matmul_direct_kernel<float, float>), dim3(grid_for(total)), dim3(256), 0, st, N, H, C, W,
                           (const float*)a, (const float*)b, 0, 0, (float*)out);
        return "matmul_direct_f32";
    }
    return nullptr;
}

const char* launch_conv_i16_direct(hipStream_t st, bool depthwise, const ConvGeom& g, const void* in, const void* w,
                                   const void* bias, int32_t w_zp, void* out)
{
    const int64_t total = (int64_t)g.N * g.OH * g.OW * g.OC;
    if (total == 0)
        return "conv_direct_empty";
    if (depthwise)
        hipLaunchKernelGGL((conv_i16_direct_kernel<true>), dim3(grid_for(total)), dim3(256), 0, st, g, (const int16_t*)in,
                           (const int8_t*)w, (const int64_t*)bias, w_zp, (int64_t*)out);
    else
        hipLaunchKernelGGL((conv_i16_direct_kernel<false>), dim3(grid_for(total)), dim3(256), 0, st, g, (const int16_t*)in,
                           (const int8_t*)w, (const int64_t*)bias, w_zp, (int64_t*)out);
    return depthwise ? "depthwise_direct_i16_i48" : "conv2d_direct_i16_i48";
}

const char* launch_matmul_i16_direct(hipStream_t st, int32_t N, int32_t H, int32_t C, int32_t W, const void* a, const void* b,
                                     void* out)
{
    const int64_t total = (int64_t)N * H * W;
    if (total == 0)
        return "matmul_direct_empty";
    hipLaunchKernelGGL(matmul_i16_direct_kernel, dim3(grid_for(total)), dim3(256), 0, st, N, H, C, W, (const int16_t*)a,
                       (const int16_t*)b, (int64_t*)out);
    return "matmul_direct_i16_i48";
}

}    // namespace tmi
