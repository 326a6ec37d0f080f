// The two extra passes of the reference's floating-point compliance flow, on the device:
//
//  * precise mode (--precise_mode: every floating-point tensor is evaluated in fp64) of CONV2D,
//    DEPTHWISE_CONV2D and MATMUL: operands in their storage type (fp16 / bf16 / fp32), products and sums in
//    fp64 in the reference's loop order - taps (ky, kx, ic), bias added last - so the result is the same
//    fp64 number the reference's loop nest produces (tensor_ops.cpp:843-882, 1291-1334, 1463-1500);
//  * bounds mode (bounds_mode: the same sums over absolute values, tensor_ops.cpp:757-765);
//  * the DOT_PRODUCT check of the verifier library (reference_model/src/verify/verify_dot_product.cpp:30-139)
//    as a reduction: per element the error in units of the bound, then sum, sum of squares, largest
//    magnitude and the number of elements that fail on their own.
//
// These are checkers for the fast kernels at shapes where a scalar CPU pass takes seconds to minutes; one
// output element per lane, nothing tiled.
#include "tmi_kernels.h"

namespace tmi
{

typedef int pr_v4i __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ double widen(const void* p, size_t i);
template <>
__device__ __forceinline__ double widen<_Float16>(const void* p, size_t i)
{
    return (double)reinterpret_cast<const _Float16*>(p)[i];
}
template <>
__device__ __forceinline__ double widen<bf16_t>(const void* p, size_t i)
{
    return (double)bf16_to_float(reinterpret_cast<const bf16_t*>(p)[i]);
}
template <>
__device__ __forceinline__ double widen<float>(const void* p, size_t i)
{
    return (double)reinterpret_cast<const float*>(p)[i];
}

struct PreciseConvArgs
{
    ConvGeom g;
    const void* in;
    const void* w;
    const void* bias;
    double* out;
    int64_t total;
    int32_t abs_mode;
    int32_t depthwise;
    int32_t vec;    // channel vectors are whole, aligned 16-byte pieces
    // bounds mode without local_bound (tensor_ops.cpp:797-801, 1252-1256): every input element is replaced by the
    // largest magnitude of the input tensor, found by absmax_kernel; nullptr otherwise
    const double* input_abs_max;
};

// The largest |x| of a tensor into *out (zero before the launch; non-negative doubles order like their bit patterns).
template <typename T>
__global__ __launch_bounds__(256) void absmax_kernel(const void* x, int64_t n, double* out)
{
    __shared__ double red[256];
    double m             = 0.0;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        m = fmax(m, fabs(widen<T>(x, (size_t)i)));
    red[threadIdx.x] = m;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1)
    {
        if ((int)threadIdx.x < s)
            red[threadIdx.x] = fmax(red[threadIdx.x], red[threadIdx.x + s]);
        __syncthreads();
    }
    if (threadIdx.x == 0)
        atomicMax(reinterpret_cast<unsigned long long*>(out), (unsigned long long)__double_as_longlong(red[0]));
}

__global__ void store_zero_kernel(double* p)
{
    *p = 0.0;
}

template <typename T>
__global__ __launch_bounds__(256) void precise_conv_kernel(PreciseConvArgs a)
{
    const ConvGeom& g    = a.g;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const bool flat      = a.input_abs_max != nullptr;    // the input is one constant
    const double gmax    = flat ? *a.input_abs_max : 0.0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.total; i += stride)
    {
        const int oc      = (int)(i % g.OC);
        const int64_t pix = i / g.OC;
        const int ow      = (int)(pix % g.OW);
        const int oh      = (int)((pix / g.OW) % g.OH);
        const int n       = (int)(pix / ((int64_t)g.OW * g.OH));
        double acc        = 0.0;
        for (int ky = 0; ky < g.KH; ky++)
        {
            const int y = oh * g.stride_y - g.pad_top + ky * g.dil_y;
            if (y < 0 || y >= g.IH)
                continue;
            for (int kx = 0; kx < g.KW; kx++)
            {
                const int x = ow * g.stride_x - g.pad_left + kx * g.dil_x;
                if (x < 0 || x >= g.IW)
                    continue;
                const size_t in_base = (((size_t)n * g.IH + y) * g.IW + x) * g.IC;
                if (a.depthwise)
                {
                    // weight [KH, KW, C, M], output channel c * M + m
                    const int c = oc / g.M, m = oc - c * g.M;
                    double u = widen<T>(a.in, in_base + c);
                    double v = widen<T>(a.w, (((size_t)ky * g.KW + kx) * g.IC + c) * g.M + m);
                    if (a.abs_mode)
                        u = flat ? gmax : fabs(u), v = fabs(v);
                    acc = acc + u * v;
                }
                else
                {
                    const size_t w_base = (((size_t)oc * g.KH + ky) * g.KW + kx) * g.IC;
                    int ic              = 0;
                    if (a.vec)
                    {
                        // 16 bytes of both rows per step; the products still enter the sum one by one, in order
                        constexpr int V = 16 / (int)sizeof(T);
                        for (; ic + V <= g.IC; ic += V)
                        {
                            alignas(16) T xu[V], xw[V];
                            *reinterpret_cast<pr_v4i*>(xu) =
                                *reinterpret_cast<const pr_v4i*>(reinterpret_cast<const T*>(a.in) + in_base + ic);
                            *reinterpret_cast<pr_v4i*>(xw) =
                                *reinterpret_cast<const pr_v4i*>(reinterpret_cast<const T*>(a.w) + w_base + ic);
#pragma unroll
                            for (int e = 0; e < V; e++)
                            {
                                double u = widen<T>(xu, e), v = widen<T>(xw, e);
                                if (a.abs_mode)
                                    u = flat ? gmax : fabs(u), v = fabs(v);
                                acc = acc + u * v;
                            }
                        }
                    }
                    for (; ic < g.IC; ic++)
                    {
                        double u = widen<T>(a.in, in_base + ic);
                        double v = widen<T>(a.w, w_base + ic);
                        if (a.abs_mode)
                            u = flat ? gmax : fabs(u), v = fabs(v);
                        acc = acc + u * v;
                    }
                }
            }
        }
        double b = widen<T>(a.bias, g.bias_len == 1 ? 0 : oc);
        if (a.abs_mode)
            b = fabs(b);
        a.out[i] = acc + b;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void precise_matmul_kernel(int32_t H, int32_t C, int32_t W, int64_t total,
                                                             const void* av, const void* bv, int32_t abs_mode,
                                                             int32_t vec, double* out)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride)
    {
        const int w       = (int)(i % W);
        const int64_t row = i / W;    // n * H + h
        const int64_t n   = row / H;
        double acc        = 0.0;
        int c             = 0;
        if (vec)
        {
            constexpr int V = 16 / (int)sizeof(T);
            for (; c + V <= C; c += V)
            {
                alignas(16) T xu[V];
                *reinterpret_cast<pr_v4i*>(xu) =
                    *reinterpret_cast<const pr_v4i*>(reinterpret_cast<const T*>(av) + (size_t)row * C + c);
#pragma unroll
                for (int e = 0; e < V; e++)
                {
                    double u = widen<T>(xu, e);
                    double v = widen<T>(bv, ((size_t)n * C + c + e) * W + w);
                    if (abs_mode)
                        u = fabs(u), v = fabs(v);
                    acc = acc + u * v;
                }
            }
        }
        for (; c < C; c++)
        {
            double u = widen<T>(av, (size_t)row * C + c);
            double v = widen<T>(bv, ((size_t)n * C + c) * W + w);
            if (abs_mode)
                u = fabs(u), v = fabs(v);
            acc = acc + u * v;
        }
        out[i] = acc;
    }
}

static int grid_for(int64_t total)
{
    int64_t blocks = (total + 255) / 256;
    return (int)(blocks > 256 * 64 ? 256 * 64 : blocks);
}

const char* launch_conv_precise(hipStream_t st, int32_t in_dtype, bool depthwise, const ConvGeom& g, const void* in,
                                const void* w, const void* bias, int32_t abs_mode, double* abs_max_slot, double* out)
{
    PreciseConvArgs a{};
    a.g = g, a.in = in, a.w = w, a.bias = bias, a.out = out, a.abs_mode = abs_mode, a.depthwise = depthwise ? 1 : 0;
    a.total = (int64_t)g.N * g.OH * g.OW * g.OC;
    const int eb = in_dtype == TMI_FP32 ? 4 : 2;
    a.vec        = ((int64_t)g.IC * eb) % 16 == 0 && (((uintptr_t)in | (uintptr_t)w) & 15) == 0;
    if (abs_mode && abs_max_slot)
    {
        // the bounds pass of an operator without local_bound: the input tensor's largest magnitude first
        const int64_t n_in = (int64_t)g.N * g.IH * g.IW * g.IC;
        const dim3 rgrid(grid_for(n_in)), rblock(256);
        hipLaunchKernelGGL(store_zero_kernel, dim3(1), dim3(1), 0, st, abs_max_slot);
        switch (in_dtype)
        {
            case TMI_FP16: hipLaunchKernelGGL(absmax_kernel<_Float16>, rgrid, rblock, 0, st, in, n_in, abs_max_slot); break;
            case TMI_BF16: hipLaunchKernelGGL(absmax_kernel<bf16_t>, rgrid, rblock, 0, st, in, n_in, abs_max_slot); break;
            case TMI_FP32: hipLaunchKernelGGL(absmax_kernel<float>, rgrid, rblock, 0, st, in, n_in, abs_max_slot); break;
            default: return nullptr;
        }
        a.input_abs_max = abs_max_slot;
    }
    switch (in_dtype)
    {
        case TMI_FP16: hipLaunchKernelGGL(precise_conv_kernel<_Float16>, dim3(grid_for(a.total)), dim3(256), 0, st, a); break;
        case TMI_BF16: hipLaunchKernelGGL(precise_conv_kernel<bf16_t>, dim3(grid_for(a.total)), dim3(256), 0, st, a); break;
        case TMI_FP32: hipLaunchKernelGGL(precise_conv_kernel<float>, dim3(grid_for(a.total)), dim3(256), 0, st, a); break;
        default: return nullptr;
    }
    return abs_mode ? "conv_bounds_f64" : "conv_precise_f64";
}

const char* launch_matmul_precise(hipStream_t st, int32_t in_dtype, int32_t N, int32_t H, int32_t C, int32_t W,
                                  const void* a, const void* b, int32_t abs_mode, double* out)
{
    const int64_t total = (int64_t)N * H * W;
    const dim3 grid(grid_for(total)), block(256);
    const int eb      = in_dtype == TMI_FP32 ? 4 : 2;
    const int32_t vec = ((int64_t)C * eb) % 16 == 0 && ((uintptr_t)a & 15) == 0;
    switch (in_dtype)
    {
        case TMI_FP16: hipLaunchKernelGGL(precise_matmul_kernel<_Float16>, grid, block, 0, st, H, C, W, total, a, b, abs_mode, vec, out); break;
        case TMI_BF16: hipLaunchKernelGGL(precise_matmul_kernel<bf16_t>, grid, block, 0, st, H, C, W, total, a, b, abs_mode, vec, out); break;
        case TMI_FP32: hipLaunchKernelGGL(precise_matmul_kernel<float>, grid, block, 0, st, H, C, W, total, a, b, abs_mode, vec, out); break;
        default: return nullptr;
    }
    return abs_mode ? "matmul_bounds_f64" : "matmul_precise_f64";
}

// ---- DOT_PRODUCT check ---------------------------------------------------------------------------------------
// results: [0] sum of errors, [1] sum of squared errors, [2] largest |error| (as a double whose bit pattern is
// ordered like the value: non-negative), counts: [0] elements that fail on their own
struct DpCheckArgs
{
    const void* imp;
    const double* ref;
    const double* bnd;
    int64_t n;
    int32_t abs_bound;
    int32_t normal_frac;
    double normal_min;
    double* results;
    unsigned long long* counts;
};

template <typename T>
__device__ __forceinline__ bool overflows(double v);
template <>
__device__ __forceinline__ bool overflows<_Float16>(double v)
{
    return isinf((float)(_Float16)v);
}
template <>
__device__ __forceinline__ bool overflows<bf16_t>(double v)
{
    return isinf(bf16_to_float(float_to_bf16((float)v)));
}
template <>
__device__ __forceinline__ bool overflows<float>(double v)
{
    return isinf((float)v);
}

template <typename T>
__global__ __launch_bounds__(256) void dp_check_kernel(DpCheckArgs a)
{
    __shared__ double red[3][256];
    __shared__ unsigned long long bad_s[256];
    double sum = 0.0, sumsq = 0.0, worst = 0.0;
    unsigned long long bad = 0;
    const double unit_scale = exp2(-1.0 - a.normal_frac);
    const int64_t stride    = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n; i += stride)
    {
        const double ref = a.ref[i], bnd = a.bnd[i], imp = widen<T>(a.imp, (size_t)i);
        double err = 0.0;
        bool ok    = true;
        if (ref != ref)
            ok = imp != imp;    // a NaN reference must be matched
        else if (bnd != bnd)
            ok = true;          // no accuracy requirement under a NaN bound
        else if (overflows<T>(bnd * (1.0 + a.abs_bound * unit_scale)))
            ok = true;          // the dot product may overflow: no accuracy limit
        else if (bnd == 0.0)
            ok = ref == 0.0 && imp == 0.0;
        else
        {
            const double unit = fmax(bnd * unit_scale, a.normal_min);
            err               = (imp - ref) / unit;
            ok                = fabs(err) <= (double)a.abs_bound;
        }
        if (!ok)
            bad++;
        sum += err, sumsq += err * err;
        worst = fmax(worst, fabs(err));
    }
    const int t = threadIdx.x;
    red[0][t] = sum, red[1][t] = sumsq, red[2][t] = worst, bad_s[t] = bad;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1)
    {
        if (t < s)
        {
            red[0][t] += red[0][t + s];
            red[1][t] += red[1][t + s];
            red[2][t] = fmax(red[2][t], red[2][t + s]);
            bad_s[t] += bad_s[t + s];
        }
        __syncthreads();
    }
    if (t == 0)
    {
        atomicAdd(&a.results[0], red[0][0]);
        atomicAdd(&a.results[1], red[1][0]);
        // non-negative doubles order like their bit patterns
        atomicMax(reinterpret_cast<unsigned long long*>(&a.results[2]),
                  (unsigned long long)__double_as_longlong(red[2][0]));
        atomicAdd(&a.counts[0], bad_s[0]);
    }
}

// results (3 doubles) and counts (1 word) must be zero before the launch
const char* launch_dp_check(hipStream_t st, int32_t out_dtype, int64_t n, const void* imp, const double* ref,
                            const double* bnd, int32_t abs_bound, double* results, unsigned long long* counts)
{
    DpCheckArgs a{};
    a.imp = imp, a.ref = ref, a.bnd = bnd, a.n = n, a.abs_bound = abs_bound, a.results = results, a.counts = counts;
    int64_t blocks = (n + 255) / 256;
    const dim3 grid((int)(blocks > 2048 ? 2048 : blocks)), block(256);
    switch (out_dtype)
    {
        case TMI_FP16:
            a.normal_frac = 10, a.normal_min = 0x1p-14;
            hipLaunchKernelGGL(dp_check_kernel<_Float16>, grid, block, 0, st, a);
            break;
        case TMI_BF16:
            a.normal_frac = 7, a.normal_min = 0x1p-126;
            hipLaunchKernelGGL(dp_check_kernel<bf16_t>, grid, block, 0, st, a);
            break;
        case TMI_FP32:
            a.normal_frac = 23, a.normal_min = 0x1p-126;
            hipLaunchKernelGGL(dp_check_kernel<float>, grid, block, 0, st, a);
            break;
        default: return nullptr;
    }
    return "dot_product_check";
}

}    // namespace tmi
