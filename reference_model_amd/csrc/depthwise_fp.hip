// DEPTHWISE_CONV2D for fp16 / bf16 (channel multiplier 1, channels a multiple of 8): the bandwidth-bound case.
//
//   out[n][oy][ox][c] = bias[c] + sum_{ky,kx inside the image} in[n][oy*sy - pt + ky*dy][ox*sx - pl + kx*dx][c] * w[ky][kx][c]
//                                                                       (tensor_ops.cpp:1262-1340 with fp32 accumulation)
//
// A lane owns 8 consecutive channels (16 bytes) and produces them for one output pixel per iteration: consecutive lanes
// take consecutive channel groups of a pixel, then the next pixel, so every tap load and the store of a wave are contiguous
// runs of NHWC memory.  The sum runs over the taps in (ky, kx) order in fp32, a tap outside the image is skipped as the
// reference skips it, and the bias is added last: the same arithmetic as the reference's loop nest, operation for operation
// (a product of two fp16 or two bf16 values is exact in fp32, so the fused multiply-add rounds as multiply and add would).
// For 3 x 3 taps the lane's weights stay in registers, packed as they lie in memory, for all the pixels it visits, and a
// wave whose pixels are all interior issues its nine tap loads before it uses the first.
#include <type_traits>

#include "tmi_mfma.h"

namespace tmi
{

struct DwFpArgs
{
    ConvGeom g;
    const uint8_t* in;
    const uint8_t* w;
    const void* bias;
    uint8_t* out;
    int32_t cgs;         // channel groups of 8 per pixel
    int32_t ppi;         // pixels a workgroup covers per iteration = 256 / cgs
    int32_t iters;       // iterations per workgroup
    int32_t total_px;    // N * OH * OW
    int32_t blocks;      // workgroups that have work
    FastDiv div_cgs, div_ow, div_oh;
};

template <typename T>
__device__ __forceinline__ void unpack8(const v4i& raw, float (&f)[8])
{
    if constexpr (std::is_same<T, _Float16>::value)
    {
        const v8h h = __builtin_bit_cast(v8h, raw);
#pragma unroll
        for (int i = 0; i < 8; i++)
            f[i] = (float)h[i];
    }
    else
    {
#pragma unroll
        for (int i = 0; i < 4; i++)
        {
            f[2 * i]     = __uint_as_float((uint32_t)raw[i] << 16);
            f[2 * i + 1] = __uint_as_float((uint32_t)raw[i] & 0xffff0000u);
        }
    }
}

template <typename T>
__device__ __forceinline__ void accumulate8(const v4i& x, const v4i& w, float (&acc)[8])
{
    float xf[8], wf[8];
    unpack8<T>(x, xf);
    unpack8<T>(w, wf);
#pragma unroll
    for (int i = 0; i < 8; i++)
        acc[i] = __builtin_fmaf(xf[i], wf[i], acc[i]);
}

template <typename T, bool K33>
__global__ __launch_bounds__(256) void depthwise_fp_vec_kernel(DwFpArgs a)
{
    asm volatile("" ::"s"(a.g.N), "s"(a.g.bias_len), "s"(a.out), "s"(a.blocks), "s"(a.div_oh.d));
    const ConvGeom& g  = a.g;
    const int tid      = threadIdx.x;
    const int slot     = fdiv(tid, a.div_cgs);    // pixel slot of this lane inside an iteration
    const bool lane_on = slot < a.ppi;
    const int cg       = lane_on ? tid - slot * a.cgs : 0;
    const int cb       = cg * 16;                 // byte offset of the lane's channels inside a pixel
    const int CB       = g.IC * 2;                // bytes of a pixel

    // consecutive workgroups are dealt to the 8 XCDs in turn: give each XCD a contiguous run of pixels, so that the input
    // rows shared by vertically adjacent outputs are found in its L2
    const uint32_t per = gridDim.x >> 3;
    const uint32_t bid = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
    if (bid >= (uint32_t)a.blocks)
        return;

    float bias[8];
    {
        const T* bp = reinterpret_cast<const T*>(a.bias);
#pragma unroll
        for (int i = 0; i < 8; i++)
            bias[i] = load_as_float<T>(bp, g.bias_len == 1 ? 0 : cg * 8 + i);
    }
    v4i wreg[K33 ? 9 : 1];
    if constexpr (K33)
    {
#pragma unroll
        for (int t = 0; t < 9; t++)
            wreg[t] = *reinterpret_cast<const v4i*>(a.w + (uint32_t)(t * CB + cb));
    }

    for (int it = 0; it < a.iters; it++)
    {
        const int pix  = (bid * a.iters + it) * a.ppi + slot;
        const bool on  = lane_on && pix < a.total_px;
        const int pixc = on ? pix : 0;
        const int row  = fdiv(pixc, a.div_ow);    // n * OH + oy
        const int ox   = pixc - row * g.OW;
        const int n    = fdiv(row, a.div_oh);
        const int oy   = row - n * g.OH;
        // (a lane without a pixel reads as if its window lay at the image's origin, and stores nothing)
        const int y0   = on ? oy * g.stride_y - g.pad_top : 0;
        const int x0   = on ? ox * g.stride_x - g.pad_left : 0;
        // byte offset of tap (0, 0) in the input tensor (below 2^31 in magnitude; it may be negative at the top / left
        // border, the taps that are used bring it back into the tensor)
        const int voff = ((n * g.IH + y0) * g.IW + x0) * CB + cb;
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; i++)
            acc[i] = 0.0f;
        if constexpr (K33)
        {
            const bool interior = y0 >= 0 && x0 >= 0 && y0 + 2 * g.dil_y < g.IH && x0 + 2 * g.dil_x < g.IW;
            if (__all(interior))
            {
                v4i d[9];
#pragma unroll
                for (int t = 0; t < 9; t++)
                    d[t] = *reinterpret_cast<const v4i*>(a.in + ((t / 3) * g.dil_y * g.IW + (t % 3) * g.dil_x) * CB + voff);
#pragma unroll
                for (int t = 0; t < 9; t++)
                    accumulate8<T>(d[t], wreg[t], acc);
            }
            else
            {
#pragma unroll
                for (int t = 0; t < 9; t++)
                {
                    const int y = y0 + (t / 3) * g.dil_y, x = x0 + (t % 3) * g.dil_x;
                    if ((uint32_t)y < (uint32_t)g.IH && (uint32_t)x < (uint32_t)g.IW)
                    {
                        const v4i d = *reinterpret_cast<const v4i*>(a.in + ((t / 3) * g.dil_y * g.IW + (t % 3) * g.dil_x) * CB + voff);
                        accumulate8<T>(d, wreg[t], acc);
                    }
                }
            }
        }
        else
        {
            for (int ky = 0; ky < g.KH; ky++)
            {
                const int y = y0 + ky * g.dil_y;
                if ((uint32_t)y >= (uint32_t)g.IH)
                    continue;
                for (int kx = 0; kx < g.KW; kx++)
                {
                    const int x = x0 + kx * g.dil_x;
                    if ((uint32_t)x >= (uint32_t)g.IW)
                        continue;
                    const v4i d  = *reinterpret_cast<const v4i*>(a.in + (ky * g.dil_y * g.IW + kx * g.dil_x) * CB + voff);
                    const v4i wv = *reinterpret_cast<const v4i*>(a.w + (uint32_t)((ky * g.KW + kx) * CB + cb));
                    accumulate8<T>(d, wv, acc);
                }
            }
        }
        if (on)
        {
            union
            {
                T e[8];
                v4i q;
            } u;
#pragma unroll
            for (int i = 0; i < 8; i++)
                store_from_float(&u.e[i], bias[i] + acc[i]);
            *reinterpret_cast<v4i*>(a.out + (size_t)(uint32_t)pix * CB + cb) = u.q;
        }
    }
}

template <typename T>
static void launch_dw_fp(hipStream_t st, const DwFpArgs& a, int grid, bool k33)
{
    if (k33)
        hipLaunchKernelGGL((depthwise_fp_vec_kernel<T, true>), dim3(grid), dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL((depthwise_fp_vec_kernel<T, false>), dim3(grid), dim3(256), 0, st, a);
}

// Eligible: fp16 / bf16 in and out, multiplier 1, channels a multiple of 8 (at most 2048), 16-byte aligned tensors.
// nullptr otherwise; the caller then goes to the one-result-per-lane kernel.
const char* launch_depthwise_fp_vec(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                                    const void* w, const void* bias, void* out)
{
    if ((in_dtype != TMI_FP16 && in_dtype != TMI_BF16) || out_dtype != in_dtype || g.M != 1 || (g.IC & 7) != 0 || g.IC == 0 ||
        g.IC > 2048)
        return nullptr;
    if (((((uintptr_t)in | (uintptr_t)w | (uintptr_t)out) & 15) != 0) || ((uintptr_t)bias & 1) != 0)
        return nullptr;
    const int64_t total_px = (int64_t)g.N * g.OH * g.OW;
    // 32-bit byte offsets inside both tensors and exact multiply-high divisions of the pixel index
    if (total_px == 0 || total_px * g.OW >= (int64_t(1) << 31) || (total_px / g.OW + 1) * g.OH >= (int64_t(1) << 31) ||
        (int64_t)g.N * g.IH * g.IW * g.IC * 2 >= (int64_t(1) << 31) || total_px * g.IC * 2 >= (int64_t(1) << 32) ||
        (int64_t)g.KH * g.KW * g.IC * 2 >= (int64_t(1) << 31))
        return nullptr;

    DwFpArgs a{};
    a.g = g, a.in = (const uint8_t*)in, a.w = (const uint8_t*)w, a.bias = bias, a.out = (uint8_t*)out;
    a.cgs      = g.IC / 8;
    a.ppi      = 256 / a.cgs;
    a.total_px = (int)total_px;
    // enough workgroups to give every CU several, few enough that a lane's weights serve a few pixels
    const int64_t px_iters = (total_px + a.ppi - 1) / a.ppi;
    a.iters                = px_iters >= 256 * 64 ? 8 : (px_iters >= 256 * 16 ? 4 : (px_iters >= 256 * 8 ? 2 : 1));
    a.blocks               = (int)((px_iters + a.iters - 1) / a.iters);
    a.div_cgs              = make_fastdiv(a.cgs);
    a.div_ow               = make_fastdiv(g.OW);
    a.div_oh               = make_fastdiv(g.OH);
    const int grid         = ((a.blocks + 7) / 8) * 8;
    const bool k33         = g.KH == 3 && g.KW == 3;
    if (in_dtype == TMI_FP16)
        launch_dw_fp<_Float16>(st, a, grid, k33);
    else
        launch_dw_fp<bf16_t>(st, a, grid, k33);
    return in_dtype == TMI_FP16 ? "depthwise_vec_f16" : "depthwise_vec_bf16";
}

}    // namespace tmi
