// DEPTHWISE_CONV2D for the bandwidth-bound case (channel multiplier 1, channels a multiple of 16):
// every lane produces 16 consecutive channels of one output pixel from KH*KW 16-byte NHWC loads, with the
// bias / zero-point / RESCALE / CLAMP epilogue fused, so the op reads the input once (plus tap overlap served
// by L1/L2) and writes 1 byte per output element.  Consecutive lanes take consecutive 16-channel chunks of the
// same pixel, then the next pixel, so loads and stores of a wave are contiguous runs of NHWC memory.
//
// Out-of-image taps contribute nothing in the reference (tensor_ops.cpp:1302-1313); they are skipped here too,
// which keeps the arithmetic the plain sum((a - za) * (w - zw)).
#include "tmi_kernels.h"

namespace tmi
{

typedef int v4i __attribute__((ext_vector_type(4)));

template <bool RESCALE>
__global__ __launch_bounds__(256) void depthwise_vec16_kernel(ConvGeom g, const int8_t* __restrict__ in,
                                                              const int8_t* __restrict__ w,
                                                              const int32_t* __restrict__ bias, int32_t za,
                                                              int32_t zw, RescaleParams rp, int32_t out_dtype,
                                                              void* __restrict__ out, uint32_t* flag_word)
{
    const int chunks     = g.IC >> 4;
    const int64_t total  = (int64_t)g.N * g.OH * g.OW * chunks;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    uint32_t flags       = 0;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride)
    {
        const int ch = (int)(idx % chunks);
        int64_t t    = idx / chunks;
        const int ox = (int)(t % g.OW);
        t /= g.OW;
        const int oy = (int)(t % g.OH);
        const int n  = (int)(t / g.OH);
        const int c0 = ch << 4;

        int32_t acc[16];
#pragma unroll
        for (int c = 0; c < 16; c++)
            acc[c] = 0;
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
                const v4i av = *reinterpret_cast<const v4i*>(in + (((int64_t)n * g.IH + y) * g.IW + x) * g.IC + c0);
                const v4i wv = *reinterpret_cast<const v4i*>(w + ((int64_t)ky * g.KW + kx) * g.IC + c0);
#pragma unroll
                for (int c = 0; c < 16; c++)
                {
                    const int32_t a = (int32_t)(int8_t)(av[c >> 2] >> (8 * (c & 3))) - za;
                    const int32_t b = (int32_t)(int8_t)(wv[c >> 2] >> (8 * (c & 3))) - zw;
                    acc[c] += a * b;
                }
            }
        }
        const int64_t o = (((int64_t)n * g.OH + oy) * g.OW + ox) * g.OC + c0;
        int32_t res[16];
#pragma unroll
        for (int q = 0; q < 4; q++)
        {
            v4i b4;
            if (g.bias_len == 1)
                b4 = v4i{ bias[0], bias[0], bias[0], bias[0] };
            else
                b4 = *reinterpret_cast<const v4i*>(bias + c0 + 4 * q);
#pragma unroll
            for (int r = 0; r < 4; r++)
                res[4 * q + r] = acc[4 * q + r] + b4[r];
            if constexpr (RESCALE)
            {
                v4i m4;
                int sh;
                if (rp.per_channel)
                {
                    m4 = *reinterpret_cast<const v4i*>(reinterpret_cast<const int32_t*>(rp.multiplier) + c0 + 4 * q);
                    sh = *reinterpret_cast<const int*>(rp.shift + c0 + 4 * q);
                }
                else
                {
                    const int32_t m = reinterpret_cast<const int32_t*>(rp.multiplier)[0];
                    const int s1    = rp.shift[0] & 0xff;
                    m4              = v4i{ m, m, m, m };
                    sh              = s1 * 0x01010101;
                }
#pragma unroll
                for (int r = 0; r < 4; r++)
                {
                    const ChannelScale cs =
                        make_channel_scale(m4[r], (int32_t)(int8_t)(sh >> (8 * r)), rp.double_round, flags);
                    res[4 * q + r] = fast_rescale(res[4 * q + r], cs, rp.out_zp, rp.lo, rp.hi, flags);
                }
            }
        }
        if (!RESCALE || out_dtype == TMI_INT32)
        {
            int32_t* p = reinterpret_cast<int32_t*>(out) + o;
#pragma unroll
            for (int q = 0; q < 4; q++)
                *reinterpret_cast<v4i*>(p + 4 * q) = v4i{ res[4 * q], res[4 * q + 1], res[4 * q + 2], res[4 * q + 3] };
        }
        else if (out_dtype == TMI_INT8)
        {
            v4i pk;
#pragma unroll
            for (int q = 0; q < 4; q++)
                pk[q] = (res[4 * q] & 0xff) | ((res[4 * q + 1] & 0xff) << 8) | ((res[4 * q + 2] & 0xff) << 16) |
                        ((res[4 * q + 3] & 0xff) << 24);
            *reinterpret_cast<v4i*>(reinterpret_cast<int8_t*>(out) + o) = pk;
        }
        else
        {
            v4i pk[2];
#pragma unroll
            for (int q = 0; q < 8; q++)
                pk[q >> 2][q & 3] = (res[2 * q] & 0xffff) | ((res[2 * q + 1] & 0xffff) << 16);
            reinterpret_cast<v4i*>(reinterpret_cast<int16_t*>(out) + o)[0] = pk[0];
            reinterpret_cast<v4i*>(reinterpret_cast<int16_t*>(out) + o)[1] = pk[1];
        }
    }
    raise_flags(flag_word, flags);
}

// Eligible: INT8, multiplier 1, channels a multiple of 16, 16-byte aligned tensors, and either no RESCALE or
// one that qualifies for fast_rescale() with 32-bit per-channel or per-tensor multipliers.
const char* launch_depthwise_vec(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g,
                                 const void* in, const void* w, const void* bias, int32_t in_zp, int32_t w_zp,
                                 const RescaleParams& rp, void* out, uint32_t* flag_word)
{
    if (in_dtype != TMI_INT8 || g.M != 1 || (g.IC & 15) != 0 || g.IC == 0)
        return nullptr;
    if ((((uintptr_t)in | (uintptr_t)w | (uintptr_t)out | (uintptr_t)bias) & 15) != 0)
        return nullptr;
    if (rp.enabled && (!rp.fast || (((uintptr_t)rp.multiplier & 15) != 0) || (((uintptr_t)rp.shift & 3) != 0)))
        return nullptr;
    const int64_t total = (int64_t)g.N * g.OH * g.OW * (g.IC >> 4);
    if (total == 0)
        return nullptr;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 32)
        blocks = 256 * 32;
    if (rp.enabled)
        hipLaunchKernelGGL(depthwise_vec16_kernel<true>, dim3((int)blocks), dim3(256), 0, st, g, (const int8_t*)in,
                           (const int8_t*)w, (const int32_t*)bias, in_zp, w_zp, rp, out_dtype, out, flag_word);
    else
        hipLaunchKernelGGL(depthwise_vec16_kernel<false>, dim3((int)blocks), dim3(256), 0, st, g, (const int8_t*)in,
                           (const int8_t*)w, (const int32_t*)bias, in_zp, w_zp, rp, out_dtype, out, flag_word);
    return rp.enabled ? "depthwise_vec16_i8_rescale" : "depthwise_vec16_i8";
}

}    // namespace tmi
