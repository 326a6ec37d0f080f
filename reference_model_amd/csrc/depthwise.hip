// DEPTHWISE_CONV2D for the bandwidth-bound case (int8, channel multiplier 1, channels a multiple of 4).
//
// A lane owns 4 consecutive channels and produces them for one output pixel per iteration: consecutive lanes
// take consecutive channel groups of a pixel, then the next pixel, so every tap load and the store of a wave
// are contiguous runs of NHWC memory (one dword per lane).  The per-channel constants of a lane -- its
// weights, bias, zero-point terms, RESCALE multiplier / shift / rounding terms -- are set up once in registers
// and reused for every pixel the lane visits.
//
// Arithmetic: there is no sum across channels to feed a dot-product instruction, but there is one across taps.
// Four taps of the lane's four channels arrive as four dwords (tap-major); eight byte permutes transpose them
// to channel-major and four v_dot4_i32_i8 against the equally transposed weights give 16 multiply-adds, 12
// instructions where the scalar formulation needs about 50.  Zero points follow the identity
//   sum((a - za)(w - zw)) = sum(a*w) - zw*sum(a) - za*sum(w) + T*za*zw   (T = KH*KW)
// with out-of-image taps read as `za`: the reference skips them (tensor_ops.cpp:1302-1313), and a tap whose
// input equals za contributes (za - za)(w - zw) = 0 all the same.  sum(w) is a per-channel constant; sum(a)
// costs one more dot4 per channel and group and is only compiled into the zw != 0 instantiation.
//
// The bias / zero-point / RESCALE / CLAMP epilogue is fused, so the op reads the input once (tap overlap is
// served by L1/L2) and writes one byte per output element.
#include "tmi_kernels.h"

namespace tmi
{

struct DwArgs
{
    ConvGeom g;
    const int8_t* in;
    const int8_t* w;
    const int32_t* bias;
    void* out;
    uint32_t* flag_word;
    RescaleParams rp;
    int32_t za, zw;
    int32_t out_dtype;
    int32_t cgs;          // channel groups of 4 per pixel
    int32_t ppi;          // pixels a workgroup covers per iteration = 256 / cgs
    int32_t iters;        // iterations per workgroup
    int32_t total_px;     // N * OH * OW
    int32_t blocks;       // workgroups that have work
    FastDiv div_cgs, div_ow, div_oh;
};

// 4x4 byte transpose: d[j] holds bytes (c0..c3) of tap j; e[c] receives bytes (tap0..tap3) of channel c.
__device__ __forceinline__ void transpose4x4(const int (&d)[4], int (&e)[4])
{
    const int t01_lo = __builtin_amdgcn_perm(d[1], d[0], 0x05010400);    // d0.b0 d1.b0 d0.b1 d1.b1
    const int t01_hi = __builtin_amdgcn_perm(d[1], d[0], 0x07030602);    // d0.b2 d1.b2 d0.b3 d1.b3
    const int t23_lo = __builtin_amdgcn_perm(d[3], d[2], 0x05010400);
    const int t23_hi = __builtin_amdgcn_perm(d[3], d[2], 0x07030602);
    e[0]             = __builtin_amdgcn_perm(t23_lo, t01_lo, 0x05040100);
    e[1]             = __builtin_amdgcn_perm(t23_lo, t01_lo, 0x07060302);
    e[2]             = __builtin_amdgcn_perm(t23_hi, t01_hi, 0x05040100);
    e[3]             = __builtin_amdgcn_perm(t23_hi, t01_hi, 0x07060302);
}

// NG: groups of four taps held in registers (KH*KW <= 4*NG).  K33: the kernel is 3x3 (NG = 3).  ZW: weight_zp != 0.
template <int NG, bool K33, bool ZW, bool RESCALE>
__global__ __launch_bounds__(256) void depthwise_dot4_kernel(DwArgs a)
{
    // one field of every cache line of the kernel arguments up front: a single scalar-cache round trip instead
    // of one per line along the start-up path
    asm volatile("" ::"s"(a.g.N), "s"(a.g.bias_len), "s"(a.out), "s"(a.rp.shift), "s"(a.rp.lo), "s"(a.za), "s"(a.blocks),
                 "s"(a.div_oh.d));
    const ConvGeom& g = a.g;
    const int tid     = threadIdx.x;
    const int slot    = fdiv(tid, a.div_cgs);    // pixel slot of this lane inside an iteration
    const bool lane_on = slot < a.ppi;
    const int cg      = lane_on ? tid - slot * a.cgs : 0;
    const int c0      = cg * 4;
    const int T       = g.KH * g.KW;
    const int C       = g.IC;

    // consecutive workgroups are dealt to the 8 XCDs in turn: give each XCD a contiguous run of pixels, so
    // that the input rows shared by vertically adjacent outputs are found in its L2
    const uint32_t per = gridDim.x >> 3;
    const uint32_t bid = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
    if (bid >= (uint32_t)a.blocks)
        return;

    const int za_word = (a.za & 0xff) * 0x01010101;

    // All tap loads of a pixel are issued before any is used; a tap outside the image (or past the last tap)
    // reads a valid address and is replaced by the input zero point.
    auto load_taps = [&](int it, int (&d)[NG][4], bool& on, int& pix) {
        pix            = (bid * a.iters + it) * a.ppi + slot;
        on             = lane_on && pix < a.total_px;
        const int pixc = on ? pix : 0;
        const int row  = fdiv(pixc, a.div_ow);    // n * OH + oy
        const int ox   = pixc - row * g.OW;
        const int n    = fdiv(row, a.div_oh);
        const int oy   = row - n * g.OH;
        const int y0   = oy * g.stride_y - g.pad_top;
        const int x0   = ox * g.stride_x - g.pad_left;
        // byte offset of tap (0, 0) in the input tensor (below 2^31 in magnitude; it may be negative at the
        // top/left border, the taps that are used bring it back into the tensor)
        const int voff = ((n * g.IH + y0) * g.IW + x0) * C + c0;
        // Most waves see interior pixels only: every tap of every lane is inside the image, so the loads need
        // neither predicates nor a per-lane address (scalar tap base + the lane's offset).
        const bool interior = y0 >= 0 && x0 >= 0 && y0 + (g.KH - 1) * g.dil_y < g.IH &&
                              x0 + (g.KW - 1) * g.dil_x < g.IW;
        if (__all(interior))
        {
            int ky = 0, kx = 0;
#pragma unroll
            for (int t = 0; t < (K33 ? 9 : 4 * NG); t++)
            {
                const int tky = K33 ? t / 3 : ky, tkx = K33 ? t % 3 : kx;
                const bool tap = K33 || t < T;    // uniform
                const int8_t* tb = a.in + (tap ? (tky * g.dil_y * g.IW + tkx * g.dil_x) * C : 0);
                d[t / 4][t % 4]  = *reinterpret_cast<const int*>(tb + (uint32_t)voff);
                if (++kx == g.KW)
                    kx = 0, ky++;
            }
            if constexpr (K33)
            {
                d[2][1] = d[2][2] = d[2][3] = za_word;    // the slots past the ninth tap
                return 0xfffu;
            }
            return (1u << T) - 1u;
        }
        uint32_t m = 0;    // which slots hold an in-image tap: the others are patched to za once loaded
        if constexpr (K33)
        {
            // 3x3: row and column validity once per pixel, tap offsets are scalars
            bool yv[3], xv[3];
#pragma unroll
            for (int k = 0; k < 3; k++)
            {
                yv[k] = (uint32_t)(y0 + k * g.dil_y) < (uint32_t)g.IH;
                xv[k] = (uint32_t)(x0 + k * g.dil_x) < (uint32_t)g.IW;
            }
#pragma unroll
            for (int t = 0; t < 9; t++)
            {
                const bool ok    = yv[t / 3] && xv[t % 3];
                const int toff   = ((t / 3) * g.dil_y * g.IW + (t % 3) * g.dil_x) * C;
                const uint32_t o = ok ? (uint32_t)(voff + toff) : 0u;
                d[t / 4][t % 4]  = *reinterpret_cast<const int*>(a.in + o);
                m |= (ok ? 1u : 0u) << t;
            }
            d[2][1] = d[2][2] = d[2][3] = za_word;    // the slots past the ninth tap
            m |= 0xe00u;
        }
        else
        {
            int ky = 0, kx = 0;
#pragma unroll
            for (int gq = 0; gq < NG; gq++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                {
                    const bool ok = 4 * gq + j < T && (uint32_t)(y0 + ky * g.dil_y) < (uint32_t)g.IH &&
                                    (uint32_t)(x0 + kx * g.dil_x) < (uint32_t)g.IW;
                    const int toff   = (ky * g.dil_y * g.IW + kx * g.dil_x) * C;
                    const uint32_t o = ok ? (uint32_t)(voff + toff) : 0u;
                    d[gq][j]         = *reinterpret_cast<const int*>(a.in + o);
                    m |= (ok ? 1u : 0u) << (4 * gq + j);
                    if (++kx == g.KW)
                        kx = 0, ky++;
                }
        }
        return m;
    };

    // The first pixel's loads go out before anything else, the loads of the per-lane constants right behind
    // them: one trip to memory covers both.
    int d_cur[NG][4];
    bool on_cur;
    int pix_cur;
    uint32_t ok_cur = load_taps(0, d_cur, on_cur, pix_cur);

    // ---- per-lane constants ----------------------------------------------------------------------------
    int wraw[NG][4];
    int32_t braw[4], mraw[4], sraw[4];
#pragma unroll
    for (int gq = 0; gq < NG; gq++)
#pragma unroll
        for (int j = 0; j < 4; j++)
        {
            const int t = 4 * gq + j < T ? 4 * gq + j : 0;
            wraw[gq][j] = *reinterpret_cast<const int*>(a.w + (size_t)t * C + c0);
        }
#pragma unroll
    for (int c = 0; c < 4; c++)
    {
        braw[c] = a.bias[g.bias_len == 1 ? 0 : c0 + c];
        if constexpr (RESCALE)
        {
            // the fast RESCALE path has 32-bit multipliers
            const int i = a.rp.per_channel ? c0 + c : 0;
            mraw[c]     = reinterpret_cast<const int32_t*>(a.rp.multiplier)[i];
            sraw[c]     = (int32_t)a.rp.shift[i];
        }
    }
    int wq[NG][4];    // [tap group][channel]: the weights of four taps of one channel
    int wsum[4] = { 0, 0, 0, 0 };
#pragma unroll
    for (int gq = 0; gq < NG; gq++)
    {
        int d[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
            d[j] = 4 * gq + j < T ? wraw[gq][j] : 0;
        transpose4x4(d, wq[gq]);
#pragma unroll
        for (int c = 0; c < 4; c++)
            wsum[c] = __builtin_amdgcn_sdot4(wq[gq][c], 0x01010101, wsum[c], false);
    }
    uint32_t flags = 0;
    int32_t corr[4];    // bias - za*sum(w) + T*za*zw
    int32_t mul[4], sh[4], zp_post[4] = { 0, 0, 0, 0 };
    uint32_t lim[4];
    int64_t rnd_pos[4], rnd_neg[4];
    bool check = false;    // some channel of this lane has a shift below 32: the value range must be tested
#pragma unroll
    for (int c = 0; c < 4; c++)
    {
        corr[c] = braw[c] - a.za * wsum[c] + T * a.za * a.zw;
        if constexpr (RESCALE)
        {
            const ChannelScale cs = make_channel_scale(mraw[c], sraw[c], a.rp.double_round, flags);
            // the output zero point rides in the rounding term where that cannot overflow, else it is added last
            const bool fold       = cs.s <= zp_fold_max_shift(a.rp.out_zp);
            const int64_t zp_term = fold ? ((int64_t)a.rp.out_zp << cs.s) : 0;
            zp_post[c]            = fold ? 0 : a.rp.out_zp;
            mul[c] = cs.m, sh[c] = cs.s, lim[c] = cs.lim;
            rnd_pos[c] = cs.rnd_pos + zp_term, rnd_neg[c] = cs.rnd_neg + zp_term;
            check |= cs.lim != 0x80000000u;
        }
    }
    if (!lane_on)
        flags = 0;    // idle lanes mirror channel group 0; only the lanes that own it report its constants

    // ---- pixels ----------------------------------------------------------------------------------------
    for (int it = 0; it < a.iters; it++)
    {
        // the next pixel's loads are in flight while this one is computed
        int d_next[NG][4];
        bool on_next   = false;
        int pix_next   = 0;
        uint32_t ok_next = 0;
        if (it + 1 < a.iters)
            ok_next = load_taps(it + 1, d_next, on_next, pix_next);
        const bool on = on_cur;
        const int pix = pix_cur;
        // slots without an in-image tap read as the input zero point; a wave of interior pixels under a kernel
        // that fills its slots has none
        const uint32_t full = 4 * NG >= 32 ? 0xffffffffu : (1u << (4 * NG)) - 1u;
        if (__any(ok_cur != full))
#pragma unroll
            for (int gq = 0; gq < NG; gq++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    d_cur[gq][j] = (ok_cur >> (4 * gq + j)) & 1u ? d_cur[gq][j] : za_word;
        auto& d = d_cur;
        int32_t acc[4] = { 0, 0, 0, 0 };
        int32_t asum[4] = { 0, 0, 0, 0 };
#pragma unroll
        for (int gq = 0; gq < NG; gq++)
        {
            int e[4];
            transpose4x4(d[gq], e);
#pragma unroll
            for (int c = 0; c < 4; c++)
            {
                acc[c] = __builtin_amdgcn_sdot4(e[c], wq[gq][c], acc[c], false);
                if constexpr (ZW)
                    asum[c] = __builtin_amdgcn_sdot4(e[c], 0x01010101, asum[c], false);
            }
        }
        int32_t res[4];
#pragma unroll
        for (int c = 0; c < 4; c++)
        {
            int32_t v = acc[c] + corr[c];
            if constexpr (ZW)    // slots past the last tap hold za: take them out of sum(a) again
                v -= a.zw * (asum[c] - (4 * NG - T) * a.za);
            if constexpr (RESCALE)
            {
                if (check && on && (uint32_t)v + lim[c] > 2u * lim[c] - 1u)
                    flags |= TMI_FLAG_SCALE_VALUE;
                const int64_t pr = (int64_t)v * (int64_t)mul[c] + (v >= 0 ? rnd_pos[c] : rnd_neg[c]);
                v                = (int32_t)(pr >> sh[c]) + zp_post[c];
                v                = v < a.rp.lo ? a.rp.lo : v;
                v                = v > a.rp.hi ? a.rp.hi : v;
            }
            res[c] = v;
        }
        const size_t o = (size_t)pix * C + c0;
        if (!on)
        {}
        else if (!RESCALE || a.out_dtype == TMI_INT32)
        {
            int32_t* p = reinterpret_cast<int32_t*>(a.out) + o;
            p[0] = res[0], p[1] = res[1], p[2] = res[2], p[3] = res[3];
        }
        else if (a.out_dtype == TMI_INT8)
            *reinterpret_cast<int*>(reinterpret_cast<int8_t*>(a.out) + o) =
                (res[0] & 0xff) | ((res[1] & 0xff) << 8) | ((res[2] & 0xff) << 16) | ((res[3] & 0xff) << 24);
        else
        {
            int* p = reinterpret_cast<int*>(reinterpret_cast<int16_t*>(a.out) + o);
            p[0]   = (res[0] & 0xffff) | ((res[1] & 0xffff) << 16);
            p[1]   = (res[2] & 0xffff) | ((res[3] & 0xffff) << 16);
        }
#pragma unroll
        for (int gq = 0; gq < NG; gq++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                d_cur[gq][j] = d_next[gq][j];
        on_cur = on_next, pix_cur = pix_next, ok_cur = ok_next;
    }
    raise_flags(a.flag_word, flags);
}

template <int NG, bool K33>
static void launch_dot4(hipStream_t st, const DwArgs& a, int grid, bool zw, bool rescale)
{
    if (zw && rescale)
        hipLaunchKernelGGL((depthwise_dot4_kernel<NG, K33, true, true>), dim3(grid), dim3(256), 0, st, a);
    else if (zw)
        hipLaunchKernelGGL((depthwise_dot4_kernel<NG, K33, true, false>), dim3(grid), dim3(256), 0, st, a);
    else if (rescale)
        hipLaunchKernelGGL((depthwise_dot4_kernel<NG, K33, false, true>), dim3(grid), dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL((depthwise_dot4_kernel<NG, K33, false, false>), dim3(grid), dim3(256), 0, st, a);
}

// Eligible: INT8, multiplier 1, channels a multiple of 4 (at most 1024), at most 28 taps, 4-byte aligned
// tensors, and either no RESCALE or one that qualifies for fast_rescale().
const char* launch_depthwise_vec(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g,
                                 const void* in, const void* w, const void* bias, int32_t in_zp, int32_t w_zp,
                                 const RescaleParams& rp, void* out, uint32_t* flag_word)
{
    const int T = g.KH * g.KW;
    if (in_dtype != TMI_INT8 || g.M != 1 || (g.IC & 3) != 0 || g.IC == 0 || g.IC > 1024 || T > 28)
        return nullptr;
    if ((((uintptr_t)in | (uintptr_t)w | (uintptr_t)out | (uintptr_t)bias) & 3) != 0)
        return nullptr;
    if (rp.enabled && !rp.fast)
        return nullptr;
    const int64_t total_px = (int64_t)g.N * g.OH * g.OW;
    // 32-bit offsets inside the input tensor and exact multiply-high divisions of the pixel index
    if (total_px == 0 || total_px * g.OW >= (int64_t(1) << 31) || (total_px / g.OW + 1) * g.OH >= (int64_t(1) << 31) ||
        (int64_t)g.N * g.IH * g.IW * g.IC >= (int64_t(1) << 31))
        return nullptr;

    DwArgs a{};
    a.g = g, a.in = (const int8_t*)in, a.w = (const int8_t*)w, a.bias = (const int32_t*)bias, a.out = out;
    a.flag_word = flag_word, a.rp = rp, a.za = in_zp, a.zw = w_zp, a.out_dtype = out_dtype;
    a.cgs      = g.IC / 4;
    a.ppi      = 256 / a.cgs;
    a.total_px = (int)total_px;
    // enough workgroups to give every CU several, few enough that a lane's constants serve a few pixels
    const int64_t px_iters = (total_px + a.ppi - 1) / a.ppi;
    a.iters                = px_iters >= 256 * 64 ? 8 : (px_iters >= 256 * 16 ? 4 : (px_iters >= 256 * 8 ? 2 : 1));
    a.blocks               = (int)((px_iters + a.iters - 1) / a.iters);
    a.div_cgs              = make_fastdiv(a.cgs);
    a.div_ow               = make_fastdiv(g.OW);
    a.div_oh               = make_fastdiv(g.OH);
    const int grid         = ((a.blocks + 7) / 8) * 8;
    if (g.KH == 3 && g.KW == 3)
        launch_dot4<3, true>(st, a, grid, w_zp != 0, rp.enabled);
    else if (T <= 4)
        launch_dot4<1, false>(st, a, grid, w_zp != 0, rp.enabled);
    else if (T <= 12)
        launch_dot4<3, false>(st, a, grid, w_zp != 0, rp.enabled);
    else
        launch_dot4<7, false>(st, a, grid, w_zp != 0, rp.enabled);
    return rp.enabled ? "depthwise_dot4_i8_rescale" : "depthwise_dot4_i8";
}

}    // namespace tmi
