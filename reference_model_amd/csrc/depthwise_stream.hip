// DEPTHWISE_CONV2D (int8, channel multiplier 1, 3x3 taps, weight_zp = 0) on the matrix cores, without LDS.
//
// The arithmetic is that of depthwise_slab.hip: D[channel, pixel] = sum over taps t of diag(w[t, .]) x X_t, one
// v_mfma_i32_32x32x32_i8 per tap for a unit of 32 channels x 32 pixels.  What differs is where the operands live.
// The pixel operand of the matrix instruction is the natural NHWC layout - lane (pixel li, half lh) holds the 16
// channels [16 lh, 16 lh + 16) of its pixel under the tap - so a lane can fetch it straight from global memory
// with one 16-byte load per tap: no patch in LDS, no barrier, and the waves of a workgroup have nothing to do with
// each other.  A wave keeps one channel block for its whole life; the block's diagonal operands (36 registers) and
// bias terms (16) are built once and stay in registers, its requantisation constants lie in a piece of LDS that only
// this wave touches, and the wave walks a sequence of pixel tiles with the nine loads of the next tile in flight
// while the current one is multiplied, requantised and stored.  The overlap of loads and arithmetic that workgroups with a barrier have to get from
// their neighbours on the CU comes here from every wave by itself.
//
// The taps of neighbouring pixels and the three or more channel blocks of a pixel read the same cache lines: the
// waves of a workgroup take consecutive (pixel tile, channel block) pairs, so those reads meet in the CU's L1, and
// workgroup b works in the b % 8-th eighth of the layer, so that neighbouring tiles share an L2.
#include "tmi_mfma.h"

namespace tmi
{

struct DwStreamArgs
{
    const uint8_t* in;
    const int8_t* w;
    const int32_t* bias;
    const uint8_t* pad_page;    // 64 bytes of input_zp
    void* out;
    uint32_t* flag_word;
    RescaleParams rp;
    int32_t N, IH, IW, C, OH, OW;
    int32_t sy, sx, dy, dx, pad_top, pad_left;
    int32_t ltw;            // a pixel tile is (32 >> ltw) rows of (1 << ltw) output pixels
    int32_t tiles_x, tiles_y;
    int32_t n_cblk;         // channel blocks of 32
    int32_t bias_len, za;
    int32_t out_kind;       // 0: int32 accumulators, 1: int8 through the RESCALE, 2: int16 through the RESCALE
    int32_t n_tiles;        // pixel tiles of the layer
    int32_t tiles_per_grp;  // pixel tiles per group of workgroups (group = workgroup index % 8)
    int32_t n_streams;      // waves per group and channel block
    FastDiv div_tiles_x, div_tiles_y, div_cblk;
};

template <bool ZA, bool FUSED>
__global__ __launch_bounds__(512) void depthwise_stream_kernel(DwStreamArgs a)
{
    constexpr int TAPS = 9;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nw   = blockDim.x >> 6;
    const int li = lane & 31, lh = lane >> 5;
    const int C  = a.C;

    // ---- the wave's channel block and its sequence of pixel tiles ------------------------------------------------
    const int grp    = blockIdx.x & 7;
    const int gw     = (blockIdx.x >> 3) * nw + wave;
    const int stream = (int)fdiv((uint32_t)gw, a.div_cblk);
    const int cb     = gw - stream * a.n_cblk;
    int pt           = grp * a.tiles_per_grp + stream;
    int pt_end       = (grp + 1) * a.tiles_per_grp;
    pt_end           = pt_end < a.n_tiles ? pt_end : a.n_tiles;
    if (stream >= a.n_streams || pt >= pt_end)
        return;
    const int c0 = cb * 32;
    const int cl = c0 + 16 * lh;     // (lane, register e) = channel cl + e of pixel li
    const bool cl_ok = cl < C;       // C is a multiple of 16
    const int clc = cl_ok ? cl : 0;

    // ---- once per wave: diagonal operands, bias terms, requantisation constants ----------------------------------
    // operand row li of the diagonal matrix stands for channel wr of the block; it is non-zero at K index wr only, which
    // lies in this lane's K half when wr / 16 == lh: byte wr % 4 of word (wr / 4) % 4 of the lane's 16 operand bytes
    const int wr = 4 * (li & 4) + ((li >> 1) & 12) + (li & 3);
    v4i fa[TAPS];
    {
        const int c     = c0 + wr;
        const bool c_ok = c < C && (wr >> 4) == lh;
        const int8_t* wp = a.w + (c < C ? c : 0);
        int wt[TAPS];
#pragma unroll
        for (int t = 0; t < TAPS; t++)
            wt[t] = wp[t * C];
        const int sel = (wr >> 2) & 3;
        const int msk = c_ok ? 0xff << ((wr & 3) * 8) : 0;
#pragma unroll
        for (int t = 0; t < TAPS; t++)
        {
            const int rep = __builtin_amdgcn_perm(wt[t], wt[t], 0x04040404) & msk;
            fa[t]         = v4i{ sel == 0 ? rep : 0, sel == 1 ? rep : 0, sel == 2 ? rep : 0, sel == 3 ? rep : 0 };
        }
    }
    v16i bterm;
    {
#pragma unroll
        for (int q = 0; q < 4; q++)
        {
            v4i b4;
            if (a.bias_len == 1)
            {
                const int b0 = a.bias[0];
                b4           = v4i{ b0, b0, b0, b0 };
            }
            else
                b4 = *reinterpret_cast<const v4i*>(a.bias + clc + 4 * q);
            bterm[4 * q] = b4[0], bterm[4 * q + 1] = b4[1], bterm[4 * q + 2] = b4[2], bterm[4 * q + 3] = b4[3];
        }
        if constexpr (ZA)
        {
            // sum(w) per channel in the accumulators' own layout: the nine diagonal operands against a tile of ones
            const v4i ones = v4i{ 0x01010101, 0x01010101, 0x01010101, 0x01010101 };
            v16i sw        = { 0 };
#pragma unroll
            for (int t = 0; t < TAPS; t++)
                sw = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[t], ones, sw, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 16; e++)
                bterm[e] -= a.za * sw[e];
        }
    }
    uint32_t flags = 0;
    // requantisation: lane l derives the constants of channel c0 + l % 32 and leaves them in the wave's own piece of LDS
    // (no other wave reads it, so no barrier); an element's constants are one ds_read_b128 in the epilogue.  The
    // high-word form per channel where every shift of the block allows it (form 1; 2 when no value's sign is needed for
    // the rounding term), else fast_rescale() (form 0).
    __shared__ HighWordScale s_hw[8][32];
    __shared__ ChannelScale s_cs[8][32];
    const HighWordScale* tab_hw = &s_hw[wave][16 * lh];
    const ChannelScale* tab_cs  = &s_cs[wave][16 * lh];
    int form = 0;
    if constexpr (FUSED)
    {
        const int ch     = c0 + li;
        const bool ch_ok = ch < C;
        const int32_t m  = load_multiplier(a.rp, ch_ok ? ch : 0);
        const int32_t s  = load_shift(a.rp, ch_ok ? ch : 0);
        uint32_t f       = 0;
        const ChannelScale cs = make_channel_scale(m, s, a.rp.double_round != 0, f);
        if (ch_ok && lh == 0)
            flags |= f;
        if (lh == 0)
        {
            s_cs[wave][li] = cs;
            s_hw[wave][li] = make_high_word_scale(cs, a.rp.out_zp);
        }
        const int s_min  = a.rp.double_round ? 33 : 32;
        const bool folds = !ch_ok || (cs.s >= s_min && cs.s <= zp_fold_max_shift(a.rp.out_zp));
        const bool relu  = a.rp.double_round && a.rp.lo >= a.rp.out_zp && __all(!ch_ok || cs.m >= 0);
        form             = __all(folds) ? ((a.rp.double_round && !relu) ? 1 : 2) : 0;
    }

    // ---- the lane's place in a pixel tile ----------------------------------------------------------------------------
    const int ty = li >> a.ltw, tx = li & ((1 << a.ltw) - 1);
    const int th = 32 >> a.ltw, tw = 1 << a.ltw;
    const uint8_t* pad_src = a.pad_page + 16 * lh;
    const int row_step = a.dy * a.IW * C, col_step = a.dx * C;

    // the nine loads of pixel tile p
    auto request = [&](int p, v4i(&fb)[TAPS]) {
        const uint32_t trow = fdiv((uint32_t)p, a.div_tiles_x);
        const int txi       = p - trow * a.tiles_x;
        const int n         = (int)fdiv(trow, a.div_tiles_y);
        const int tyi       = trow - n * a.tiles_y;
        const int oy = tyi * th + ty, ox = txi * tw + tx;
        const int iy0 = oy * a.sy - a.pad_top, ix0 = ox * a.sx - a.pad_left;
        const bool px_ok = cl_ok && oy < a.OH && ox < a.OW;
        // the tensor has fewer than 2^31 bytes (checked by the launcher)
        const int base = ((n * a.IH + iy0) * a.IW + ix0) * C + cl;
        bool rok[3], cok[3];
#pragma unroll
        for (int k = 0; k < 3; k++)
        {
            rok[k] = px_ok && (unsigned)(iy0 + k * a.dy) < (unsigned)a.IH;
            cok[k] = (unsigned)(ix0 + k * a.dx) < (unsigned)a.IW;
        }
#pragma unroll
        for (int t = 0; t < TAPS; t++)
        {
            const uint8_t* src = (rok[t / 3] && cok[t % 3]) ? a.in + (base + (t / 3) * row_step + (t % 3) * col_step) : pad_src;
            fb[t]              = *reinterpret_cast<const v4i*>(src);
        }
    };

    // multiply, requantise and store pixel tile p
    auto finish = [&](int p, const v4i(&fb)[TAPS]) {
        v16i acc = bterm;
#pragma unroll
        for (int t = 0; t < TAPS; t++)
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[t], fb[t], acc, 0, 0, 0);
        const uint32_t trow = fdiv((uint32_t)p, a.div_tiles_x);
        const int txi       = p - trow * a.tiles_x;
        const int n         = (int)fdiv(trow, a.div_tiles_y);
        const int tyi       = trow - n * a.tiles_y;
        const int oy = tyi * th + ty, ox = txi * tw + tx;
        const bool ok = cl_ok && oy < a.OH && ox < a.OW;
        const size_t obase = (uint32_t)(((n * a.OH + oy) * a.OW + ox) * C + cl);
        if constexpr (!FUSED)
        {
            if (ok)
            {
                int32_t* o = reinterpret_cast<int32_t*>(a.out) + obase;
#pragma unroll
                for (int q = 0; q < 4; q++)
                    *reinterpret_cast<v4i*>(o + 4 * q) = v4i{ acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3] };
            }
        }
        else
        {
            int32_t r[16];
            if (form == 2)
            {
#pragma unroll
                for (int e = 0; e < 16; e++)
                {
                    const HighWordScale c = tab_hw[e];
                    r[e] = clamp_med3(high_word_rescale64<false>(acc[e], c), a.rp.lo, a.rp.hi);
                }
            }
            else if (form == 1)
            {
#pragma unroll
                for (int e = 0; e < 16; e++)
                {
                    const HighWordScale c = tab_hw[e];
                    r[e] = clamp_med3(high_word_rescale64<true>(acc[e], c), a.rp.lo, a.rp.hi);
                }
            }
            else
            {
                uint32_t eflags = 0;
#pragma unroll
                for (int e = 0; e < 16; e++)
                {
                    const ChannelScale cs = tab_cs[e];
                    r[e]                  = fast_rescale(acc[e], cs, a.rp.out_zp, a.rp.lo, a.rp.hi, eflags);
                }
                if (ok)
                    flags |= eflags;    // pixels and channels outside the tensor raise nothing
            }
            if (ok)
            {
                if (a.out_kind == 1)
                {
                    v4i pk;
#pragma unroll
                    for (int q = 0; q < 4; q++)
                    {
                        const int lo2 = __builtin_amdgcn_perm(r[4 * q + 1], r[4 * q], 0x0c0c0400);
                        const int hi2 = __builtin_amdgcn_perm(r[4 * q + 3], r[4 * q + 2], 0x04000c0c);
                        pk[q]         = lo2 | hi2;
                    }
                    *reinterpret_cast<v4i*>(reinterpret_cast<int8_t*>(a.out) + obase) = pk;
                }
                else
                {
                    int16_t* o = reinterpret_cast<int16_t*>(a.out) + obase;
#pragma unroll
                    for (int half = 0; half < 2; half++)
                    {
                        v4i pk;
#pragma unroll
                        for (int q = 0; q < 4; q++)
                            pk[q] = (r[8 * half + 2 * q] & 0xffff) | ((r[8 * half + 2 * q + 1] & 0xffff) << 16);
                        *reinterpret_cast<v4i*>(o + 8 * half) = pk;
                    }
                }
            }
        }
    };

    // ---- the tiles, two at a time: the next tile's loads are in flight while this one is worked on.  The request past
    // the wave's last tile repeats that tile, so that the loop has no branch between a request and its use. ----
    v4i fb0[TAPS], fb1[TAPS];
    request(pt, fb0);
    for (;;)
    {
        int pn = pt + a.n_streams;
        request(pn < pt_end ? pn : pt, fb1);
        __builtin_amdgcn_sched_barrier(0);
        finish(pt, fb0);
        if (pn >= pt_end)
            break;
        pt = pn, pn = pt + a.n_streams;
        request(pn < pt_end ? pn : pt, fb0);
        __builtin_amdgcn_sched_barrier(0);
        finish(pt, fb1);
        if (pn >= pt_end)
            break;
        pt = pn;
    }
    raise_flags(a.flag_word, flags);
}

// nullptr when the layer is not one this kernel takes.
const char* launch_depthwise_stream(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                                    const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                                    void* out, const void* pad_page, uint32_t* flag_word)
{
    if (in_dtype != TMI_INT8 || g.M != 1 || g.KH != 3 || g.KW != 3 || w_zp != 0 || !pad_page || !flag_word)
        return nullptr;
    if ((g.IC & 15) || g.IC < 32 || g.OC != g.IC)
        return nullptr;
    if (rp.enabled ? (!rp.fast || (out_dtype != TMI_INT8 && out_dtype != TMI_INT16)) : out_dtype != TMI_INT32)
        return nullptr;
    if ((((uintptr_t)in | (uintptr_t)out | (uintptr_t)pad_page | (uintptr_t)bias) & 15) || g.N < 1 || g.OH < 1 || g.OW < 1)
        return nullptr;
    // 32-bit byte offsets into both tensors, tap offsets included
    if ((int64_t)g.N * g.IH * g.IW * g.IC + (int64_t)3 * g.dil_y * g.IW * g.IC >= (int64_t(1) << 31) ||
        (int64_t)g.N * (g.OH + 32) * (g.OW + 32) * g.IC >= (int64_t(1) << 31))
        return nullptr;

    const int C = g.IC, n_cblk = (C + 31) / 32;
    // the tile shape (rows x columns = 32) that reads the fewest input pixels over the layer; ties go to the wider one
    int best_l = 0;
    int64_t best_px = 0;
    for (int l = 0; l <= 5; l++)
    {
        const int tw = 1 << l, th = 32 >> l;
        const int64_t ph = (th - 1) * g.stride_y + 2 * g.dil_y + 1, pw = (tw - 1) * g.stride_x + 2 * g.dil_x + 1;
        const int64_t px = (int64_t)((g.OH + th - 1) / th) * ((g.OW + tw - 1) / tw) * ph * pw;
        if (l == 0 || px <= best_px)
            best_l = l, best_px = px;
    }
    DwStreamArgs a{};
    a.in = (const uint8_t*)in, a.w = (const int8_t*)w, a.bias = (const int32_t*)bias, a.out = out;
    a.pad_page = (const uint8_t*)pad_page, a.flag_word = flag_word, a.rp = rp;
    a.N = g.N, a.IH = g.IH, a.IW = g.IW, a.C = C, a.OH = g.OH, a.OW = g.OW;
    a.sy = g.stride_y, a.sx = g.stride_x, a.dy = g.dil_y, a.dx = g.dil_x, a.pad_top = g.pad_top, a.pad_left = g.pad_left;
    a.ltw = best_l;
    const int tw = 1 << best_l, th = 32 >> best_l;
    a.tiles_x = (g.OW + tw - 1) / tw, a.tiles_y = (g.OH + th - 1) / th;
    a.n_cblk = n_cblk, a.bias_len = g.bias_len, a.za = in_zp;
    a.out_kind = !rp.enabled ? 0 : (out_dtype == TMI_INT8 ? 1 : 2);
    const int64_t n_tiles = (int64_t)g.N * a.tiles_y * a.tiles_x;
    if (n_tiles >= (int64_t(1) << 24) || !tile_decode_is_exact(n_tiles, 1u, (uint32_t)a.tiles_x, (uint32_t)a.tiles_y))
        return nullptr;
    a.n_tiles       = (int32_t)n_tiles;
    a.tiles_per_grp = (int32_t)((n_tiles + 7) / 8);
    // eight waves per workgroup and CU (two per SIMD: a wave holds up to 256 registers), 32 workgroups per group at most
    constexpr int NW = 8;
    int64_t wgs = ((int64_t)a.tiles_per_grp * n_cblk + NW - 1) / NW;
    wgs         = wgs < 32 ? wgs : 32;
    while (wgs * NW < n_cblk)
        wgs++;
    a.n_streams = (int32_t)(wgs * NW / n_cblk);
    a.div_tiles_x = make_fastdiv((uint32_t)a.tiles_x), a.div_tiles_y = make_fastdiv((uint32_t)a.tiles_y);
    a.div_cblk = make_fastdiv((uint32_t)n_cblk);
    const int grid = (int)wgs * 8;
    if (in_zp != 0)
    {
        if (rp.enabled)
            hipLaunchKernelGGL((depthwise_stream_kernel<true, true>), dim3(grid), dim3(NW * 64), 0, st, a);
        else
            hipLaunchKernelGGL((depthwise_stream_kernel<true, false>), dim3(grid), dim3(NW * 64), 0, st, a);
    }
    else
    {
        if (rp.enabled)
            hipLaunchKernelGGL((depthwise_stream_kernel<false, true>), dim3(grid), dim3(NW * 64), 0, st, a);
        else
            hipLaunchKernelGGL((depthwise_stream_kernel<false, false>), dim3(grid), dim3(NW * 64), 0, st, a);
    }
    return rp.enabled ? "depthwise_stream_i8_rescale" : "depthwise_stream_i8";
}

}    // namespace tmi
