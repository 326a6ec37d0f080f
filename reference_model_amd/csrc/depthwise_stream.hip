// DEPTHWISE_CONV2D (int8, channel multiplier 1, 3x3 taps, weight_zp = 0) on the matrix cores, without a patch in LDS.
//
// The arithmetic is that of depthwise_slab.hip: D[channel, pixel] = sum over taps t of diag(w[t, .]) x X_t, one
// v_mfma_i32_32x32x32_i8 per tap for a unit of 32 channels x 32 pixels.  What differs is where the pixel operand comes
// from.  It is the natural NHWC layout - lane (pixel li, half lh) holds the 16 channels [16 lh, 16 lh + 16) of its
// pixel under the tap - so a lane fetches it straight from global memory with one 16-byte load per tap: no patch in
// LDS, and after the one barrier behind the per-channel tables the waves of a workgroup have nothing to do with each
// other.  A wave keeps a group of G channel blocks (G x 32 consecutive channels) for its whole life and walks a sequence
// of pixel tiles: the 9 G loads of a tile are requested tap by tap with the G blocks of a tap back to back (they read the
// same cache lines: a load instruction takes 32 of a pixel's bytes, and what the L1 fetched for the first block serves
// the others), the 9 G matrix instructions run when they have landed, the next tile's loads are requested, and the G
// blocks are requantised and stored while those loads fly.  The overlap of loads and arithmetic that workgroups with a
// barrier have to get from their neighbours on the CU comes here from every wave by itself.
//
// Workgroup b works in the b % 8-th eighth of the layer, so that tiles with common halo rows share an L2.
#include "tmi_mfma.h"

namespace tmi
{

struct DwStreamArgs
{
    const uint8_t* in;
    const int8_t* w;
    const int32_t* bias;
    void* out;
    uint32_t* flag_word;
    RescaleParams rp;
    int32_t N, IH, IW, C, OH, OW;
    int32_t sy, sx, dy, dx, pad_top, pad_left;
    int32_t ltw;            // a pixel tile is (32 >> ltw) rows of (1 << ltw) output pixels
    int32_t tiles_x, tiles_y;
    int32_t n_grp;          // groups of G channel blocks
    int32_t bias_len, za;
    int32_t out_kind;       // 0: int32 accumulators, 1: int8 through the RESCALE, 2: int16 through the RESCALE
    int32_t n_tiles;        // pixel tiles of the layer
    int32_t tiles_per_part; // pixel tiles per part of the layer (part = workgroup index % 8)
    int32_t n_streams;      // waves per part and channel group
    FastDiv div_tiles_x, div_tiles_y, div_grp;
};

template <bool ZA, bool FUSED, int G>
__global__ __launch_bounds__(512) void depthwise_stream_kernel(DwStreamArgs a)
{
    constexpr int TAPS = 9;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw   = blockDim.x >> 6;
    const int li = lane & 31, lh = lane >> 5;
    const int C  = a.C;
    // LDS: [weights: 9 x C words, the byte in all four bytes][C x ChannelScale][C x HighWordScale][C x (bias - za * sum(w))]
    //      [the epilogue's form per 64 channels]
    int32_t* wtab         = reinterpret_cast<int32_t*>(lds);
    ChannelScale* tab_cs  = reinterpret_cast<ChannelScale*>(lds + TAPS * C * 4);
    HighWordScale* tab_hw = reinterpret_cast<HighWordScale*>(tab_cs + C);
    int32_t* tab_b        = reinterpret_cast<int32_t*>(tab_hw + C);
    int32_t* tab_form     = tab_b + C;

    // ---- the wave's channel group and its sequence of pixel tiles ------------------------------------------------
    const int part   = blockIdx.x & 7;
    const int gw     = (blockIdx.x >> 3) * nw + wave;
    const int stream = (int)fdiv((uint32_t)gw, a.div_grp);
    const int cg     = gw - stream * a.n_grp;
    int pt           = part * a.tiles_per_part + stream;
    int pt_end       = (part + 1) * a.tiles_per_part;
    pt_end           = pt_end < a.n_tiles ? pt_end : a.n_tiles;
    const bool idle  = stream >= a.n_streams || pt >= pt_end;    // such a wave still builds its share of the tables
    const int c0 = cg * 32 * G;
    const int cl = c0 + 16 * lh;     // (lane, block g, register e) = channel cl + 32 g + e of pixel li

    // ---- the lane's place in a pixel tile; the first tile's loads ------------------------------------------------
    const int ty = li >> a.ltw, tx = li & ((1 << a.ltw) - 1);
    const int th = 32 >> a.ltw, tw = 1 << a.ltw;
    const int row_step = a.dy * a.IW * C, col_step = a.dx * C;
    bool g_ok[G];    // C is a multiple of 16: a lane's 16 channels exist or do not
#pragma unroll
    for (int g = 0; g < G; g++)
        g_ok[g] = cl + 32 * g < C;

    // The nine tap addresses of a lane are one 32-bit offset from the tensor's base each (the G blocks of a tap lie 32
    // bytes apart: an immediate).  A tap outside the image, and every tap of a lane whose pixel or channels do not exist,
    // loads the tensor's first bytes instead and is replaced by input_zp before use; the return value has bit t set when
    // tap t is a real one.
    const bool lane_has_channels = G > 1 || g_ok[0];    // (with G > 1 the launcher takes whole groups only)
    const bool all_channels      = G > 1 || c0 + 32 <= C;
    auto request = [&](int p, v4i(&fb)[TAPS][G]) -> uint32_t {
        const uint32_t trow = fdiv((uint32_t)p, a.div_tiles_x);
        const int txi       = p - trow * a.tiles_x;
        const int n         = (int)fdiv(trow, a.div_tiles_y);
        const int tyi       = trow - n * a.tiles_y;
        const int oy = tyi * th + ty, ox = txi * tw + tx;
        const int iy0 = oy * a.sy - a.pad_top, ix0 = ox * a.sx - a.pad_left;
        // the tensor has fewer than 2^31 bytes (checked by the launcher)
        const uint32_t base = (uint32_t)(((n * a.IH + iy0) * a.IW + ix0) * C + cl);
        // a tile whose pixels all exist and whose windows all lie inside the image (a test on scalars): nine additions
        const int ty0 = tyi * th, tx0 = txi * tw;
        const bool inside = all_channels && ty0 + th <= a.OH && tx0 + tw <= a.OW && ty0 * a.sy >= a.pad_top &&
                            tx0 * a.sx >= a.pad_left && (ty0 + th - 1) * a.sy - a.pad_top + 2 * a.dy < a.IH &&
                            (tx0 + tw - 1) * a.sx - a.pad_left + 2 * a.dx < a.IW;
        if (inside)
        {
#pragma unroll
            for (int t = 0; t < TAPS; t++)
            {
                const uint32_t voff = base + (uint32_t)((t / 3) * row_step + (t % 3) * col_step);
#pragma unroll
                for (int g = 0; g < G; g++)
                    fb[t][g] = *reinterpret_cast<const v4i*>(a.in + voff + 32 * g);
            }
            return 0x1ffu;
        }
        const bool px_ok = lane_has_channels && oy < a.OH && ox < a.OW;
        bool rok[3], cok[3];
#pragma unroll
        for (int k = 0; k < 3; k++)
        {
            rok[k] = px_ok && (unsigned)(iy0 + k * a.dy) < (unsigned)a.IH;
            cok[k] = (unsigned)(ix0 + k * a.dx) < (unsigned)a.IW;
        }
        uint32_t real = 0;
#pragma unroll
        for (int t = 0; t < TAPS; t++)
        {
            const bool ok       = rok[t / 3] && cok[t % 3];
            const uint32_t voff = ok ? base + (uint32_t)((t / 3) * row_step + (t % 3) * col_step) : 0u;
            real |= ok ? 1u << t : 0u;
#pragma unroll
            for (int g = 0; g < G; g++)
                fb[t][g] = *reinterpret_cast<const v4i*>(a.in + voff + 32 * g);
        }
        return real;
    };
    v4i fb[TAPS][G];
    uint32_t real = 0x1ff;
    if (!idle)
        real = request(pt, fb);
    const int za_word = (a.za & 0xff) * 0x01010101;

    // ---- per-channel tables, by all waves of the workgroup -----------------------------------------------------------
    uint32_t flags = 0;
    for (int ch0 = wave * 64; ch0 < C; ch0 += nw * 64)    // whole waves, so that the votes below see 64 channels
    {
        const int ch     = ch0 + lane;
        const bool ch_ok = ch < C;
        const int chc    = ch_ok ? ch : 0;
        int8_t t_w[TAPS];
#pragma unroll
        for (int t = 0; t < TAPS; t++)
            t_w[t] = a.w[t * C + chc];
        const int32_t t_bias = a.bias[a.bias_len == 1 ? 0 : chc];
        int wsum = 0;
#pragma unroll
        for (int t = 0; t < TAPS; t++)
            wsum += (int)t_w[t];
        if constexpr (FUSED)
        {
            const int32_t t_mult  = load_multiplier(a.rp, chc);
            const int32_t t_shift = load_shift(a.rp, chc);
            // lanes past C take the wave's first shift, so that they do not break a wave whose channels share a form
            const int32_t s_first = __builtin_amdgcn_readfirstlane(t_shift);
            uint32_t f            = 0;
            const ChannelScale cs = make_channel_scale(ch_ok ? t_mult : 0, ch_ok ? t_shift : s_first, a.rp.double_round != 0, f);
            // The epilogue's form per 64 channels: every shift large enough for the high-word form (tmi_device.h) and small
            // enough for output_zp * 2^shift to ride in the 64-bit rounding term (1; 2 where, with double rounding, the
            // result is clamped at or above output_zp and no multiplier is negative, so that a negative value ends at the
            // lower limit with either rounding term and its sign need not be looked at); anything else: fast_rescale() (0).
            const int s_min = a.rp.double_round ? 33 : 32;
            const int folds = __all(cs.s >= s_min && cs.s <= zp_fold_max_shift(a.rp.out_zp));
            const int relu  = a.rp.double_round && a.rp.lo >= a.rp.out_zp && __all(cs.m >= 0);
            if (ch_ok)
            {
                flags |= f;
                tab_cs[ch] = cs;
                tab_hw[ch] = make_high_word_scale(cs, a.rp.out_zp);
            }
            if (lane == 0)
                tab_form[ch0 >> 6] = folds ? ((a.rp.double_round && !relu) ? 1 : 2) : 0;
        }
        if (ch_ok)
        {
            tab_b[ch]   = t_bias - (ZA ? a.za * wsum : 0);
            int32_t* wp = wtab + ch;
#pragma unroll
            for (int t = 0; t < TAPS; t++, wp += C)    // byte 0 in all four bytes: one permute, no multiply
                *wp = __builtin_amdgcn_perm((int)t_w[t], (int)t_w[t], 0x04040404);
        }
    }
    __syncthreads();
    if (idle)
    {
        raise_flags(a.flag_word, flags);
        return;
    }

    // operand row li of the diagonal matrix stands for channel wr of the block; it is non-zero at K index wr only, which
    // lies in this lane's K half when wr / 16 == lh: byte wr % 4 of word (wr / 4) % 4 of the lane's 16 operand bytes
    const int wr = 4 * (li & 4) + ((li >> 1) & 12) + (li & 3);
    int wmask[4];
#pragma unroll
    for (int k = 0; k < 4; k++)
        wmask[k] = ((wr >> 4) == lh && ((wr >> 2) & 3) == k) ? 0xff << ((wr & 3) * 8) : 0;

    for (;;)
    {
        // ---- the 9 G matrix instructions of this tile ------------------------------------------------------------------
        if (__any(real != 0x1ff))
        {
#pragma unroll
            for (int t = 0; t < TAPS; t++)
#pragma unroll
                for (int g = 0; g < G; g++)
                {
                    const bool ok = (real >> t) & 1;
                    fb[t][g] = v4i{ ok ? fb[t][g][0] : za_word, ok ? fb[t][g][1] : za_word, ok ? fb[t][g][2] : za_word,
                                    ok ? fb[t][g][3] : za_word };
                }
        }
        v16i acc[G];
#pragma unroll
        for (int g = 0; g < G; g++)
        {
            const int c   = c0 + 32 * g + wr;
            const int cc  = c < C ? c : 0;
            const int clc = g_ok[g] ? cl + 32 * g : 0;
            int wv[TAPS];
#pragma unroll
            for (int t = 0; t < TAPS; t++)
                wv[t] = wtab[t * C + cc];
#pragma unroll
            for (int q = 0; q < 4; q++)
            {
                const v4i b4 = *reinterpret_cast<const v4i*>(tab_b + clc + 4 * q);
                acc[g][4 * q] = b4[0], acc[g][4 * q + 1] = b4[1], acc[g][4 * q + 2] = b4[2], acc[g][4 * q + 3] = b4[3];
            }
            int wm[4];
#pragma unroll
            for (int k = 0; k < 4; k++)
                wm[k] = c < C ? wmask[k] : 0;
#pragma unroll
            for (int t = 0; t < TAPS; t++)
            {
                const v4i fa = v4i{ wv[t] & wm[0], wv[t] & wm[1], wv[t] & wm[2], wv[t] & wm[3] };
                acc[g]       = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb[t][g], acc[g], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // ---- the next tile's loads ---------------------------------------------------------------------------------------
        // They land in the registers the matrix instructions above read.  A matrix instruction runs for 16 passes after it
        // has been issued and nothing orders a later load's data behind its operand reads (a load of a line that the L1 holds,
        // issued right behind the matrix instruction of its tap, was seen to replace the operand's last bytes in time to
        // change the product), so the requests wait for a value of the last matrix instruction's result.
        {
            const int done = __builtin_amdgcn_readfirstlane(acc[G - 1][15]);
            asm volatile("" ::"s"(done));
        }
        __builtin_amdgcn_sched_barrier(0);
        const int pn        = pt + a.n_streams;
        const bool has_next = pn < pt_end;
        if (has_next)
            real = request(pn, fb);
        __builtin_amdgcn_sched_barrier(0);

        // ---- epilogue ------------------------------------------------------------------------------------------------
        const uint32_t trow = fdiv((uint32_t)pt, a.div_tiles_x);
        const int txi       = pt - trow * a.tiles_x;
        const int n         = (int)fdiv(trow, a.div_tiles_y);
        const int tyi       = trow - n * a.tiles_y;
        const int oy = tyi * th + ty, ox = txi * tw + tx;
        const bool px_ok = oy < a.OH && ox < a.OW;
        // the tensor has fewer than 2^31 elements (checked by the launcher): 32-bit arithmetic
        const uint32_t opix = (uint32_t)(((n * a.OH + oy) * a.OW + ox) * C + cl);
#pragma unroll
        for (int g = 0; g < G; g++)
        {
            const bool ok      = px_ok && g_ok[g];
            const size_t obase = opix + 32 * g;
            const int clc      = g_ok[g] ? cl + 32 * g : 0;
            if constexpr (!FUSED)
            {
                if (ok)
                {
                    int32_t* o = reinterpret_cast<int32_t*>(a.out) + obase;
#pragma unroll
                    for (int q = 0; q < 4; q++)
                        *reinterpret_cast<v4i*>(o + 4 * q) =
                            v4i{ acc[g][4 * q], acc[g][4 * q + 1], acc[g][4 * q + 2], acc[g][4 * q + 3] };
                }
            }
            else
            {
                int32_t r[16];
                const int form = __builtin_amdgcn_readfirstlane(tab_form[(c0 + 32 * g < C ? c0 + 32 * g : 0) >> 6]);
                if (form == 2)
                {
#pragma unroll
                    for (int e = 0; e < 16; e++)
                    {
                        const HighWordScale c = tab_hw[clc + e];
                        r[e] = clamp_med3(high_word_rescale64<false>(acc[g][e], c), a.rp.lo, a.rp.hi);
                    }
                }
                else if (form == 1)
                {
#pragma unroll
                    for (int e = 0; e < 16; e++)
                    {
                        const HighWordScale c = tab_hw[clc + e];
                        r[e] = clamp_med3(high_word_rescale64<true>(acc[g][e], c), a.rp.lo, a.rp.hi);
                    }
                }
                else
                {
                    uint32_t eflags = 0;
#pragma unroll
                    for (int e = 0; e < 16; e++)
                    {
                        const ChannelScale cs = tab_cs[clc + e];
                        r[e]                  = fast_rescale(acc[g][e], cs, a.rp.out_zp, a.rp.lo, a.rp.hi, eflags);
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
        }
        if (!has_next)
            break;
        pt = pn;
    }
    raise_flags(a.flag_word, flags);
}

template <bool ZA, bool FUSED, int G>
static bool launch_dwstream_kernel(hipStream_t st, const DwStreamArgs& a, int grid, int threads, int lds_bytes)
{
    auto kern = depthwise_stream_kernel<ZA, FUSED, G>;
    static LdsLimit granted{};
    if (!ensure_dynamic_lds(reinterpret_cast<const void*>(kern), (size_t)lds_bytes, granted))
        return false;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), lds_bytes, st, a);
    return true;
}

template <int G>
static bool launch_dwstream_g(hipStream_t st, const DwStreamArgs& a, bool za, bool fused, int grid, int threads, int lds_bytes)
{
    if (za)
        return fused ? launch_dwstream_kernel<true, true, G>(st, a, grid, threads, lds_bytes)
                     : launch_dwstream_kernel<true, false, G>(st, a, grid, threads, lds_bytes);
    return fused ? launch_dwstream_kernel<false, true, G>(st, a, grid, threads, lds_bytes)
                 : launch_dwstream_kernel<false, false, G>(st, a, grid, threads, lds_bytes);
}

// nullptr when the layer is not one this kernel takes.
const char* launch_depthwise_stream(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                                    const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                                    void* out, uint32_t* flag_word)
{
    if (in_dtype != TMI_INT8 || g.M != 1 || g.KH != 3 || g.KW != 3 || w_zp != 0 || !flag_word)
        return nullptr;
    if ((g.IC & 15) || g.IC < 32 || g.IC > 1024 || g.OC != g.IC || (int64_t)g.N * g.IH * g.IW * g.IC < 128)
        return nullptr;
    if (rp.enabled ? (!rp.fast || (out_dtype != TMI_INT8 && out_dtype != TMI_INT16)) : out_dtype != TMI_INT32)
        return nullptr;
    if ((((uintptr_t)in | (uintptr_t)out) & 15) || ((uintptr_t)bias & 3) || g.N < 1 || g.OH < 1 || g.OW < 1)
        return nullptr;
    // 32-bit byte offsets into both tensors, tap offsets included
    if ((int64_t)g.N * g.IH * g.IW * g.IC + (int64_t)3 * g.dil_y * g.IW * g.IC >= (int64_t(1) << 31) ||
        (int64_t)g.N * (g.OH + 32) * (g.OW + 32) * g.IC >= (int64_t(1) << 31))
        return nullptr;

    const int C = g.IC, n_cblk = (C + 31) / 32;
    // blocks per wave: three or two where the channels come in whole groups of that many blocks
    const int G = C % 96 == 0 ? 3 : (C % 64 == 0 ? 2 : 1);
    const int n_grp = (n_cblk + G - 1) / G;
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
    a.flag_word = flag_word, a.rp = rp;
    a.N = g.N, a.IH = g.IH, a.IW = g.IW, a.C = C, a.OH = g.OH, a.OW = g.OW;
    a.sy = g.stride_y, a.sx = g.stride_x, a.dy = g.dil_y, a.dx = g.dil_x, a.pad_top = g.pad_top, a.pad_left = g.pad_left;
    a.ltw = best_l;
    const int tw = 1 << best_l, th = 32 >> best_l;
    a.tiles_x = (g.OW + tw - 1) / tw, a.tiles_y = (g.OH + th - 1) / th;
    a.n_grp = n_grp, a.bias_len = g.bias_len, a.za = in_zp;
    a.out_kind = !rp.enabled ? 0 : (out_dtype == TMI_INT8 ? 1 : 2);
    const int64_t n_tiles = (int64_t)g.N * a.tiles_y * a.tiles_x;
    if (n_tiles >= (int64_t(1) << 24) || !tile_decode_is_exact(n_tiles, 1u, (uint32_t)a.tiles_x, (uint32_t)a.tiles_y))
        return nullptr;
    a.n_tiles       = (int32_t)n_tiles;
    a.tiles_per_part = (int32_t)((n_tiles + 7) / 8);
    // eight waves per workgroup; a CU holds one workgroup (two waves per SIMD: a wave of the fused kernel holds 190 to 254
    // registers), with single blocks two (at most 128 registers), and a part of the layer has 32 CUs
    constexpr int NW      = 8;
    const int64_t wgs_max = G == 1 ? 64 : 32;
    int64_t wgs = ((int64_t)a.tiles_per_part * n_grp + NW - 1) / NW;
    wgs         = wgs < wgs_max ? wgs : wgs_max;
    while (wgs * NW < n_grp)
        wgs++;
    a.n_streams = (int32_t)(wgs * NW / n_grp);
    a.div_tiles_x = make_fastdiv((uint32_t)a.tiles_x), a.div_tiles_y = make_fastdiv((uint32_t)a.tiles_y);
    a.div_grp = make_fastdiv((uint32_t)n_grp);
    const int grid = (int)wgs * 8;
    const int lds_bytes = 9 * C * 4 + C * (int)(sizeof(ChannelScale) + sizeof(HighWordScale)) + C * 4 + 64;
    const bool ok = G == 3 ? launch_dwstream_g<3>(st, a, in_zp != 0, rp.enabled != 0, grid, NW * 64, lds_bytes)
                  : G == 2 ? launch_dwstream_g<2>(st, a, in_zp != 0, rp.enabled != 0, grid, NW * 64, lds_bytes)
                           : launch_dwstream_g<1>(st, a, in_zp != 0, rp.enabled != 0, grid, NW * 64, lds_bytes);
    if (!ok)
        return nullptr;
    return rp.enabled ? "depthwise_stream_i8_rescale" : "depthwise_stream_i8";
}

}    // namespace tmi
