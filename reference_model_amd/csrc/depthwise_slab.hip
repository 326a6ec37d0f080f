// DEPTHWISE_CONV2D (int8, channel multiplier 1, 3x3 taps, weight_zp = 0) on the matrix cores.
//
// A depthwise convolution has no sum across channels, so it is not a GEMM; the vector kernel (depthwise.hip) spends
// about 150 vector instructions per (pixel, four channels), most of them on tap addresses, byte transposes and the
// per-pixel setup, and the layer ends up bound by instruction issue rather than by the 12 MB it moves.  The matrix
// cores do the same arithmetic as a by-product of a wasteful but nearly free formulation:
//
//     D[channel, pixel] = sum over taps t of  diag(w[t, .]) x X_t          (32 channels x 32 pixels per tile)
//
// where X_t[channel, pixel] is the input under tap t and diag(w[t, .]) a 32 x 32 diagonal matrix of the tap's
// weights: one v_mfma_i32_32x32x32_i8 per tap.  31/32 of the multiplies are by zero, and still the nine MFMAs of a
// tile take 288 cycles for 9216 useful multiply-adds, a fifth of what the vector formulation needs.  The rest
// is the slab kernel's machinery (conv2d_slab.hip):
//   - the input patch of a TH x TW tile of output pixels (all channels) goes straight into LDS with
//     global_load_lds_dwordx4; a pixel outside the image reads the page of input_zp bytes, so no tap needs a
//     predicate and sum((a - za) w) = sum(a w) - za sum(w) holds with all nine taps;
//   - the pixel operand of the MFMA is the natural NHWC layout: lane (pixel li, half lh) reads the 16 channels
//     [16 lh, 16 lh + 16) of the block under the tap, one ds_read_b128;
//   - the diagonal operand lives in registers (4 per tap), built once per channel block from a small weight table in
//     LDS; operand row r stands for channel 16*((r>>2)&1) + 4*(r>>3) + (r&3), which makes a lane's 16 accumulators
//     16 consecutive channels of one pixel: the RESCALE (+ CLAMP) epilogue of the slab kernel and one 16-byte store;
//   - bias, sum(w), multiplier and shift become per-channel tables in LDS, built by the first C lanes while the
//     patch loads are in flight.
// A wave owns units (pixel tile, channel block) of the workgroup's tile in turn.
#include <cstring>

#include "tmi_mfma.h"

namespace tmi
{

struct DwSlabArgs
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
    int32_t TH, TW, PH, PW, tiles_x, tiles_y;
    int32_t bias_len, za;
    int32_t out_kind;    // 0: int32 accumulators, 1: int8 through the RESCALE, 2: int16 through the RESCALE
    int32_t xcd_remap;    // 0, or grid / 8: workgroup b takes tile (b % 8) * (grid / 8) + b / 8
    int32_t cpp;         // 16-byte chunks per pixel = C / 16
    int32_t ppitch;      // chunks per patch pixel in LDS (odd)
    int32_t pitch;       // chunks per patch row in LDS
    int32_t step_row, step_px, step_ch;    // one round of loads (64 slots per wave) = step_row rows + step_px pixels + step_ch chunks
    int32_t wrap_px, wrap_ch;    // a patch row in pixels and chunks: pitch = wrap_px * ppitch + wrap_ch (padding included)
    int32_t n_cblk;      // channel blocks of 32
    int32_t n_units;     // (pixel tiles of 32) x channel blocks
    FastDiv div_tw, div_pitch, div_ppitch, div_tiles_x, div_tiles_y, div_cblk;
};

__device__ __forceinline__ void dwslab_load(const void* src, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_addr) : "memory");
}

template <bool ZA, bool FUSED>
__global__ __launch_bounds__(1024) void depthwise_slab_kernel(DwSlabArgs a)
{
    asm volatile("" ::"s"(a.in), "s"(a.rp.shift), "s"(a.rp.lo), "s"(a.N), "s"(a.TH), "s"(a.bias_len), "s"(a.n_units),
                 "s"(a.div_cblk.d));
    constexpr int TAPS = 9;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid     = threadIdx.x;
    const int lane    = tid & 63;
    const int wave    = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves  = blockDim.x >> 6;
    const int li      = lane & 31;
    const int lh      = lane >> 5;
    const int C       = a.C;
    const int p_slots = a.PH * a.pitch;
    const int p_loads = (p_slots + 63) >> 6;
    // LDS: [patch][weights: 9 x C bytes][C x ChannelScale][C x HighWordScale][C multipliers][C x (bias - za * sum(w))][common shift per table wave]
    uint8_t* pl          = lds;
    int32_t* wtab        = reinterpret_cast<int32_t*>(lds + p_loads * 1024);    // the weight byte in all four bytes of a word
    const int wtab_bytes = TAPS * C * 4;
    ChannelScale* tab_cs = reinterpret_cast<ChannelScale*>(lds + p_loads * 1024 + wtab_bytes);
    HighWordScale* tab_hw = reinterpret_cast<HighWordScale*>(tab_cs + C);
    int32_t* tab_m       = reinterpret_cast<int32_t*>(tab_hw + C);
    int32_t* tab_b       = tab_m + C;
    int32_t* uni_shift   = tab_b + C;    // a word per table wave: 16

    uint32_t bid = blockIdx.x;
    if (a.xcd_remap)
    {
        const uint32_t per = (uint32_t)a.xcd_remap;    // an eighth of the grid: no hidden-argument load for gridDim
        bid                = (bid & 7) * per + (bid >> 3);
    }
    const uint32_t trow = fdiv(bid, a.div_tiles_x);
    const int txi       = bid - trow * a.tiles_x;
    const int n         = fdiv(trow, a.div_tiles_y);
    const int tyi       = trow - n * a.tiles_y;
    const int oy0 = tyi * a.TH, ox0 = txi * a.TW;
    const int y0 = oy0 * a.sy - a.pad_top, x0 = ox0 * a.sx - a.pad_left;

    // ---- per-channel operands: requested first, used after the patch loads have been issued ---------------------
    uint32_t flags = 0;
    const bool tab_lane = tid < C;
    int32_t t_bias = 0, t_mult = 0, t_shift = 32;
    int8_t t_w[TAPS];
    if (tab_lane)
    {
        t_bias = a.bias[a.bias_len == 1 ? 0 : tid];
        if constexpr (FUSED)
        {
            t_mult  = load_multiplier(a.rp, tid);
            t_shift = load_shift(a.rp, tid);
        }
#pragma unroll
        for (int t = 0; t < TAPS; t++)
            t_w[t] = a.w[t * C + tid];
    }

    // ---- the input patch: straight into LDS ----------------------------------------------------------------------
    {
        const uint32_t lbase = (uint32_t)(uintptr_t)lds;
        const uint8_t* in_n  = a.in + (size_t)n * a.IH * a.IW * C;
        const int s0         = wave * 64 + lane;
        // slot s0 = (patch row py, pixel px, chunk ch); a round of loads later it is step_row rows, step_px pixels and
        // step_ch chunks further on, wrapped with additions only (a row ends with row_pad spare chunks)
        int py       = fdiv(s0, a.div_pitch);
        const int r0 = s0 - py * a.pitch;
        int px       = fdiv(r0, a.div_ppitch);
        int ch       = r0 - px * a.ppitch;
        uint32_t dst = lbase + wave * 1024;
        for (int l = wave; l < p_loads; l += nwaves)
        {
            const int iy = y0 + py, ix = x0 + px;
            const bool img = py < a.PH && px < a.PW && (unsigned)iy < (unsigned)a.IH && (unsigned)ix < (unsigned)a.IW;
            const int cc   = ch < a.cpp ? ch : 0;    // the spare chunk of a pixel reads its first one
            const uint8_t* src = img ? in_n + mad_u24(mad_u24((uint32_t)iy, (uint32_t)a.IW, (uint32_t)ix), (uint32_t)C, (uint32_t)(cc * 16))
                                     : a.pad_page + (cc & 3) * 16;
            dwslab_load(src, dst);
            dst += nwaves * 1024;
            py += a.step_row, px += a.step_px, ch += a.step_ch;
            if (ch >= a.ppitch)
                ch -= a.ppitch, px++;
            // past the end of the row (pixels PW .. hold the row's spare chunks): on to the next row
            if (__mul24(px, a.ppitch) + ch >= a.pitch)
            {
                ch -= a.wrap_ch, px -= a.wrap_px, py++;
                if (ch < 0)
                    ch += a.ppitch, px--;
            }
        }
    }

    // ---- tables ----------------------------------------------------------------------------------------------------
    if (tid < ((C + 63) & ~63))    // whole waves, so that the wave-wide votes below see every lane
    {
        int wsum = 0;
#pragma unroll
        for (int t = 0; t < TAPS; t++)
            wsum += tab_lane ? (int)t_w[t] : 0;
        int32_t m = 0;
        if constexpr (FUSED)
        {
            // lanes past C take the wave's first shift, so that they do not break a wave whose channels share one
            const int32_t s_first = __builtin_amdgcn_readfirstlane(t_shift);
            const ChannelScale cs =
                make_channel_scale(tab_lane ? t_mult : 0, tab_lane ? t_shift : s_first, a.rp.double_round != 0, flags);
            m             = cs.m;
            // The epilogue has three forms, chosen per group of 64 channels (one table wave):
            //   every shift large enough for the high-word form (tmi_device.h) and small enough for output_zp * 2^shift
            //   to ride in the 64-bit rounding term: 16 bytes of constants per channel, no value-range test (-2);
            //   the same with one shift for all 64 channels: rounding term and shift are scalars (the shift itself);
            //   anything else: fast_rescale() with its range test and a 64-bit shift (-1).
            // With double rounding a value below zero takes a rounding term 2^31 smaller; where the result is clamped at or
            // above output_zp anyway, a negative value ends at the lower limit with either term (the scaled value is at
            // most 0 for a multiplier >= 0), and the first two forms skip the sign test (bit 8 of the shift; -3).
            const int s_min = a.rp.double_round ? 33 : 32;
            const int folds = __all(cs.s >= s_min && cs.s <= zp_fold_max_shift(a.rp.out_zp));
            const int uni   = folds && __all(cs.s == s_first);
            const int relu  = a.rp.double_round && a.rp.lo >= a.rp.out_zp && __all(cs.m >= 0);
            if (tab_lane)
            {
                tab_cs[tid] = cs;
                tab_hw[tid] = make_high_word_scale(cs, a.rp.out_zp);
            }
            if (lane == 0)
                uni_shift[wave] = uni ? (s_first | (relu << 8)) : (folds ? (relu ? -3 : -2) : -1);
        }
        if (tab_lane)
        {
            tab_m[tid] = m;
            tab_b[tid] = t_bias - (ZA ? a.za * wsum : 0);
            int32_t* wp = wtab + tid;
#pragma unroll
            for (int t = 0; t < TAPS; t++, wp += C)    // byte 0 in all four bytes: one permute, no multiply
                *wp = __builtin_amdgcn_perm((int)t_w[t], (int)t_w[t], 0x04040404);
        }
        else
            flags = 0;    // lanes without a channel report nothing
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // ---- units: (pixel tile of 32, channel block of 32) ---------------------------------------------------------
    const int P        = a.TH * a.TW;
    const int row_step = a.dy * a.pitch * 16;
    const int col_step = a.dx * a.ppitch * 16;
    // operand row li of the diagonal matrix stands for channel wr of the block
    const int wr = 4 * (li & 4) + ((li >> 1) & 12) + (li & 3);
    // row li is non-zero at K index wr only, which lies in this lane's K half when wr / 16 == lh: byte wr % 4 of word
    // (wr / 4) % 4 of the lane's 16 operand bytes
    int wmask[4];
#pragma unroll
    for (int k = 0; k < 4; k++)
        wmask[k] = ((wr >> 4) == lh && ((wr >> 2) & 3) == k) ? 0xff << ((wr & 3) * 8) : 0;
    for (int u = wave; u < a.n_units; u += nwaves)
    {
        const int pxt = fdiv(u, a.div_cblk);
        const int cb  = u - pxt * a.n_cblk;
        const int c0  = cb * 32;
        int p         = pxt * 32 + li;
        const bool p_in_tile = p < P;
        p             = p_in_tile ? p : 0;
        const int ty  = fdiv(p, a.div_tw);
        const int tx  = p - ty * a.TW;
        // Everything the nine MFMAs need is requested up front, in a pinned order: left alone, the compiler requests a
        // tap's pixel fragment right before its MFMA and a wave waits out the LDS latency nine times in a row.
        // The diagonal operands of this channel block are built from the replicated weight bytes (channels past C:
        // zero rows).
        const int c          = c0 + wr;
        const int32_t* wcol  = wtab + (c < C ? c : 0);
        // the nine tap addresses are this one plus scalars; kept opaque so that the products are not redistributed
        // over the taps (a 32-bit vector multiply runs at a quarter of the rate)
        uint32_t pbase = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)pl +
                         (uint32_t)((ty * a.sy * a.pitch + tx * a.sx * a.ppitch) * 16 + c0 + lh * 16);
        asm volatile("" : "+v"(pbase));
        // (lane, register e) = channel c0 + 16 lh + e of pixel li; the accumulators start at the channel's bias term
        const int cl  = c0 + 16 * lh;
        const int clc = cl < C ? cl : 0;    // C is a multiple of 16
        v16i acc;
#pragma unroll
        for (int q = 0; q < 4; q++)
        {
            const v4i b4 = *reinterpret_cast<const v4i*>(tab_b + clc + 4 * q);
            acc[4 * q] = b4[0], acc[4 * q + 1] = b4[1], acc[4 * q + 2] = b4[2], acc[4 * q + 3] = b4[3];
        }
        int wv[TAPS];
        v4i fb[TAPS];
#pragma unroll
        for (int t = 0; t < TAPS; t++)
            wv[t] = wcol[t * C];
#pragma unroll
        for (int t = 0; t < TAPS; t++)
            fb[t] = *(const __attribute__((address_space(3))) v4i*)(uintptr_t)(pbase + (uint32_t)((t / 3) * row_step + (t % 3) * col_step));
        __builtin_amdgcn_sched_barrier(0);
        int wm[4];
#pragma unroll
        for (int k = 0; k < 4; k++)
            wm[k] = c < C ? wmask[k] : 0;
#pragma unroll
        for (int t = 0; t < TAPS; t++)
        {
            const v4i fa = v4i{ wv[t] & wm[0], wv[t] & wm[1], wv[t] & wm[2], wv[t] & wm[3] };
            acc          = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb[t], acc, 0, 0, 0);
        }

        // ---- epilogue ------------------------------------------------------------------------------------------------
        const int oy = oy0 + ty, ox = ox0 + tx;
        const bool ok = p_in_tile && oy < a.OH && ox < a.OW && cl < C;
        // the tensor has fewer than 2^31 elements (checked by the launcher): 32-bit arithmetic
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
            const int s_form = __builtin_amdgcn_readfirstlane(uni_shift[c0 >> 6]);    // the form of this block's group
            const bool sign_test = a.rp.double_round && (s_form >= 0 ? (s_form >> 8) == 0 : s_form == -2);
            if (s_form >= 0)
            {
                // one shift for all 64 channels: the high-word form with its constants in scalar registers
                const int s_uni   = s_form & 255;
                const int64_t rnd = (int64_t(1) << (s_uni - 1)) + (a.rp.double_round ? (int64_t(1) << 30) : 0) +
                                    ((int64_t)a.rp.out_zp << s_uni);
                const int sh        = s_uni - 32;
                int32_t cm[16];
#pragma unroll
                for (int q = 0; q < 4; q++)
                {
                    const v4i m4 = *reinterpret_cast<const v4i*>(tab_m + clc + 4 * q);
                    cm[4 * q] = m4[0], cm[4 * q + 1] = m4[1], cm[4 * q + 2] = m4[2], cm[4 * q + 3] = m4[3];
                }
                if (sign_test)
                {
#pragma unroll
                    for (int e = 0; e < 16; e++)
                        r[e] = clamp_med3(high_word_rescale64<true>(acc[e], cm[e], rnd, sh), a.rp.lo, a.rp.hi);
                }
                else
                {
#pragma unroll
                    for (int e = 0; e < 16; e++)
                        r[e] = clamp_med3(high_word_rescale64<false>(acc[e], cm[e], rnd, sh), a.rp.lo, a.rp.hi);
                }
            }
            else if (s_form <= -2)
            {
                if (sign_test)
                {
#pragma unroll
                    for (int e = 0; e < 16; e++)
                    {
                        const HighWordScale c = tab_hw[clc + e];
                        r[e] = clamp_med3(high_word_rescale64<true>(acc[e], c), a.rp.lo, a.rp.hi);
                    }
                }
                else
                {
#pragma unroll
                    for (int e = 0; e < 16; e++)
                    {
                        const HighWordScale c = tab_hw[clc + e];
                        r[e] = clamp_med3(high_word_rescale64<false>(acc[e], c), a.rp.lo, a.rp.hi);
                    }
                }
            }
            else
            {
                uint32_t eflags = 0;
#pragma unroll
                for (int e = 0; e < 16; e++)
                {
                    const ChannelScale cs = tab_cs[clc + e];
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
    }
    raise_flags(a.flag_word, flags);
}

template <bool ZA, bool FUSED>
static bool launch_dwslab_kernel(hipStream_t st, const DwSlabArgs& a, int grid, int threads, int lds_bytes)
{
    auto kern = depthwise_slab_kernel<ZA, FUSED>;
    static LdsLimit granted{};
    if (!ensure_dynamic_lds(reinterpret_cast<const void*>(kern), (size_t)lds_bytes, granted))
        return false;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), lds_bytes, st, a);
    return true;
}

// nullptr when the layer is not one this kernel takes; the caller then goes to the vector kernel.
const char* launch_depthwise_slab(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                                  const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                                  void* out, const void* pad_page, uint32_t* flag_word)
{
    if (in_dtype != TMI_INT8 || g.M != 1 || g.KH != 3 || g.KW != 3 || w_zp != 0 || !pad_page || !flag_word)
        return nullptr;
    if ((g.IC & 15) || g.IC < 32 || g.IC > 1024 || g.OC != g.IC)
        return nullptr;
    if (rp.enabled ? (!rp.fast || (out_dtype != TMI_INT8 && out_dtype != TMI_INT16)) : out_dtype != TMI_INT32)
        return nullptr;
    if ((((uintptr_t)in | (uintptr_t)out | (uintptr_t)pad_page) & 15) || ((uintptr_t)bias & 3) || g.N < 1 || g.OH < 1 ||
        g.OW < 1)
        return nullptr;
    if ((int64_t)g.IH * g.IW >= (1 << 24) || (int64_t)g.IH * g.IW * g.IC >= (int64_t(1) << 31) ||
        (int64_t)g.N * g.OH * g.OW * g.IC >= (int64_t(1) << 31))
        return nullptr;

    const int C = g.IC, cpp = C / 16, ppitch = cpp | 1, n_cblk = (C + 31) / 32;
    // The tile: at most 128 pixels (four pixel tiles of 32); a workgroup of NW waves shares the units
    // (pixel tile, channel block) and the patch loads.  Rounds of 256 workgroups count; within a workgroup the loads
    // per wave and the units per wave do.  The search depends on the geometry only: the last answer is kept.
    struct Choice
    {
        int32_t key[8];
        int th, tw, nw;
    };
    static thread_local Choice last = { { 0, 0, 0, 0, 0, 0, 0, 0 }, 0, 0, 0 };
    const int32_t key[8] = { g.N, g.OH, g.OW, C, g.stride_y, g.stride_x, g.dil_y, g.dil_x };
    int best_th = 0, best_tw = 0, best_nw = 0;
    // weights, both forms of the requantisation constants, multipliers, bias terms, the table waves' shifts
    const int table_bytes = 9 * C * 4 + C * (int)(sizeof(ChannelScale) + sizeof(HighWordScale)) + C * 8 + 64;
    constexpr int lds_max = 160 * 1024;
    if (memcmp(key, last.key, sizeof(key)) == 0)
        best_th = last.th, best_tw = last.tw, best_nw = last.nw;
    else
    {
        int64_t best_cost = 0, best_busy = 0, best_moved = 0;
        for (int th = 1; th <= g.OH && th <= 128; th++)
            for (int tw = 1; tw <= g.OW && th * tw <= 128; tw++)
            {
                const int ph = (th - 1) * g.stride_y + 2 * g.dil_y + 1;
                const int pw = (tw - 1) * g.stride_x + 2 * g.dil_x + 1;
                const int64_t slots = (int64_t)ph * (pw * ppitch + 15);
                // (the patch is rounded up to whole rounds of 64 slots, and a row may take up to 15 chunks of padding)
                if (slots >= (1 << 16) || slots * 16 > 96 * 1024 || slots * 16 + 1024 + table_bytes > lds_max)
                    continue;
                const int units        = ((th * tw + 31) / 32) * n_cblk;
                const int64_t tiles    = (int64_t)g.N * ((g.OH + th - 1) / th) * ((g.OW + tw - 1) / tw);
                const int64_t rounds   = (tiles + 255) / 256;
                // A single round of workgroups (one per CU) is as fast as its slowest wave: up to 16 waves, so that a
                // wave has one unit.  With more rounds two workgroups of at most 8 waves share a CU and overlap.
                for (int nw = (rounds == 1 ? 16 : 8); nw >= 4; nw -= 2)    // equal cost: the larger workgroup
                {
                    if (nw * 64 < C)    // the first C lanes build the per-channel tables
                        continue;
                    const int64_t loads = (slots / 64 + nw) / nw, turns = (units + nw - 1) / nw;
                    // per workgroup: a fixed part, the loads a wave issues, the units a wave works through
                    const int64_t cost = rounds * (60 + 5 * loads + 30 * turns);
                    // equal cost: the shape that keeps more of the 256 CUs busy, then the one that moves the fewest
                    // chunks into LDS over the whole layer, then the larger tile (measured on the MobileNet layer, us:
                    // 7x15 and 14x7 tiles on 256 CUs 5.06 and 5.01, 7x17 5.23, 8x14 tiles on 224 CUs 5.16)
                    const int64_t busy = tiles < 256 ? tiles : 256, moved = tiles * slots;
                    if (!best_th || cost < best_cost ||
                        (cost == best_cost &&
                         (busy > best_busy ||
                          (busy == best_busy && (moved < best_moved || (moved == best_moved && th * tw > best_th * best_tw))))))
                        best_th = th, best_tw = tw, best_nw = nw, best_cost = cost, best_busy = busy, best_moved = moved;
                }
            }
        memcpy(last.key, key, sizeof(key));
        last.th = best_th, last.tw = best_tw, last.nw = best_nw;
    }
    if (!best_th)
        return nullptr;

    DwSlabArgs a{};
    a.in = (const uint8_t*)in, a.w = (const int8_t*)w, a.bias = (const int32_t*)bias, a.out = out;
    a.pad_page = (const uint8_t*)pad_page, a.flag_word = flag_word, a.rp = rp;
    a.N = g.N, a.IH = g.IH, a.IW = g.IW, a.C = C, a.OH = g.OH, a.OW = g.OW;
    a.sy = g.stride_y, a.sx = g.stride_x, a.dy = g.dil_y, a.dx = g.dil_x, a.pad_top = g.pad_top, a.pad_left = g.pad_left;
    a.TH = best_th, a.TW = best_tw;
    a.PH = (best_th - 1) * g.stride_y + 2 * g.dil_y + 1;
    a.PW = (best_tw - 1) * g.stride_x + 2 * g.dil_x + 1;
    a.tiles_y = (g.OH + best_th - 1) / best_th, a.tiles_x = (g.OW + best_tw - 1) / best_tw;
    a.bias_len = g.bias_len, a.za = in_zp;
    a.out_kind = !rp.enabled ? 0 : (out_dtype == TMI_INT8 ? 1 : 2);
    a.cpp = cpp, a.ppitch = ppitch, a.n_cblk = n_cblk;
    a.n_units = ((best_th * best_tw + 31) / 32) * n_cblk;
    // The chunk of tile pixel p = ty * TW + tx under tap (0, 0) is ty * sy * pitch + tx * sx * ppitch; the 16 lanes a
    // ds_read_b128 serves together differ modulo 16, so the reads are free of bank conflicts when that chunk is an odd
    // multiple of p plus a constant (modulo 16): sx * ppitch odd and sy * pitch = sx * ppitch * TW (mod 16).  Odd
    // strides get there with up to 15 chunks of padding per patch row; even strides keep their conflicts.
    int pad = 0;
    if ((g.stride_x & 1) && (g.stride_y & 1))
        for (pad = 0; pad < 16; pad++)
            if (((g.stride_y * (a.PW * ppitch + pad) - g.stride_x * ppitch * a.TW) & 15) == 0)
                break;
    a.pitch = a.PW * ppitch + (pad & 15);
    const int per_round = best_nw * 64;
    a.wrap_px = a.pitch / ppitch, a.wrap_ch = a.pitch % ppitch;
    a.step_row = per_round / a.pitch;
    a.step_px = (per_round % a.pitch) / ppitch, a.step_ch = (per_round % a.pitch) % ppitch;
    const int64_t grid = (int64_t)g.N * a.tiles_y * a.tiles_x;
    if (!tile_decode_is_exact(grid, 1u, (uint32_t)a.tiles_x, (uint32_t)a.tiles_y))
        return nullptr;
    a.xcd_remap = grid % 8 == 0 ? (int32_t)(grid / 8) : 0;
    a.div_tw = make_fastdiv((uint32_t)a.TW), a.div_pitch = make_fastdiv((uint32_t)a.pitch);
    a.div_ppitch = make_fastdiv((uint32_t)ppitch);
    a.div_tiles_x = make_fastdiv((uint32_t)a.tiles_x), a.div_tiles_y = make_fastdiv((uint32_t)a.tiles_y);
    a.div_cblk = make_fastdiv((uint32_t)n_cblk);
    const int p_loads   = (a.PH * a.pitch + 63) / 64;
    const int lds_bytes = p_loads * 1024 + table_bytes;
    if (lds_bytes > lds_max)
        return nullptr;
    bool ok;
    if (in_zp != 0)
        ok = rp.enabled ? launch_dwslab_kernel<true, true>(st, a, (int)grid, per_round, lds_bytes)
                        : launch_dwslab_kernel<true, false>(st, a, (int)grid, per_round, lds_bytes);
    else
        ok = rp.enabled ? launch_dwslab_kernel<false, true>(st, a, (int)grid, per_round, lds_bytes)
                        : launch_dwslab_kernel<false, false>(st, a, (int)grid, per_round, lds_bytes);
    if (!ok)
        return nullptr;
    return rp.enabled ? "depthwise_mfma_i8_rescale" : "depthwise_mfma_i8";
}

}    // namespace tmi
