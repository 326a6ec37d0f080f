// Small int8 CONV2D layers with taps and a long reduction (3x3 over 128 ... 512 channels on images of 14 x 14 or 7 x 7
// pixels: the last stages of a classification network), with or without the fused RESCALE (+ CLAMP).
//
//   out[n][oy][ox][oc] = sum_{ky,kx,ic} (in[n][oy*sy - pt + ky*dy][ox*sx - pl + kx*dx][ic] - input_zp) * w[oc][ky][kx][ic]
//                        + bias[oc]                                                     (tensor_ops.cpp:828-882)
//
// Such a layer has few output tiles (8 x 14 x 14 pixels x 256 channels: 26 tiles of 128 x 128) and K = 2304 ... 4608, so a
// kernel that gives a workgroup a large tile keeps a tenth of the chip busy.  Here a workgroup of NW waves (4, 8 or 16) owns a
// tile of 32 output channels x 32 pixels and splits the K steps (ky, kx, 32 channels) between its waves; both operands go
// straight from global memory into the registers the matrix instruction reads - the weight rows are K-contiguous as they
// lie, a pixel fragment is 16 bytes of the input pixel under the step's tap, or of the context's page of input_zp bytes
// where that tap falls outside the image - with every load of the tile in flight at once.  Each wave's accumulators start
// from its share of bias - input_zp * sum(w); the partial tiles meet in LDS and the first four waves requantise and store
// a quarter of the tile each (4 consecutive channels per lane).
//
// weight_zp must be 0, IC a multiple of 32, OC a multiple of 8, and K at most 160 steps (16 waves of 10).
#include "tmi_mfma.h"

namespace tmi
{

struct ConvSplitArgs
{
    const uint8_t* in;
    const int8_t* w;
    const int32_t* bias;
    const uint8_t* pad_page;    // 64 bytes of input_zp
    void* out;
    uint32_t* flag_word;
    RescaleParams rp;
    int32_t P, IC, OC;    // output pixels (N * OH * OW), input and output channels
    int32_t IH, IW, OH, OW, KW;
    int32_t sy, sx, dy, dx, pad_top, pad_left;
    int32_t za, bias_len;
    int32_t out_kind;     // 0: int32 accumulators, 1: int8 through the RESCALE, 2: int16 through the RESCALE
    int32_t n_oct, n_pt, n_groups;
    int32_t steps;        // K steps in all = taps * IC / 32
    int32_t spt;          // K steps per tap = IC / 32
    int32_t ksw;          // K steps per wave
    FastDiv div_oct, div_spt, div_kw, div_ow, div_oh;
};

// apply_scale_32 + output_zp + clip (+ CLAMP) from the multiplier and the validated shift (see pointwise.hip)
__device__ __forceinline__ int32_t split_rescale_from_shift(int32_t v, int32_t m, int32_t s, bool double_round, int32_t out_zp,
                                                            int32_t lo, int32_t hi, uint32_t& flags)
{
    if (s <= 31)
    {
        const int32_t high = 1 << (s - 1);
        if (v < -high || v >= high)
            flags |= TMI_FLAG_SCALE_VALUE;
    }
    int64_t round = int64_t(1) << (s - 1);
    if (double_round && s > 31)
        round += v >= 0 ? (int64_t(1) << 30) : -(int64_t(1) << 30);
    const int64_t p = (int64_t)v * (int64_t)m + round;
    int32_t r       = (int32_t)(p >> s) + out_zp;
    r               = r < lo ? lo : r;
    return r > hi ? hi : r;
}

template <int KS, int NW, bool ZA>
__global__ __launch_bounds__(NW * 64, NW == 16 ? 4 : 2) void conv_ksplit_i8_kernel(ConvSplitArgs a)
{
    // [NW waves x 4 quarters x 64 lanes x 16 bytes][32 x HighWordScale][32 x (m, s)][NW waves x 32 start values][form]
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const uint32_t g = blockIdx.x;
    const int q = (int)fdiv(g, a.div_oct), oct = (int)g - q * a.n_oct;
    const int G = a.n_groups;
    HighWordScale* tab_hw = reinterpret_cast<HighWordScale*>(lds + NW * 4096);
    v2i* tab_ms           = reinterpret_cast<v2i*>(tab_hw + 32);
    int32_t* wave_start   = reinterpret_cast<int32_t*>(tab_ms + 32) + wave * 32;
    int32_t* form_word    = reinterpret_cast<int32_t*>(tab_ms + 32) + NW * 32;
    const int ksw   = a.ksw;
    const int step0 = wave * ksw;    // first K step of the wave's share
    const int nvalid = a.steps - step0 < ksw ? (a.steps - step0 > 0 ? a.steps - step0 : 0) : ksw;    // steps of the share that exist
    const int kbytes = a.steps * 32; // bytes of a weight row

    // ---- pixel fragments: lane (li, lh) holds bytes [16 lh, + 16) of the 32 channels of step s under the step's tap ------
    auto load_pixels = [&](v4i (&fb)[KS], int pt) {
        int p = pt * 32 + li;
        p     = p < a.P ? p : a.P - 1;    // a pixel past the end: the last one again, never stored
        const int row = (int)fdiv((uint32_t)p, a.div_ow);    // n * OH + oy
        const int ox  = p - row * a.OW;
        const int n   = (int)fdiv((uint32_t)row, a.div_oh);
        const int oy  = row - n * a.OH;
        const int iy0 = oy * a.sy - a.pad_top, ix0 = ox * a.sx - a.pad_left;
        const uint8_t* img = a.in + (size_t)n * a.IH * a.IW * a.IC;
        // A wave with one wave on its SIMD issues an instruction every eight clocks or so, so what a step costs is its
        // instruction count: the tap's pixel is worked out once per tap (the wave's first step with divisions, the following
        // taps by stepping: scalar work, the same for all lanes) and a step inside a tap is a load and an addition.
        int tap = (int)fdiv((uint32_t)step0, a.div_spt);
        int cs  = step0 - tap * a.spt;    // which 32 channels of the tap
        int ky  = (int)fdiv((uint32_t)tap, a.div_kw);
        int kx  = tap - ky * a.KW;
        const uint8_t* cur = nullptr;
        uint32_t inc       = 0;
        auto at_tap        = [&]() {
            const int iy = iy0 + ky * a.dy, ix = ix0 + kx * a.dx;
            const bool inside  = (unsigned)iy < (unsigned)a.IH && (unsigned)ix < (unsigned)a.IW;
            const uint32_t off = (uint32_t)((iy * a.IW + ix) * a.IC + cs * 32 + 16 * lh);    // one image is below 2^31 bytes
            cur                = inside ? img + off : a.pad_page + 16 * lh;
            inc                = inside ? 32u : 0u;    // outside the image every step reads the page of input_zp bytes
        };
        at_tap();
#pragma unroll
        for (int s = 0; s < KS; s++)
        {
            if (s < nvalid)    // (a test per step, not a loop exit: the register array keeps constant indices)
            {
                fb[s] = *reinterpret_cast<const v4i*>(cur);
                cur += inc;
                cs++;
                if (cs == a.spt)
                {
                    cs = 0, kx++;
                    if (kx == a.KW)
                        kx = 0, ky++;
                    at_tap();
                }
            }
        }
    };
    v4i fb[KS];
    load_pixels(fb, q);

    // ---- weight fragments: MFMA operand row li is channel 16 * ((li >> 2) & 1) + 4 * (li >> 3) + (li & 3) of the tile -------
    const int wr = 4 * (li & 4) + ((li >> 1) & 12) + (li & 3);
    const int ch = oct * 32 + wr;
    v4i fa[KS];
    {
        // one 32-bit offset per lane; the steps are the instruction's offset field (the weights are below 2^31 bytes)
        const uint32_t woff = (uint32_t)((ch < a.OC ? ch : a.OC - 1) * kbytes + step0 * 32 + 16 * lh);
#pragma unroll
        for (int s = 0; s < KS; s++)
        {
            if (s < nvalid)
                fa[s] = *reinterpret_cast<const v4i*>(a.w + woff + s * 32);
        }
    }
    // (rows past OC are zeroed further down, once, so that no load is waited for before the next one is issued)
    uint32_t flags = 0;
    if (wave == 0)
    {
        // the first wave derives the constants of the tile's 32 channels for all
        const int oc  = oct * 32 + li;
        const bool ok = oc < a.OC;
        const int occ = ok ? oc : oct * 32;
        if (a.rp.enabled)
        {
            const int32_t m_raw   = load_multiplier(a.rp, occ);
            const int32_t s_raw   = load_shift(a.rp, occ);
            const int32_t s_first = __builtin_amdgcn_readfirstlane(s_raw);
            const ChannelScale cs = make_channel_scale(ok ? m_raw : 0, ok ? s_raw : s_first, a.rp.double_round != 0, flags);
            const int s_min       = a.rp.double_round ? 33 : 32;
            // bit 0: the high-word form for all 32 channels; bit 1: no sign test in it (a negative value is clamped away
            // with either rounding term: the result's lower limit is at or above output_zp and no multiplier is negative)
            const int form = (__all(cs.s >= s_min && cs.s <= zp_fold_max_shift(a.rp.out_zp)) ? 1 : 0) |
                             (a.rp.lo >= a.rp.out_zp && __all(cs.m >= 0) ? 2 : 0);
            if (lh == 0)
            {
                tab_ms[li] = v2i{ cs.m, cs.s };
                tab_hw[li] = make_high_word_scale(cs, a.rp.out_zp);
            }
            if (lane == 0)
                *form_word = form;
        }
    }
    if (ch >= a.OC)
    {
#pragma unroll
        for (int s = 0; s < KS; s++)
            fa[s] = v4i{ 0, 0, 0, 0 };
    }
    {
        int32_t b = wave == 0 ? a.bias[a.bias_len == 1 ? 0 : (ch < a.OC ? ch : oct * 32)] : 0;
        if constexpr (ZA)
        {
            int sum = 0;
#pragma unroll
            for (int s = 0; s < KS; s++)
                if (s < nvalid)
                    sum += dot4_ones(fa[s]);
            sum += __builtin_amdgcn_ds_bpermute((lane ^ 32) * 4, sum);
            b = (int32_t)((uint32_t)b - (uint32_t)a.za * (uint32_t)sum);
        }
        if (lh == 0)
            wave_start[wr] = ch < a.OC ? b : 0;
        __builtin_amdgcn_wave_barrier();    // the wave's own LDS accesses complete in order
    }
    // (a tile's start values are read from the wave's table again for every tile: the registers are needed for the loads)
    auto start_values = [&]() {
        int first = 16 * lh;
        asm volatile("" : "+v"(first));    // (hidden from the compiler, which would otherwise keep them across the loop)
        v16i start;
#pragma unroll
        for (int gq = 0; gq < 4; gq++)
        {
            const v4i b4 = *reinterpret_cast<const v4i*>(wave_start + first + 4 * gq);
            start[4 * gq] = b4[0], start[4 * gq + 1] = b4[1], start[4 * gq + 2] = b4[2], start[4 * gq + 3] = b4[3];
        }
        return start;
    };
    const int oc_lane = oct * 32 + 16 * lh + 4 * (wave & 3);    // first of the 4 channels a lane of waves 0 .. 3 stores
    const bool ch_ok  = oc_lane < a.OC;                         // OC is a multiple of 8: the four are in or out together
    const int32_t v_lo = a.rp.lo, v_hi = a.rp.hi;
    for (int pt = q; pt < a.n_pt; pt += G)
    {
        v16i acc = start_values();
#pragma unroll
        for (int s = 0; s < KS; s++)
            if (s < nvalid)
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[s], fb[s], acc, 0, 0, 0);
        if (pt + G < a.n_pt)
            load_pixels(fb, pt + G);    // in flight across the exchange and the requantisation
        // the partial tiles meet in LDS: [wave][quarter][lane] of 16 bytes
        if (pt != q)
            __syncthreads();    // every wave has read the tile before
#pragma unroll
        for (int gq = 0; gq < 4; gq++)
            *reinterpret_cast<v4i*>(lds + ((wave * 4 + gq) * 64 + lane) * 16) = v4i{ acc[4 * gq], acc[4 * gq + 1], acc[4 * gq + 2], acc[4 * gq + 3] };
        __syncthreads();    // also publishes the first wave's tables
        if (wave >= 4)
            continue;
        v4i sum = *reinterpret_cast<const v4i*>(lds + ((0 * 4 + wave) * 64 + lane) * 16);
#pragma unroll
        for (int w2 = 1; w2 < NW; w2++)
        {
            const v4i o = *reinterpret_cast<const v4i*>(lds + ((w2 * 4 + wave) * 64 + lane) * 16);
            sum.x += o.x, sum.y += o.y, sum.z += o.z, sum.w += o.w;
        }
        const int p      = pt * 32 + li;
        const bool store = p < a.P && ch_ok;
        const size_t at  = (size_t)(p < a.P ? p : 0) * a.OC + (ch_ok ? oc_lane : 0);
        if (a.out_kind == 0)
        {
            if (store)
                *reinterpret_cast<v4i*>(reinterpret_cast<int32_t*>(a.out) + at) = sum;
            continue;
        }
        const int form = *form_word;
        int32_t r[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
        {
            const int c = 16 * lh + 4 * wave + j;
            if (form & 1)
                r[j] = (a.rp.double_round && !(form & 2)) ? clamp_med3(high_word_rescale64<true>(sum[j], tab_hw[c]), v_lo, v_hi)
                                                          : clamp_med3(high_word_rescale64<false>(sum[j], tab_hw[c]), v_lo, v_hi);
            else
            {
                uint32_t f   = 0;
                const v2i ms = tab_ms[c];
                r[j]         = split_rescale_from_shift(sum[j], ms.x, ms.y, a.rp.double_round != 0, a.rp.out_zp, v_lo, v_hi, f);
                flags |= store ? f : 0u;
            }
        }
        if (a.out_kind == 1)
        {
            const int lo2 = __builtin_amdgcn_perm(r[1], r[0], 0x0c0c0400);
            const int hi2 = __builtin_amdgcn_perm(r[3], r[2], 0x04000c0c);
            if (store)
                *reinterpret_cast<int*>(reinterpret_cast<int8_t*>(a.out) + at) = lo2 | hi2;
        }
        else if (store)
            *reinterpret_cast<v2i*>(reinterpret_cast<int16_t*>(a.out) + at) =
                v2i{ (r[0] & 0xffff) | ((r[1] & 0xffff) << 16), (r[2] & 0xffff) | ((r[3] & 0xffff) << 16) };
    }
    raise_flags(a.flag_word, flags);
}

template <int KS, int NW, bool ZA>
static bool launch_conv_ksplit_za(hipStream_t st, const ConvSplitArgs& a, int grid)
{
    constexpr int lds_bytes = NW * 4096 + 32 * 16 + 32 * 8 + NW * 128 + 16;
    static LdsLimit granted{};
    auto kern = conv_ksplit_i8_kernel<KS, NW, ZA>;
    if (!ensure_dynamic_lds(reinterpret_cast<const void*>(kern), (size_t)lds_bytes, granted))
        return false;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), lds_bytes, st, a);
    last_launch_shape[0] = grid, last_launch_shape[1] = NW * 64, last_launch_shape[2] = lds_bytes;
    return true;
}

template <int KS, int NW>
static bool launch_conv_ksplit(hipStream_t st, const ConvSplitArgs& a, int grid)
{
    return a.za != 0 ? launch_conv_ksplit_za<KS, NW, true>(st, a, grid) : launch_conv_ksplit_za<KS, NW, false>(st, a, grid);
}

// nullptr when the layer is not one this kernel takes.
const char* launch_conv2d_ksplit(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                                 const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                                 void* out, const void* pad_page, uint32_t* flag_word)
{
    if (in_dtype != TMI_INT8 || w_zp != 0 || !flag_word || !pad_page)
        return nullptr;
    const int taps = g.KH * g.KW;
    if (taps < 2 || (g.IC & 31) || g.IC < 32 || (g.OC & 7) || g.OC < 8 || g.OC > 4096)
        return nullptr;
    if (rp.enabled ? (!rp.fast || (out_dtype != TMI_INT8 && out_dtype != TMI_INT16)) : out_dtype != TMI_INT32)
        return nullptr;
    if ((((uintptr_t)in | (uintptr_t)w | (uintptr_t)out | (uintptr_t)pad_page) & 15) || ((uintptr_t)bias & 3))
        return nullptr;
    const int64_t P = (int64_t)g.N * g.OH * g.OW;
    if (P < 1 || (int64_t)g.N * g.IH * g.IW * g.IC >= (int64_t(1) << 31) || P * g.OC >= (int64_t(1) << 31) ||
        (int64_t)g.OC * taps * g.IC >= (int64_t(1) << 31))
        return nullptr;
    // 4, 8 or 16 waves a workgroup: at most 10 K steps a wave (a wave's time is its instruction count)
    const int steps = taps * (g.IC / 32);
    const int nw    = steps > 80 ? 16 : (steps > 40 ? 8 : 4);
    const int ksw   = (steps + nw - 1) / nw;
    if (ksw > 10)
        return nullptr;

    ConvSplitArgs a{};
    a.in = (const uint8_t*)in, a.w = (const int8_t*)w, a.bias = (const int32_t*)bias, a.out = out;
    a.pad_page = (const uint8_t*)pad_page, a.flag_word = flag_word, a.rp = rp;
    a.P = (int32_t)P, a.IC = g.IC, a.OC = g.OC;
    a.IH = g.IH, a.IW = g.IW, a.OH = g.OH, a.OW = g.OW, a.KW = g.KW;
    a.sy = g.stride_y, a.sx = g.stride_x, a.dy = g.dil_y, a.dx = g.dil_x, a.pad_top = g.pad_top, a.pad_left = g.pad_left;
    a.za = in_zp, a.bias_len = g.bias_len;
    a.out_kind = !rp.enabled ? 0 : (out_dtype == TMI_INT8 ? 1 : 2);
    a.n_oct    = (g.OC + 31) / 32;
    a.n_pt     = (int32_t)((P + 31) / 32);
    a.steps = steps, a.spt = g.IC / 32, a.ksw = ksw;
    // At most one workgroup per CU, each walking its pixel tiles with the weight fragments in registers (us for a
    // workgroup per tile / at most 256 workgroups, 3x3, fused RESCALE: [8,14,14,256]->256 10.9 / 9.0, [16,14,14,256]->256
    // 18.5 / 12.8, [4,28,28,256]->256 19.6 / 12.9, [8,14,14,384]->384 24.1 / 15.3; 320 workgroups: 17.0 and 23.0 on the last
    // two, 192: 14.8 and 18.2).
    const int max_groups = 256 / a.n_oct > 0 ? 256 / a.n_oct : 1;
    const int per_group  = (a.n_pt + max_groups - 1) / max_groups;    // pixel tiles a workgroup walks: the same for all
    a.n_groups = (a.n_pt + per_group - 1) / per_group;
    a.div_oct = make_fastdiv((uint32_t)a.n_oct), a.div_spt = make_fastdiv((uint32_t)a.spt);
    a.div_kw = make_fastdiv((uint32_t)g.KW), a.div_ow = make_fastdiv((uint32_t)g.OW), a.div_oh = make_fastdiv((uint32_t)g.OH);
    const int grid = a.n_groups * a.n_oct;
    if (!fastdiv_exact_up_to((uint64_t)grid, (uint32_t)a.n_oct) || !fastdiv_exact_up_to((uint64_t)P, (uint32_t)g.OW) ||
        !fastdiv_exact_up_to((uint64_t)P / g.OW + 1, (uint32_t)g.OH) || !fastdiv_exact_up_to((uint64_t)steps, (uint32_t)a.spt) ||
        !fastdiv_exact_up_to((uint64_t)taps, (uint32_t)g.KW))
        return nullptr;
    bool ok;
    if (nw == 4)
        ok = ksw <= 4 ? launch_conv_ksplit<4, 4>(st, a, grid) : launch_conv_ksplit<10, 4>(st, a, grid);
    else if (nw == 8)
        ok = launch_conv_ksplit<10, 8>(st, a, grid);
    else
        ok = launch_conv_ksplit<10, 16>(st, a, grid);
    if (!ok)
        return nullptr;
    return rp.enabled ? "conv2d_ksplit_i8_rescale" : "conv2d_ksplit_i8";
}

}    // namespace tmi
