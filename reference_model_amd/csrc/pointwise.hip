// Pointwise (1x1, unit stride, no padding) int8 CONV2D with few input channels, with or without the fused RESCALE
// (+ CLAMP): the layers of MobileNet-like networks that expand or project 16 ... 160 channels.
//
//   out[p][oc] = sum_ic (in[p][ic] - input_zp) * w[oc][ic] + bias[oc]      (tensor_ops.cpp:843-882 with one tap)
//
// Such a layer moves more bytes than it multiplies, and a workgroup that stages operands in LDS and meets at barriers
// spends its time on that set-up.  Here nothing is staged and no wave waits for another: a wave owns one tile of 32
// output channels for its whole life.  It fetches its weight fragments (K steps x 16 bytes per lane) straight from global
// memory into the registers the matrix instruction reads, derives sum(w) from them (dot products with a word of ones),
// builds the 32 channels' RESCALE constants in a wave-private piece of LDS, and then walks pixel tiles of 32: the pixel
// fragments come straight from global memory as well (a lane reads 16 bytes of its pixel's channel vector; two tiles
// ahead are in flight), K steps of v_mfma_i32_32x32x32_i8 start from
// bias - input_zp * sum(w), and a lane requantises and stores the 16 consecutive channels of one pixel it ends up with.
// Waves that share pixel tiles (the channel tiles of one pixel tile) are neighbours in a workgroup, so the pixel bytes
// they all read come from HBM once.
//
// weight_zp must be 0 (the usual case for int8 weights); IC is a multiple of 8 from 16 to 160 and OC a multiple of 8.  The
// K bytes past IC (the rest of the last K step of 32) are zeros in the weight fragments, so whatever the pixel fragment
// holds there contributes nothing.
#include <type_traits>

#include "tmi_mfma.h"

namespace tmi
{

struct PointwiseArgs
{
    const uint8_t* in;
    const int8_t* w;
    const int32_t* bias;
    void* out;
    uint32_t* flag_word;
    RescaleParams rp;
    int32_t P, IC, OC;    // pixels (N * OH * OW), input and output channels
    int32_t za, bias_len;
    int32_t out_kind;    // 0: int32 accumulators, 1: int8 through the RESCALE, 2: int16 through the RESCALE
    int32_t n_oct;       // channel tiles of 32
    int32_t n_pt;        // pixel tiles of 32
    int32_t n_groups;    // groups of n_oct waves; group q takes the pixel tiles q, q + n_groups, ...
    int32_t ksw;         // the form that splits K over a workgroup's waves: K steps per wave
    FastDiv div_oct;
    // The first layer of a network (STEM): `in` is a copy of the image with its padding materialised, rows of row_bytes
    // bytes, a pixel every 4 bytes (or every IC); a K step is one row of taps, the at most 32 contiguous bytes under it; `w`
    // holds 32 bytes per (channel, tap row) in the same arrangement, so IC above is 32 * KH for the weight loads
    int32_t row_bytes, rows, OH, OW;     // padded image: bytes per row, rows per image
    int32_t step_y, step_x, step_k;      // bytes from one output row / output pixel / tap row to the next
    FastDiv div_ow, div_oh;
};

constexpr int kPointwiseWaves   = 4;
constexpr int kPointwiseWaveLds = 32 * (int)sizeof(HighWordScale) + 32 * 8 + 32 * 4;

// apply_scale_32 + output_zp + clip (+ CLAMP) from the multiplier and the (validated) shift alone: fast_rescale() with
// its per-channel constants worked out on the spot, for the channel tiles whose shifts rule out the high-word form.  Few
// registers matter more here than few instructions.
__device__ __forceinline__ int32_t rescale_from_shift(int32_t v, int32_t m, int32_t s, bool double_round, int32_t out_zp,
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

template <int KSTEPS, bool ZA, bool STEM = false>
__global__ __launch_bounds__(kPointwiseWaves * 64, KSTEPS <= 2 ? 3 : 2) void pointwise_i8_kernel(PointwiseArgs a)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[kPointwiseWaves][kPointwiseWaveLds];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const uint32_t g = blockIdx.x * kPointwiseWaves + wave;
    if (g >= (uint32_t)(a.n_groups * a.n_oct))
        return;
    const int q = (int)fdiv(g, a.div_oct), oct = (int)g - q * a.n_oct;
    const int G = a.n_groups;
    HighWordScale* tab_hw = reinterpret_cast<HighWordScale*>(lds[wave]);
    v2i* tab_ms           = reinterpret_cast<v2i*>(tab_hw + 32);    // multiplier and validated shift
    int32_t* wave_start   = reinterpret_cast<int32_t*>(tab_ms + 32);

    // ---- pixel fragments: lane (li, lh) holds bytes [32 s + 16 lh, + 16) of pixel 32 pt + li ---------------------------
    // (channel vectors of whole 16-byte chunks, or of 8-byte pieces: 24, 40, 56 ... channels, fetched 8 bytes at a time)
    const bool by8 = (a.IC & 8) != 0;
    auto load_pixels = [&](v4i (&fb)[KSTEPS], int pt) {
        int p = pt * 32 + li;
        p     = p < a.P ? p : a.P - 1;    // a pixel past the end: the last one again, never stored
        if constexpr (STEM)
        {
            // 16 of the 32 bytes that start under the window's tap (ky, 0): KW pixels of them are the row of taps, the rest
            // meets zero weights; the address is a multiple of 4 where the copy's pixels are 4 bytes apart and has no
            // alignment otherwise (the compiler is told the latter and chooses the load)
            const int r  = (int)fdiv((uint32_t)p, a.div_ow);    // n * OH + oy
            const int ox = p - r * a.OW;
            const int n  = (int)fdiv((uint32_t)r, a.div_oh);
            const int oy = r - n * a.OH;
            const uint8_t* win = a.in + (uint32_t)((n * a.rows) * a.row_bytes + oy * a.step_y + ox * a.step_x + 16 * lh);
#pragma unroll
            for (int s = 0; s < KSTEPS; s++)
                __builtin_memcpy(&fb[s], win + s * a.step_k, 16);
            return;
        }
        const uint8_t* row = a.in + (size_t)p * a.IC;
#pragma unroll
        for (int s = 0; s < KSTEPS; s++)
        {
            const int k0 = 32 * s + 16 * lh;
            if (!by8)
                fb[s] = *reinterpret_cast<const v4i*>(row + (k0 < a.IC ? k0 : 0));    // past IC: any bytes, times zero weights
            else
            {
                const v2i lo = *reinterpret_cast<const v2i*>(row + (k0 < a.IC ? k0 : 0));
                const v2i hi = *reinterpret_cast<const v2i*>(row + (k0 + 8 < a.IC ? k0 + 8 : 0));
                fb[s]        = v4i{ lo.x, lo.y, hi.x, hi.y };
            }
        }
    };
    v4i fb0[KSTEPS], fb1[KSTEPS];
    load_pixels(fb0, q);
    if (q + G < a.n_pt)
        load_pixels(fb1, q + G);

    // ---- weight fragments: MFMA operand row li is channel 16 * ((li >> 2) & 1) + 4 * (li >> 3) + (li & 3) of the tile, so
    // that a lane's 16 accumulators are 16 consecutive channels of its pixel -------------------------------------------
    const int wr = 4 * (li & 4) + ((li >> 1) & 12) + (li & 3);
    const int ch = oct * 32 + wr;
    v4i fa[KSTEPS];
    {
        const int8_t* row = a.w + (size_t)(ch < a.OC ? ch : a.OC - 1) * a.IC;
#pragma unroll
        for (int s = 0; s < KSTEPS; s++)
        {
            const int k0 = 32 * s + 16 * lh;
            const v2i lo = *reinterpret_cast<const v2i*>(row + (k0 < a.IC ? k0 : 0));
            const v2i hi = *reinterpret_cast<const v2i*>(row + (k0 + 8 < a.IC ? k0 + 8 : 0));
            fa[s]        = v4i{ lo.x, lo.y, hi.x, hi.y };
        }
        // what lies past IC or past OC is zeroed once all loads have been issued (a test in the loop above would wait for
        // every load before the next)
#pragma unroll
        for (int s = 0; s < KSTEPS; s++)
        {
            const int k0  = 32 * s + 16 * lh;
            const bool r0 = ch < a.OC && k0 < a.IC, r1 = ch < a.OC && k0 + 8 < a.IC;
            fa[s]         = v4i{ r0 ? fa[s].x : 0, r0 ? fa[s].y : 0, r1 ? fa[s].z : 0, r1 ? fa[s].w : 0 };
        }
    }
    // ---- per-channel constants: lane li (both halves alike) derives those of channel 32 oct + li ------------------------
    uint32_t flags = 0;
    int form       = 0;    // 1: every channel of the tile takes the high-word form of the requantisation
    // With double rounding a value below zero takes a rounding term 2^31 smaller; where the result is clamped at or above
    // output_zp anyway, a negative value ends at the lower limit with either term (the scaled value is at most 0 for a
    // multiplier >= 0), and the high-word form needs no sign test.
    bool sign_free = false;
    {
        const int oc  = oct * 32 + li;
        const bool ok = oc < a.OC;
        const int occ = ok ? oc : oct * 32;
        int32_t b     = a.bias[a.bias_len == 1 ? 0 : (ch < a.OC ? ch : oct * 32)];    // of the row this lane holds weights of
        if (a.rp.enabled)
        {
            const int32_t m_raw   = load_multiplier(a.rp, occ);
            const int32_t s_raw   = load_shift(a.rp, occ);
            const int32_t s_first = __builtin_amdgcn_readfirstlane(s_raw);
            const ChannelScale cs = make_channel_scale(ok ? m_raw : 0, ok ? s_raw : s_first, a.rp.double_round != 0, flags);
            const int s_min       = a.rp.double_round ? 33 : 32;
            form                  = __all(cs.s >= s_min && cs.s <= zp_fold_max_shift(a.rp.out_zp)) ? 1 : 0;
            sign_free             = a.rp.lo >= a.rp.out_zp && __all(cs.m >= 0);
            if (lh == 0)
            {
                tab_ms[li] = v2i{ cs.m, cs.s };
                tab_hw[li] = make_high_word_scale(cs, a.rp.out_zp);
            }
        }
        if constexpr (ZA)
        {
            int sum = 0;
#pragma unroll
            for (int s = 0; s < KSTEPS; s++)
                sum += dot4_ones(fa[s]);
            sum += __builtin_amdgcn_ds_bpermute((lane ^ 32) * 4, sum);
            b = (int32_t)((uint32_t)b - (uint32_t)a.za * (uint32_t)sum);
        }
        if (lh == 0)
            wave_start[wr] = ch < a.OC ? b : 0;
        __builtin_amdgcn_wave_barrier();    // the wave's own LDS accesses complete in order
    }
    v16i start;
#pragma unroll
    for (int gq = 0; gq < 4; gq++)
    {
        const v4i b4 = *reinterpret_cast<const v4i*>(wave_start + 16 * lh + 4 * gq);
        start[4 * gq] = b4[0], start[4 * gq + 1] = b4[1], start[4 * gq + 2] = b4[2], start[4 * gq + 3] = b4[3];
    }
    const int oc_lane = oct * 32 + 16 * lh;                        // first of the lane's 16 channels
    int cnt           = a.OC - oc_lane;                            // how many of them exist: 16, 8 or none (OC is a multiple of 8)
    cnt               = cnt < 0 ? 0 : (cnt > 16 ? 16 : cnt);
    const bool whole  = (a.OC & 15) == 0;                          // int8 rows of whole 16-byte pieces
    const int32_t v_lo = a.rp.lo, v_hi = a.rp.hi;

    // FORM 0: int32 results; 1: the high-word requantisation; 2: the general form
    auto run = [&](auto FORM, auto DOUBLE) {
        constexpr int kForm    = decltype(FORM)::value;
        constexpr bool kDouble = decltype(DOUBLE)::value;
        auto tile = [&](const v4i (&fb)[KSTEPS], int pt) {
            // The constants of the lane's 16 channels are read from the wave's table for every tile (32 lanes read one
            // address: four LDS cycles a read) rather than held in 64 registers, which would halve the waves a SIMD holds;
            // the offset is hidden from the compiler so that it does not move the reads out of the loop over the tiles.
            int first = 16 * lh;
            asm volatile("" : "+v"(first));
            const HighWordScale* hw = tab_hw + first;
            const v2i* ms           = tab_ms + first;
            v16i acc = start;
#pragma unroll
            for (int s = 0; s < KSTEPS; s++)
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[s], fb[s], acc, 0, 0, 0);
            const int p      = pt * 32 + li;
            const bool store = p < a.P && cnt > 0;
            const size_t at  = (size_t)(p < a.P ? p : 0) * a.OC + oc_lane;
            if constexpr (kForm == 0)
            {
                int32_t* o = reinterpret_cast<int32_t*>(a.out) + at;
                if (store)
                {
#pragma unroll
                    for (int gq = 0; gq < 4; gq++)
                        if (4 * gq < cnt)
                            *reinterpret_cast<v4i*>(o + 4 * gq) = v4i{ acc[4 * gq], acc[4 * gq + 1], acc[4 * gq + 2], acc[4 * gq + 3] };
                }
                return;
            }
            int32_t r[16];
#pragma unroll
            for (int e = 0; e < 16; e++)
            {
                if constexpr (kForm == 1)
                    r[e] = clamp_med3(high_word_rescale64<kDouble>(acc[e], hw[e]), v_lo, v_hi);
                else
                {
                    // (elements that are not stored raise nothing)
                    uint32_t f = 0;
                    const v2i c = ms[e];
                    r[e]        = rescale_from_shift(acc[e], c.x, c.y, a.rp.double_round != 0, a.rp.out_zp, v_lo, v_hi, f);
                    flags |= (store && e < cnt) ? f : 0u;
                }
                if ((e & 3) == 3)
                    __builtin_amdgcn_sched_barrier(0);    // four elements' constants at a time: the registers are few
            }
            if (a.out_kind == 1)
            {
                v4i pk;
#pragma unroll
                for (int gq = 0; gq < 4; gq++)
                {
                    const int lo2 = __builtin_amdgcn_perm(r[4 * gq + 1], r[4 * gq], 0x0c0c0400);
                    const int hi2 = __builtin_amdgcn_perm(r[4 * gq + 3], r[4 * gq + 2], 0x04000c0c);
                    pk[gq]        = lo2 | hi2;
                }
                int8_t* o = reinterpret_cast<int8_t*>(a.out) + at;
                if (store)
                {
                    if (whole)
                        *reinterpret_cast<v4i*>(o) = pk;
                    else
                    {
                        *reinterpret_cast<v2i*>(o) = v2i{ pk[0], pk[1] };
                        if (cnt > 8)
                            *reinterpret_cast<v2i*>(o + 8) = v2i{ pk[2], pk[3] };
                    }
                }
            }
            else
            {
                v4i pk, pk2;
#pragma unroll
                for (int gq = 0; gq < 4; gq++)
                {
                    pk[gq]  = (r[2 * gq] & 0xffff) | ((r[2 * gq + 1] & 0xffff) << 16);
                    pk2[gq] = (r[8 + 2 * gq] & 0xffff) | ((r[8 + 2 * gq + 1] & 0xffff) << 16);
                }
                int16_t* o = reinterpret_cast<int16_t*>(a.out) + at;
                if (store)
                {
                    *reinterpret_cast<v4i*>(o) = pk;
                    if (cnt > 8)
                        *reinterpret_cast<v4i*>(o + 8) = pk2;
                }
            }
        };
        // two pixel tiles are in flight while one is multiplied
        for (int pt = q; pt < a.n_pt; pt += 2 * G)
        {
            tile(fb0, pt);
            if (pt + 2 * G < a.n_pt)
                load_pixels(fb0, pt + 2 * G);
            if (pt + G < a.n_pt)
            {
                tile(fb1, pt + G);
                if (pt + 3 * G < a.n_pt)
                    load_pixels(fb1, pt + 3 * G);
            }
        }
    };
    if (!a.rp.enabled)
        run(std::integral_constant<int, 0>{}, std::false_type{});
    else if (form == 1)
        (a.rp.double_round && !sign_free) ? run(std::integral_constant<int, 1>{}, std::true_type{})
                                          : run(std::integral_constant<int, 1>{}, std::false_type{});
    else
        run(std::integral_constant<int, 2>{}, std::false_type{});
    raise_flags(a.flag_word, flags);
}

// The same layers with long channel vectors (up to 2048 input channels): the four waves of a workgroup share one tile of
// 32 output channels x 32 pixels and split K between them, a quarter each, again with both operands straight from global
// memory into registers - all loads of a tile are in flight at once, so a tile costs one trip to memory however deep K is.
// Each wave's accumulators start from its share of bias - input_zp * sum(w) (the bias with the first wave); the four
// partial tiles meet in LDS (16 KB, two buffers, one barrier per tile), and every wave requantises and stores a quarter of
// the tile: 4 consecutive channels per lane.  What a projection layer of a small image offers is few tiles and a long
// reduction (8 x 7 x 7 pixels x 512 channels over K = 2048: 208 tiles of 64 K steps), which this form spreads over 832
// waves where a 128 x 128 GEMM tile would keep 32 CUs busy.
constexpr int kSplitWaves = 4;

template <int KS, bool ZA>
__global__ __launch_bounds__(kSplitWaves * 64, 2) void pointwise_ksplit_i8_kernel(PointwiseArgs a)
{
    // [two buffers x 4 waves x 4 quarters x 64 lanes x 16 bytes][32 x HighWordScale][32 x (m, s)][4 waves x 32 start values][form]
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * 16384 + 32 * 16 + 32 * 8 + kSplitWaves * 128 + 16];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const uint32_t g = blockIdx.x;
    const int q = (int)fdiv(g, a.div_oct), oct = (int)g - q * a.n_oct;
    const int G = a.n_groups;
    HighWordScale* tab_hw = reinterpret_cast<HighWordScale*>(lds + 2 * 16384);
    v2i* tab_ms           = reinterpret_cast<v2i*>(tab_hw + 32);
    int32_t* wave_start   = reinterpret_cast<int32_t*>(tab_ms + 32) + wave * 32;
    int32_t* form_word    = reinterpret_cast<int32_t*>(tab_ms + 32) + kSplitWaves * 32;
    const int ksw = a.ksw;                     // K steps of a wave's share (at most KS)
    const int kbase = wave * ksw * 32;         // first K byte of the share
    const bool by8 = (a.IC & 8) != 0;

    auto load_pixels = [&](v4i (&fb)[KS], int pt) {
        int p = pt * 32 + li;
        p     = p < a.P ? p : a.P - 1;
        const uint8_t* row = a.in + (size_t)p * a.IC;
#pragma unroll
        for (int s = 0; s < KS; s++)
        {
            const int k0 = kbase + 32 * s + 16 * lh;
            if (s < ksw)    // (a test per step, not a loop exit: the register array keeps constant indices)
            {
                if (!by8)
                    fb[s] = *reinterpret_cast<const v4i*>(row + (k0 < a.IC ? k0 : 0));
                else
                {
                    const v2i lo = *reinterpret_cast<const v2i*>(row + (k0 < a.IC ? k0 : 0));
                    const v2i hi = *reinterpret_cast<const v2i*>(row + (k0 + 8 < a.IC ? k0 + 8 : 0));
                    fb[s]        = v4i{ lo.x, lo.y, hi.x, hi.y };
                }
            }
        }
    };
    v4i fb[KS];
    load_pixels(fb, q);

    const int wr = 4 * (li & 4) + ((li >> 1) & 12) + (li & 3);
    const int ch = oct * 32 + wr;
    v4i fa[KS];
    {
        const int8_t* row = a.w + (size_t)(ch < a.OC ? ch : a.OC - 1) * a.IC;
#pragma unroll
        for (int s = 0; s < KS; s++)
        {
            const int k0 = kbase + 32 * s + 16 * lh;
            if (s < ksw)
            {
                // (a load instruction costs the memory pipeline the same for 8 or 16 bytes a lane)
                if (!by8)
                    fa[s] = *reinterpret_cast<const v4i*>(row + (k0 < a.IC ? k0 : 0));
                else
                {
                    const v2i lo = *reinterpret_cast<const v2i*>(row + (k0 < a.IC ? k0 : 0));
                    const v2i hi = *reinterpret_cast<const v2i*>(row + (k0 + 8 < a.IC ? k0 + 8 : 0));
                    fa[s]        = v4i{ lo.x, lo.y, hi.x, hi.y };
                }
            }
        }
        // what lies past IC or past OC is zeroed once all loads have been issued
#pragma unroll
        for (int s = 0; s < KS; s++)
        {
            const int k0  = kbase + 32 * s + 16 * lh;
            const bool r0 = ch < a.OC && k0 < a.IC, r1 = ch < a.OC && k0 + 8 < a.IC;
            if (s < ksw)
                fa[s] = v4i{ r0 ? fa[s].x : 0, r0 ? fa[s].y : 0, r1 ? fa[s].z : 0, r1 ? fa[s].w : 0 };
        }
    }
    uint32_t flags = 0;
    if (wave == 0)
    {
        // the first wave derives the constants of the tile's 32 channels for all four
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
    {
        int32_t b = wave == 0 ? a.bias[a.bias_len == 1 ? 0 : (ch < a.OC ? ch : oct * 32)] : 0;
        if constexpr (ZA)
        {
            int sum = 0;
#pragma unroll
            for (int s = 0; s < KS; s++)
                if (s < ksw)
                    sum += dot4_ones(fa[s]);
            sum += __builtin_amdgcn_ds_bpermute((lane ^ 32) * 4, sum);
            b = (int32_t)((uint32_t)b - (uint32_t)a.za * (uint32_t)sum);
        }
        if (lh == 0)
            wave_start[wr] = ch < a.OC ? b : 0;
        __builtin_amdgcn_wave_barrier();
    }
    v16i start;
#pragma unroll
    for (int gq = 0; gq < 4; gq++)
    {
        const v4i b4 = *reinterpret_cast<const v4i*>(wave_start + 16 * lh + 4 * gq);
        start[4 * gq] = b4[0], start[4 * gq + 1] = b4[1], start[4 * gq + 2] = b4[2], start[4 * gq + 3] = b4[3];
    }
    const int oc_lane = oct * 32 + 16 * lh + 4 * wave;    // first of the 4 channels this lane requantises and stores
    const bool ch_ok  = oc_lane < a.OC;                   // OC is a multiple of 8: the four are in or out together
    const int32_t v_lo = a.rp.lo, v_hi = a.rp.hi;
    int buf = 0;
    for (int pt = q; pt < a.n_pt; pt += G)
    {
        v16i acc = start;
#pragma unroll
        for (int s = 0; s < KS; s++)
            if (s < ksw)
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[s], fb[s], acc, 0, 0, 0);
        if (pt + G < a.n_pt)
            load_pixels(fb, pt + G);    // in flight across the exchange and the requantisation
        // the partial tiles meet in LDS: [wave][quarter][lane] of 16 bytes
        uint8_t* red = lds + buf * 16384;
#pragma unroll
        for (int gq = 0; gq < 4; gq++)
            *reinterpret_cast<v4i*>(red + ((wave * 4 + gq) * 64 + lane) * 16) = v4i{ acc[4 * gq], acc[4 * gq + 1], acc[4 * gq + 2], acc[4 * gq + 3] };
        __syncthreads();    // also publishes the first wave's tables
        v4i sum = *reinterpret_cast<const v4i*>(red + ((0 * 4 + wave) * 64 + lane) * 16);
#pragma unroll
        for (int w2 = 1; w2 < kSplitWaves; w2++)
        {
            const v4i o = *reinterpret_cast<const v4i*>(red + ((w2 * 4 + wave) * 64 + lane) * 16);
            sum.x += o.x, sum.y += o.y, sum.z += o.z, sum.w += o.w;
        }
        buf ^= 1;
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
                r[j]         = rescale_from_shift(sum[j], ms.x, ms.y, a.rp.double_round != 0, a.rp.out_zp, v_lo, v_hi, f);
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

template <int KS>
static bool launch_pointwise_ksplit(hipStream_t st, const PointwiseArgs& a, int grid)
{
    if (a.za != 0)
        hipLaunchKernelGGL((pointwise_ksplit_i8_kernel<KS, true>), dim3(grid), dim3(kSplitWaves * 64), 0, st, a);
    else
        hipLaunchKernelGGL((pointwise_ksplit_i8_kernel<KS, false>), dim3(grid), dim3(kSplitWaves * 64), 0, st, a);
    return true;
}

template <int KSTEPS>
static bool launch_pointwise(hipStream_t st, const PointwiseArgs& a, int grid)
{
    if (a.za != 0)
        hipLaunchKernelGGL((pointwise_i8_kernel<KSTEPS, true>), dim3(grid), dim3(kPointwiseWaves * 64), 0, st, a);
    else
        hipLaunchKernelGGL((pointwise_i8_kernel<KSTEPS, false>), dim3(grid), dim3(kPointwiseWaves * 64), 0, st, a);
    return true;
}

// nullptr when the layer is not one this kernel takes.
const char* launch_conv2d_pointwise(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                                    const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                                    void* out, uint32_t* flag_word)
{
    if (in_dtype != TMI_INT8 || g.KH != 1 || g.KW != 1 || g.stride_y != 1 || g.stride_x != 1 || g.pad_top != 0 ||
        g.pad_left != 0 || g.OH != g.IH || g.OW != g.IW || w_zp != 0 || !flag_word)
        return nullptr;
    if ((g.IC & 7) || g.IC < 16 || g.IC > 2048 || (g.OC & 7) || g.OC < 8 || g.OC > 4096)
        return nullptr;
    if (rp.enabled ? (!rp.fast || (out_dtype != TMI_INT8 && out_dtype != TMI_INT16)) : out_dtype != TMI_INT32)
        return nullptr;
    if ((((uintptr_t)in | (uintptr_t)w | (uintptr_t)out) & 15) || ((uintptr_t)bias & 3))
        return nullptr;
    const int64_t P = (int64_t)g.N * g.OH * g.OW;
    if (P < 1 || P * g.IC >= (int64_t(1) << 31) || P * g.OC >= (int64_t(1) << 31))
        return nullptr;

    PointwiseArgs a{};
    a.in = (const uint8_t*)in, a.w = (const int8_t*)w, a.bias = (const int32_t*)bias, a.out = out;
    a.flag_word = flag_word, a.rp = rp;
    a.P = (int32_t)P, a.IC = g.IC, a.OC = g.OC, a.za = in_zp, a.bias_len = g.bias_len;
    a.out_kind = !rp.enabled ? 0 : (out_dtype == TMI_INT8 ? 1 : 2);
    a.n_oct    = (g.OC + 31) / 32;
    a.n_pt     = (int32_t)((P + 31) / 32);
    a.div_oct  = make_fastdiv((uint32_t)a.n_oct);
    if (g.IC > 160)
    {
        // K split over the four waves of a workgroup.  A workgroup walks several pixel tiles with its weight fragments in
        // registers once the layer has more than 640 tiles: about two workgroups per CU is where the weight loads saved and
        // the tiles a workgroup works through one after the other balance (us for 1 / 2 / 3 / 4 tiles a workgroup, fused
        // RESCALE: [8,28,28,512]->128 6.8 / 6.5 / 7.0 / -, [8,14,14,1024]->512 10.6 / 8.6 / 9.2 / 8.8, [8,28,28,512]->256
        // 11.1 / 9.0 / 8.8 / 9.2, [8,56,56,256]->64 8.7 / - / 7.0 / 7.5, [8,14,14,256]->1024 8.3 / - / 6.7 / 7.4).
        const int ksteps = (g.IC + 31) / 32;
        a.ksw            = (ksteps + kSplitWaves - 1) / kSplitWaves;
        const int max_groups = 640 / a.n_oct > 0 ? 640 / a.n_oct : 1;
        const int per_group = (a.n_pt + max_groups - 1) / max_groups;    // pixel tiles a workgroup walks: the same for all
        a.n_groups       = (a.n_pt + per_group - 1) / per_group;
        const int grid   = a.n_groups * a.n_oct;
        if (!fastdiv_exact_up_to((uint64_t)grid, (uint32_t)a.n_oct))
            return nullptr;
        if (a.ksw <= 2)
            launch_pointwise_ksplit<2>(st, a, grid);
        else if (a.ksw <= 4)
            launch_pointwise_ksplit<4>(st, a, grid);
        else if (a.ksw <= 8)
            launch_pointwise_ksplit<8>(st, a, grid);
        else
            launch_pointwise_ksplit<16>(st, a, grid);
        last_launch_shape[0] = grid, last_launch_shape[1] = kSplitWaves * 64, last_launch_shape[2] = 34064;
        return rp.enabled ? "conv2d_pointwise_ksplit_i8_rescale" : "conv2d_pointwise_ksplit_i8";
    }
    // as many groups as there are pixel tiles, up to the waves the 256 CUs hold at once (12 each up to 64 input channels,
    // 8 beyond: the fragments of two pixel tiles in flight take the registers)
    const int per_cu     = g.IC <= 64 ? 12 : 8;
    const int max_groups = 256 * per_cu / a.n_oct > 0 ? 256 * per_cu / a.n_oct : 1;
    a.n_groups = a.n_pt < max_groups ? a.n_pt : max_groups;
    const int64_t waves = (int64_t)a.n_groups * a.n_oct;
    if (!fastdiv_exact_up_to((uint64_t)waves + kPointwiseWaves, (uint32_t)a.n_oct))
        return nullptr;
    const int grid   = (int)((waves + kPointwiseWaves - 1) / kPointwiseWaves);
    const int ksteps = (g.IC + 31) / 32;
    bool ok          = false;
    switch (ksteps)
    {
        case 1: ok = launch_pointwise<1>(st, a, grid); break;
        case 2: ok = launch_pointwise<2>(st, a, grid); break;
        case 3: ok = launch_pointwise<3>(st, a, grid); break;
        case 4: ok = launch_pointwise<4>(st, a, grid); break;
        case 5: ok = launch_pointwise<5>(st, a, grid); break;
        default: break;
    }
    if (!ok)
        return nullptr;
    last_launch_shape[0] = grid, last_launch_shape[1] = kPointwiseWaves * 64, last_launch_shape[2] = kPointwiseWaves * kPointwiseWaveLds;
    return rp.enabled ? "conv2d_pointwise_i8_rescale" : "conv2d_pointwise_i8";
}

// ---- the first layer of a network: 3 x 3 ... 7 x 7 taps over at most 4 channels -------------------------------------------
//
// With at most 4 input channels the whole row of taps of a 7 x 7 window is at most 28 contiguous bytes of an image whose
// pixels are 4 bytes apart: a K step of the matrix instruction (32 bytes) per tap row, read where it lies.  What stands in
// the way is the padding (a window at the border reads input_zp for the pixels outside), the pixel pitch (3 channels: odd
// addresses) and the weight layout; a first launch writes the image with its padding materialised and a pixel every 4
// bytes (rows of (IW + pad_left + pad_right) * 4 bytes, input_zp outside; where 4 * KW exceeds 32, a pixel every IC bytes)
// and the weights as 32 bytes per (channel, tap row) in the same arrangement, zeros where no tap and no channel is, into
// the caller's scratch buffer; the pointwise kernel above then runs with a wave per tile of 32 output channels, K steps =
// tap rows (STEM).  dilation_x must be 1.
struct StemPrepArgs
{
    const uint8_t* in;
    const int8_t* w;
    uint8_t* padded;
    int8_t* wrep;
    int32_t N, IH, IW, IC, OC, KH, KW;
    int32_t rows, row_bytes, pad_top, pad_left, za;
    int32_t image_words, weight_words;    // 4-byte words of the padded images / of the weight rows
    int32_t PP;                           // bytes from one pixel to the next in the copy: 4, or IC where KW * 4 exceeds a K step
    FastDiv div_rw, div_rows, div_pp;
};

__global__ __launch_bounds__(256) void stem_prepass_kernel(StemPrepArgs a)
{
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < (uint32_t)a.image_words)
    {
        const uint32_t rw = (uint32_t)a.row_bytes / 4;
        const uint32_t r  = fdiv(i, a.div_rw);    // n * rows + y
        const uint32_t b0 = (i - r * rw) * 4;     // first of the word's four bytes in the row
        const uint32_t n  = fdiv(r, a.div_rows);
        const int iy      = (int)(r - n * a.rows) - a.pad_top;
        uint32_t word     = 0;
#pragma unroll
        for (int k = 0; k < 4; k++)
        {
            const uint32_t x = fdiv(b0 + k, a.div_pp);
            const int c      = (int)(b0 + k - x * a.PP);
            const int ix     = (int)x - a.pad_left;
            int v            = a.za;    // (also in the bytes between IC and the pixel pitch, which meet zero weights)
            if (n < (uint32_t)a.N && (unsigned)iy < (unsigned)a.IH && (unsigned)ix < (unsigned)a.IW && c < a.IC)    // (n = N: the spare bytes behind the last image)
                v = a.in[((size_t)(n * a.IH + iy) * a.IW + ix) * a.IC + c];
            word |= (uint32_t)(v & 0xff) << (8 * k);
        }
        reinterpret_cast<uint32_t*>(a.padded)[i] = word;
        return;
    }
    const uint32_t j = i - a.image_words;
    if (j < (uint32_t)a.weight_words)
    {
        const uint32_t row = j >> 3;    // (channel, tap row): 32 bytes, 8 words
        const uint32_t b0  = (j & 7) * 4;
        const int len      = a.KW * a.IC;
        uint32_t word      = 0;
#pragma unroll
        for (int k = 0; k < 4; k++)
        {
            const uint32_t kx = fdiv(b0 + k, a.div_pp);    // byte b of the row is channel b % PP under tap b / PP
            const int c       = (int)(b0 + k - kx * a.PP);
            if ((int)kx < a.KW && c < a.IC)
                word |= (uint32_t)(a.w[(size_t)row * len + kx * a.IC + c] & 0xff) << (8 * k);
        }
        reinterpret_cast<uint32_t*>(a.wrep)[j] = word;
    }
}

template <int KSTEPS>
static void launch_stem(hipStream_t st, const PointwiseArgs& a, int grid)
{
    if (a.za != 0)
        hipLaunchKernelGGL((pointwise_i8_kernel<KSTEPS, true, true>), dim3(grid), dim3(kPointwiseWaves * 64), 0, st, a);
    else
        hipLaunchKernelGGL((pointwise_i8_kernel<KSTEPS, false, true>), dim3(grid), dim3(kPointwiseWaves * 64), 0, st, a);
}

// Bytes from one pixel to the next in the padded copy.  Four where a row of taps then still fits a K step: every window
// starts on a 4-byte boundary, and a 16-byte load from such an address costs the memory pipeline a third less than one from
// an odd address (ResNet-50's first layer at batch 8: 14.8 -> 10.9 us).
static int stem_pixel_pitch(const ConvGeom& g)
{
    return g.KW * 4 <= 32 ? 4 : g.IC;
}

// Bytes of scratch the first-layer form needs for this layer, or 0 when it does not take it.
size_t conv2d_stem_scratch_bytes(int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, int32_t w_zp, const RescaleParams& rp)
{
    if (in_dtype != TMI_INT8 || w_zp != 0 || g.IC < 1 || g.IC > 4 || g.KW * g.IC > 32 || g.dil_x != 1)
        return 0;
    if ((g.KH != 3 && g.KH != 5 && g.KH != 7) || g.KW < 2 || (g.OC & 7) || g.OC < 8 || g.OC > 4096)
        return 0;
    if (rp.enabled ? (!rp.fast || (out_dtype != TMI_INT8 && out_dtype != TMI_INT16)) : out_dtype != TMI_INT32)
        return 0;
    // rows and columns the windows reach: what the declared output size needs, not more than the padded image
    const int64_t rows = (int64_t)(g.OH - 1) * g.stride_y + (int64_t)(g.KH - 1) * g.dil_y + 1;
    const int64_t cols = (int64_t)(g.OW - 1) * g.stride_x + g.KW;
    const int64_t row_bytes = (cols * stem_pixel_pitch(g) + 3) / 4 * 4;
    const int64_t image = (int64_t)g.N * rows * row_bytes;
    if (image + 64 >= (int64_t(1) << 31) || (int64_t)g.N * g.OH * g.OW * g.OC >= (int64_t(1) << 31))
        return 0;
    return (size_t)((image + 64 + 255) / 256 * 256 + (int64_t)g.OC * g.KH * 32);
}

// nullptr when the layer is not one this form takes; `scratch` holds conv2d_stem_scratch_bytes() bytes, 256-byte aligned.
const char* launch_conv2d_stem(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                               const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp, void* out,
                               void* scratch, uint32_t* flag_word)
{
    if (!conv2d_stem_scratch_bytes(in_dtype, out_dtype, g, w_zp, rp) || !scratch || !flag_word)
        return nullptr;
    if ((((uintptr_t)out | (uintptr_t)scratch) & 15) || ((uintptr_t)bias & 3))
        return nullptr;
    const int rows = (g.OH - 1) * g.stride_y + (g.KH - 1) * g.dil_y + 1;
    const int cols = (g.OW - 1) * g.stride_x + g.KW;
    const int pp   = stem_pixel_pitch(g);
    const int row_bytes = (cols * pp + 3) / 4 * 4;
    const int64_t image = (int64_t)g.N * rows * row_bytes;
    StemPrepArgs pa{};
    pa.in = (const uint8_t*)in, pa.w = (const int8_t*)w;
    pa.padded = (uint8_t*)scratch, pa.wrep = (int8_t*)scratch + (image + 64 + 255) / 256 * 256;
    pa.N = g.N, pa.IH = g.IH, pa.IW = g.IW, pa.IC = g.IC, pa.OC = g.OC, pa.KH = g.KH, pa.KW = g.KW;
    pa.rows = rows, pa.row_bytes = row_bytes, pa.pad_top = g.pad_top, pa.pad_left = g.pad_left, pa.za = in_zp;
    pa.image_words = (int32_t)((image + 64) / 4), pa.weight_words = g.OC * g.KH * 8;
    pa.div_rw = make_fastdiv((uint32_t)(row_bytes / 4)), pa.div_rows = make_fastdiv((uint32_t)rows);
    pa.PP = pp, pa.div_pp = make_fastdiv((uint32_t)pp);
    // (the 64 bytes behind the last image belong to no row: they are written as a row past the last image would be)
    if (!fastdiv_exact_up_to((uint64_t)pa.image_words, (uint32_t)(row_bytes / 4)) ||
        !fastdiv_exact_up_to((uint64_t)pa.image_words / (row_bytes / 4) + 1, (uint32_t)rows) ||
        !fastdiv_exact_up_to((uint64_t)row_bytes + 36, (uint32_t)pp))
        return nullptr;
    const int64_t P = (int64_t)g.N * g.OH * g.OW;
    PointwiseArgs a{};
    a.in = pa.padded, a.w = pa.wrep, a.bias = (const int32_t*)bias, a.out = out, a.flag_word = flag_word, a.rp = rp;
    a.P = (int32_t)P, a.IC = g.KH * 32, a.OC = g.OC, a.za = in_zp, a.bias_len = g.bias_len;
    a.out_kind = !rp.enabled ? 0 : (out_dtype == TMI_INT8 ? 1 : 2);
    a.n_oct = (g.OC + 31) / 32, a.n_pt = (int32_t)((P + 31) / 32);
    a.div_oct = make_fastdiv((uint32_t)a.n_oct);
    a.row_bytes = row_bytes, a.rows = rows, a.OH = g.OH, a.OW = g.OW;
    a.step_y = g.stride_y * row_bytes, a.step_x = g.stride_x * pp, a.step_k = g.dil_y * row_bytes;
    a.div_ow = make_fastdiv((uint32_t)g.OW), a.div_oh = make_fastdiv((uint32_t)g.OH);
    const int max_groups = 256 * 8 / a.n_oct > 0 ? 256 * 8 / a.n_oct : 1;
    a.n_groups = a.n_pt < max_groups ? a.n_pt : max_groups;
    const int64_t waves = (int64_t)a.n_groups * a.n_oct;
    if (!fastdiv_exact_up_to((uint64_t)waves + kPointwiseWaves, (uint32_t)a.n_oct) || !fastdiv_exact_up_to((uint64_t)P, (uint32_t)g.OW) ||
        !fastdiv_exact_up_to((uint64_t)P / g.OW + 1, (uint32_t)g.OH))
        return nullptr;
    const int prep_grid = (pa.image_words + pa.weight_words + 255) / 256;
    hipLaunchKernelGGL(stem_prepass_kernel, dim3(prep_grid), dim3(256), 0, st, pa);
    const int grid = (int)((waves + kPointwiseWaves - 1) / kPointwiseWaves);
    if (g.KH == 3)
        launch_stem<3>(st, a, grid);
    else if (g.KH == 5)
        launch_stem<5>(st, a, grid);
    else
        launch_stem<7>(st, a, grid);
    last_launch_shape[0] = grid, last_launch_shape[1] = kPointwiseWaves * 64, last_launch_shape[2] = kPointwiseWaves * kPointwiseWaveLds;
    return rp.enabled ? "conv2d_stem_i8_rescale" : "conv2d_stem_i8";
}

}    // namespace tmi
