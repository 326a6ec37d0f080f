// Device-side helpers shared by every kernel: the RESCALE arithmetic and the epilogue that turns an
// int32 accumulator into the stored output element.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tosa_mi355.h"

namespace tmi
{

// n / d for n*d < 2^32 as one multiply-high (magic = floor(2^32/d) + 1; d == 1 is special-cased).
struct FastDiv
{
    uint32_t magic, d;
};

inline FastDiv make_fastdiv(uint32_t d)
{
    FastDiv f;
    f.d     = d;
    f.magic = d <= 1 ? 0u : (uint32_t)((uint64_t(1) << 32) / d) + 1u;
    return f;
}

__device__ __forceinline__ uint32_t fdiv(uint32_t n, FastDiv f)
{
    return f.d <= 1 ? n : __umulhi(n, f.magic);
}

// a * b + c on the 24-bit multiplier with three 32-bit operands (a and b below 2^24).  Left to the compiler, a * b + c
// becomes a 64-bit multiply-add whose addend's upper half is whatever register is at hand, and where that register is the
// destination of a load in flight, the instruction - and every load the wave has yet to issue - waits for that load.
__device__ __forceinline__ uint32_t mad_u24(uint32_t a, uint32_t b, uint32_t c)
{
    uint32_t r;
    asm("v_mad_u32_u24 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// The same quotient on the host (the multiply-high written out).
inline uint32_t fdiv_host(uint32_t n, FastDiv f)
{
    return f.d <= 1 ? n : (uint32_t)(((uint64_t)n * f.magic) >> 32);
}

// fdiv(n, make_fastdiv(d)) is exact for every n <= max_n.
inline bool fastdiv_exact_up_to(uint64_t max_n, uint32_t d)
{
    return d <= 1 || max_n * (uint64_t)d < (uint64_t(1) << 32);
}

// The tiled kernels turn a block index into (channel block, tile column, tile row, image) with three FastDiv
// divisions: block / n_ocb, then / tiles_x, then / tiles_y.  True when all three are exact for every block of the
// grid; a launcher whose layer fails this leaves the layer to a kernel with another decomposition.
inline bool tile_decode_is_exact(int64_t grid, uint32_t n_ocb, uint32_t tiles_x, uint32_t tiles_y)
{
    if (grid <= 0 || grid >= (int64_t(1) << 31) || !n_ocb || !tiles_x || !tiles_y)
        return false;
    const uint64_t max_bid = (uint64_t)grid - 1, max_tile = max_bid / n_ocb, max_trow = max_tile / tiles_x;
    return fastdiv_exact_up_to(max_bid, n_ocb) && fastdiv_exact_up_to(max_tile, tiles_x) &&
           fastdiv_exact_up_to(max_trow, tiles_y);
}

// Everything a kernel needs to apply RESCALE (and an optional CLAMP) to one value.  Filled on the host
// after validation, passed by value.
struct RescaleParams
{
    const void* multiplier;    // int32[n] when scale32 else int16[n]
    const int8_t* shift;       // int8[n]
    int32_t in_zp;             // sign/zero-extended input zero point
    int32_t out_zp;            // sign/zero-extended output zero point
    int32_t qmin, qmax;        // clip range of the output type
    int32_t clamp_min, clamp_max;
    // inexact_round: 0 SINGLE / DOUBLE rounding; 1 INEXACT_ROUND in FP32; 2 in FP64 (precise mode); 3 / 4 the same moved to the
    // lower / upper edge of the compliance error bound (normal / bounds pass)
    uint8_t scale32, double_round, inexact_round, per_channel;
    uint8_t in_bits, in_unsigned, has_clamp, enabled;
    // Set by the host when the input is a signed INT32 value with zero input_zp, scale32 is on and the
    // rounding is SINGLE or DOUBLE: the kernels may then use fast_rescale() with the merged range [lo, hi]
    // (output clip followed by CLAMP) instead of the general rescale_value().
    uint8_t fast;
    int32_t lo, hi;
};

// Per-channel constants of the fast path, derived once per channel and reused for every pixel.
struct ChannelScale
{
    int32_t m, s;
    int64_t rnd_pos, rnd_neg;    // rounding constant for value >= 0 / value < 0 (double round folded in)
    uint32_t lim, lim2;          // value v is legal iff (uint32)(v + lim) <= lim2
};

// value_extend64_impl of the reference (type_conversion.cpp:183-221); INT48 is stored as int64 and never
// unsigned here (the host rejects it, :132).
__device__ __forceinline__ int64_t value_extend(int64_t v, int bits, bool is_unsigned)
{
    if (bits == 48)
        return (v & 0x800000000000ll) ? (int64_t)((uint64_t)v | 0xFFFF000000000000ull) : v;
    if (bits == 8)
        return is_unsigned ? (int64_t)(uint8_t)v : (int64_t)(int8_t)v;
    if (bits == 16)
        return is_unsigned ? (int64_t)(uint16_t)v : (int64_t)(int16_t)v;
    return is_unsigned ? (int64_t)(uint32_t)v : (int64_t)(int32_t)v;
}

// QuantUtil::apply_scale_32 (quant_util.h:45-84).  Violated preconditions set bits in `flags`.
__device__ __forceinline__ int32_t apply_scale_32(int32_t value, int32_t multiplier, int32_t shift,
                                                  bool double_round, uint32_t& flags)
{
    if (multiplier < 0)
        flags |= TMI_FLAG_SCALE_MULTIPLIER;
    if (shift < 2 || shift > 62)
    {
        flags |= TMI_FLAG_SCALE_SHIFT;
        return 0;
    }
    if (shift <= 31)
    {
        const int32_t high = 1 << (shift - 1);
        if (value < -high || value >= high)
            flags |= TMI_FLAG_SCALE_VALUE;
    }
    int64_t round = int64_t(1) << (shift - 1);
    if (double_round && shift > 31)
        round += (value >= 0) ? (int64_t(1) << 30) : -(int64_t(1) << 30);
    int64_t result = (int64_t)value * (int64_t)multiplier + round;
    result >>= shift;
    if (result < -(int64_t(1) << 31) || result >= (int64_t(1) << 31))
        flags |= TMI_FLAG_SCALE_RESULT;
    return (int32_t)result;
}

// QuantUtil::apply_scale_16 (quant_util.h:86-108).
__device__ __forceinline__ int32_t apply_scale_16(int64_t value, int32_t multiplier, int32_t shift, uint32_t& flags)
{
    if (multiplier < 0)
        flags |= TMI_FLAG_SCALE_MULTIPLIER;
    if (shift < 2 || shift > 62)
    {
        flags |= TMI_FLAG_SCALE_SHIFT;
        return 0;
    }
    int64_t result = (int64_t)((uint64_t)value * (uint64_t)(int64_t)multiplier + (uint64_t(1) << (shift - 1)));
    result >>= shift;
    if (result < -(int64_t(1) << 31) || result >= (int64_t(1) << 31))
        flags |= TMI_FLAG_SCALE_RESULT;
    return (int32_t)result;
}

// The rescale_func lambda of OpRescale::eval (type_conversion.cpp:305-370) followed by the optional
// CLAMP (arith_util.h:389-413).  `stored` is the raw stored input value, `m`/`s` the channel's constants.
//
// PRECISE chooses which INEXACT_ROUND forms the instantiation holds: false, the integer roundings and FP32 (inexact_round
// 0 and 1); true, only the FP64 forms of precise mode (2, 3, 4).  A kernel is built for one or the other and the host
// picks it by RescaleParams::inexact_round, so that the integer kernels carry no FP64 code.
template <bool PRECISE = false>
__device__ __forceinline__ int32_t rescale_value(const RescaleParams& p, int64_t stored, int32_t m, int32_t s,
                                                 uint32_t& flags)
{
    const int64_t v = value_extend(stored, p.in_bits, p.in_unsigned) - (int64_t)p.in_zp;
    int32_t scaled;
    if constexpr (PRECISE)
    {
        // INEXACT_ROUND in precise mode (type_conversion.cpp:326-346): the scaled value in FP64, truncated; in compliance
        // mode it is first moved to the edge of the error bound that the specification grants an FP32 implementation,
        // the lower edge in the normal pass (3) and the upper edge in the bounds pass (4).
        double x = (double)v * (double)m * ldexp(1.0, -s);
        if (p.inexact_round >= 3)
        {
            const double with_zp = x + (double)p.out_zp;
            const double bound   = 0.5 + (3.0 * fabs(x) + fabs(with_zp)) * ldexp(1.0, -24);
            x                    = p.inexact_round == 4 ? floor(x + bound) : ceil(x - bound);
        }
        // outside int32: the same convention as for the FP32 form below
        scaled = (x > -2147483649.0 && x < 2147483648.0) ? (int32_t)x : INT32_MIN;
    }
    else if (p.inexact_round)
    {
        const float t = (float)v * (float)m;
        const float u = rintf(t * ldexpf(1.0f, -s));    // 2^-s is exact
        // Outside the int32 range the reference's cast (type_conversion.cpp:323) is undefined; an x86-64 build of it
        // returns INT32_MIN for every such value (the conversion instruction's "integer indefinite"), and so does
        // this one, rather than the saturated value the device's own conversion would give.
        scaled = (u >= -2147483648.0f && u < 2147483648.0f) ? (int32_t)u : INT32_MIN;
    }
    else if (p.scale32)
        scaled = apply_scale_32((int32_t)v, m, s, p.double_round, flags);
    else
        scaled = apply_scale_16(v, m, s, flags);
    const int64_t res = (int64_t)scaled + (int64_t)p.out_zp;
    if (res > (int64_t)INT32_MAX || res < (int64_t)INT32_MIN)
        flags |= TMI_FLAG_ZP_RESULT;
    int32_t r = (int32_t)res;
    r         = r < p.qmin ? p.qmin : r;
    r         = r > p.qmax ? p.qmax : r;
    if (p.has_clamp)
    {
        r = r >= p.clamp_min ? r : p.clamp_min;
        r = r < p.clamp_max ? r : p.clamp_max;
    }
    return r;
}

__device__ __forceinline__ ChannelScale make_channel_scale(int32_t m, int32_t s, bool double_round, uint32_t& flags)
{
    if (m < 0)
        flags |= TMI_FLAG_SCALE_MULTIPLIER;
    if (s < 2 || s > 62)
    {
        flags |= TMI_FLAG_SCALE_SHIFT;
        s = 2;
    }
    ChannelScale c;
    c.m               = m;
    c.s               = s;
    const int64_t rnd = int64_t(1) << (s - 1);
    const int64_t adj = (double_round && s > 31) ? (int64_t(1) << 30) : 0;
    c.rnd_pos         = rnd + adj;
    c.rnd_neg         = rnd - adj;
    c.lim             = s <= 31 ? (1u << (s - 1)) : 0x80000000u;
    c.lim2            = 2u * c.lim - 1u;    // 0xffffffff when every int32 value is legal
    return c;
}

// (p + rnd) >> s + zp == (p + rnd + zp * 2^s) >> s lets the output zero point ride in the 64-bit rounding term,
// but only while the sum stays inside int64: |value * multiplier| < 2^62 and rnd <= 2^61 + 2^30 leave room for
// |zp| * 2^s <= 2^60.  Returns the largest shift for which the fold is safe.
__device__ __forceinline__ int zp_fold_max_shift(int32_t out_zp)
{
    const uint32_t mag = (uint32_t)(out_zp < 0 ? -(int64_t)out_zp : (int64_t)out_zp);
    return mag == 0 ? 62 : 60 - (32 - __clz((int)mag));
}

// High-word form of apply_scale_32 + output_zp for a channel whose shift s is at least 32 (33 with double rounding)
// and at most zp_fold_max_shift(): (v * m + rnd(v)) >> s == ((v * m + rnd(v)) >> 32) >> (s - 32), and the value-range
// test of apply_scale_32 cannot fire.  rnd(v) = R for v >= 0 and R - 2^31 for v < 0 when double rounding, with
// R = 2^(s-1) + 2^30 + output_zp * 2^s: the low word of R is 2^30, so the low word of rnd(v) is R.lo | (sign << 31)
// and its high word R.hi + (v >> 31).  Without double rounding rnd(v) = R = 2^(s-1) + output_zp * 2^s.
struct alignas(16) HighWordScale
{
    uint32_t lo;    // low word of R
    int32_t hi;     // R >> 32: next to the low word, the two are the 64-bit addend of the multiply-add
    int32_t m;      // multiplier
    int32_t sh;     // s - 32
};

__device__ __forceinline__ HighWordScale make_high_word_scale(const ChannelScale& c, int32_t out_zp)
{
    const int64_t r = c.rnd_pos + ((int64_t)out_zp << c.s);
    return HighWordScale{ (uint32_t)r, (int32_t)(r >> 32), c.m, c.s - 32 };
}

template <bool DOUBLE_ROUND>
__device__ __forceinline__ int32_t high_word_rescale(int32_t v, int32_t m, int32_t hi, uint32_t lo, int32_t sh)
{
    if (DOUBLE_ROUND)
    {
        const int32_t t = v >> 31;
        lo |= (uint32_t)t << 31;
        hi += t;
    }
    const int64_t pr = (int64_t)v * (int64_t)m + (int64_t)(((uint64_t)(uint32_t)hi << 32) | lo);
    return (int32_t)(pr >> 32) >> sh;
}

// The same with the rounding term as one 64-bit value R (a scalar, or the lo / hi pair of a HighWordScale): v * m + R is
// one multiply-add, and with double rounding a second one takes the 2^31 off again for a negative value,
// (v >>> 31) * -2^31 + (v * m + R), instead of the three instructions that patch the sign into the two words of R.
// (64-bit multiply-adds issue at the full rate on gfx950.)
template <bool DOUBLE_ROUND>
__device__ __forceinline__ int32_t high_word_rescale64(int32_t v, int32_t m, int64_t rnd, int32_t sh)
{
    int64_t pr = (int64_t)v * (int64_t)m + rnd;
    if (DOUBLE_ROUND)
    {
        const int32_t neg = (int32_t)((uint32_t)v >> 31);
        uint64_t carry;
        asm("v_mad_i64_i32 %0, %1, %2, %3, %4" : "=v"(pr), "=s"(carry) : "v"(neg), "v"(INT32_MIN), "v"(pr));
    }
    return (int32_t)(pr >> 32) >> sh;
}

template <bool DOUBLE_ROUND>
__device__ __forceinline__ int32_t high_word_rescale64(int32_t v, const HighWordScale& c)
{
    return high_word_rescale64<DOUBLE_ROUND>(v, c.m, (int64_t)(((uint64_t)(uint32_t)c.hi << 32) | c.lo), c.sh);
}

// The same for a rounding term that does not depend on the value's sign (single rounding, or double rounding where a
// negative value is clamped away anyway): the whole 64-bit term is the addend of the multiply-add, one instruction.
__device__ __forceinline__ int32_t high_word_rescale_const(int32_t v, int32_t m, int64_t rnd, int32_t sh)
{
    int64_t pr;
    asm("v_mad_i64_i32 %0, vcc, %1, %2, %3" : "=v"(pr) : "v"(v), "v"(m), "s"(rnd) : "vcc");
    return (int32_t)(pr >> 32) >> sh;
}

// apply_scale_32 + output_zp + clip (+ CLAMP) for a signed int32 value with zero input_zp.  With a legal
// value |v| < 2^(s-1) and m < 2^31 the scaled result is below 2^30 in magnitude, so neither of the
// reference's int32 range checks (quant_util.h:78-82, type_conversion.cpp:352-360) can fire here.
__device__ __forceinline__ int32_t fast_rescale(int32_t v, const ChannelScale& c, int32_t out_zp, int32_t lo,
                                                int32_t hi, uint32_t& flags)
{
    if ((uint32_t)v + c.lim > c.lim2)
        flags |= TMI_FLAG_SCALE_VALUE;
    const int64_t p = (int64_t)v * (int64_t)c.m + (v >= 0 ? c.rnd_pos : c.rnd_neg);
    int32_t r       = (int32_t)(p >> c.s) + out_zp;
    r               = r < lo ? lo : r;
    r               = r > hi ? hi : r;
    return r;
}

__device__ __forceinline__ int32_t load_multiplier(const RescaleParams& p, int c)
{
    const int i = p.per_channel ? c : 0;
    return p.scale32 ? reinterpret_cast<const int32_t*>(p.multiplier)[i]
                     : (int32_t) reinterpret_cast<const int16_t*>(p.multiplier)[i];
}

__device__ __forceinline__ int32_t load_shift(const RescaleParams& p, int c)
{
    return (int32_t)p.shift[p.per_channel ? c : 0];
}

// Latches REQUIRE conditions into the context's flag word (one vector atomic per lane that saw one).
__device__ __forceinline__ void raise_flags(uint32_t* flag_word, uint32_t flags)
{
    if (flags)
        atomicOr(flag_word, flags);
}

}    // namespace tmi
