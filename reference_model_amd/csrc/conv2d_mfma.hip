// CONV2D as an implicit GEMM on the matrix cores (MFMA), with the bias / zero-point / RESCALE / CLAMP
// epilogue fused so that the int32 accumulators never reach HBM.
//
// One workgroup (4 waves) computes a TH x TW tile of output pixels of one image for a block of OCB =
// 16*OCT output channels.  Per block of 64 bytes of input channels it stages in LDS
//   - the input patch that the tile needs (PH x PW pixels, out-of-image pixels filled with input_zp, so the
//     zero-point identity below holds with the full K), each pixel a row of CH 16-byte chunks, and
//   - the weight slab [tap][channel row][CH chunks],
// both with a row stride chosen so that the 16 lanes of a ds_read_b128 phase hit distinct banks.
// Every input byte is read from HBM/L2 once per workgroup (plus the halo) and reused KH*KW*OCB times
// from LDS.
//
// MFMA operand roles: the weights are the "A" operand (rows of D = output channels), the pixels the "B"
// operand (columns of D = pixels).  With the 16x16 accumulator layout (lane l, register r) = D[4*(l/16)+r]
// [l%16], assigning output channel 4*OCT*(i/4) + 4*t + i%4 to row i of channel tile t makes every lane own
// 4*OCT consecutive channels of one pixel, i.e. one 16-byte store of int8 results for OCT = 4.
//
// A K-step feeds each lane 16 bytes of one (tap, channel chunk) pair; lane group g = l/16 takes pair
// 4*step+g.  Integer dot products are order independent, so which pair lands in which lane group does not
// matter as long as both operands agree.
//
// Zero points: sum((a-za)(w-zw)) = sum(a*w) - zw*sum(a) - za*sum(w) + K*za*zw.  sum(w) per channel and
// sum(a) per pixel are accumulated from the very fragments fed to the MFMA with v_dot4 against 0x01010101.
#include "tmi_kernels.h"

namespace tmi
{

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8b __attribute__((ext_vector_type(8)));

struct PatchArgs
{
    ConvGeom g;
    const uint8_t* in;
    const uint8_t* w;
    const void* bias;
    void* out;
    uint32_t* flag_word;
    RescaleParams rp;
    int32_t za, zw;
    int32_t TH, TW, tiles_y, tiles_x, oc_blocks;
    int32_t PH, PW;
    int32_t CH;               // 16-byte chunks per pixel row in LDS (1, 2 or 4)
    int32_t pstride, wstride; // LDS row strides in bytes
    int32_t n_icb;            // blocks of CH*16 bytes along the input channels
    int32_t ksteps;           // MFMA K-steps per channel block = ceil(taps*CH/4)
    int32_t n_tiles;          // N * tiles_y * tiles_x
    int32_t out_dtype;
    int32_t xcd_remap;
};

template <typename T>
struct Mma;

template <>
struct Mma<int8_t>
{
    using acc_t                  = v4i;
    static constexpr bool is_int = true;
    __device__ static v4i mma(v4i a, v4i b, v4i c)
    {
        return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
    }
};
template <>
struct Mma<_Float16>
{
    using acc_t                  = v4f;
    static constexpr bool is_int = false;
    __device__ static v4f mma(v4i a, v4i b, v4f c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0,
                                                      0, 0);
    }
};
template <>
struct Mma<bf16_t>
{
    using acc_t                  = v4f;
    static constexpr bool is_int = false;
    __device__ static v4f mma(v4i a, v4i b, v4f c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8b, a), __builtin_bit_cast(v8b, b), c, 0,
                                                       0, 0);
    }
};

__device__ __forceinline__ int dot4_ones(v4i v)
{
    int s = __builtin_amdgcn_sdot4(v.x, 0x01010101, 0, false);
    s     = __builtin_amdgcn_sdot4(v.y, 0x01010101, s, false);
    s     = __builtin_amdgcn_sdot4(v.z, 0x01010101, s, false);
    return __builtin_amdgcn_sdot4(v.w, 0x01010101, s, false);
}

// 16 bytes starting at byte offset `off` of a row of `row_bytes` bytes; bytes past the row end read as 0.
// `vec_ok` says that every row start and `off` are 16-byte aligned and the row length is a multiple of 16.
__device__ __forceinline__ v4i load_chunk(const uint8_t* row, int off, int row_bytes, bool vec_ok)
{
    if (vec_ok)
    {
        if (off < row_bytes)
            return *reinterpret_cast<const v4i*>(row + off);
        return v4i{ 0, 0, 0, 0 };
    }
    union
    {
        v4i v;
        uint8_t b[16];
    } u;
    u.v = v4i{ 0, 0, 0, 0 };
    for (int j = 0; j < 16; j++)
        if (off + j < row_bytes)
            u.b[j] = row[off + j];
    return u.v;
}

// 16 bytes of the fill value (input_zp in every byte) limited to the row, zero beyond it.
__device__ __forceinline__ v4i fill_chunk(int off, int row_bytes, int fill_byte)
{
    const int word = (fill_byte & 0xff) * 0x01010101;
    if (off + 16 <= row_bytes)
        return v4i{ word, word, word, word };
    union
    {
        v4i v;
        uint8_t b[16];
    } u;
    u.v = v4i{ 0, 0, 0, 0 };
    for (int j = 0; j < 16; j++)
        if (off + j < row_bytes)
            u.b[j] = (uint8_t)fill_byte;
    return u.v;
}

template <typename OutT>
__device__ __forceinline__ OutT to_out(float v);
template <>
__device__ __forceinline__ _Float16 to_out<_Float16>(float v)
{
    return (_Float16)v;
}
template <>
__device__ __forceinline__ bf16_t to_out<bf16_t>(float v)
{
    return float_to_bf16(v);
}

template <typename T, int OCT, int PXT>
__global__ __launch_bounds__(256) void conv2d_patch_kernel(PatchArgs a)
{
    using M                = Mma<T>;
    using acc_t            = typename M::acc_t;
    constexpr int EB       = sizeof(T);
    constexpr int OCB      = 16 * OCT;
    constexpr int STAGE_U  = 8;    // global loads in flight per lane while staging
    const ConvGeom& g      = a.g;
    const int tid          = threadIdx.x;
    const int lane         = tid & 63;
    const int wave         = tid >> 6;
    const int li           = lane & 15;    // row of the A fragment / column (pixel) of D
    const int lg           = lane >> 4;    // K chunk taken by this lane / row group of D
    const int taps         = g.KH * g.KW;
    const int row_bytes    = g.IC * EB;    // bytes of one pixel's (or one weight tap's) channel vector
    const int blk_bytes    = a.CH * 16;
    const bool vec_ok      = (row_bytes % 16) == 0;

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    int* tapoff        = reinterpret_cast<int*>(lds);
    const int tab_bytes = (taps * 4 + 15) & ~15;
    uint8_t* wl        = lds + tab_bytes;
    uint8_t* pl        = wl + (size_t)taps * OCB * a.wstride;

#ifdef TMI_X_EARLY_RETURN
    if (a.ksteps < 1000) return;
#endif
    // ---- which tile --------------------------------------------------------------------------------
    int bid = blockIdx.x;
    if (a.xcd_remap)
    {
        // consecutive workgroups are dealt to the 8 XCDs in turn; give each XCD a contiguous run of tiles
        // so that neighbouring tiles (which share halo rows) share an L2
        const int per = gridDim.x >> 3;
        bid           = (bid & 7) * per + (bid >> 3);
    }
    const int ocb   = bid / a.n_tiles;
    int tile        = bid - ocb * a.n_tiles;
    const int txi   = tile % a.tiles_x;
    tile /= a.tiles_x;
    const int tyi   = tile % a.tiles_y;
    const int n     = tile / a.tiles_y;
    const int oy0   = tyi * a.TH;
    const int ox0   = txi * a.TW;
    const int oc0   = ocb * OCB;
    const int y0    = oy0 * g.stride_y - g.pad_top;
    const int x0    = ox0 * g.stride_x - g.pad_left;
    const int P     = a.TH * a.TW;

    for (int t = tid; t < taps; t += 256)
        tapoff[t] = ((t / g.KW) * g.dil_y * a.PW + (t % g.KW) * g.dil_x) * a.pstride;

    // ---- per-lane pixel bases ----------------------------------------------------------------------
    int pbase[PXT];
#pragma unroll
    for (int i = 0; i < PXT; i++)
    {
        int p = (wave * PXT + i) * 16 + li;
        if (p >= P)
            p = 0;
        pbase[i] = ((p / a.TW) * g.stride_y * a.PW + (p % a.TW) * g.stride_x) * a.pstride;
    }

    acc_t acc[PXT][OCT];
#pragma unroll
    for (int i = 0; i < PXT; i++)
#pragma unroll
        for (int t = 0; t < OCT; t++)
            acc[i][t] = acc_t{ 0, 0, 0, 0 };
    int wsum[OCT];
    int asum[PXT];
#pragma unroll
    for (int t = 0; t < OCT; t++)
        wsum[t] = 0;
#pragma unroll
    for (int i = 0; i < PXT; i++)
        asum[i] = 0;

    const int ch_shift = a.CH == 4 ? 2 : (a.CH == 2 ? 1 : 0);
    const int n_pairs  = taps * a.CH;
    const bool wave_active = wave * PXT * 16 < P;

    for (int icb = 0; icb < a.n_icb; icb++)
    {
        const int ic_off = icb * blk_bytes;
        if (icb)
            __syncthreads();
        // ---- stage weights [tap][row][CH chunks] and the input patch [py][px][CH chunks] ------------------
        // Loads are issued in batches of STAGE_U per lane before any of them is written to LDS, so that
        // the HBM/L2 latency is paid once per batch rather than once per chunk.
#ifndef TMI_X_NO_STAGE
        {
            const int w_total = OCB * taps * a.CH;
            const int p_total = a.PH * a.PW * a.CH;
            for (int base = tid; base < w_total; base += 256 * STAGE_U)
            {
                v4i v[STAGE_U];
                int dst[STAGE_U];
#pragma unroll
                for (int u = 0; u < STAGE_U; u++)
                {
                    const int idx = base + u * 256;
                    v[u]          = v4i{ 0, 0, 0, 0 };
                    dst[u]        = -1;
                    if (idx < w_total)
                    {
                        const int cc  = idx & (a.CH - 1);
                        const int r2  = idx >> ch_shift;
                        const int ocl = r2 / taps;
                        const int tap = r2 - ocl * taps;
                        if (oc0 + ocl < g.OC)
                            v[u] = load_chunk(a.w + ((size_t)(oc0 + ocl) * taps + tap) * row_bytes, ic_off + cc * 16,
                                              row_bytes, vec_ok);
                        const int grp = ocl / (4 * OCT), rem = ocl % (4 * OCT);
                        const int row = (rem >> 2) * 16 + grp * 4 + (rem & 3);
                        dst[u]        = (tap * OCB + row) * a.wstride + cc * 16;
                    }
                }
#pragma unroll
                for (int u = 0; u < STAGE_U; u++)
                    if (dst[u] >= 0)
                        *reinterpret_cast<v4i*>(wl + dst[u]) = v[u];
            }
            for (int base = tid; base < p_total; base += 256 * STAGE_U)
            {
                v4i v[STAGE_U];
                int dst[STAGE_U];
#pragma unroll
                for (int u = 0; u < STAGE_U; u++)
                {
                    const int idx = base + u * 256;
                    v[u]          = v4i{ 0, 0, 0, 0 };
                    dst[u]        = -1;
                    if (idx < p_total)
                    {
                        const int cc  = idx & (a.CH - 1);
                        const int pix = idx >> ch_shift;
                        const int py  = pix / a.PW;
                        const int px  = pix - py * a.PW;
                        const int iy = y0 + py, ix = x0 + px;
                        if (iy >= 0 && iy < g.IH && ix >= 0 && ix < g.IW)
                            v[u] = load_chunk(a.in + (((size_t)n * g.IH + iy) * g.IW + ix) * row_bytes,
                                              ic_off + cc * 16, row_bytes, vec_ok);
                        else
                            v[u] = fill_chunk(ic_off + cc * 16, row_bytes, M::is_int ? a.za : 0);
                        dst[u] = pix * a.pstride + cc * 16;
                    }
                }
#pragma unroll
                for (int u = 0; u < STAGE_U; u++)
                    if (dst[u] >= 0)
                        *reinterpret_cast<v4i*>(pl + dst[u]) = v[u];
            }
        }
#endif
        __syncthreads();

        // ---- MFMA over the (tap, chunk) pairs of this channel block -----------------------------------
#ifndef TMI_X_NO_MFMA
        if (wave_active)
#else
        if (wave_active && a.ksteps > 1000)
#endif
        {
            for (int s = 0; s < a.ksteps; s++)
            {
                const int q     = 4 * s + lg;
                const bool live = q < n_pairs;
                const int tap   = live ? (q >> ch_shift) : 0;
                const int cc    = q & (a.CH - 1);
                v4i af[OCT], bf[PXT];
                const uint8_t* wp = wl + (size_t)(tap * OCB + li) * a.wstride + cc * 16;
#pragma unroll
                for (int t = 0; t < OCT; t++)
                    af[t] = live ? *reinterpret_cast<const v4i*>(wp + t * 16 * a.wstride) : v4i{ 0, 0, 0, 0 };
                const int to = tapoff[tap] + cc * 16;
#pragma unroll
                for (int i = 0; i < PXT; i++)
                    bf[i] = live ? *reinterpret_cast<const v4i*>(pl + pbase[i] + to) : v4i{ 0, 0, 0, 0 };
#pragma unroll
                for (int i = 0; i < PXT; i++)
#pragma unroll
                    for (int t = 0; t < OCT; t++)
                        acc[i][t] = M::mma(af[t], bf[i], acc[i][t]);
                if constexpr (M::is_int)
                {
                    if (a.za != 0)
#pragma unroll
                        for (int t = 0; t < OCT; t++)
                            wsum[t] += dot4_ones(af[t]);
                    if (a.zw != 0)
#pragma unroll
                        for (int i = 0; i < PXT; i++)
                            asum[i] += dot4_ones(bf[i]);
                }
            }
        }
    }

    if (!wave_active)
        return;
#ifdef TMI_X_NO_EPILOGUE_AT_ALL
    if (a.ksteps < 1000) { if (acc[0][0][0] == 0x12345678) a.flag_word[1] = 1; return; }
#endif

    // ---- epilogue -------------------------------------------------------------------------------------
    uint32_t flags = 0;
    const int ocl0 = 4 * OCT * lg;    // first of this lane's 4*OCT consecutive channels inside the block
    if constexpr (M::is_int)
    {
        // finish the K-chunk reduction of the side sums (lanes li, li+16, li+32, li+48 hold partials)
        int corr[OCT][4];
        if (a.za != 0)
        {
#pragma unroll
            for (int t = 0; t < OCT; t++)
            {
                int v = wsum[t];
                v += __shfl_xor(v, 16);
                v += __shfl_xor(v, 32);
                // D row 4*lg + r of tile t is weight row (A fragment lane) 4*lg + r
#pragma unroll
                for (int r = 0; r < 4; r++)
                    corr[t][r] = __shfl(v, 4 * lg + r) * a.za;
            }
        }
        else
        {
#pragma unroll
            for (int t = 0; t < OCT; t++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    corr[t][r] = 0;
        }
        const int kzz = g.KH * g.KW * g.IC * a.za * a.zw;
        // per pixel group: validity, output offset and the zero-point term that depends on the pixel
        bool pix_ok[PXT];
        size_t obase[PXT];
        int pcorr[PXT];
#pragma unroll
        for (int i = 0; i < PXT; i++)
        {
            int sa = asum[i];
            if (a.zw != 0)
            {
                sa += __shfl_xor(sa, 16);
                sa += __shfl_xor(sa, 32);
            }
            pcorr[i]     = kzz - a.zw * sa;
            const int p  = (wave * PXT + i) * 16 + li;
            const int ty = p / a.TW, tx = p - ty * a.TW;
            const int oy = oy0 + ty, ox = ox0 + tx;
            pix_ok[i]    = p < P && oy < g.OH && ox < g.OW;
            obase[i]     = (((size_t)n * g.OH + oy) * g.OW + ox) * g.OC + oc0 + ocl0;
        }
        const bool full    = (oc0 + ocl0 + 4 * OCT <= g.OC);
        const bool vec_out = full && (g.OC % (4 * OCT)) == 0 && ((uintptr_t)a.out & 15) == 0;
        // bias / multiplier / shift / int32 output rows of four channels can be moved as one vector
        const bool vec_par = full && (g.OC & 3) == 0 && (oc0 + ocl0) % 4 == 0 &&
                             (((uintptr_t)a.bias | (uintptr_t)a.out | (a.rp.enabled ? (uintptr_t)a.rp.multiplier : 0)) & 15) == 0 &&
                             (!a.rp.enabled || ((uintptr_t)a.rp.shift & 3) == 0);
        int packed[PXT][OCT];    // int8 results, four channels per word

        // channel tile by channel tile: fetch the four channels' constants once, use them for every pixel
#pragma unroll
        for (int t = 0; t < OCT; t++)
        {
            const int c0 = oc0 + ocl0 + 4 * t;
            int32_t bias4[4], mult4[4], shift4[4];
#pragma unroll
            for (int r = 0; r < 4; r++)
                bias4[r] = mult4[r] = 0, shift4[r] = 32;    // neutral: every value legal, result 0
            if (g.bias_len == 1)
            {
                const int32_t b = reinterpret_cast<const int32_t*>(a.bias)[0];
#pragma unroll
                for (int r = 0; r < 4; r++)
                    bias4[r] = b;
            }
            else if (vec_par)
            {
                const v4i b = *reinterpret_cast<const v4i*>(reinterpret_cast<const int32_t*>(a.bias) + c0);
                bias4[0] = b.x, bias4[1] = b.y, bias4[2] = b.z, bias4[3] = b.w;
            }
            else
            {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (c0 + r < g.OC)
                        bias4[r] = reinterpret_cast<const int32_t*>(a.bias)[c0 + r];
            }
            ChannelScale cs[4];
            if (a.rp.enabled)
            {
                if (vec_par && a.rp.per_channel && a.rp.scale32)
                {
                    const v4i m = *reinterpret_cast<const v4i*>(reinterpret_cast<const int32_t*>(a.rp.multiplier) + c0);
                    const int sh = *reinterpret_cast<const int*>(a.rp.shift + c0);
                    mult4[0] = m.x, mult4[1] = m.y, mult4[2] = m.z, mult4[3] = m.w;
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        shift4[r] = (int32_t)(int8_t)(sh >> (8 * r));
                }
                else
                {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (c0 + r < g.OC)
                            mult4[r] = load_multiplier(a.rp, c0 + r), shift4[r] = load_shift(a.rp, c0 + r);
                }
                if (a.rp.fast)
                {
                    // channels past OC carry the neutral constants (0, 32) set above and raise nothing
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        cs[r] = make_channel_scale(mult4[r], shift4[r], a.rp.double_round, flags);
                }
            }
#pragma unroll
            for (int i = 0; i < PXT; i++)
            {
                int32_t res[4];
#pragma unroll
                for (int r = 0; r < 4; r++)
                {
                    int32_t v = acc[i][t][r] + pcorr[i] - corr[t][r] + bias4[r];
#ifndef TMI_X_NO_EPI
                    if (a.rp.enabled)
                    {
                        if (a.rp.fast)
                        {
                            uint32_t f = 0;
                            v          = fast_rescale(v, cs[r], a.rp.out_zp, a.rp.lo, a.rp.hi, f);
                            flags |= pix_ok[i] ? f : 0u;    // pixels outside the image must not raise anything
                        }
                        else if (pix_ok[i] && c0 + r < g.OC)
                            v = rescale_value(a.rp, v, mult4[r], shift4[r], flags);
                    }
#endif
                    res[r] = v;
                }
                if (!pix_ok[i])
                    continue;
                if (a.out_dtype == TMI_INT32)
                {
                    int32_t* o = reinterpret_cast<int32_t*>(a.out) + obase[i] + 4 * t;
                    if (vec_par)
                        *reinterpret_cast<v4i*>(o) = v4i{ res[0], res[1], res[2], res[3] };
                    else
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            if (c0 + r < g.OC)
                                o[r] = res[r];
                }
                else if (a.out_dtype == TMI_INT8)
                {
                    if (vec_out)
                        packed[i][t] = (res[0] & 0xff) | ((res[1] & 0xff) << 8) | ((res[2] & 0xff) << 16) |
                                       ((res[3] & 0xff) << 24);
                    else
                    {
                        int8_t* o = reinterpret_cast<int8_t*>(a.out) + obase[i] + 4 * t;
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            if (c0 + r < g.OC)
                                o[r] = (int8_t)res[r];
                    }
                }
                else
                {
                    int16_t* o = reinterpret_cast<int16_t*>(a.out) + obase[i] + 4 * t;
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (c0 + r < g.OC)
                            o[r] = (int16_t)res[r];
                }
            }
        }
        if (a.out_dtype == TMI_INT8 && vec_out)
        {
#pragma unroll
            for (int i = 0; i < PXT; i++)
            {
                if (!pix_ok[i])
                    continue;
                int8_t* o = reinterpret_cast<int8_t*>(a.out) + obase[i];
                if constexpr (OCT == 4)
                    *reinterpret_cast<v4i*>(o) = v4i{ packed[i][0], packed[i][1], packed[i][2], packed[i][3] };
                else
#pragma unroll
                    for (int t = 0; t < OCT; t++)
                        reinterpret_cast<int*>(o)[t] = packed[i][t];
            }
        }
        raise_flags(a.flag_word, flags);
    }
    else
    {
#pragma unroll
        for (int i = 0; i < PXT; i++)
        {
            const int p = (wave * PXT + i) * 16 + li;
            const int ty = p / a.TW, tx = p - ty * a.TW;
            const int oy = oy0 + ty, ox = ox0 + tx;
            if (!(p < P && oy < g.OH && ox < g.OW))
                continue;
            const size_t obase = (((size_t)n * g.OH + oy) * g.OW + ox) * g.OC + oc0 + ocl0;
            T* o               = reinterpret_cast<T*>(a.out) + obase;
            const T* bias      = reinterpret_cast<const T*>(a.bias);
#pragma unroll
            for (int t = 0; t < OCT; t++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                {
                    const int j  = 4 * t + r;
                    const int oc = oc0 + ocl0 + j;
                    if (oc < g.OC)
                    {
                        float b;
                        if constexpr (sizeof(T) == 2 && !__is_same(T, bf16_t))
                            b = (float)bias[g.bias_len == 1 ? 0 : oc];
                        else
                            b = bf16_to_float(reinterpret_cast<const bf16_t*>(a.bias)[g.bias_len == 1 ? 0 : oc]);
                        o[j] = to_out<T>(b + acc[i][t][r]);
                    }
                }
        }
    }
}

// ---- host side: tile choice and launch -----------------------------------------------------------------

static constexpr int kMaxLds = 160 * 1024;

template <typename T, int OCT, int PXT>
static bool launch_patch(hipStream_t st, PatchArgs& a, size_t lds_bytes, int blocks)
{
    auto kern = conv2d_patch_kernel<T, OCT, PXT>;
    static size_t configured = 0;    // largest dynamic LDS size this instantiation was configured for
    if (lds_bytes > configured)
    {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds_bytes) != hipSuccess)
            return false;
        configured = lds_bytes;
    }
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), lds_bytes, st, a);
    return true;
}

template <typename T>
static const char* launch_conv2d_mfma_t(hipStream_t st, const ConvGeom& g, int32_t out_dtype, const void* in,
                                        const void* w, const void* bias, int32_t in_zp, int32_t w_zp,
                                        const RescaleParams& rp, void* out, uint32_t* flag_word, const char* label)
{
    constexpr int EB  = sizeof(T);
    constexpr int PXT = 2;
    const int row_bytes = g.IC * EB;
    if (row_bytes <= 0 || g.OC <= 0 || (int64_t)g.N * g.OH * g.OW == 0)
        return nullptr;

    PatchArgs a{};
    a.g = g, a.in = (const uint8_t*)in, a.w = (const uint8_t*)w, a.bias = bias, a.out = out;
    a.flag_word = flag_word, a.rp = rp, a.za = in_zp, a.zw = w_zp, a.out_dtype = out_dtype;
    a.CH      = row_bytes <= 16 ? 1 : (row_bytes <= 32 ? 2 : 4);
    a.pstride = a.CH == 1 ? 16 : a.CH * 16 + 16;
    a.wstride = a.pstride;
    a.n_icb   = (row_bytes + a.CH * 16 - 1) / (a.CH * 16);
    const int taps = g.KH * g.KW;
    a.ksteps  = (taps * a.CH + 3) / 4;

    const int OCT = g.OC > 32 ? 4 : (g.OC > 16 ? 2 : 1);
    const int OCB = 16 * OCT;
    a.oc_blocks   = (g.OC + OCB - 1) / OCB;

    // tile: up to 4 waves x PXT groups x 16 pixels; prefer full output rows
    const int max_px = 4 * PXT * 16;
    int TW = g.OW < max_px ? g.OW : max_px;
    int TH = max_px / TW;
    if (TH > g.OH)
        TH = g.OH;
    if (TH < 1)
        TH = 1;
    const size_t tab_bytes = ((size_t)taps * 4 + 15) & ~(size_t)15;
    const size_t w_bytes   = (size_t)taps * OCB * a.wstride;
    size_t lds_bytes       = 0;
    for (;;)
    {
        a.PH      = (TH - 1) * g.stride_y + (g.KH - 1) * g.dil_y + 1;
        a.PW      = (TW - 1) * g.stride_x + (g.KW - 1) * g.dil_x + 1;
        lds_bytes = tab_bytes + w_bytes + (size_t)a.PH * a.PW * a.pstride;
        if (lds_bytes <= (size_t)kMaxLds)
            break;
        if (TH > 1)
            TH = (TH + 1) / 2;
        else if (TW > 16)
            TW = (TW + 1) / 2;
        else
            return nullptr;    // the weight slab alone does not fit: not eligible
    }
    a.TH = TH, a.TW = TW;
    a.tiles_y = (g.OH + TH - 1) / TH;
    a.tiles_x = (g.OW + TW - 1) / TW;
    const int64_t n_tiles = (int64_t)g.N * a.tiles_y * a.tiles_x;
    const int64_t blocks  = n_tiles * a.oc_blocks;
    if (blocks > 0x7fffffff)
        return nullptr;
    a.n_tiles   = (int)n_tiles;
    a.xcd_remap = (blocks % 8) == 0 && blocks >= 16;

    bool ok = false;
    switch (OCT)
    {
        case 4:
            ok = launch_patch<T, 4, PXT>(st, a, lds_bytes, (int)blocks);
            break;
        case 2:
            ok = launch_patch<T, 2, PXT>(st, a, lds_bytes, (int)blocks);
            break;
        default:
            ok = launch_patch<T, 1, PXT>(st, a, lds_bytes, (int)blocks);
            break;
    }
    return ok ? label : nullptr;
}

const char* launch_conv2d_mfma(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                               const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                               void* out, uint32_t* flag_word)
{
    if (in_dtype == TMI_INT8)
        return launch_conv2d_mfma_t<int8_t>(st, g, out_dtype, in, w, bias, in_zp, w_zp, rp, out, flag_word,
                                            rp.enabled ? "conv2d_mfma_i8_rescale" : "conv2d_mfma_i8");
    if (in_dtype == TMI_FP16 && out_dtype == TMI_FP16)
        return launch_conv2d_mfma_t<_Float16>(st, g, out_dtype, in, w, bias, 0, 0, rp, out, flag_word,
                                              "conv2d_mfma_f16");
    if (in_dtype == TMI_BF16 && out_dtype == TMI_BF16)
        return launch_conv2d_mfma_t<bf16_t>(st, g, out_dtype, in, w, bias, 0, 0, rp, out, flag_word,
                                            "conv2d_mfma_bf16");
    return nullptr;
}

}    // namespace tmi
