// CONV2D as an implicit GEMM on the matrix cores (MFMA), with the bias / zero-point / RESCALE / CLAMP
// epilogue fused so that the int32 accumulators never reach HBM.
//
// One workgroup (8 waves) computes a TH x TW tile of output pixels of one image for a block of OCB =
// 32*WOC output channels; wave w owns channel tile w / (8/WOC) and PXT pixel tiles of 32 pixels.  Two waves
// per SIMD is what hides LDS and VALU latency here: the named shapes are far too small to fill the chip with
// bigger per-wave tiles.  Per block of 64 bytes of input channels the workgroup stages in LDS
//   - the input patch that the tile needs (PH x PW pixels, out-of-image pixels filled with input_zp, so the
//     zero-point identity below holds with the full K): one row of CH 16-byte chunks per pixel, and
//   - the weight slab: one row per output channel holding its KH*KW*CH chunks in (tap, chunk) order, which
//     is the order they have in HBM.
// Every input byte is read from HBM/L2 once per workgroup (plus the halo) and reused KH*KW*OCB times
// from LDS.
//
// The MFMA is the 32x32 shape (v_mfma_i32_32x32x32_i8, v_mfma_f32_32x32x16_{f16,bf16}), which on this chip
// runs at the full int8 rate while the 16x16x64 shape does not.  A fragment gives every lane 16 bytes: lane
// l holds row l%32, K half l/32.  Both LDS row strides are kept congruent to 16 modulo 32 bytes, the layout
// for which ds_read_b128 of such a fragment runs at the full LDS rate (measured: 16/48/80/.. bytes reach
// ~230 B/clk/CU, 32/64/96 bytes half or less).
//
// Operand roles: the weights are the "A" operand (rows of D = output channels), the pixels the "B" operand
// (columns of D = pixels).  With the 32x32 accumulator layout (lane l, register 4q+j) = D[8q + 4(l/32) + j]
// [l%32], giving row 8q+4h+j of a channel tile the output channel 16h + 4q + j makes every lane own 16
// consecutive channels of one pixel: its int8 results leave as one 16-byte store.
//
// A K-step feeds each lane 16 bytes of one (tap, chunk) pair; lane half h takes pair 2*step+h.  The K loop is
// software pipelined three deep (fragments of step s+2 are requested before the MFMAs of step s issue) and a
// dead pair (odd pair count) is read from a zeroed LDS chunk so that no instruction has to touch a fragment
// between its load and its MFMA.  Integer dot
// products are order independent, so the assignment of pairs to lanes is free as long as both operands
// agree; the floating-point variants are compared against fp64 with the reference's DOT_PRODUCT bound.
//
// Zero points: sum((a-za)(w-zw)) = sum(a*w) - zw*sum(a) - za*sum(w) + K*za*zw.  sum(w) per channel and
// sum(a) per pixel are accumulated from the very fragments fed to the MFMA with v_dot4 against 0x01010101.
//
// Epilogue: the per-channel constants (bias, multiplier, shift and the 64-bit rounding terms derived from
// them) are computed once per workgroup by OCB lanes while the staging loads are in flight and kept in an
// LDS table; every lane then spends about ten instructions per output element.
#include <type_traits>

#include "tmi_kernels.h"

namespace tmi
{

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8b __attribute__((ext_vector_type(8)));

// n / d for n*d < 2^32 as one multiply-high (magic = floor(2^32/d) + 1; d == 1 is special-cased).
struct FastDiv
{
    uint32_t magic, d;
};

static FastDiv make_fastdiv(uint32_t d)
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
    int32_t TH, TW, tiles_y, tiles_x;
    int32_t PH, PW;
    int32_t CH;                  // 16-byte chunks per pixel row in LDS (1, 2 or 4)
    int32_t pstride, wstride;    // LDS row strides in bytes, both = 16 (mod 32)
    int32_t n_icb;               // blocks of CH*16 bytes along the input channels
    int32_t ksteps;              // MFMA K-steps per channel block = ceil(taps*CH/2)
    int32_t n_tiles;             // N * tiles_y * tiles_x
    int32_t out_dtype;
    int32_t xcd_remap;
    int64_t w_batch_stride;    // bytes between the weights of consecutive images (0: shared; MATMUL: per batch)
    FastDiv div_tw, div_pw, div_rch, div_tiles_x, div_tiles_y, div_n_tiles, div_kw;
};

template <typename T>
struct Mma;

template <>
struct Mma<int8_t>
{
    using acc_t                  = v16i;
    static constexpr bool is_int = true;
    __device__ static v16i mma(v4i a, v4i b, v16i c)
    {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
    }
};
template <>
struct Mma<_Float16>
{
    using acc_t                  = v16f;
    static constexpr bool is_int = false;
    __device__ static v16f mma(v4i a, v4i b, v16f c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0,
                                                      0, 0);
    }
};
template <>
struct Mma<bf16_t>
{
    using acc_t                  = v16f;
    static constexpr bool is_int = false;
    __device__ static v16f mma(v4i a, v4i b, v16f c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8b, a), __builtin_bit_cast(v8b, b), c, 0,
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

// Byte-wise version of a chunk load for channel vectors whose length is not a multiple of 16 bytes
// (rows are then unaligned): bytes past the row end read as 0.  The rare path.
__device__ __forceinline__ v4i load_chunk_bytes(const uint8_t* row, int off, int row_bytes)
{
    v4i r;
#pragma unroll
    for (int k = 0; k < 4; k++)
    {
        uint32_t word = 0;
#pragma unroll
        for (int b = 0; b < 4; b++)
            if (off + 4 * k + b < row_bytes)
                word |= (uint32_t)row[off + 4 * k + b] << (8 * b);
        r[k] = (int)word;
    }
    return r;
}

// 16 bytes of the fill byte limited to the row, zero beyond it.
__device__ __forceinline__ v4i fill_chunk(int off, int row_bytes, int fill_byte)
{
    const int word = (fill_byte & 0xff) * 0x01010101;
    const int n    = row_bytes - off;    // bytes of this chunk that belong to the row
    if (n >= 16)
        return v4i{ word, word, word, word };
    v4i r;
#pragma unroll
    for (int k = 0; k < 4; k++)
    {
        const int m = n - 4 * k;    // bytes of word k inside the row
        r[k]        = m >= 4 ? word : (m <= 0 ? 0 : (word & ((1 << (8 * m)) - 1)));
    }
    return r;
}

template <typename T>
__device__ __forceinline__ float load_as_float(const void* p, int i);
template <>
__device__ __forceinline__ float load_as_float<_Float16>(const void* p, int i)
{
    return (float)reinterpret_cast<const _Float16*>(p)[i];
}
template <>
__device__ __forceinline__ float load_as_float<bf16_t>(const void* p, int i)
{
    return bf16_to_float(reinterpret_cast<const bf16_t*>(p)[i]);
}
template <>
__device__ __forceinline__ float load_as_float<int8_t>(const void*, int)
{
    return 0.0f;
}

__device__ __forceinline__ void store_from_float(_Float16* p, float v)
{
    *p = (_Float16)v;
}
__device__ __forceinline__ void store_from_float(bf16_t* p, float v)
{
    *p = float_to_bf16(v);
}
__device__ __forceinline__ void store_from_float(int8_t*, float)
{}

enum
{
    EPI_PLAIN   = 0,    // int32 (or floating-point) result stored as is
    EPI_FAST    = 1,    // RESCALE (+CLAMP) through fast_rescale()
    EPI_GENERIC = 2     // any other RESCALE, staged through LDS
};

// Per-channel constants of the integer epilogues, one 32-byte LDS entry per channel of the block.
struct alignas(16) ChanEntry
{
    int32_t m, s, bias;
    uint32_t lim;
    int64_t rnd_pos, rnd_neg;
};

template <typename T, int WOC, int PXT, int EPI, bool VEC>
__global__ __launch_bounds__(512) void conv2d_patch_kernel(PatchArgs a)
{
    using M              = Mma<T>;
    using acc_t          = typename M::acc_t;
    constexpr int EB     = sizeof(T);
    constexpr int NT     = 512;          // lanes per workgroup
    constexpr int WPX    = 8 / WOC;      // waves along the pixel dimension
    constexpr int OCB    = 32 * WOC;     // output channels per workgroup
    constexpr int WU     = 5;            // weight chunks in flight per lane in one staging round
    constexpr int PU     = 2;            // patch chunks in flight per lane in one staging round
    const ConvGeom& g    = a.g;
    const int tid        = threadIdx.x;
    const int lane       = tid & 63;
    // wave-uniform values are made scalar explicitly: with two waves per SIMD the vector ALU (4 cycles per
    // wave64 instruction) is the scarce resource, so everything uniform must run on the scalar unit
    const int wave       = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int woc        = wave / WPX;   // channel tile of this wave
    const int wpx        = wave % WPX;   // first pixel tile of this wave is wpx*PXT
    const int li         = lane & 31;    // row of the A fragment / column (pixel) of D
    const int lh         = lane >> 5;    // K half taken by this lane / row half of D
    const int taps       = g.KH * g.KW;
    const int row_bytes  = g.IC * EB;    // bytes of one pixel's (or one weight tap's) channel vector
    const int blk_bytes  = a.CH * 16;
    const int ch_shift   = a.CH == 4 ? 2 : (a.CH == 2 ? 1 : 0);
    const int n_pairs    = taps * a.CH;  // (tap, chunk) pairs per channel block = chunks per weight row
    const int fill_word  = M::is_int ? (a.za & 0xff) * 0x01010101 : 0;    // out-of-image pixels hold input_zp

    // LDS: [channel table][16 zero bytes][pair offset table][weight rows][input patch]
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    ChanEntry* ctab        = reinterpret_cast<ChanEntry*>(lds);
    float* ftab            = reinterpret_cast<float*>(lds);    // floating point: bias as float
    constexpr int kCtab    = OCB * (int)sizeof(ChanEntry);
    uint8_t* zero_chunk    = lds + kCtab;
    int* need_check        = reinterpret_cast<int*>(lds + kCtab + 16);    // set when some channel has shift < 32
    int* pairoff           = reinterpret_cast<int*>(lds + kCtab + 32);
    const int tab_entries  = n_pairs + 32;    // 2*(ksteps + 3G) + 1 < n_pairs + 32 for G = 3    // slack: the pipeline reads a few entries past the end
    const int tab_bytes    = (tab_entries * 4 + 15) & ~15;
    uint8_t* wl            = lds + kCtab + 32 + tab_bytes;
    uint8_t* pl            = wl + OCB * a.wstride;

    // ---- which tile ------------------------------------------------------------------------------------
    uint32_t bid = blockIdx.x;
    if (a.xcd_remap)
    {
        // consecutive workgroups are dealt to the 8 XCDs in turn; give each XCD a contiguous run of tiles
        // so that neighbouring tiles (which share halo rows) share an L2
        const uint32_t per = gridDim.x >> 3;
        bid                = (bid & 7) * per + (bid >> 3);
    }
    const uint32_t ocb  = fdiv(bid, a.div_n_tiles);
    uint32_t tile       = bid - ocb * a.n_tiles;
    const uint32_t trow = fdiv(tile, a.div_tiles_x);
    const int txi       = tile - trow * a.tiles_x;
    const int n         = fdiv(trow, a.div_tiles_y);
    const int tyi       = trow - n * a.tiles_y;
    const int oy0       = tyi * a.TH;
    const int ox0       = txi * a.TW;
    const int oc0       = ocb * OCB;
    const int y0        = oy0 * g.stride_y - g.pad_top;
    const int x0        = ox0 * g.stride_x - g.pad_left;
    const int P         = a.TH * a.TW;
    const uint8_t* wbase_ptr = a.w + (size_t)n * a.w_batch_stride;

    // ---- tables ----------------------------------------------------------------------------------------
    uint32_t flags = 0;
    if (tid < 4)
        reinterpret_cast<int*>(zero_chunk)[tid] = 0;
    // An odd pair count leaves the upper K half of the last step empty: the spare chunk behind every weight
    // row is zero, so that half contributes nothing whatever the pixel operand holds.
    if ((n_pairs & 1) && tid < OCB)
        *reinterpret_cast<v4i*>(wl + tid * a.wstride + n_pairs * 16) = v4i{ 0, 0, 0, 0 };
    for (int q = tid; q < tab_entries; q += NT)
    {
        int off = 0;
        if (q < n_pairs)
        {
            const int tap = q >> ch_shift;
            const int ky  = fdiv(tap, a.div_kw);
            const int kx  = tap - ky * g.KW;
            off           = (ky * g.dil_y * a.PW + kx * g.dil_x) * a.pstride + (q & (a.CH - 1)) * 16;
        }
        pairoff[q] = off;
    }
    if (tid < OCB)
    {
        const int oc  = oc0 + tid;
        const bool ok = oc < g.OC;
        if constexpr (M::is_int)
        {
            ChanEntry e;
            e.bias = ok ? reinterpret_cast<const int32_t*>(a.bias)[g.bias_len == 1 ? 0 : oc] : 0;
            e.m = 0, e.s = 32, e.lim = 0x80000000u, e.rnd_pos = e.rnd_neg = 0;
            if constexpr (EPI == EPI_FAST)
            {
                // channels past OC get neutral constants (0, 32): every value legal, nothing raised
                const int32_t m       = ok ? load_multiplier(a.rp, oc) : 0;
                const int32_t sh      = ok ? load_shift(a.rp, oc) : 32;
                const ChannelScale cs = make_channel_scale(m, sh, a.rp.double_round, flags);
                // (p + rnd) >> s + zp == (p + rnd + zp * 2^s) >> s: the output zero point rides in the rounding term
                const int64_t zp_term = (int64_t)a.rp.out_zp << cs.s;
                e.m = cs.m, e.s = cs.s, e.lim = cs.lim, e.rnd_pos = cs.rnd_pos + zp_term, e.rnd_neg = cs.rnd_neg + zp_term;
                // a shift below 32 somewhere: apply_scale_32's value range can be violated and must be checked.
                // All table lanes sit in wave 0, so one ballot decides and a single lane writes the word.
                const int any_check = __any(cs.lim != 0x80000000u);
                if (tid == 0)
                    *need_check = any_check;
            }
            ctab[tid] = e;
        }
        else
            ftab[tid] = ok ? load_as_float<T>(a.bias, g.bias_len == 1 ? 0 : oc) : 0.0f;
    }

    // ---- per-lane pixel bases --------------------------------------------------------------------------
    int pbase[PXT];
#pragma unroll
    for (int i = 0; i < PXT; i++)
    {
        int p = (wpx * PXT + i) * 32 + li;
        if (p >= P)
            p = 0;
        const int ty = fdiv(p, a.div_tw);
        pbase[i]     = (ty * g.stride_y * a.PW + (p - ty * a.TW) * g.stride_x) * a.pstride;
    }

    acc_t acc[PXT];
#pragma unroll
    for (int i = 0; i < PXT; i++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            acc[i][r] = 0;
    int asum[PXT];
#pragma unroll
    for (int i = 0; i < PXT; i++)
        asum[i] = 0;

    const bool wave_active = wpx * PXT * 32 < P;

    for (int icb = 0; icb < a.n_icb; icb++)
    {
        const int ic_off = icb * blk_bytes;
        int staged_w_sum = 0;
        if (icb)
            __syncthreads();
        // ---- stage the weight rows and the input patch ---------------------------------------------------
        // Nothing hides memory latency here except the loads themselves: every round issues up to WU weight
        // chunks and PU patch chunks per lane before any of them is written to LDS, so a round costs one trip
        // to HBM/L2.  The 3x3 / 64-channel shape needs a single round.  In the VEC instantiation (channel
        // vectors are whole, aligned 16-byte chunks) the loads are unconditional: out-of-range work items read
        // a clamped, valid address and the result is replaced afterwards, which keeps the round free of
        // branches so that its loads really are in flight together.
        {
            // weight rows: NT/OCB lanes share a row and walk its chunks, so no division is needed
            constexpr int LPR = NT / OCB;
            const int w_ocl   = tid / LPR;
            const int w_part  = tid % LPR;
            const int w_r32   = w_ocl & 31;    // output channel -> row of the MFMA operand (see the header comment)
            const int w_row   = (w_ocl & ~31) + ((w_r32 >> 2) & 3) * 8 + (w_r32 >> 4) * 4 + (w_r32 & 3);
            const bool w_oc_ok = oc0 + w_ocl < g.OC;
            const size_t w_src_row = (size_t)(oc0 + w_ocl) * taps * row_bytes;
            int w_sum = 0;
            const int p_total = a.PH * a.PW * a.CH;
            for (int wj0 = w_part, pbase_idx = tid; wj0 < n_pairs || pbase_idx < p_total;
                 wj0 += LPR * WU, pbase_idx += NT * PU)
            {
                v4i wv[WU], pv[PU];
                int wdst[WU], pdst[PU];
#pragma unroll
                for (int u = 0; u < PU; u++)
                {
                    const int idx  = pbase_idx + u * NT;
                    const bool ok  = idx < p_total;
                    const int idc  = ok ? idx : 0;
                    const int cc   = idc & (a.CH - 1);
                    const int pix  = idc >> ch_shift;
                    const int py   = fdiv(pix, a.div_pw);
                    const int px   = pix - py * a.PW;
                    const int iy = y0 + py, ix = x0 + px;
                    const int off  = ic_off + cc * 16;
                    const bool img = iy >= 0 && iy < g.IH && ix >= 0 && ix < g.IW;
                    pdst[u]        = ok ? pix * a.pstride + cc * 16 : -1;
                    if constexpr (VEC)
                    {
                        const bool ld    = img && off < row_bytes;
                        const size_t src = ld ? (((size_t)n * g.IH + iy) * g.IW + ix) * row_bytes + off : 0;
                        const v4i v      = *reinterpret_cast<const v4i*>(a.in + src);
                        const int fw     = off < row_bytes ? fill_word : 0;    // whole chunks only in this path
                        const v4i f      = v4i{ fw, fw, fw, fw };
                        pv[u]            = ld ? v : (img ? v4i{ 0, 0, 0, 0 } : f);
                    }
                    else
                    {
                        pv[u] = v4i{ 0, 0, 0, 0 };
                        if (ok)
                            pv[u] = img ? load_chunk_bytes(a.in + (((size_t)n * g.IH + iy) * g.IW + ix) * row_bytes,
                                                           off, row_bytes)
                                        : fill_chunk(off, row_bytes, M::is_int ? a.za : 0);
                    }
                }
#pragma unroll
                for (int u = 0; u < WU; u++)
                {
                    const int j   = wj0 + u * LPR;    // (tap, chunk) pair inside the row
                    const bool ok = j < n_pairs;
                    const int jc  = ok ? j : 0;
                    const int off = ic_off + (jc & (a.CH - 1)) * 16;
                    const bool ld = ok && w_oc_ok && off < row_bytes;
                    wdst[u]       = ok ? w_row * a.wstride + j * 16 : -1;
                    const size_t src = w_src_row + (size_t)(jc >> ch_shift) * row_bytes + off;
                    if constexpr (VEC)
                    {
                        const v4i v = *reinterpret_cast<const v4i*>(wbase_ptr + (ld ? src : 0));
                        wv[u]       = ld ? v : v4i{ 0, 0, 0, 0 };
                    }
                    else
                    {
                        wv[u] = v4i{ 0, 0, 0, 0 };
                        if (ld)
                            wv[u] = load_chunk_bytes(wbase_ptr + w_src_row + (size_t)(jc >> ch_shift) * row_bytes, off,
                                                     row_bytes);
                    }
                }
#pragma unroll
                for (int u = 0; u < PU; u++)
                    if (pdst[u] >= 0)
                        *reinterpret_cast<v4i*>(pl + pdst[u]) = pv[u];
#pragma unroll
                for (int u = 0; u < WU; u++)
                    if (wdst[u] >= 0)
                        *reinterpret_cast<v4i*>(wl + wdst[u]) = wv[u];
                // sum(w) of this lane's share of its weight row, taken while the chunks are in registers
                if constexpr (M::is_int)
                    if (a.za != 0)
#pragma unroll
                        for (int u = 0; u < WU; u++)
                            w_sum += dot4_ones(wv[u]);
                staged_w_sum = w_sum;
            }
        }
        __syncthreads();

        // ---- sum(w) per output channel, for the zero-point correction -----------------------------------------
        // The NT/OCB lanes that share a weight row finish its byte sum with a butterfly and -za*sum(w) goes
        // straight into the channel table's bias (one LDS atomic per row, all rows distinct; the table was
        // written before the barrier above).  The K loop stays free of side computations.
        if constexpr (M::is_int)
        {
            if (a.za != 0)
            {
                constexpr int LPR = NT / OCB;    // lanes per row: 8 or 16
                int sum           = staged_w_sum;
#pragma unroll
                for (int m = 1; m < LPR; m <<= 1)
                    sum += __shfl_xor(sum, m);
                if ((tid % LPR) == 0)
                    atomicAdd(&ctab[tid / LPR].bias, -a.za * sum);    // the lanes of row group r staged channel r
            }
        }

        // ---- MFMA over the (tap, chunk) pairs of this channel block -----------------------------------
        if (wave_active)
        {
            // Double buffered in groups of G steps: at the top of a round the fragments of the next group are
            // requested (their patch offsets were read from the table one round earlier), then the current
            // group's MFMAs issue, so the wait in front of an MFMA only meets loads that have had a whole
            // group of matrix instructions to complete.  The main loop runs on whole pairs of groups and has no
            // branch in its body; what is left (fewer than 2G steps) goes through the checked tail.  Loads past
            // the last step are clamped to it and never used.
            constexpr int G     = 3;
            const uint8_t* wrow = wl + (woc * 32 + li) * a.wstride + lh * 16;
            const int* tab      = pairoff + lh;
            const int last_step = a.ksteps - 1;
            v4i fa[2][G], fb[2][G][PXT];
            int po[G];
            auto load_group = [&](int s0, v4i(&ga)[G], v4i(&gb)[G][PXT]) {
#pragma unroll
                for (int u = 0; u < G; u++)
                {
                    const int sc = s0 + u < last_step ? s0 + u : last_step;
                    ga[u]        = *reinterpret_cast<const v4i*>(wrow + sc * 32);
#pragma unroll
                    for (int i = 0; i < PXT; i++)
                        gb[u][i] = *reinterpret_cast<const v4i*>(pl + pbase[i] + po[u]);
                }
#pragma unroll
                for (int u = 0; u < G; u++)
                    po[u] = tab[2 * (s0 + G + u)];    // offsets of the group after that one
            };
            // ZW: the weight zero point is non-zero, so sum(a) per pixel is needed as well; it is accumulated
            // from the pixel fragments here (the upper K half of an odd last step holds no pair)
            auto run = [&](auto zw_tag) {
                constexpr bool ZW = decltype(zw_tag)::value;
                auto compute = [&](int s, const v4i& ga, const v4i(&gb)[PXT]) {
#pragma unroll
                    for (int i = 0; i < PXT; i++)
                        acc[i] = M::mma(ga, gb[i], acc[i]);
                    if constexpr (ZW)
                    {
                        const bool live = 2 * s + lh < n_pairs;
#pragma unroll
                        for (int i = 0; i < PXT; i++)
                            asum[i] += live ? dot4_ones(gb[i]) : 0;
                    }
                };
#pragma unroll
                for (int u = 0; u < G; u++)
                    po[u] = tab[2 * u];
                load_group(0, fa[0], fb[0]);
                int s = 0;
                for (; s + 2 * G <= a.ksteps; s += 2 * G)
                {
                    load_group(s + G, fa[1], fb[1]);
#pragma unroll
                    for (int u = 0; u < G; u++)
                        compute(s + u, fa[0][u], fb[0][u]);
                    load_group(s + 2 * G, fa[0], fb[0]);
#pragma unroll
                    for (int u = 0; u < G; u++)
                        compute(s + G + u, fa[1][u], fb[1][u]);
                }
                if (s < a.ksteps)
                {
                    load_group(s + G, fa[1], fb[1]);
#pragma unroll
                    for (int u = 0; u < G; u++)
                        if (s + u < a.ksteps)
                            compute(s + u, fa[0][u], fb[0][u]);
#pragma unroll
                    for (int u = 0; u < G; u++)
                        if (s + G + u < a.ksteps)
                            compute(s + G + u, fa[1][u], fb[1][u]);
                }
            };
            if (M::is_int && a.zw != 0)
                run(std::true_type{});
            else
                run(std::false_type{});
        }
    }

    // ---- epilogue -------------------------------------------------------------------------------------
    // per pixel tile: validity and output offset of this lane's pixel; the lane owns channels
    // [ocl0, ocl0 + 16) of the block
    bool pix_ok[PXT];
    size_t obase[PXT];
    const int ocl0 = woc * 32 + 16 * lh;
#pragma unroll
    for (int i = 0; i < PXT; i++)
    {
        const int p  = (wpx * PXT + i) * 32 + li;
        const int ty = fdiv(p, a.div_tw);
        const int oy = oy0 + ty, ox = ox0 + (p - ty * a.TW);
        pix_ok[i]    = wave_active && p < P && oy < g.OH && ox < g.OW;
        obase[i]     = (((size_t)n * g.OH + oy) * g.OW + ox) * g.OC + oc0 + ocl0;
    }
    const bool full = (oc0 + ocl0 + 16 <= g.OC);

    if constexpr (!M::is_int)
    {
        // floating point: out = bias + acc, rounded to the output type (16 channels = 32 bytes per pixel), or
        // kept in fp32 (MATMUL: 64 bytes per pixel)
        const bool vec_out = full && (g.OC & 7) == 0 && ((uintptr_t)a.out & 15) == 0;
#pragma unroll
        for (int i = 0; i < PXT; i++)
        {
            if (a.out_dtype == TMI_FP32)
            {
                float* o = reinterpret_cast<float*>(a.out) + obase[i];
#pragma unroll
                for (int q = 0; q < 4; q++)
                {
                    const v4f b = *reinterpret_cast<const v4f*>(ftab + ocl0 + 4 * q);
                    v4f r;
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        r[j] = b[j] + acc[i][4 * q + j];
                    if (!pix_ok[i])
                        continue;
                    if (vec_out)
                        *reinterpret_cast<v4f*>(o + 4 * q) = r;
                    else
#pragma unroll
                        for (int j = 0; j < 4; j++)
                            if (oc0 + ocl0 + 4 * q + j < g.OC)
                                o[4 * q + j] = r[j];
                }
                continue;
            }
            union
            {
                v4i v[2];
                T e[16];
            } u;
#pragma unroll
            for (int q = 0; q < 4; q++)
            {
                const v4f b = *reinterpret_cast<const v4f*>(ftab + ocl0 + 4 * q);
#pragma unroll
                for (int r = 0; r < 4; r++)
                    store_from_float(&u.e[4 * q + r], b[r] + acc[i][4 * q + r]);
            }
            if (!pix_ok[i])
                continue;
            T* o = reinterpret_cast<T*>(a.out) + obase[i];
            if (vec_out)
            {
                reinterpret_cast<v4i*>(o)[0] = u.v[0];
                reinterpret_cast<v4i*>(o)[1] = u.v[1];
            }
            else
            {
#pragma unroll
                for (int j = 0; j < 16; j++)
                    if (oc0 + ocl0 + j < g.OC)
                        o[j] = u.e[j];
            }
        }
    }
    else
    {
        const int kzz = g.KH * g.KW * g.IC * a.za * a.zw;
        int pcorr[PXT];    // the zero-point terms that depend on the pixel only
#pragma unroll
        for (int i = 0; i < PXT; i++)
        {
            int sa = asum[i];
            if (a.zw != 0)
                sa += __shfl_xor(sa, 32);
            pcorr[i] = kzz - a.zw * sa;
        }
        // -za*sum(w) was added to the channel table's bias after staging: make it visible to every wave
        if (a.za != 0)
            __syncthreads();
        // int32 rows of four channels can be stored as one vector; int8 rows of 16 channels likewise
        const bool vec4  = full && (g.OC & 3) == 0 && ((uintptr_t)a.out & 15) == 0;
        const bool vec16 = full && (g.OC & 15) == 0 && ((uintptr_t)a.out & 15) == 0;
        int packed[PXT][4];    // int8 results, four channels per word

        if constexpr (EPI == EPI_GENERIC)
            __syncthreads();    // every wave is done reading the operands: LDS becomes the staging area
        int32_t* stage = reinterpret_cast<int32_t*>(lds + kCtab);    // [pixel of the tile][channel of the block]

        // The common case -- RESCALE to int8, whole aligned 16-channel rows -- as straight-line code: about ten
        // vector instructions per element and no branch; `checked` adds apply_scale_32's value-range test and
        // is only taken when some channel's shift is below 32.
        const bool fast_i8 = EPI == EPI_FAST && a.out_dtype == TMI_INT8 && vec16;
        if constexpr (EPI == EPI_FAST)
        {
            if (fast_i8)
            {
                auto rows = [&](auto checked_tag) {
                    constexpr bool CHECKED = decltype(checked_tag)::value;
#pragma unroll
                    for (int q = 0; q < 4; q++)
                    {
                        ChanEntry ce[4];
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            ce[r] = ctab[ocl0 + 4 * q + r];
#pragma unroll
                        for (int i = 0; i < PXT; i++)
                        {
                            int32_t res[4];
#pragma unroll
                            for (int r = 0; r < 4; r++)
                            {
                                const int32_t v = acc[i][4 * q + r] + pcorr[i] + ce[r].bias;
                                if constexpr (CHECKED)
                                    if ((uint32_t)v + ce[r].lim > 2u * ce[r].lim - 1u && pix_ok[i])
                                        flags |= TMI_FLAG_SCALE_VALUE;    // pixels outside the image raise nothing
                                const int64_t pr = (int64_t)v * (int64_t)ce[r].m + (v >= 0 ? ce[r].rnd_pos : ce[r].rnd_neg);
                                int32_t o        = (int32_t)(pr >> ce[r].s);
                                o                = o < a.rp.lo ? a.rp.lo : o;
                                res[r]           = o > a.rp.hi ? a.rp.hi : o;
                            }
                            packed[i][q] = (res[0] & 0xff) | ((res[1] & 0xff) << 8) | ((res[2] & 0xff) << 16) |
                                           ((res[3] & 0xff) << 24);
                        }
                    }
                };
                if (*need_check)
                    rows(std::true_type{});
                else
                    rows(std::false_type{});
            }
        }

        // every other combination: four channels at a time, constants fetched once and used for every pixel
        if (!fast_i8)
#pragma unroll
        for (int q = 0; q < 4; q++)
        {
            const int c0 = oc0 + ocl0 + 4 * q;
            ChanEntry ce[4];
            int32_t cb[4];    // bias minus za * sum(w)
#pragma unroll
            for (int r = 0; r < 4; r++)
            {
                ce[r] = ctab[ocl0 + 4 * q + r];
                cb[r] = ce[r].bias;
            }
#pragma unroll
            for (int i = 0; i < PXT; i++)
            {
                int32_t res[4];
#pragma unroll
                for (int r = 0; r < 4; r++)
                {
                    int32_t v = acc[i][4 * q + r] + pcorr[i] + cb[r];
                    if constexpr (EPI == EPI_FAST)
                    {
                        if ((uint32_t)v + ce[r].lim > 2u * ce[r].lim - 1u && pix_ok[i])
                            flags |= TMI_FLAG_SCALE_VALUE;    // pixels outside the image raise nothing
                        const int64_t pr = (int64_t)v * (int64_t)ce[r].m + (v >= 0 ? ce[r].rnd_pos : ce[r].rnd_neg);
                        v                = (int32_t)(pr >> ce[r].s);    // output_zp rides in the rounding term
                        v                = v < a.rp.lo ? a.rp.lo : v;
                        v                = v > a.rp.hi ? a.rp.hi : v;
                    }
                    res[r] = v;
                }
                if constexpr (EPI == EPI_GENERIC)
                {
                    const int p = (wpx * PXT + i) * 32 + li;
                    if (wave_active && p < P)
                        *reinterpret_cast<v4i*>(stage + (size_t)p * OCB + ocl0 + 4 * q) =
                            v4i{ res[0], res[1], res[2], res[3] };
                    continue;
                }
                if (!pix_ok[i])
                    continue;
                if (EPI == EPI_PLAIN || a.out_dtype == TMI_INT32)
                {
                    int32_t* o = reinterpret_cast<int32_t*>(a.out) + obase[i] + 4 * q;
                    if (vec4)
                        *reinterpret_cast<v4i*>(o) = v4i{ res[0], res[1], res[2], res[3] };
                    else
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            if (c0 + r < g.OC)
                                o[r] = res[r];
                }
                else if (a.out_dtype == TMI_INT8)
                {
                    if (vec16)
                        packed[i][q] = (res[0] & 0xff) | ((res[1] & 0xff) << 8) | ((res[2] & 0xff) << 16) |
                                       ((res[3] & 0xff) << 24);
                    else
                    {
                        int8_t* o = reinterpret_cast<int8_t*>(a.out) + obase[i] + 4 * q;
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            if (c0 + r < g.OC)
                                o[r] = (int8_t)res[r];
                    }
                }
                else
                {
                    int16_t* o = reinterpret_cast<int16_t*>(a.out) + obase[i] + 4 * q;
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (c0 + r < g.OC)
                            o[r] = (int16_t)res[r];
                }
            }
        }
        if constexpr (EPI == EPI_FAST)
        {
            if (a.out_dtype == TMI_INT8 && vec16)
            {
#pragma unroll
                for (int i = 0; i < PXT; i++)
                    if (pix_ok[i])
                        *reinterpret_cast<v4i*>(reinterpret_cast<int8_t*>(a.out) + obase[i]) =
                            v4i{ packed[i][0], packed[i][1], packed[i][2], packed[i][3] };
            }
        }
        if constexpr (EPI == EPI_GENERIC)
        {
            // the general RESCALE (16-bit scale, inexact rounding, split clip/clamp ranges, ...): every lane
            // takes elements of the staged int32 tile in turn
            __syncthreads();
            const int total = P * OCB;
#pragma nounroll
            for (int idx = tid; idx < total; idx += NT)
            {
                const int p   = idx / OCB;
                const int ocl = idx % OCB;
                const int oc  = oc0 + ocl;
                const int ty  = fdiv(p, a.div_tw);
                const int oy = oy0 + ty, ox = ox0 + (p - ty * a.TW);
                if (oc >= g.OC || oy >= g.OH || ox >= g.OW)
                    continue;
                const int32_t r =
                    rescale_value(a.rp, stage[idx], load_multiplier(a.rp, oc), load_shift(a.rp, oc), flags);
                const size_t o = (((size_t)n * g.OH + oy) * g.OW + ox) * g.OC + oc;
                if (a.out_dtype == TMI_INT8)
                    reinterpret_cast<int8_t*>(a.out)[o] = (int8_t)r;
                else if (a.out_dtype == TMI_INT16)
                    reinterpret_cast<int16_t*>(a.out)[o] = (int16_t)r;
                else
                    reinterpret_cast<int32_t*>(a.out)[o] = r;
            }
        }
        raise_flags(a.flag_word, flags);
    }
}

// ---- host side: tile choice and launch -----------------------------------------------------------------

static constexpr int kMaxLds = 160 * 1024;

template <typename T, int WOC, int PXT, int EPI, bool VEC>
static bool launch_patch(hipStream_t st, PatchArgs& a, size_t lds_bytes, int blocks)
{
    auto kern                = conv2d_patch_kernel<T, WOC, PXT, EPI, VEC>;
    static size_t configured = 0;    // largest dynamic LDS size this instantiation was configured for
    if (lds_bytes > configured)
    {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds_bytes) != hipSuccess)
            return false;
        configured = lds_bytes;
    }
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(512), lds_bytes, st, a);
    return true;
}

template <typename T>
static const char* launch_conv2d_mfma_t(hipStream_t st, const ConvGeom& g, int32_t out_dtype, const void* in,
                                        const void* w, const void* bias, int32_t in_zp, int32_t w_zp,
                                        const RescaleParams& rp, void* out, uint32_t* flag_word, const char* label,
                                        int64_t w_batch_stride)
{
    constexpr int EB    = sizeof(T);
    const int row_bytes = g.IC * EB;
    const int64_t n_px  = (int64_t)g.N * g.OH * g.OW;
    if (row_bytes <= 0 || g.OC <= 0 || n_px == 0)
        return nullptr;

    PatchArgs a{};
    a.g = g, a.in = (const uint8_t*)in, a.w = (const uint8_t*)w, a.bias = bias, a.out = out;
    a.flag_word = flag_word, a.rp = rp, a.za = in_zp, a.zw = w_zp, a.out_dtype = out_dtype;
    a.w_batch_stride = w_batch_stride;
    a.CH           = row_bytes <= 16 ? 1 : (row_bytes <= 32 ? 2 : 4);
    a.pstride      = a.CH == 1 ? 16 : a.CH * 16 + 16;    // 16, 48, 80: all = 16 (mod 32)
    a.n_icb        = (row_bytes + a.CH * 16 - 1) / (a.CH * 16);
    const int taps = g.KH * g.KW;
    const int rch  = taps * a.CH;    // chunks per weight row
    a.wstride      = (rch + (rch & 1)) * 16 + 16;    // room for a spare zero chunk; = 16 (mod 32)
    a.ksteps       = (rch + 1) / 2;

    const int WOC           = g.OC > 32 ? 2 : 1;
    const int OCB           = 32 * WOC;
    const int64_t oc_blocks = (g.OC + OCB - 1) / OCB;

    // channel vectors made of whole, aligned 16-byte chunks take the branch-free staging path
    const bool vec = (row_bytes & 15) == 0 && (((uintptr_t)in | (uintptr_t)w) & 15) == 0;
    // Pixel tiles per wave: two when that still leaves at least two workgroups per CU, else one.
    const int max_px1 = 32 * (8 / WOC);
    const int PXT     = (vec && n_px * oc_blocks >= (int64_t)256 * 2 * 2 * max_px1) ? 2 : 1;
    const int max_px  = max_px1 * PXT;
    // tile: prefer full output rows
    int TW = g.OW < max_px ? g.OW : max_px;
    int TH = max_px / TW;
    if (TH > g.OH)
        TH = g.OH;
    if (TH < 1)
        TH = 1;
    const size_t fixed_bytes = (size_t)OCB * 32 + 32 + ((((size_t)rch + 32) * 4 + 15) & ~(size_t)15);
    const size_t w_bytes     = (size_t)OCB * a.wstride;
    size_t lds_bytes         = 0;
    for (;;)
    {
        a.PH      = (TH - 1) * g.stride_y + (g.KH - 1) * g.dil_y + 1;
        a.PW      = (TW - 1) * g.stride_x + (g.KW - 1) * g.dil_x + 1;
        lds_bytes = fixed_bytes + w_bytes + (size_t)a.PH * a.PW * a.pstride;
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
    const int64_t blocks  = n_tiles * oc_blocks;
    if (blocks > 0x3fffffff || (int64_t)a.PH * a.PW * a.CH > (1 << 20))
        return nullptr;
    a.n_tiles     = (int)n_tiles;
    a.xcd_remap   = (blocks % 8) == 0 && blocks >= 16;
    a.div_tw      = make_fastdiv(TW);
    a.div_pw      = make_fastdiv(a.PW);
    a.div_rch     = make_fastdiv(rch);
    a.div_tiles_x = make_fastdiv(a.tiles_x);
    a.div_tiles_y = make_fastdiv(a.tiles_y);
    a.div_n_tiles = make_fastdiv(a.n_tiles);
    a.div_kw      = make_fastdiv(g.KW);
    // fdiv is exact for n*d < 2^32: every dividend but the block index is bounded by the LDS capacity;
    // guard the products that involve the block index
    if ((uint64_t)blocks * (uint64_t)a.n_tiles >= (uint64_t(1) << 32) ||
        (uint64_t)n_tiles * (uint64_t)a.tiles_x >= (uint64_t(1) << 32) ||
        (uint64_t)(n_tiles / a.tiles_x + 1) * (uint64_t)a.tiles_y >= (uint64_t(1) << 32))
        return nullptr;

    const int epi = !rp.enabled ? EPI_PLAIN : (rp.fast ? EPI_FAST : EPI_GENERIC);
    if (epi == EPI_GENERIC)
    {
        // the int32 tile is staged in LDS (behind the channel table) before the general RESCALE
        const size_t stage_bytes = (size_t)OCB * 32 + (size_t)TH * TW * OCB * 4;
        if (stage_bytes > lds_bytes)
            lds_bytes = stage_bytes;
        if (lds_bytes > (size_t)kMaxLds)
            return nullptr;
    }
    bool ok = false;
#define TMI_PATCH_CASE(O, P, E)                                                                                      \
    if (WOC == O && PXT == P && epi == E)                                                                            \
        ok = launch_patch<T, O, P, E, true>(st, a, lds_bytes, (int)blocks);
#define TMI_PATCH_CASE_BYTES(O, E)                                                                                   \
    if (WOC == O && epi == E)                                                                                        \
        ok = launch_patch<T, O, 1, E, false>(st, a, lds_bytes, (int)blocks);
    if (vec)
    {
        TMI_PATCH_CASE(1, 1, EPI_PLAIN)
        TMI_PATCH_CASE(1, 2, EPI_PLAIN)
        TMI_PATCH_CASE(2, 1, EPI_PLAIN)
        TMI_PATCH_CASE(2, 2, EPI_PLAIN)
        if constexpr (Mma<T>::is_int)
        {
            TMI_PATCH_CASE(1, 1, EPI_FAST)
            TMI_PATCH_CASE(1, 2, EPI_FAST)
            TMI_PATCH_CASE(2, 1, EPI_FAST)
            TMI_PATCH_CASE(2, 2, EPI_FAST)
            TMI_PATCH_CASE(1, 1, EPI_GENERIC)
            TMI_PATCH_CASE(1, 2, EPI_GENERIC)
            TMI_PATCH_CASE(2, 1, EPI_GENERIC)
            TMI_PATCH_CASE(2, 2, EPI_GENERIC)
        }
    }
    else
    {
        TMI_PATCH_CASE_BYTES(1, EPI_PLAIN)
        TMI_PATCH_CASE_BYTES(2, EPI_PLAIN)
        if constexpr (Mma<T>::is_int)
        {
            TMI_PATCH_CASE_BYTES(1, EPI_FAST)
            TMI_PATCH_CASE_BYTES(2, EPI_FAST)
            TMI_PATCH_CASE_BYTES(1, EPI_GENERIC)
            TMI_PATCH_CASE_BYTES(2, EPI_GENERIC)
        }
    }
#undef TMI_PATCH_CASE_BYTES
#undef TMI_PATCH_CASE
    return ok ? label : nullptr;
}

const char* launch_conv2d_mfma(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                               const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                               void* out, uint32_t* flag_word, int64_t w_batch_stride)
{
    if (in_dtype == TMI_INT8)
        return launch_conv2d_mfma_t<int8_t>(st, g, out_dtype, in, w, bias, in_zp, w_zp, rp, out, flag_word,
                                            rp.enabled ? "conv2d_mfma_i8_rescale" : "conv2d_mfma_i8", w_batch_stride);
    if (in_dtype == TMI_FP16 && (out_dtype == TMI_FP16 || out_dtype == TMI_FP32))
        return launch_conv2d_mfma_t<_Float16>(st, g, out_dtype, in, w, bias, 0, 0, rp, out, flag_word,
                                              "conv2d_mfma_f16", w_batch_stride);
    if (in_dtype == TMI_BF16 && (out_dtype == TMI_BF16 || out_dtype == TMI_FP32))
        return launch_conv2d_mfma_t<bf16_t>(st, g, out_dtype, in, w, bias, 0, 0, rp, out, flag_word,
                                            "conv2d_mfma_bf16", w_batch_stride);
    return nullptr;
}

}    // namespace tmi
