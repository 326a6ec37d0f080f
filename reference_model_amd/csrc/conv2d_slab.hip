// CONV2D for layers whose channel vector is 64, 96 or 128 bytes (int8 with IC = 64, 96 or 128), 3x3 or 1x1 taps: the small,
// latency-bound layers of a ResNet stem, where a launch does well under a microsecond of matrix work and everything else is
// overhead.  The kernel is the shortest path from memory to the matrix cores this chip offers:
//
//   - A workgroup (8 waves) owns a TH x TW tile of output pixels of one image and a block of 64 output channels.
//     It needs the weight slab of the block (64 rows x taps x 64 bytes) and the input patch of the tile with its
//     halo (PH x PW pixels x 64 bytes).  Both go from global memory straight into LDS with
//     global_load_lds_dwordx4 (64 lanes x 16 bytes to 1 KB of LDS per instruction): no staging registers, no LDS
//     stores, and only address arithmetic on the vector ALU.  Seven waves issue about seven loads each.
//   - An LDS destination is fixed (M0 + 16 * lane) but every lane names its own source, so the layout is chosen
//     by the mapping slot -> source: weight rows take taps*CH + 1 chunks and patch pixels CH + 1, the odd chunk being
//     padding, and a patch row gets up to 15 more chunks of padding.  The 16 lanes that a ds_read_b128 serves
//     together then read 16 different bank groups, for the weight fragments and (odd strides) the pixel fragments.
//   - A pixel outside the image reads a 64-byte page of input_zp bytes, so it contributes
//     (zp - zp) * w = 0 like the reference's skipped tap (tensor_ops.cpp:845-852), and the zero-point identity
//     sum((a - za) w) = sum(a w) - za * sum(w) holds with the full K.  za * sum(w) per channel costs nothing: a
//     wave's 32 MFMA columns are 31 pixels and one "zero-point pixel" (input_zp bytes in LDS wherever a tap can
//     read), whose accumulators are those terms, already in the register order of the lanes that need them.
//     The accumulators of the 31 pixels start at the bias, those of the zero-point column at zero.
//   - While the loads are in flight the eighth wave, which issues none, turns bias / multiplier / shift into
//     the per-channel constants of the RESCALE in LDS.
//   - One barrier, then 18 MFMA steps per wave (one accumulator tile of 32 channels x 32 columns), then the fused
//     RESCALE (+ CLAMP) epilogue of the patch kernel: a lane owns 16 consecutive channels of a pixel and stores
//     them as 16 bytes (int8), 32 (int16) or 64 (int32).
//
// weight_zp must be 0 (the usual case for int8 weights); the patch kernel takes everything else.
#include <cstring>
#include <type_traits>

#include "tmi_mfma.h"

namespace tmi
{

struct SlabArgs
{
    const uint8_t* in;
    const uint8_t* w;
    const int32_t* bias;
    const uint8_t* pad_page;    // 64 bytes of input_zp
    void* out;
    uint32_t* flag_word;
    RescaleParams rp;
    int32_t N, IH, IW, OC, OH, OW;
    int32_t sy, sx, dy, dx, pad_top, pad_left;
    int32_t TH, TW, PH, PW, tiles_x, tiles_y;
    int32_t bias_len, za;
    int32_t n_ocb;
    int32_t out_kind;    // 0: int32 accumulators, 1: int8 through the RESCALE, 2: int16 through the RESCALE
    int32_t xcd_remap;    // 0, or grid / 8: workgroup b takes tile (b % 8) * (grid / 8) + b / 8
    int32_t pitch;               // 16-byte chunks per patch row in LDS: 5 per pixel plus the padding that spreads the banks
    int32_t step_row, step_chunk;    // 448 = step_row * pitch + step_chunk: how far 7 loads (448 slots) move
    FastDiv div_tw, div_pitch, div_tiles_x, div_tiles_y, div_ocb;
    // TRANSPOSE_CONV2D: IH x IW above are those of the input with up_y - 1 (up_x - 1) holes between its rows (columns),
    // which is never materialised; the tensor in memory is IHr x IWr
    int32_t up_y, up_x, IHr, IWr;
    FastDiv div_up_y, div_up_x;
    // CONV3D: image n above is output slice (n / OD, n % OD); chunk group kd of a pixel comes from input slice
    // od * sd + kd * dd - pd0 of a volume of ID slices
    int32_t ID, OD, sd, dd, pd0;
    FastDiv div_od;
};

__device__ __forceinline__ void slab_load(const void* src, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_addr) : "memory");
}

// the same with a 64-bit scalar base and a 32-bit per-lane byte offset: no 64-bit vector arithmetic per load
__device__ __forceinline__ void slab_load_off(uint32_t off, const void* base, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(lds_addr)
                 : "memory");
}

// A workgroup barrier that waits for this wave's LDS accesses and nothing else: loads into LDS that are still in flight
// (counted by vmcnt) stay in flight across it.
__device__ __forceinline__ void slab_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// CH: 16-byte chunks of a channel vector (4, 6, 8: 64, 96, 128 input channels)
// TC: TRANSPOSE_CONV2D (tensor_ops.cpp:2138-2187) as the stride-1 CONV2D with flipped taps over the input with holes:
// a hole reads the page of input_zp bytes like a pixel outside the image (it contributes (zp - zp) * w = 0, as the
// reference's skipped tap does), and the flip is applied where a K step picks its place in the patch, so neither
// operand is copied.
// KD > 1: CONV3D (tensor_ops.cpp:1058-1108) with the KD depth taps as channel groups of a CONV2D over the output
// slices: the patch loader takes chunk group kd of a pixel from input slice od * sd + kd * dd - pd0 (a slice outside
// the volume reads the input_zp page), and the weights stay in their own [OC][KD][KH][KW][IC] order, a K step
// (tap, kd, half) finding its place in the row at compile time.  Neither operand is copied.
// NPT: accumulator tiles (of 32 columns) per wave.  Two of them share every weight fragment, which cuts the LDS
// traffic of the K loop by a quarter; the workgroup's tile is then up to 252 pixels, which only pays when the layer
// has more tiles than the chip has CUs.
// T: int8_t, or _Float16 / bf16_t: the same loads and LDS layout on channel vectors of CH * 8 values, fp32 accumulators that
// start at the bias, results rounded to T (tensor_ops.cpp:828-882 with fp32 accumulation); no zero points, no RESCALE.
template <int KH, int KW, int CH, bool ZA, bool FUSED, bool TC = false, int KD = 1, int NPT = 1, typename T = int8_t>
__global__ __launch_bounds__(512) void conv2d_slab_kernel(SlabArgs a)
{
    static_assert(Mma<T>::is_int || (!ZA && !FUSED && !TC && KD == 1), "floating point: plain CONV2D only");
    // one field of every cache line of the arguments up front: a single scalar-cache round trip
    // every scalar argument the kernel reads, named once so that they are fetched together at the top (fields
    // first needed later are otherwise loaded one at a time, each with its own wait)
    asm volatile("" ::"s"(a.in), "s"(a.rp.shift), "s"(a.rp.out_zp), "s"(*reinterpret_cast<const uint32_t*>(&a.rp.scale32)),
                 "s"(*reinterpret_cast<const uint32_t*>(&a.rp.in_bits)), "s"(a.rp.lo), "s"(a.N), "s"(a.TH), "s"(a.bias_len),
                 "s"(a.div_ocb.d));
    constexpr int TAPS   = KH * KW;
    constexpr int RW     = TAPS * CH + 1;    // chunks per weight row in LDS (odd)
    constexpr int KB     = CH * 16;          // bytes of a channel vector
    constexpr int WSLOTS = 64 * RW;
    constexpr int WLOADS = (WSLOTS + 63) / 64;
    constexpr int RP     = CH + 1;          // chunks per patch pixel in LDS (odd)
    constexpr int LWAVES = 7;               // waves that issue loads; the eighth builds the tables
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // LDS: [weight rows][patch][zero-point pixel][64 x ChannelScale][64 x HighWordScale][64 multipliers][64 biases, 16 zeros][the block's common shift]
    const int tid    = threadIdx.x;
    const int lane   = tid & 63;
    const int wave   = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li     = lane & 31;
    const int lh     = lane >> 5;
    const int p_slots = a.PH * a.pitch;
    const int p_loads = (p_slots + 63) >> 6;
    uint8_t* wl       = lds;
    uint8_t* pl       = lds + WLOADS * 1024;
    // fragment offsets of the taps inside the patch, and the zero-point pixel: input_zp bytes wherever a tap can read
    const int row_step   = a.dy * a.pitch * 16;
    const int col_step   = a.dx * RP * 16;
    const int ones_bytes = ZA ? ((KH - 1) * row_step + (KW - 1) * col_step + KB) : 0;
    uint8_t* ones        = pl + p_loads * 1024;
    uint8_t* tabs        = ones + ones_bytes;
    ChannelScale* tab_cs = reinterpret_cast<ChannelScale*>(tabs);
    HighWordScale* tab_hw = reinterpret_cast<HighWordScale*>(tabs + 64 * sizeof(ChannelScale));
    int32_t* tab_m       = reinterpret_cast<int32_t*>(tab_hw + 64);                         // multipliers
    int32_t* tab_b       = tab_m + 64;                                                      // biases, then 16 zeros
    int32_t* uni_shift   = tab_b + 80;                                                      // 4 words, one used

    uint32_t bid = blockIdx.x;
    if (a.xcd_remap)
    {
        // consecutive workgroups go to the 8 XCDs in turn: give each XCD a contiguous run of tiles, whose halos
        // then meet in one L2
        const uint32_t per = (uint32_t)a.xcd_remap;    // an eighth of the grid: no hidden-argument load for gridDim
        bid                = (bid & 7) * per + (bid >> 3);
    }
    const uint32_t tile = fdiv(bid, a.div_ocb);
    const int ocb       = bid - tile * a.n_ocb;
    const uint32_t trow = fdiv(tile, a.div_tiles_x);
    const int txi       = tile - trow * a.tiles_x;
    const int n         = fdiv(trow, a.div_tiles_y);
    const int tyi       = trow - n * a.tiles_y;
    const int oy0 = tyi * a.TH, ox0 = txi * a.TW;
    const int oc0 = ocb * 64;
    const int y0 = oy0 * a.sy - a.pad_top, x0 = ox0 * a.sx - a.pad_left;

    uint32_t flags = 0;
    if (wave < LWAVES)
    {
        // Load l fills LDS bytes [1024 l, 1024 l + 1024); wave v issues l = v, v + 7, ...  The per-lane source is
        // worked out once with divisions and then walked: 7 loads on are 448 slots, i.e. 12 weight rows and 4 chunks,
        // or step_row patch rows and step_chunk chunks.  (Integer multiplies and divides run at a quarter of the
        // vector rate; with them in the loop, issuing the loads took three times as long as the loads themselves.)
        const uint32_t lbase = (uint32_t)(uintptr_t)lds;
        {
            // Weights: LDS row r is channel r of the block, so slot s = (row, chunk) reads byte 16 (s - row) of the
            // block's weights and the walk is two additions; the spare chunk of a row reads the next row's first
            // chunk, and whatever lies past the block's last channel (a ragged last block, the last spare chunk)
            // is clamped to its last chunk: valid memory whose results are never stored.
            const int s0         = wave * 64 + lane;
            const int row0       = s0 / RW;
            int ch               = s0 - row0 * RW;
            uint32_t off         = 16u * (uint32_t)(s0 - row0);
            const int rows       = a.OC - oc0 < 64 ? a.OC - oc0 : 64;
            const uint32_t limit = (uint32_t)rows * (TAPS * KB) - 16u;
            const uint8_t* wb    = a.w + (size_t)oc0 * (TAPS * KB);
            uint32_t dst         = lbase + wave * 1024;
            for (int l = wave; l < WLOADS; l += LWAVES)
            {
                slab_load_off(off < limit ? off : limit, wb, dst);
                dst += LWAVES * 1024;
                off += 16u * (LWAVES * 64 - (LWAVES * 64) / RW);
                ch += (LWAVES * 64) % RW;
                if (ch >= RW)
                    ch -= RW, off -= 16u;
            }
        }
        {
            const uint8_t* in_n = a.in + (size_t)n * (TC ? a.IHr * a.IWr : a.IH * a.IW) * KB;
            constexpr int ICC   = CH / KD;    // chunks of a channel vector in memory
            const int nb        = KD > 1 ? (int)fdiv(n, a.div_od) : 0;
            const int slice0    = nb * a.ID;                              // first slice of the volume
            const int z0        = (n - nb * a.OD) * a.sd - a.pd0;         // slice under depth tap 0
            int lp              = wave + ((WLOADS - wave + LWAVES - 1) / LWAVES) * LWAVES - WLOADS;    // first patch load of this wave
            const int s0        = lp * 64 + lane;
            int py              = fdiv(s0, a.div_pitch);    // patch row and chunk inside the row
            int r               = s0 - py * a.pitch;
            uint32_t dst        = lbase + (WLOADS + lp) * 1024;
            for (; lp < p_loads; lp += LWAVES)
            {
                const int px   = (int)((uint32_t)r / (uint32_t)RP);
                const int ch   = r - px * RP;
                const int iy = y0 + py, ix = x0 + px;
                bool img       = py < a.PH && px < a.PW && (unsigned)iy < (unsigned)a.IH && (unsigned)ix < (unsigned)a.IW;
                const int c16  = (ch < CH ? ch : 0) * 16;
                uint32_t pixel = __umul24(iy, a.IW) + ix;
                if constexpr (TC)
                {
                    const int ry = fdiv(img ? iy : 0, a.div_up_y), rx = fdiv(img ? ix : 0, a.div_up_x);
                    img          = img && ry * a.up_y == iy && rx * a.up_x == ix;
                    pixel        = __umul24(ry, a.IWr) + rx;
                }
                const uint8_t* src = img ? in_n + (uint32_t)(pixel * KB + c16) : a.pad_page + (c16 & 48);
                if constexpr (KD > 1)
                {
                    const int chc = ch < CH ? ch : 0;
                    const int kd  = chc / ICC, cc = chc - kd * ICC;
                    const int z   = z0 + kd * a.dd;
                    img           = img && (unsigned)z < (unsigned)a.ID;
                    src           = img ? a.in + (((uint32_t)(slice0 + z) * (uint32_t)(a.IH * a.IW) + pixel) * (ICC * 16) + cc * 16)
                                        : a.pad_page + (c16 & 48);
                }
                slab_load(src, dst);
                dst += LWAVES * 1024;
                r += a.step_chunk, py += a.step_row;
                if (r >= a.pitch)
                    r -= a.pitch, py++;
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    else
    {
        // the table wave: bias and the per-channel RESCALE constants, one channel per lane
        const int oc    = oc0 + lane;
        const bool ok   = oc < a.OC;
        const int occ   = ok ? oc : 0;
        int32_t b;    // the accumulator's start value: an int32, or the bits of a float
        if constexpr (Mma<T>::is_int)
            b = a.bias[a.bias_len == 1 ? 0 : occ];
        else
            b = __float_as_int(load_as_float<T>(a.bias, a.bias_len == 1 ? 0 : occ));
        int32_t m       = 0;
        if constexpr (FUSED)
        {
            const int32_t m_raw   = load_multiplier(a.rp, occ);
            const int32_t s_raw   = load_shift(a.rp, occ);
            // channels past OC take the first channel's shift, so that they do not break a block whose channels
            // all share one
            const int32_t s_first = __builtin_amdgcn_readfirstlane(s_raw);
            const ChannelScale cs = make_channel_scale(ok ? m_raw : 0, ok ? s_raw : s_first, a.rp.double_round != 0, flags);
            m                     = cs.m;
            // The epilogue has three forms:
            //   every shift large enough for the high-word form (tmi_device.h) and small enough for output_zp * 2^shift
            //   to ride in the 64-bit rounding term: 16 bytes of constants per channel, no value-range test (-2);
            //   the same with one shift for the whole block: the rounding term and the shift are scalars and a channel
            //   needs its multiplier only (the shift itself);
            //   anything else: fast_rescale() with its range test and a 64-bit shift (-1).
            const int s_min = a.rp.double_round ? 33 : 32;
            const int folds = __all(cs.s >= s_min && cs.s <= zp_fold_max_shift(a.rp.out_zp));
            const int uni   = folds && __all(cs.s == s_first);
            tab_cs[lane]    = cs;
            tab_hw[lane]    = make_high_word_scale(cs, a.rp.out_zp);
            // With double rounding, a value below zero takes a rounding term 2^31 smaller; when the result is clamped at
            // or above output_zp anyway, a negative value ends at the lower limit with either term (the scaled value is at
            // most 0 for a multiplier >= 0), so that form skips the sign test (bit 8).
            const int relu = a.rp.double_round && a.rp.lo >= a.rp.out_zp && __all(cs.m >= 0);
            if (lane == 0)
                *uni_shift = uni ? (s_first | (relu << 8)) : (folds ? (relu ? -3 : -2) : -1);
        }
        tab_m[lane] = m;
        tab_b[lane] = ok ? b : 0;
        if (lane < 16)
            tab_b[64 + lane] = 0;
        const int za4 = (a.za & 0xff) * 0x01010101;
        for (int i = lane * 16; i < ones_bytes; i += 1024)
            *reinterpret_cast<v4i*>(ones + i) = v4i{ za4, za4, za4, za4 };
    }
    __syncthreads();

    // ---- MFMA: wave = (channel tile, pixel tile) ---------------------------------------------------------------
    const int oct = wave >> 2, pxt = wave & 3;
    // A wave's first 32 MFMA columns are 31 pixels and, in column 31, the zero-point pixel: its accumulators are
    // input_zp * sum(w) of the wave's 32 channels, for the price of nothing (the column would be computed anyway).
    // A second accumulator tile (NPT = 2) holds 32 more pixels.
    constexpr int PXW  = 31;
    constexpr int WPIX = PXW + 32 * (NPT - 1);    // pixels of a wave
    const int P        = a.TH * a.TW;
    bool p_in_tile[NPT];
    int ty[NPT], tx[NPT];
#pragma unroll
    for (int k = 0; k < NPT; k++)
    {
        int p        = pxt * WPIX + (k ? PXW + 32 * (k - 1) : 0) + li;
        p_in_tile[k] = (k || li < PXW) && p < P;
        p            = p_in_tile[k] ? p : 0;
        ty[k]        = fdiv(p, a.div_tw);
        tx[k]        = p - ty[k] * a.TW;
    }
    // The accumulators start at the bias of the lane's 16 channels (the zero-point column at zero).
    const int ocl = oct * 32 + 16 * lh;    // first of the lane's 16 channels inside the block
    typename Mma<T>::acc_t acc[NPT];
#pragma unroll
    for (int k = 0; k < NPT; k++)
    {
        const int32_t* b16 = tab_b + ((ZA && k == 0 && li == PXW) ? 64 : ocl);
#pragma unroll
        for (int q = 0; q < 4; q++)
        {
            const v4i b4 = *reinterpret_cast<const v4i*>(b16 + 4 * q);
#pragma unroll
            for (int j = 0; j < 4; j++)
            {
                if constexpr (Mma<T>::is_int)
                    acc[k][4 * q + j] = b4[j];
                else
                    acc[k][4 * q + j] = __int_as_float(b4[j]);
            }
        }
    }
    const bool wave_active = pxt * WPIX < P;                     // wave-uniform
    const bool second_active = NPT > 1 && pxt * WPIX + PXW < P;  // wave-uniform: the second tile has a pixel
    if (wave_active)
    {
        // MFMA operand row li holds channel 16*((li>>2)&1) + 4*(li>>3) + (li&3) of the wave's 32: a lane's 16
        // accumulators are then 16 consecutive channels.  (The 16 lanes a ds_read_b128 serves together still read
        // rows that differ modulo 16, which the odd row stride turns into 16 different bank groups.)
        const int wr        = 4 * (li & 4) + ((li >> 1) & 12) + (li & 3);
        const uint8_t* wrow = wl + ((oct * 32 + wr) * RW) * 16 + lh * 16;
        const uint8_t* prow[NPT];
#pragma unroll
        for (int k = 0; k < NPT; k++)
            prow[k] = pl + (ty[k] * a.sy * a.pitch + tx[k] * a.sx * RP) * 16 + lh * 16;
        if (ZA && li == PXW)
            prow[0] = ones + lh * 16;
        // K step s = (tap s / (CH/2), half s % (CH/2)).  The fragments of step s + DEPTH are requested before the
        // MFMA of step s and the order is pinned: an LDS read takes several MFMA times to come back with eight waves
        // asking, and left alone the scheduler requests a step's fragments only one MFMA ahead.
        constexpr int STEPS = TAPS * (CH / 2);
        constexpr int AHEAD = NPT > 1 ? 5 : 8;    // two tiles: fewer steps ahead, to stay within 128 registers
        constexpr int DEPTH = STEPS < AHEAD ? STEPS : AHEAD;
        v4i fa[STEPS], fb[NPT][STEPS];
        auto request = [&](int s) {
            const int tap = s / (CH / 2), h = s % (CH / 2);
            const int at  = TC ? TAPS - 1 - tap : tap;    // flipped taps: weight tap (ky, kx) meets patch tap (KH-1-ky, KW-1-kx)
            int aoff      = s * 32;
            if constexpr (KD > 1)
            {
                constexpr int ICH = CH / KD / 2;    // 32-byte pieces of a channel vector in memory
                aoff              = (((h / ICH) * TAPS + tap) * ICH + h % ICH) * 32;
            }
            fa[s] = *reinterpret_cast<const v4i*>(wrow + aoff);
#pragma unroll
            for (int k = 0; k < NPT; k++)
                fb[k][s] = *reinterpret_cast<const v4i*>(prow[k] + (at / KW) * row_step + (at % KW) * col_step + h * 32);
        };
#pragma unroll
        for (int s = 0; s < DEPTH; s++)
            request(s);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < STEPS; s++)
        {
            if (s + DEPTH < STEPS)
                request(s + DEPTH);
#pragma unroll
            for (int k = 0; k < NPT; k++)
                acc[k] = Mma<T>::mma(fa[s], fb[k][s], acc[k]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- epilogue ----------------------------------------------------------------------------------------------
    // (lane, register 4q + j) = D[row 8q + 4 lh + j][pixel li] = channel 32 oct + 16 lh + 4q + j
    if constexpr (ZA)
    {
        // Lane 31 + 32 lh of the first tile holds in register e the zero-point column for channel 16 lh + e:
        // input_zp * sum(w) of exactly the channel this lane has in register e (of either tile).
        const int src = (PXW + 32 * lh) * 4;
#pragma unroll
        for (int e = 0; e < 16; e++)
        {
            const int zsum = __builtin_amdgcn_ds_bpermute(src, acc[0][e]);
#pragma unroll
            for (int k = 0; k < NPT; k++)
                acc[k][e] -= zsum;
        }
    }
    const bool chan_ok = oc0 + ocl < a.OC;    // OC is a multiple of 16: a lane's 16 channels are in or out together
#pragma unroll
    for (int k = 0; k < NPT; k++)
    {
    if (k > 0 && !second_active)
        break;
    const auto& acck = acc[k];
    const int oy = oy0 + ty[k], ox = ox0 + tx[k];
    const bool pix_ok  = p_in_tile[k] && wave_active && oy < a.OH && ox < a.OW;
    // the tensor has fewer than 2^31 elements (checked by the launcher): 32-bit arithmetic, scalar where it can be
    const size_t obase = (uint32_t)(((n * a.OH + oy) * a.OW + ox) * a.OC + oc0 + ocl);
    if constexpr (!Mma<T>::is_int)
    {
        // 16 consecutive channels of one pixel, rounded to the tensor's type: 32 bytes
        if (pix_ok && chan_ok)
        {
            union
            {
                T e[16];
                v4i q[2];
            } u;
#pragma unroll
            for (int e = 0; e < 16; e++)
                store_from_float(&u.e[e], acck[e]);
            v4i* o = reinterpret_cast<v4i*>(reinterpret_cast<T*>(a.out) + obase);
            o[0] = u.q[0], o[1] = u.q[1];
        }
    }
    else if constexpr (!FUSED)
    {
        if (pix_ok && chan_ok)
        {
            int32_t* o = reinterpret_cast<int32_t*>(a.out) + obase;
#pragma unroll
            for (int q = 0; q < 4; q++)
                *reinterpret_cast<v4i*>(o + 4 * q) = v4i{ acck[4 * q], acck[4 * q + 1], acck[4 * q + 2], acck[4 * q + 3] };
        }
    }
    else
    {
        int32_t r[16];
        const int form  = __builtin_amdgcn_readfirstlane(*uni_shift);
        const int s_uni = form >= 0 ? (form & 255) : form;
        const int relu  = form >= 0 ? (form >> 8) : (form == -3);    // (-3: the per-channel high-word form without the sign test)
        if (s_uni >= 0)
        {
            // one shift for every channel: the high-word form with its constants in scalar registers
            const int64_t rnd = (int64_t(1) << (s_uni - 1)) + (a.rp.double_round ? (int64_t(1) << 30) : 0) +
                                ((int64_t)a.rp.out_zp << s_uni);
            const int32_t hi_p  = (int32_t)(rnd >> 32);
            const uint32_t lo_p = (uint32_t)rnd;
            const int sh        = s_uni - 32;
            int32_t cm[16];    // multipliers of the lane's channels
#pragma unroll
            for (int q = 0; q < 4; q++)
            {
                const v4i m4 = *reinterpret_cast<const v4i*>(tab_m + ocl + 4 * q);
                cm[4 * q] = m4[0], cm[4 * q + 1] = m4[1], cm[4 * q + 2] = m4[2], cm[4 * q + 3] = m4[3];
            }
            if (a.rp.double_round && !relu)
            {
#pragma unroll
                for (int e = 0; e < 16; e++)
                    r[e] = clamp_med3(high_word_rescale<true>(acck[e], cm[e], hi_p, lo_p, sh), a.rp.lo, a.rp.hi);
            }
            else
            {
#pragma unroll
                for (int e = 0; e < 16; e++)
                    r[e] = clamp_med3(high_word_rescale<false>(acck[e], cm[e], hi_p, lo_p, sh), a.rp.lo, a.rp.hi);
            }
        }
        else if (s_uni <= -2)
        {
            if (a.rp.double_round && !relu)
            {
#pragma unroll
                for (int e = 0; e < 16; e++)
                {
                    const HighWordScale c = tab_hw[ocl + e];
                    r[e] = clamp_med3(high_word_rescale<true>(acck[e], c.m, c.hi, c.lo, c.sh), a.rp.lo, a.rp.hi);
                }
            }
            else
            {
#pragma unroll
                for (int e = 0; e < 16; e++)
                {
                    const HighWordScale c = tab_hw[ocl + e];
                    r[e] = clamp_med3(high_word_rescale<false>(acck[e], c.m, c.hi, c.lo, c.sh), a.rp.lo, a.rp.hi);
                }
            }
        }
        else
        {
            uint32_t eflags = 0;
#pragma unroll
            for (int e = 0; e < 16; e++)
            {
                const ChannelScale cs = tab_cs[ocl + e];
                r[e]                  = fast_rescale(acck[e], cs, a.rp.out_zp, a.rp.lo, a.rp.hi, eflags);
            }
            if (pix_ok && chan_ok)
                flags |= eflags;    // pixels and channels outside the tensor raise nothing
        }
        if (pix_ok && chan_ok)
        {
            if (a.out_kind == 1)
            {
                v4i pk;
#pragma unroll
                for (int q = 0; q < 4; q++)
                {
                    // the low bytes of four clamped values into one word
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

// 3x3 layers with 64 input channels, unit stride and a fused RESCALE (the headline layer and its larger batches): tiles of
// up to several hundred pixels, and the weights in registers.  A wave owns one of the block's two channel tiles of 32
// for the whole workgroup, so after the barrier it reads its 18 weight fragments (72 registers) from LDS once and then
// walks the tile's pixel tiles of 32 (wave w: channel tile w % 2, pixel tiles w / 2, w / 2 + 4, ...).  A K step is one
// fragment read and one matrix instruction (the kernel above reads 2.5 fragments per matrix instruction with one
// accumulator tile per wave and 1.5 with two) and a workgroup loads the weight slab once for all its pixels.
// input_zp * sum(w) comes from the weight registers (dot products with a word of ones, once per wave), so all 32
// columns of a pixel tile are pixels, and a tile starts from bias - input_zp * sum(w) as the third operand of its first
// matrix instruction.  What bounds a workgroup once its operands have landed is the rate at which a wave issues
// instructions (two waves per SIMD: about one instruction per eight clocks each), so the loop is written to issue as
// few as it can: with one shift for all channels the requantisation of a pixel tile is dealt over the K steps of the
// wave's next one, four instructions per output element, and the fragments of the next tile are requested in the last
// steps of the current one.
template <bool ZA, bool VL>
__global__ __launch_bounds__(512) void conv2d_slab_wreg_kernel(SlabArgs a)
{
    constexpr int KH = 3, KW = 3, CH = 4;    // 3x3 taps of 64 input channels: 18 weight fragments, 72 registers
    constexpr int NW = 8;
    asm volatile("" ::"s"(a.in), "s"(a.rp.shift), "s"(a.rp.out_zp), "s"(*reinterpret_cast<const uint32_t*>(&a.rp.scale32)),
                 "s"(*reinterpret_cast<const uint32_t*>(&a.rp.in_bits)), "s"(a.rp.lo), "s"(a.N), "s"(a.TH), "s"(a.bias_len),
                 "s"(a.div_ocb.d));
    constexpr int TAPS   = KH * KW;
    constexpr int RW     = TAPS * CH + 1;    // chunks per weight row in LDS (odd)
    constexpr int KB     = CH * 16;          // bytes of a channel vector
    constexpr int WSLOTS = 64 * RW;
    constexpr int WLOADS = (WSLOTS + 63) / 64;
    constexpr int RP     = CH + 1;          // chunks per patch pixel in LDS (odd)
    constexpr int LWAVES = NW - 1;          // waves that issue loads; the eighth builds the tables
    constexpr int STEPS  = TAPS * (CH / 2);
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // LDS: [weight rows][patch][64 x ChannelScale][64 x HighWordScale][64 multipliers][64 biases][the block's common shift]
    //      [8 waves x 32 start values]
    const int tid    = threadIdx.x;
    const int lane   = tid & 63;
    const int wave   = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li     = lane & 31;
    const int lh     = lane >> 5;
    const int p_slots = a.PH * a.pitch;
    const int p_loads = (p_slots + 63) >> 6;
    uint8_t* wl       = lds;
    uint8_t* pl       = lds + WLOADS * 1024;
    const int row_step   = a.dy * a.pitch * 16;
    const int col_step   = a.dx * RP * 16;
    uint8_t* tabs        = pl + p_loads * 1024;
    ChannelScale* tab_cs = reinterpret_cast<ChannelScale*>(tabs);
    HighWordScale* tab_hw = reinterpret_cast<HighWordScale*>(tabs + 64 * sizeof(ChannelScale));
    int32_t* tab_m       = reinterpret_cast<int32_t*>(tab_hw + 64);    // multipliers
    int32_t* tab_b       = tab_m + 64;                                 // biases
    int32_t* uni_shift   = tab_b + 64;                                 // 4 words, one used
    int32_t* wave_start  = uni_shift + 4 + wave * 32;                  // this wave's start values

    uint32_t bid = blockIdx.x;
    if (a.xcd_remap)
    {
        const uint32_t per = (uint32_t)a.xcd_remap;
        bid                = (bid & 7) * per + (bid >> 3);
    }
    const uint32_t tile = fdiv(bid, a.div_ocb);
    const int ocb       = bid - tile * a.n_ocb;
    const uint32_t trow = fdiv(tile, a.div_tiles_x);
    const int txi       = tile - trow * a.tiles_x;
    const int n         = fdiv(trow, a.div_tiles_y);
    const int tyi       = trow - n * a.tiles_y;
    const int oy0 = tyi * a.TH, ox0 = txi * a.TW;
    const int oc0 = ocb * 64;
    const int y0 = oy0 * a.sy - a.pad_top, x0 = ox0 * a.sx - a.pad_left;

    uint32_t flags = 0;
    const int ct = wave & 1, q = wave >> 1;
    // MFMA operand row li holds channel 16*((li>>2)&1) + 4*(li>>3) + (li&3) of the tile's 32, so that a lane's 16
    // accumulators are 16 consecutive channels
    const int wr  = 4 * (li & 4) + ((li >> 1) & 12) + (li & 3);
    const int ocl = ct * 32 + 16 * lh;    // first of the lane's 16 channels inside the block
    const bool chan_ok = oc0 + ocl < a.OC;    // OC is a multiple of 16: a lane's 16 channels are in or out together
    // the bias of the channel whose weight row this lane holds: asked for now, needed after the weights are in registers
    int32_t bias_row = 0;
    if constexpr (ZA)
        bias_row = oc0 + ct * 32 + wr < a.OC ? a.bias[a.bias_len == 1 ? 0 : oc0 + ct * 32 + wr] : 0;
    const uint32_t lbase = (uint32_t)(uintptr_t)lds;
    if (wave < LWAVES)
    {
        constexpr int WB = (WLOADS + LWAVES - 1) / LWAVES;
        v4i tw[VL ? WB : 1];
        {
            // Weights: LDS row r is channel r of the block, slot s = (row, chunk) reads byte 16 (s - row) of the block's
            // weights; seven loads on are 448 slots.  Whatever lies past the block's last channel is clamped to its last chunk.
            const int rows       = a.OC - oc0 < 64 ? a.OC - oc0 : 64;
            const uint32_t limit = (uint32_t)rows * (TAPS * KB) - 16u;
            const uint8_t* wb    = a.w + (size_t)oc0 * (TAPS * KB);
            if constexpr (VL)
            {
                // through registers: the wave's five or six loads are in flight together (loads into LDS leave a wave
                // one at a time), and are written to LDS after its patch loads have been issued
#pragma unroll
                for (int j = 0; j < WB; j++)
                {
                    const int l        = wave + j * LWAVES;
                    const int s0       = l * 64 + lane;
                    const int row0     = s0 / RW;
                    const uint32_t off = 16u * (uint32_t)(s0 - row0);
                    if (l < WLOADS)
                        tw[j] = *reinterpret_cast<const v4i*>(wb + (off < limit ? off : limit));
                }
            }
            else
                for (int l = wave; l < WLOADS; l += LWAVES)
                {
                    const int s0       = l * 64 + lane;
                    const int row0     = s0 / RW;
                    const uint32_t off = 16u * (uint32_t)(s0 - row0);
                    slab_load_off(off < limit ? off : limit, wb, lbase + l * 1024);
                }
        }
        {
            const uint8_t* in_n = a.in + (size_t)n * (a.IH * a.IW) * KB;
            int lp              = wave + ((WLOADS - wave + LWAVES - 1) / LWAVES) * LWAVES - WLOADS;    // first patch load of this wave
            const int s0        = lp * 64 + lane;
            int py              = fdiv(s0, a.div_pitch);    // patch row and chunk inside the row
            int r               = s0 - py * a.pitch;
            uint32_t dst        = lbase + (WLOADS + lp) * 1024;
            for (; lp < p_loads; lp += LWAVES)
            {
                const int px   = (int)((uint32_t)r / (uint32_t)RP);
                const int ch   = r - px * RP;
                const int iy = y0 + py, ix = x0 + px;
                const bool img = py < a.PH && px < a.PW && (unsigned)iy < (unsigned)a.IH && (unsigned)ix < (unsigned)a.IW;
                const int c16  = (ch < CH ? ch : 0) * 16;
                const uint32_t pixel = __umul24(iy, a.IW) + ix;
                const uint8_t* src = img ? in_n + (uint32_t)(pixel * KB + c16) : a.pad_page + (c16 & 48);
                slab_load(src, dst);
                dst += LWAVES * 1024;
                r += a.step_chunk, py += a.step_row;
                if (r >= a.pitch)
                    r -= a.pitch, py++;
            }
        }
        if constexpr (VL)
        {
#pragma unroll
            for (int j = 0; j < WB; j++)
            {
                const int l = wave + j * LWAVES;
                if (l < WLOADS)
                    *reinterpret_cast<v4i*>(lds + l * 1024 + lane * 16) = tw[j];
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    else
    {
        // the table wave: bias and the per-channel RESCALE constants, one channel per lane
        const int oc    = oc0 + lane;
        const bool ok   = oc < a.OC;
        const int occ   = ok ? oc : 0;
        {
            const int32_t m_raw   = load_multiplier(a.rp, occ);
            const int32_t s_raw   = load_shift(a.rp, occ);
            const int32_t s_first = __builtin_amdgcn_readfirstlane(s_raw);
            const ChannelScale cs = make_channel_scale(ok ? m_raw : 0, ok ? s_raw : s_first, a.rp.double_round != 0, flags);
            // the three forms of the epilogue, chosen as in the kernel above
            const int s_min = a.rp.double_round ? 33 : 32;
            const int folds = __all(cs.s >= s_min && cs.s <= zp_fold_max_shift(a.rp.out_zp));
            const int uni   = folds && __all(cs.s == s_first);
            tab_cs[lane]    = cs;
            tab_hw[lane]    = make_high_word_scale(cs, a.rp.out_zp);
            const int relu = a.rp.double_round && a.rp.lo >= a.rp.out_zp && __all(cs.m >= 0);
            if (lane == 0)
                *uni_shift = uni ? (s_first | (relu << 8)) : (folds ? (relu ? -3 : -2) : -1);
            tab_m[lane] = cs.m;
        }
        tab_b[lane] = ok ? a.bias[a.bias_len == 1 ? 0 : occ] : 0;
    }
    slab_barrier();    // weights, patch and tables are in LDS
    v4i fa[STEPS];
    {
        const uint8_t* wrow = wl + ((ct * 32 + wr) * RW) * 16 + lh * 16;
#pragma unroll
        for (int s = 0; s < STEPS; s++)
            fa[s] = *reinterpret_cast<const v4i*>(wrow + s * 32);
        if constexpr (ZA)
        {
            // sum(w) of the row this lane holds: its own half of K in every step, plus the other half from lane ^ 32;
            // four partial sums, because one dependent chain of 4 * STEPS dot products would be the longest thing a wave
            // does here
            int part[4] = { 0, 0, 0, 0 };
#pragma unroll
            for (int s = 0; s < STEPS; s++)
            {
                part[0] = __builtin_amdgcn_sdot4(fa[s].x, 0x01010101, part[0], false);
                part[1] = __builtin_amdgcn_sdot4(fa[s].y, 0x01010101, part[1], false);
                part[2] = __builtin_amdgcn_sdot4(fa[s].z, 0x01010101, part[2], false);
                part[3] = __builtin_amdgcn_sdot4(fa[s].w, 0x01010101, part[3], false);
            }
            int sum = (part[0] + part[1]) + (part[2] + part[3]);
            sum += __builtin_amdgcn_ds_bpermute((lane ^ 32) * 4, sum);
            if (lh == 0)
                wave_start[wr] = (int32_t)((uint32_t)bias_row - (uint32_t)a.za * (uint32_t)sum);
            __builtin_amdgcn_wave_barrier();    // the wave's own LDS accesses complete in order
        }
    }
    // what a tile starts from (bias - input_zp * sum(w) of the lane's 16 channels): the third operand of its first matrix
    // instruction
    v16i start;
    {
        const int32_t* b16 = ZA ? wave_start + 16 * lh : tab_b + ocl;
#pragma unroll
        for (int g = 0; g < 4; g++)
        {
            const v4i b4 = *reinterpret_cast<const v4i*>(b16 + 4 * g);
            start[4 * g] = b4[0], start[4 * g + 1] = b4[1], start[4 * g + 2] = b4[2], start[4 * g + 3] = b4[3];
        }
    }
    const int P        = a.TH * a.TW;
    const int NT       = (P + 31) >> 5;
    // the pixel fragments of step s + DEPTH are requested before the matrix instruction of step s, order pinned
    constexpr int AHEAD = 8;
    constexpr int DEPTH = STEPS < AHEAD ? STEPS : AHEAD;
    const int form = __builtin_amdgcn_readfirstlane(*uni_shift);
    if (form >= 0)
    {
        if (q < NT)
        {
            // One shift for every channel of the block (the usual case): the requantisation of a pixel tile runs between
            // the matrix instructions of the wave's next pixel tile, one output element per K step, so that the vector
            // ALU works while the matrix core does.  (Left to themselves the two waves of a SIMD run their K loops and
            // their epilogues in step, and matrix core and vector ALU take turns.)
            const int s_uni   = form & 255;
            const bool sign   = a.rp.double_round && !(form >> 8);    // the rounding term depends on the value's sign
            const int64_t rnd = (int64_t(1) << (s_uni - 1)) + (a.rp.double_round ? (int64_t(1) << 30) : 0) +
                                ((int64_t)a.rp.out_zp << s_uni);
            const int32_t hi_p  = (int32_t)(rnd >> 32);
            const uint32_t lo_p = (uint32_t)rnd;
            const int sh        = s_uni - 32;
            int32_t cm[16];    // multipliers of the lane's channels
#pragma unroll
            for (int g = 0; g < 4; g++)
            {
                const v4i m4 = *reinterpret_cast<const v4i*>(tab_m + ocl + 4 * g);
                cm[4 * g] = m4[0], cm[4 * g + 1] = m4[1], cm[4 * g + 2] = m4[2], cm[4 * g + 3] = m4[3];
            }
            const int32_t v_lo = a.rp.lo, v_hi = a.rp.hi;
            // SIGN: the rounding term depends on the value's sign; WIDE: int16 results (two stores) instead of int8
            auto pipelined = [&](auto SIGN, auto WIDE) {
                constexpr bool kSign = decltype(SIGN)::value, kWide = decltype(WIDE)::value;
                struct Place
                {
                    uint32_t prow;    // byte offset of the lane's pixel under tap (0, 0) in the patch
                    uint32_t base;    // the lane's first output element
                    uint32_t ok;      // whether the lane stores
                };
                auto place = [&](int pt) {
                    int p              = pt * 32 + li;
                    const bool in_tile = p < P;
                    p                  = in_tile ? p : 0;
                    const int ty       = fdiv(p, a.div_tw);
                    const int tx       = p - ty * a.TW;
                    const int oy = oy0 + ty, ox = ox0 + tx;
                    return Place{ (uint32_t)((ty * a.sy * a.pitch + tx * a.sx * RP) * 16 + lh * 16),
                                  (uint32_t)(((n * a.OH + oy) * a.OW + ox) * a.OC + oc0 + ocl),
                                  (uint32_t)(in_tile && oy < a.OH && ox < a.OW && chan_ok) };
                };
                v4i fb[STEPS];
                auto request = [&](const Place& at, int s) {
                    const int tap = s / (CH / 2), h = s % (CH / 2);
                    fb[s]         = *reinterpret_cast<const v4i*>(pl + at.prow + (tap / KW) * row_step + (tap % KW) * col_step + h * 32);
                };
                int32_t r[4];
                v4i pk, pk2;
                // the requantisation of tile `done` (accumulators prv), dealt over the K steps of the tile after it: step 0
                // nothing (the last matrix instruction of `done` is still running), steps 1..16 one element each, packed
                // as soon as a word is complete, step 17 stores
                auto requant_piece = [&](int s, const v16i& prv, const Place& done) {
                    if (s >= 1 && s <= 16)
                    {
                        const int e = s - 1;
                        r[e & 3]    = kSign ? clamp_med3(high_word_rescale<true>(prv[e], cm[e], hi_p, lo_p, sh), v_lo, v_hi)
                                          : clamp_med3(high_word_rescale_const(prv[e], cm[e], rnd, sh), v_lo, v_hi);
                        if constexpr (!kWide)
                        {
                            if ((e & 3) == 3)
                            {
                                const int lo2 = __builtin_amdgcn_perm(r[1], r[0], 0x0c0c0400);
                                const int hi2 = __builtin_amdgcn_perm(r[3], r[2], 0x04000c0c);
                                pk[e >> 2]    = lo2 | hi2;
                            }
                        }
                        else if (e & 1)
                        {
                            const int word = (r[(e & 3) - 1] & 0xffff) | ((r[e & 3] & 0xffff) << 16);
                            if (e < 8)
                                pk[e >> 1] = word;
                            else
                                pk2[(e - 8) >> 1] = word;
                        }
                    }
                    else if (s == 17 && done.ok)
                    {
                        if constexpr (!kWide)
                            *reinterpret_cast<v4i*>(reinterpret_cast<int8_t*>(a.out) + done.base) = pk;
                        else
                        {
                            int16_t* o                       = reinterpret_cast<int16_t*>(a.out) + done.base;
                            *reinterpret_cast<v4i*>(o)     = pk;
                            *reinterpret_cast<v4i*>(o + 8) = pk2;
                        }
                    }
                };
                // One tile: its K loop, with the first fragments of the tile after it requested in its last steps (so that
                // the matrix instructions of consecutive tiles follow each other without a gap) and the requantisation of
                // the tile before it between its matrix instructions.
                auto tile = [&](v16i& acc, const v16i& prv, const Place& cur, const Place& next, const Place& done, auto REQUANT) {
#pragma unroll
                    for (int s = 0; s < STEPS; s++)
                    {
                        if (s + DEPTH < STEPS)
                            request(cur, s + DEPTH);
                        else
                            request(next, s + DEPTH - STEPS);
                        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[s], fb[s], s == 0 ? start : acc, 0, 0, 0);
                        if constexpr (decltype(REQUANT)::value)
                            requant_piece(s, prv, done);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                };
                v16i acc0 = start, acc1 = start;
                int pt      = q;
                Place cur   = place(pt), next = pt + (NW / 2) < NT ? place(pt + (NW / 2)) : cur, done = cur;
#pragma unroll
                for (int s = 0; s < DEPTH; s++)
                    request(cur, s);
                __builtin_amdgcn_sched_barrier(0);
                tile(acc0, acc1, cur, next, done, std::false_type{});
                while (true)
                {
                    // acc0 holds tile pt; the next one goes into acc1
                    done = cur, cur = next, pt += (NW / 2);
                    if (pt >= NT)
                    {
#pragma unroll
                        for (int s = 0; s < 18; s++)
                            requant_piece(s, acc0, done);
                        break;
                    }
                    next = pt + (NW / 2) < NT ? place(pt + (NW / 2)) : cur;
                    tile(acc1, acc0, cur, next, done, std::true_type{});
                    done = cur, cur = next, pt += (NW / 2);
                    if (pt >= NT)
                    {
#pragma unroll
                        for (int s = 0; s < 18; s++)
                            requant_piece(s, acc1, done);
                        break;
                    }
                    next = pt + (NW / 2) < NT ? place(pt + (NW / 2)) : cur;
                    tile(acc0, acc1, cur, next, done, std::true_type{});
                }
            };
            if (a.out_kind == 1)
                sign ? pipelined(std::true_type{}, std::false_type{}) : pipelined(std::false_type{}, std::false_type{});
            else
                sign ? pipelined(std::true_type{}, std::true_type{}) : pipelined(std::false_type{}, std::true_type{});
        }
        raise_flags(a.flag_word, flags);
        return;
    }
    // Shifts that differ between the channels (or lie outside the high-word form): tile after tile, K loop and then the
    // requantisation with per-channel constants from the tables.
    for (int pt = q; pt < NT; pt += (NW / 2))
    {
        int p              = pt * 32 + li;
        const bool in_tile = p < P;
        p                  = in_tile ? p : 0;
        const int ty       = fdiv(p, a.div_tw);
        const int tx       = p - ty * a.TW;
        const uint8_t* prow = pl + (ty * a.sy * a.pitch + tx * a.sx * RP) * 16 + lh * 16;
        v16i acc = start;
        v4i fb[STEPS];
        auto request = [&](int s) {
            const int tap = s / (CH / 2), h = s % (CH / 2);
            fb[s]         = *reinterpret_cast<const v4i*>(prow + (tap / KW) * row_step + (tap % KW) * col_step + h * 32);
        };
#pragma unroll
        for (int s = 0; s < DEPTH; s++)
            request(s);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < STEPS; s++)
        {
            if (s + DEPTH < STEPS)
                request(s + DEPTH);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[s], fb[s], acc, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }

        // (lane, register 4g + j) = D[row 8g + 4 lh + j][pixel li] = channel 32 ct + 16 lh + 4g + j
        const int oy = oy0 + ty, ox = ox0 + tx;
        const bool pix_ok  = in_tile && oy < a.OH && ox < a.OW;
        const size_t obase = (uint32_t)(((n * a.OH + oy) * a.OW + ox) * a.OC + oc0 + ocl);
        {
            // four channels at a time, each group packed as soon as it is done
            const bool store = pix_ok && chan_ok;
            v4i pk, pk2;    // int8: pk; int16: pk, pk2
            uint32_t eflags = 0;
            auto pack = [&](int g, const int32_t (&r)[4]) {
                if (a.out_kind == 1)
                {
                    const int lo2 = __builtin_amdgcn_perm(r[1], r[0], 0x0c0c0400);
                    const int hi2 = __builtin_amdgcn_perm(r[3], r[2], 0x04000c0c);
                    pk[g]         = lo2 | hi2;
                }
                else
                {
                    const int w0 = (r[0] & 0xffff) | ((r[1] & 0xffff) << 16), w1 = (r[2] & 0xffff) | ((r[3] & 0xffff) << 16);
                    if (g < 2)
                        pk[2 * g] = w0, pk[2 * g + 1] = w1;
                    else
                        pk2[2 * g - 4] = w0, pk2[2 * g - 3] = w1;
                }
            };
            if (form <= -2)
            {
                const bool sign_test = a.rp.double_round && form == -2;    // (-3: a negative value is clamped away either way)
#pragma unroll
                for (int g = 0; g < 4; g++)
                {
                    int32_t r[4];
#pragma unroll
                    for (int j = 0; j < 4; j++)
                    {
                        const HighWordScale c = tab_hw[ocl + 4 * g + j];
                        r[j] = sign_test ? clamp_med3(high_word_rescale<true>(acc[4 * g + j], c.m, c.hi, c.lo, c.sh), a.rp.lo, a.rp.hi)
                                                 : clamp_med3(high_word_rescale<false>(acc[4 * g + j], c.m, c.hi, c.lo, c.sh), a.rp.lo, a.rp.hi);
                    }
                    pack(g, r);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            else
            {
#pragma unroll
                for (int g = 0; g < 4; g++)
                {
                    int32_t r[4];
#pragma unroll
                    for (int j = 0; j < 4; j++)
                    {
                        const ChannelScale cs = tab_cs[ocl + 4 * g + j];
                        r[j]                  = fast_rescale(acc[4 * g + j], cs, a.rp.out_zp, a.rp.lo, a.rp.hi, eflags);
                    }
                    pack(g, r);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (store)
                    flags |= eflags;    // pixels and channels outside the tensor raise nothing
            }
            if (store)
            {
                if (a.out_kind == 1)
                    *reinterpret_cast<v4i*>(reinterpret_cast<int8_t*>(a.out) + obase) = pk;
                else
                {
                    int16_t* o                       = reinterpret_cast<int16_t*>(a.out) + obase;
                    *reinterpret_cast<v4i*>(o)     = pk;
                    *reinterpret_cast<v4i*>(o + 8) = pk2;
                }
            }
        }
    }
    raise_flags(a.flag_word, flags);
}


thread_local int32_t last_launch_shape[3] = { 0, 0, 0 };

template <int KH, int KW, int CH, bool ZA, bool FUSED, bool TC = false, int KD = 1, int NPT = 1, typename T = int8_t>
static bool launch_slab_kernel(hipStream_t st, const SlabArgs& a, int grid, int lds_bytes)
{
    auto kern              = conv2d_slab_kernel<KH, KW, CH, ZA, FUSED, TC, KD, NPT, T>;
    static LdsLimit granted{};
    if (!ensure_dynamic_lds(reinterpret_cast<const void*>(kern), (size_t)lds_bytes, granted))
        return false;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds_bytes, st, a);
    last_launch_shape[0] = grid, last_launch_shape[1] = 512, last_launch_shape[2] = lds_bytes;
    return true;
}

static bool launch_slab_wreg(hipStream_t st, const SlabArgs& a, int grid, int lds_bytes)
{
    auto launch = [&](auto kern) {
        static LdsLimit granted{};
        if (!ensure_dynamic_lds(reinterpret_cast<const void*>(kern), (size_t)lds_bytes, granted))
            return false;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds_bytes, st, a);
        last_launch_shape[0] = grid, last_launch_shape[1] = 512, last_launch_shape[2] = lds_bytes;
        return true;
    };
    // Weight loads through registers from five pixel tiles per workgroup on.  Measured on MI355X, us per launch with the
    // loads into LDS / through registers, [N,56,56,64]->64: N = 4 3.59 / 3.68, 8 4.04 / 4.09, 10 4.55 / 4.57, 12 4.70 / 4.60,
    // 16 5.25 / 5.10, 20 5.67 / 5.56, 32 6.96 / 6.64, 64 11.0 / 10.47.
    const bool vl = (a.TH * a.TW + 31) / 32 >= 5;
    if (vl)
        return a.za != 0 ? launch(conv2d_slab_wreg_kernel<true, true>) : launch(conv2d_slab_wreg_kernel<false, true>);
    return a.za != 0 ? launch(conv2d_slab_wreg_kernel<true, false>) : launch(conv2d_slab_wreg_kernel<false, false>);
}

// the floating-point instantiations: fp16 (kind 1) or bf16 (kind 2)
template <int KH, int KW, int CH, bool WIDE_TOO = true>
static bool launch_slab_taps_fp(hipStream_t st, const SlabArgs& a, int grid, int lds_bytes, int kind, bool wide)
{
    if constexpr (WIDE_TOO)
    {
        if (wide)
            return kind == 1 ? launch_slab_kernel<KH, KW, CH, false, false, false, 1, 2, _Float16>(st, a, grid, lds_bytes)
                             : launch_slab_kernel<KH, KW, CH, false, false, false, 1, 2, bf16_t>(st, a, grid, lds_bytes);
    }
    else if (wide)
        return false;
    return kind == 1 ? launch_slab_kernel<KH, KW, CH, false, false, false, 1, 1, _Float16>(st, a, grid, lds_bytes)
                     : launch_slab_kernel<KH, KW, CH, false, false, false, 1, 1, bf16_t>(st, a, grid, lds_bytes);
}

template <int KH, int KW, int CH, bool WIDE_TOO = true>
static bool launch_slab_taps(hipStream_t st, const SlabArgs& a, int grid, int lds_bytes, bool fused, bool wide)
{
    if constexpr (!WIDE_TOO)
    {
        if (wide)
            return false;
    }
    else if (wide)
    {
        if (a.za != 0)
            return fused ? launch_slab_kernel<KH, KW, CH, true, true, false, 1, 2>(st, a, grid, lds_bytes)
                         : launch_slab_kernel<KH, KW, CH, true, false, false, 1, 2>(st, a, grid, lds_bytes);
        return fused ? launch_slab_kernel<KH, KW, CH, false, true, false, 1, 2>(st, a, grid, lds_bytes)
                     : launch_slab_kernel<KH, KW, CH, false, false, false, 1, 2>(st, a, grid, lds_bytes);
    }
    if (a.za != 0)
        return fused ? launch_slab_kernel<KH, KW, CH, true, true>(st, a, grid, lds_bytes)
                     : launch_slab_kernel<KH, KW, CH, true, false>(st, a, grid, lds_bytes);
    return fused ? launch_slab_kernel<KH, KW, CH, false, true>(st, a, grid, lds_bytes)
                 : launch_slab_kernel<KH, KW, CH, false, false>(st, a, grid, lds_bytes);
}

// nullptr when the layer is not one this kernel takes; the caller then goes to the patch kernel.
const char* launch_conv2d_slab(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                               const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                               void* out, const void* pad_page, uint32_t* flag_word, const SlabHoles* tc,
                               const SlabDepth* c3d)
{
    const bool k33 = g.KH == 3 && g.KW == 3, k11 = g.KH == 1 && g.KW == 1;
    // fp16 / bf16: plain CONV2D without zero points; what counts below is the bytes of a channel vector
    const int fp = in_dtype == TMI_FP16 ? 1 : (in_dtype == TMI_BF16 ? 2 : 0);
    if (fp && (tc || c3d || rp.enabled || out_dtype != in_dtype || in_zp != 0 || ((uintptr_t)bias & 1)))
        return nullptr;
    const int icb = g.IC * (fp ? 2 : 1);
    // channel vectors of 64, 96 or 128 bytes; pointwise layers also the common sizes from 160 to 1024 bytes (64 weight rows
    // of 1024 bytes and a patch of 62 pixels still fit the LDS; the K loop is unrolled, so each size is an instantiation of
    // its own, and floating point has a few less)
    const bool deep11 = k11 && !tc && !c3d &&
                        (icb == 160 || icb == 192 || icb == 256 || icb == 320 || icb == 384 || icb == 512 || icb == 768 || icb == 1024 ||
                         (!fp && (icb == 480 || icb == 576 || icb == 960)));
    if ((in_dtype != TMI_INT8 && !fp) || ((icb != 64 && icb != 96 && icb != 128) && !deep11) || !(k33 || k11) || w_zp != 0 || !pad_page ||
        !flag_word)
        return nullptr;
    if (tc && (!k33 || rp.enabled || tc->up_y < 1 || tc->up_x < 1 || g.stride_y != 1 || g.stride_x != 1))
        return nullptr;
    if (c3d)
    {
        const int icr = c3d->KD > 0 ? g.IC / c3d->KD : 0;    // channels of the tensor in memory
        const bool kd_ok = (icr == 32 && c3d->KD >= 2 && c3d->KD <= 4) || (icr == 64 && c3d->KD == 2);
        if (tc || !k33 || rp.enabled || !kd_ok || icr * c3d->KD != g.IC || c3d->OD < 1 || g.N % c3d->OD != 0)
            return nullptr;
    }
    const int taps = g.KH * g.KW;
    if (!fp && (rp.enabled ? (!rp.fast || (out_dtype != TMI_INT8 && out_dtype != TMI_INT16)) : out_dtype != TMI_INT32))
        return nullptr;
    if (g.OC < 48 || g.OC > 65536 || (g.OC & 15) || g.N < 1 || g.OH < 1 || g.OW < 1)
        return nullptr;
    if ((((uintptr_t)in | (uintptr_t)w | (uintptr_t)out | (uintptr_t)pad_page) & 15) || (!fp && ((uintptr_t)bias & 3)))
        return nullptr;
    if ((int64_t)g.N * g.IH * g.IW * icb >= (int64_t(1) << 31) || (int64_t)g.N * g.OH * g.OW * g.OC >= (int64_t(1) << 31))
        return nullptr;

    // The tile: at most 124 pixels (four tiles of 31 pixels, one per wave and channel tile).  A workgroup moves the
    // weight slab (taps * 64 rows of 64 bytes) plus PH * PW patch rows; whole rounds of 256 workgroups count.
    // The search depends on the geometry only; a caller repeats the same layer, so the last answer is kept.
    //
    // Layers of unit stride with more such tiles than the chip has CUs run the two-tiles-per-wave form on tiles of
    // up to 252 pixels instead.  Measured on MI355X, us with one / two tiles per wave (graph replays, fused RESCALE):
    // 3x3 [32,56,56,64]->64 10.5 / 8.6, [64,..] 17.5 / 15.1, [20,..] 8.2 / 7.7, [16,..] 6.0 / 5.8, [10,..] 5.4 / 5.3,
    // [8,56,56,128]->128 9.7 / 7.9, [32,28,28,128]->128 9.4 / 7.9, [64,14,14,128]->256 9.6 / 7.6; 1x1
    // [8,56,56,64]->256 6.6 / 5.9, [32,..] 17.6 / 16.9, [16,28,28,128]->512 6.8 / 6.1, [32,..] 11.8 / 12.1;
    // a single round of the small tiles is faster with them ([8,56,56,64]->64 4.3 / 5.1, [16,28,28,128]->128 5.5 / 6.4),
    // and so is stride 2, whose patch grows with the tile ([32,57,57,128]->64 9.5 / 11.7).
    const int n_ocb = (g.OC + 63) / 64;
    const int ch = icb / 16, rp_chunks = ch + 1;    // chunks of a channel vector; chunks per patch pixel in LDS
    struct TileChoice
    {
        int32_t key[8];
        int th, tw, form;
    };
    // form 0: one accumulator tile per wave, tiles of at most 124 pixels; 1: two accumulator tiles per wave, at most 252
    // pixels; 2: weights in registers (conv2d_slab_wreg_kernel), tiles as large as the LDS takes
    static thread_local TileChoice last = { { 0, 0, 0, 0, 0, 0, 0, 0 }, 0, 0, 0 };
    const int32_t key[8] = { g.N, g.OH, g.OW, (((n_ocb * 256 + ch) * 4 + g.KH) * 2 + ((tc || c3d) ? 1 : 0)) * 2 + (rp.enabled ? 1 : 0), g.stride_y, g.stride_x,
                             g.dil_y, g.dil_x };
    int best_th = 0, best_tw = 0, form = 0;
    if (memcmp(key, last.key, sizeof(key)) == 0)
        best_th = last.th, best_tw = last.tw, form = last.form;
    else
    {
        int64_t best_rounds = 0;
        auto search = [&](int max_pix, int64_t fixed) {
            int64_t best_cost = 0;
            best_th = best_tw = 0;
            for (int th = 1; th <= g.OH && th <= max_pix; th++)
                for (int tw = 1; tw <= g.OW && th * tw <= max_pix; tw++)
                {
                    const int ph = (th - 1) * g.stride_y + (g.KH - 1) * g.dil_y + 1;
                    const int pw = (tw - 1) * g.stride_x + (g.KW - 1) * g.dil_x + 1;
                    if (ph * (pw * rp_chunks + 15) >= (1 << 16) || ph * (pw * rp_chunks + 15) * 16 > 64 * 1024)
                        continue;
                    const int64_t tiles  = (int64_t)g.N * ((g.OH + th - 1) / th) * ((g.OW + tw - 1) / tw) * n_ocb;
                    const int64_t rounds = (tiles + 255) / 256;
                    // a round costs its loads plus its 32-pixel MFMA tiles whether they are full or not
                    const int64_t cost = rounds * ((taps * 64 + ph * pw) * ch / 4 + fixed);
                    if (!best_th || cost < best_cost || (cost == best_cost && th * tw > best_th * best_tw))
                        best_th = th, best_tw = tw, best_cost = cost, best_rounds = rounds;
                }
        };
        // The form with the weights in registers: a workgroup's time is its prologue (arguments, the latency of the
        // loads, the weight fragments read into registers), its loads (1 KB each) and the matrix instructions of its
        // busiest SIMD, which holds waves s and s + 4, i.e. the pixel tiles s / 2 + 4 j and s / 2 + 2 + 4 j.
        auto search_wreg = [&]() {
            int64_t best_cost = 0;
            best_th = best_tw = 0;
            const int steps = taps * ch / 2;
            for (int th = 1; th <= g.OH; th++)
                for (int tw = 1; tw <= g.OW; tw++)
                {
                    const int ph = (th - 1) * g.stride_y + (g.KH - 1) * g.dil_y + 1;
                    const int pw = (tw - 1) * g.stride_x + (g.KW - 1) * g.dil_x + 1;
                    const int64_t slots = (int64_t)ph * (pw * rp_chunks + 15);
                    if (slots >= (1 << 16) || slots * 16 + (taps * ch + 1) * 1024 > 150 * 1024)
                        break;
                    const int nt      = (th * tw + 31) / 32;
                    const int busiest = (nt + 3) / 4 + (nt > 2 ? (nt - 2 + 3) / 4 : 0);
                    const int64_t tiles  = (int64_t)g.N * ((g.OH + th - 1) / th) * ((g.OW + tw - 1) / tw) * n_ocb;
                    const int64_t rounds = (tiles + 255) / 256;
                    const int64_t cost   = rounds * (900 + 12 * (taps * ch + 1 + (slots + 63) / 64) + 15 * steps * busiest);
                    if (!best_th || cost < best_cost || (cost == best_cost && th * tw < best_th * best_tw))
                        best_th = th, best_tw = tw, best_cost = cost;
                }
        };
        // Measured on MI355X, us per launch (graph replays, fused RESCALE) with one tile per wave / two / the weights in
        // registers: 3x3 [8,56,56,64]->64 4.18 / 5.04 / 4.09, [10,..] 5.4 / 5.2 / 4.5, [16,..] 5.9 / 5.7 / 5.25, [20,..]
        // 8.0 / 7.4 / 5.8, [32,..] 10.2 / 8.5 / 7.2, [64,..] 16.6 / 14.9 / 11.8, [8,56,56,64]->128 5.7 / 5.6 / 5.1,
        // [4,28,28,64]->64 3.6 / 4.2 / 3.3; with 96 or 128 input channels the weights leave no room for the second
        // accumulator tile and the form loses ([8,56,56,128]->128 9.3 / 7.7 / 8.5), and with int32 results all three tie.
        const bool plain = !tc && !c3d;
        if (plain && k33 && ch == 4 && g.stride_y == 1 && g.stride_x == 1 && rp.enabled)
            search_wreg(), form = 2;
        else
        {
            search(124, 600);
            if (best_th && best_rounds > 1 && g.stride_y == 1 && g.stride_x == 1 && plain && ch <= 16)
            {
                const int th1 = best_th, tw1 = best_tw;
                search(252, 1100);
                form = best_th ? 1 : 0;
                if (!form)
                    best_th = th1, best_tw = tw1;
            }
        }
        memcpy(last.key, key, sizeof(key));
        last.th = best_th, last.tw = best_tw, last.form = form;
    }
    const bool wide = form == 1;
    if (!best_th)
        return nullptr;

    SlabArgs a{};
    a.in = (const uint8_t*)in, a.w = (const uint8_t*)w, a.bias = (const int32_t*)bias, a.out = out;
    a.pad_page = (const uint8_t*)pad_page, a.flag_word = flag_word, a.rp = rp;
    a.N = g.N, a.IH = g.IH, a.IW = g.IW, a.OC = g.OC, a.OH = g.OH, a.OW = g.OW;
    a.sy = g.stride_y, a.sx = g.stride_x, a.dy = g.dil_y, a.dx = g.dil_x, a.pad_top = g.pad_top, a.pad_left = g.pad_left;
    a.TH = best_th, a.TW = best_tw;
    a.PH = (best_th - 1) * g.stride_y + (g.KH - 1) * g.dil_y + 1;
    a.PW = (best_tw - 1) * g.stride_x + (g.KW - 1) * g.dil_x + 1;
    a.tiles_y = (g.OH + best_th - 1) / best_th, a.tiles_x = (g.OW + best_tw - 1) / best_tw;
    a.bias_len = g.bias_len, a.za = in_zp, a.n_ocb = n_ocb;
    a.out_kind = !rp.enabled ? 0 : (out_dtype == TMI_INT8 ? 1 : 2);
    const int64_t grid = (int64_t)g.N * a.tiles_y * a.tiles_x * n_ocb;
    if (!tile_decode_is_exact(grid, (uint32_t)n_ocb, (uint32_t)a.tiles_x, (uint32_t)a.tiles_y))
        return nullptr;
    a.xcd_remap = (grid % 8 == 0 && n_ocb == 1) ? (int32_t)(grid / 8) : 0;
    // A patch pixel is R = CH + 1 chunks; the chunk of output pixel (ty, tx) under tap (0, 0) is ty * sy * pitch + R * sx * tx.
    // A ds_read_b128 serves 16 lanes together, whose chunks must differ modulo 16.  The lanes of a wave are consecutive
    // tile pixels p = ty * TW + tx, and any 16 lanes served together differ modulo 16, so the reads are free of bank
    // conflicts when the chunk is an odd multiple of p plus a constant (modulo 16): R * sx odd and
    // sy * pitch = R * sx * TW (mod 16).  Up to 15 chunks of padding per patch row arrange that for odd strides;
    // even strides keep pitch = 5 * PW and their conflicts.
    int pad = 0;
    if ((g.stride_x & 1) && (g.stride_y & 1))
        for (pad = 0; pad < 16; pad++)
            if (((g.stride_y * (a.PW * rp_chunks + pad) - rp_chunks * g.stride_x * a.TW) & 15) == 0)
                break;
    a.pitch     = a.PW * rp_chunks + (pad & 15);
    a.step_row  = 448 / a.pitch, a.step_chunk = 448 % a.pitch;
    a.div_tw = make_fastdiv((uint32_t)a.TW), a.div_pitch = make_fastdiv((uint32_t)a.pitch);
    a.div_tiles_x = make_fastdiv((uint32_t)a.tiles_x), a.div_tiles_y = make_fastdiv((uint32_t)a.tiles_y);
    a.div_ocb = make_fastdiv((uint32_t)n_ocb);
    const int w_loads = taps * ch + 1, p_loads = (a.PH * a.pitch + 63) / 64;
    const int ones_bytes = (g.KH - 1) * g.dil_y * a.pitch * 16 + (g.KW - 1) * g.dil_x * rp_chunks * 16 + icb;
    const int lds_bytes  = (w_loads + p_loads) * 1024 + ones_bytes + 64 * (int)(sizeof(ChannelScale) + sizeof(HighWordScale)) + 64 * 4 + 80 * 4 + 16;
    const bool fused = rp.enabled != 0;
    bool ok;
    if (form == 2)
    {
        const int wreg_lds = (w_loads + p_loads) * 1024 + 64 * (int)(sizeof(ChannelScale) + sizeof(HighWordScale)) + 64 * 4 + 64 * 4 + 16 + 8 * 32 * 4;
        return launch_slab_wreg(st, a, (int)grid, wreg_lds) ? "conv2d_slab_wreg_i8_rescale" : nullptr;
    }
    if (c3d)
    {
        a.ID = c3d->ID, a.OD = c3d->OD, a.sd = c3d->stride_d, a.dd = c3d->dilation_d, a.pd0 = c3d->pad_d0;
        a.div_od = make_fastdiv((uint32_t)c3d->OD);
        if (!fastdiv_exact_up_to((uint64_t)g.N - 1, (uint32_t)c3d->OD))    // image index = volume * OD + output slice
            return nullptr;
        const bool za = a.za != 0;
        if (ch == 4)
            ok = za ? launch_slab_kernel<3, 3, 4, true, false, false, 2>(st, a, (int)grid, lds_bytes)
                    : launch_slab_kernel<3, 3, 4, false, false, false, 2>(st, a, (int)grid, lds_bytes);
        else if (ch == 6)
            ok = za ? launch_slab_kernel<3, 3, 6, true, false, false, 3>(st, a, (int)grid, lds_bytes)
                    : launch_slab_kernel<3, 3, 6, false, false, false, 3>(st, a, (int)grid, lds_bytes);
        else if (c3d->KD == 4)
            ok = za ? launch_slab_kernel<3, 3, 8, true, false, false, 4>(st, a, (int)grid, lds_bytes)
                    : launch_slab_kernel<3, 3, 8, false, false, false, 4>(st, a, (int)grid, lds_bytes);
        else
            ok = za ? launch_slab_kernel<3, 3, 8, true, false, false, 2>(st, a, (int)grid, lds_bytes)
                    : launch_slab_kernel<3, 3, 8, false, false, false, 2>(st, a, (int)grid, lds_bytes);
        return ok ? "conv3d_slab_i8" : nullptr;
    }
    if (tc)
    {
        a.up_y = tc->up_y, a.up_x = tc->up_x, a.IHr = tc->IH, a.IWr = tc->IW;
        a.div_up_y = make_fastdiv((uint32_t)tc->up_y), a.div_up_x = make_fastdiv((uint32_t)tc->up_x);
        // the divided coordinates are rows and columns of the input with its holes (g.IH x g.IW)
        if (!fastdiv_exact_up_to((uint64_t)g.IH, (uint32_t)tc->up_y) || !fastdiv_exact_up_to((uint64_t)g.IW, (uint32_t)tc->up_x))
            return nullptr;
        if (a.za != 0)
            ok = ch == 4 ? launch_slab_kernel<3, 3, 4, true, false, true>(st, a, (int)grid, lds_bytes)
                         : (ch == 6 ? launch_slab_kernel<3, 3, 6, true, false, true>(st, a, (int)grid, lds_bytes)
                                    : launch_slab_kernel<3, 3, 8, true, false, true>(st, a, (int)grid, lds_bytes));
        else
            ok = ch == 4 ? launch_slab_kernel<3, 3, 4, false, false, true>(st, a, (int)grid, lds_bytes)
                         : (ch == 6 ? launch_slab_kernel<3, 3, 6, false, false, true>(st, a, (int)grid, lds_bytes)
                                    : launch_slab_kernel<3, 3, 8, false, false, true>(st, a, (int)grid, lds_bytes));
        return ok ? "transpose_conv2d_slab_i8" : nullptr;
    }
    if (fp)
    {
        if (k33)
            ok = ch == 4 ? launch_slab_taps_fp<3, 3, 4>(st, a, (int)grid, lds_bytes, fp, wide)
                         : (ch == 6 ? launch_slab_taps_fp<3, 3, 6>(st, a, (int)grid, lds_bytes, fp, wide)
                                    : launch_slab_taps_fp<3, 3, 8>(st, a, (int)grid, lds_bytes, fp, wide));
        else
            switch (ch)
            {
                case 4: ok = launch_slab_taps_fp<1, 1, 4>(st, a, (int)grid, lds_bytes, fp, wide); break;
                case 6: ok = launch_slab_taps_fp<1, 1, 6>(st, a, (int)grid, lds_bytes, fp, wide); break;
                case 8: ok = launch_slab_taps_fp<1, 1, 8>(st, a, (int)grid, lds_bytes, fp, wide); break;
                case 10: ok = launch_slab_taps_fp<1, 1, 10>(st, a, (int)grid, lds_bytes, fp, wide); break;
                case 12: ok = launch_slab_taps_fp<1, 1, 12>(st, a, (int)grid, lds_bytes, fp, wide); break;
                case 16: ok = launch_slab_taps_fp<1, 1, 16>(st, a, (int)grid, lds_bytes, fp, wide); break;
                case 20: ok = launch_slab_taps_fp<1, 1, 20, false>(st, a, (int)grid, lds_bytes, fp, false); break;
                case 24: ok = launch_slab_taps_fp<1, 1, 24, false>(st, a, (int)grid, lds_bytes, fp, false); break;
                case 32: ok = launch_slab_taps_fp<1, 1, 32, false>(st, a, (int)grid, lds_bytes, fp, false); break;
                case 48: ok = launch_slab_taps_fp<1, 1, 48, false>(st, a, (int)grid, lds_bytes, fp, false); break;
                case 64: ok = launch_slab_taps_fp<1, 1, 64, false>(st, a, (int)grid, lds_bytes, fp, false); break;
                default: ok = false; break;
            }
        if (!ok)
            return nullptr;
        return fp == 1 ? "conv2d_slab_f16" : "conv2d_slab_bf16";
    }
    if (k33)
        ok = ch == 4 ? launch_slab_taps<3, 3, 4>(st, a, (int)grid, lds_bytes, fused, wide)
                     : (ch == 6 ? launch_slab_taps<3, 3, 6>(st, a, (int)grid, lds_bytes, fused, wide)
                                : launch_slab_taps<3, 3, 8>(st, a, (int)grid, lds_bytes, fused, wide));
    else if (ch > 8)
    {
        switch (ch)    // (one accumulator tile per wave beyond 256 channels: see the tile search)
        {
            case 10: ok = launch_slab_taps<1, 1, 10>(st, a, (int)grid, lds_bytes, fused, wide); break;
            case 12: ok = launch_slab_taps<1, 1, 12>(st, a, (int)grid, lds_bytes, fused, wide); break;
            case 16: ok = launch_slab_taps<1, 1, 16>(st, a, (int)grid, lds_bytes, fused, wide); break;
            case 20: ok = launch_slab_taps<1, 1, 20, false>(st, a, (int)grid, lds_bytes, fused, false); break;
            case 24: ok = launch_slab_taps<1, 1, 24, false>(st, a, (int)grid, lds_bytes, fused, false); break;
            case 30: ok = launch_slab_taps<1, 1, 30, false>(st, a, (int)grid, lds_bytes, fused, false); break;
            case 32: ok = launch_slab_taps<1, 1, 32, false>(st, a, (int)grid, lds_bytes, fused, false); break;
            case 36: ok = launch_slab_taps<1, 1, 36, false>(st, a, (int)grid, lds_bytes, fused, false); break;
            case 48: ok = launch_slab_taps<1, 1, 48, false>(st, a, (int)grid, lds_bytes, fused, false); break;
            case 60: ok = launch_slab_taps<1, 1, 60, false>(st, a, (int)grid, lds_bytes, fused, false); break;
            case 64: ok = launch_slab_taps<1, 1, 64, false>(st, a, (int)grid, lds_bytes, fused, false); break;
            default: ok = false; break;
        }
    }
    else
        ok = ch == 4 ? launch_slab_taps<1, 1, 4>(st, a, (int)grid, lds_bytes, fused, wide)
                     : (ch == 6 ? launch_slab_taps<1, 1, 6>(st, a, (int)grid, lds_bytes, fused, wide)
                                : launch_slab_taps<1, 1, 8>(st, a, (int)grid, lds_bytes, fused, wide));
    if (!ok)
        return nullptr;
    return rp.enabled ? "conv2d_slab_i8_rescale" : "conv2d_slab_i8";
}

}    // namespace tmi
