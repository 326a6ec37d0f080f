// CONV2D as an implicit GEMM on the matrix cores (MFMA), with the bias / zero-point / RESCALE / CLAMP
// epilogue fused so that the int32 accumulators never reach HBM.
//
// One workgroup (8 waves) computes a TH x TW tile of output pixels of one image for a block of OCB =
// 32*OCT*WOC output channels.  The waves form a WOC x (8/WOC) grid; each owns OCT channel tiles and PXT pixel
// tiles of 32, i.e. OCT*PXT accumulator tiles.  The small instantiations (one or two accumulator tiles per
// wave) are for layers too small to fill the chip otherwise, the 2x2 and 2x4 ones for GEMM-sized work, where
// fewer operand bytes pass through L1 and LDS per MFMA.  Per block of CH*16 bytes of input channels the workgroup stages in LDS
//   - the input patch that the tile needs (PH x PW pixels, out-of-image pixels filled with input_zp, so the
//     zero-point identity below holds with the full K): one row of CH 16-byte chunks per pixel, and
//   - the weight slab: one row per output channel holding its KH*KW*CH chunks in (tap, chunk) order, which
//     is the order they have in HBM.
// Every input byte is read from HBM/L2 once per workgroup (plus the halo) and reused KH*KW*OCB times
// from LDS.
//
// When the input channels need more than one block and a block is at most WU weight chunks and PU patch
// chunks per lane, the blocks are software pipelined: LDS holds two buffers, the global loads of block b+1
// are issued before the MFMA loop of block b and written to the other buffer after it, and one barrier per
// block remains.  Otherwise (single block, or blocks too large for the registers) a block is staged in
// rounds into a single buffer.
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
// double buffered in groups of G steps and a dead pair (odd pair count) is read from a zeroed LDS chunk so
// that no instruction has to touch a fragment between its load and its MFMA.  Integer dot products are order
// independent, so the assignment of pairs to lanes is free as long as both operands agree; the
// floating-point variants are compared against fp64 with the reference's DOT_PRODUCT bound.
//
// Zero points: sum((a-za)(w-zw)) = sum(a*w) - zw*sum(a) - za*sum(w) + K*za*zw.  sum(w) per channel is taken
// with v_dot4 against 0x01010101 from the registers that stage the weights, sum(a) per pixel from the patch
// chunks as they are staged (only when zw != 0; kept per patch pixel in LDS and summed over the window in
// the epilogue).
//
// Epilogue: the per-channel constants (bias, multiplier, shift and the 64-bit rounding terms derived from
// them) are computed once per workgroup by OCB lanes while the staging loads are in flight and kept in an
// LDS table; every lane then spends about ten instructions per output element.
#include <type_traits>

#include "tmi_mfma.h"

namespace tmi
{

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
    int32_t CH;                  // 16-byte chunks per pixel row in LDS (a power of two up to 16)
    int32_t ch_shift;            // log2(CH)
    int32_t pstride, wstride;    // LDS row strides in bytes, both = 16 (mod 32)
    int32_t n_icb;               // blocks of CH*16 bytes along the input channels
    int32_t ksteps;              // MFMA K-steps per channel block = ceil(taps*CH/2)
    int32_t n_tiles;             // N * tiles_y * tiles_x
    int32_t n_ocb;               // blocks of output channels
    int32_t out_dtype;
    int32_t xcd_remap;
    int32_t rounds;              // staging rounds per channel block
    int32_t pipelined;           // two LDS buffers, loads of the next block in flight during the MFMA loop
    int32_t buf_bytes;           // size of one LDS operand buffer (weight rows + patch)
    int64_t w_batch_stride;    // bytes between the weights of consecutive images (0: shared; MATMUL: per batch)
    FastDiv div_tw, div_pw, div_tiles_x, div_tiles_y, div_group, div_kw;
    int32_t row_words;         // channel vectors that are not whole 16-byte chunks but whole, aligned words: 8 or 4 (bytes), or 0
};

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

// The same for channel vectors made of whole 4-byte words at 4-byte aligned addresses (12, 20, 28 ... int8 channels, any
// even number of 16-bit ones) or whole 8-byte words (8, 24, 40, 72 ... int8 channels): a quarter and an eighth of the load
// instructions.
__device__ __forceinline__ v4i load_chunk_words(const uint8_t* row, int off, int row_bytes, int word)
{
    v4i r;
    if (word == 8)
    {
#pragma unroll
        for (int k = 0; k < 2; k++)
        {
            const v2i d = off + 8 * k < row_bytes ? *reinterpret_cast<const v2i*>(row + off + 8 * k) : v2i{ 0, 0 };
            r[2 * k] = d.x, r[2 * k + 1] = d.y;
        }
        return r;
    }
#pragma unroll
    for (int k = 0; k < 4; k++)
        r[k] = off + 4 * k < row_bytes ? *reinterpret_cast<const int*>(row + off + 4 * k) : 0;
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

// Per-lane chunk budget of one staging round (weights, patch) and K-loop group size of an instantiation.
template <int OCT, int PXT, bool MULTI>
struct TileTraits
{
    static constexpr bool big  = OCT * PXT >= 4;
    static constexpr bool huge = OCT * PXT >= 8;    // 128 accumulator registers: the staging budget shrinks
    static constexpr int WU    = huge ? 2 : 5;
    static constexpr int PU    = huge ? 4 : (big ? 8 : (MULTI ? 4 : 2));
    static constexpr int G     = big ? 1 : 3;
};

// Source descriptors of the staging: a byte offset below kFill is loaded, kFill is an out-of-image pixel
// (filled with input_zp), kNone reads as zero.  Tensors this kernel takes are smaller than kFill bytes.
static constexpr uint32_t kNone = 0xffffffffu;
static constexpr uint32_t kFill = 0xfffffffeu;

// MULTI: the input channels take more than one block (the block loop's bookkeeping is compiled in)
template <typename T, int WOC, int OCT, int PXT, int EPI, bool VEC, bool MULTI>
__global__ __launch_bounds__(512) void conv2d_patch_kernel(PatchArgs a)
{
    // The kernel arguments span several cache lines; the compiler fetches fields where they are first used,
    // which serialises one scalar-cache miss per line along the start-up path.  Asking for one field of every
    // line up front turns that into a single round trip.
    asm volatile("" ::"s"(a.g.N), "s"(a.g.bias_len), "s"(a.out), "s"(a.rp.shift), "s"(a.rp.lo), "s"(a.TH), "s"(a.CH),
                 "s"(a.n_tiles), "s"(a.rounds), "s"(a.w_batch_stride), "s"(a.div_tw.magic), "s"(a.div_kw.d));
    using M              = Mma<T>;
    using acc_t          = typename M::acc_t;
    using TT             = TileTraits<OCT, PXT, MULTI>;
    constexpr int EB     = sizeof(T);
    constexpr int NT     = 512;                // lanes per workgroup
    constexpr int WPX    = 8 / WOC;            // waves along the pixel dimension
    constexpr int OCB    = 32 * OCT * WOC;     // output channels per workgroup
    constexpr int WU     = TT::WU;             // weight chunks in flight per lane in one staging round
    constexpr int PU     = TT::PU;             // patch chunks in flight per lane in one staging round
    constexpr int LPR    = NT / OCB;           // lanes that share a weight row while staging: 4, 8 or 16
    const ConvGeom& g    = a.g;
    const int tid        = threadIdx.x;
    const int lane       = tid & 63;
    // wave-uniform values are made scalar explicitly: with two waves per SIMD the vector ALU (4 cycles per
    // wave64 instruction) is the scarce resource, so everything uniform must run on the scalar unit
    const int wave       = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int woc        = wave / WPX;   // first channel tile of this wave is woc*OCT
    const int wpx        = wave % WPX;   // first pixel tile of this wave is wpx*PXT
    const int li         = lane & 31;    // row of the A fragment / column (pixel) of D
    const int lh         = lane >> 5;    // K half taken by this lane / row half of D
    const int taps       = g.KH * g.KW;
    const int row_bytes  = g.IC * EB;    // bytes of one pixel's (or one weight tap's) channel vector
    const int blk_bytes  = a.CH * 16;
    const int ch_shift   = a.ch_shift;
    const int n_pairs    = taps * a.CH;  // (tap, chunk) pairs per channel block = chunks per weight row
    const int fill_word  = M::is_int ? (a.za & 0xff) * 0x01010101 : 0;    // out-of-image pixels hold input_zp

    // LDS: [channel table][16 zero bytes][check words][(multiplier, bias) table][1 KB dump area][pair offset table][patch byte sums]
    // [buffer 0][buffer 1 when pipelined], a buffer being the weight rows followed by the input patch
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    ChanEntry* ctab        = reinterpret_cast<ChanEntry*>(lds);
    float* ftab            = reinterpret_cast<float*>(lds);    // floating point: bias as float
    constexpr int kCtab    = OCB * (int)sizeof(ChanEntry);
    uint8_t* zero_chunk    = lds + kCtab;
    int* need_check        = reinterpret_cast<int*>(lds + kCtab + 16);    // per table wave: [0..1] some shift < 32,
                                                                          // [2..3] the wave's common shift or -1,
                                                                          // [4..5] output_zp is added after the shift
    int2* mbtab            = reinterpret_cast<int2*>(lds + kCtab + 48);    // per channel: multiplier, bias
    uint8_t* dump          = lds + kCtab + 48 + OCB * 8 + lane * 16;    // where staging work items without a destination write
    constexpr int kFixed   = kCtab + 48 + OCB * 8 + 1024;
    int* pairoff           = reinterpret_cast<int*>(lds + kFixed);
    const int tab_entries  = n_pairs + 32;    // slack: the pipeline reads up to 4G + 1 < 32 entries past the end
    const int tab_bytes    = (tab_entries * 4 + 15) & ~15;
    int* psum              = reinterpret_cast<int*>(lds + kFixed + tab_bytes);    // per patch pixel: sum of its bytes
    const int psum_bytes   = M::is_int ? ((a.PH * a.PW * 4 + 15) & ~15) : 0;
    uint8_t* buf0          = lds + kFixed + tab_bytes + psum_bytes;
    const int w_bytes      = OCB * a.wstride;

    // ---- which tile ------------------------------------------------------------------------------------
    uint32_t bid = blockIdx.x;
    if (a.xcd_remap)
    {
        // consecutive workgroups are dealt to the 8 XCDs in turn; give each XCD a contiguous run of tiles
        // so that neighbouring tiles (which share halo rows) share an L2
        const uint32_t per = gridDim.x >> 3;
        bid                = (bid & 7) * per + (bid >> 3);
    }
    // Grouped order: a run of kGroup pixel tiles times all channel blocks, the pixel tile running fastest.
    // The workgroups that are resident on an XCD together then share a few patches and a few weight blocks
    // instead of one weight block and many patches, which is what keeps GEMM-sized operands in L2.
    constexpr uint32_t kGroup = 4;
    const uint32_t grp        = fdiv(bid, a.div_group);
    const uint32_t first      = grp * kGroup;
    const uint32_t in_grp     = bid - grp * kGroup * a.n_ocb;
    const uint32_t rows       = a.n_tiles - first < kGroup ? a.n_tiles - first : kGroup;
    const uint32_t ocb        = rows == kGroup ? in_grp / kGroup : in_grp / rows;
    const uint32_t tile       = first + in_grp - ocb * rows;
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
    const uint8_t* w_n  = a.w + (size_t)n * a.w_batch_stride;                 // weights of this image
    const uint8_t* in_n = a.in + (size_t)n * g.IH * g.IW * row_bytes;        // this image

    // ---- per-lane pixel bases --------------------------------------------------------------------------
    int pidx[PXT];    // patch pixel under tap (0, 0) of this lane's output pixel
#pragma unroll
    for (int i = 0; i < PXT; i++)
    {
        int p = (wpx * PXT + i) * 32 + li;
        if (p >= P)
            p = 0;
        const int ty = fdiv(p, a.div_tw);
        pidx[i]      = ty * g.stride_y * a.PW + (p - ty * a.TW) * g.stride_x;
    }

    acc_t acc[PXT][OCT];
#pragma unroll
    for (int i = 0; i < PXT; i++)
#pragma unroll
        for (int t = 0; t < OCT; t++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][t][r] = 0;
    const bool wave_active = wpx * PXT * 32 < P;

    // ---- staging ---------------------------------------------------------------------------------------
    // A round moves up to WU weight chunks and PU patch chunks per lane: describe() works out where they come
    // from and go to (independent of the channel block), issue() starts the global loads of one channel block
    // and commit() writes them to an LDS buffer.  Nothing but the loads themselves hides memory latency inside
    // a round, so all of a round's loads are issued before any is used; in the VEC instantiation (channel
    // vectors are whole, aligned 16-byte chunks) they are unconditional: a work item without a source reads a
    // clamped, valid address and its result is replaced in commit(), which keeps the round free of branches.
    // Weight rows: LPR lanes share a row and walk its chunks, so no division is needed.
    const int w_ocl        = tid / LPR;
    const int w_part       = tid % LPR;
    const int w_r32        = w_ocl & 31;    // output channel -> row of the MFMA operand (see the header comment)
    const int w_row        = (w_ocl & ~31) + ((w_r32 >> 2) & 3) * 8 + (w_r32 >> 4) * 4 + (w_r32 & 3);
    const bool w_oc_ok     = oc0 + w_ocl < g.OC;
    const uint32_t w_src_row = (uint32_t)(oc0 + w_ocl) * (uint32_t)(taps * row_bytes);
    const int p_total      = a.PH * a.PW * a.CH;
    const int p_cc16       = (tid & (a.CH - 1)) * 16;    // NT is a multiple of CH: one chunk column per lane

    uint32_t wsrc[WU], psrc[PU];    // byte offsets of the sources (chunk column included), or kNone / kFill
    int wdst[WU], pdst[PU];         // byte offsets inside the weight rows / the patch, or -1
    int ppix[PU];                   // patch pixel of the slot, or -1
    v4i wv[WU], pv[PU];
    int wacc = 0;                   // byte sum of this lane's share of its weight row, over all blocks
    int pacc[PU];                   // byte sums of the lane's patch chunks over all blocks (one round per block only)
#pragma unroll
    for (int u = 0; u < PU; u++)
        pacc[u] = 0;

    // Single block, channel vector = block, one round: the (tap, chunk) pairs of a weight row are consecutive
    // 16-byte chunks in memory and in LDS, so the lane's slots are its first chunk plus compile-time offsets
    // and need no per-slot arithmetic; only the slot that straddles the end of the row tests its lanes.  Rows
    // past OC read row 0 of the block (valid memory) and are zeroed when written.
    const bool w_contig = !MULTI && VEC && a.rounds == 1 && row_bytes == blk_bytes;
    const int w_full    = n_pairs / LPR;    // slots in which every lane has a chunk
    const uint8_t* w_lane_src = w_n + (w_oc_ok ? w_src_row : (uint32_t)oc0 * (uint32_t)(taps * row_bytes)) + w_part * 16;
    const int w_lane_dst      = w_row * a.wstride + w_part * 16;
    auto issue_weights_contig = [&]() {
#pragma unroll
        for (int u = 0; u < WU; u++)
        {
            if (u < w_full)
                wv[u] = *reinterpret_cast<const v4i*>(w_lane_src + u * LPR * 16);
            else if (u * LPR < n_pairs)
                wv[u] = *reinterpret_cast<const v4i*>(w_lane_src + (w_part + u * LPR < n_pairs ? u * LPR * 16 : 0));
        }
    };
    auto commit_weights_contig = [&](uint8_t* wl) {
        const bool zero_rows = !__all(w_oc_ok);    // wave-uniform
#pragma unroll
        for (int u = 0; u < WU; u++)
        {
            if (u * LPR >= n_pairs)
                continue;
            v4i v = wv[u];
            if (zero_rows)
                v = w_oc_ok ? v : v4i{ 0, 0, 0, 0 };
            uint8_t* dst = wl + w_lane_dst + u * LPR * 16;
            if (u >= w_full)
            {
                const bool ok = w_part + u * LPR < n_pairs;
                v             = ok ? v : v4i{ 0, 0, 0, 0 };
                dst           = ok ? dst : dump;
            }
            *reinterpret_cast<v4i*>(dst) = v;
            if constexpr (M::is_int)
                if (a.za != 0)
                    wacc += dot4_ones(v);
        }
    };

    auto describe = [&](int round) {
#pragma unroll
        for (int u = 0; u < PU; u++)
        {
            const int idx  = tid + (round * PU + u) * NT;
            const bool ok  = idx < p_total;
            const int pix  = (ok ? idx : 0) >> ch_shift;
            const int py   = fdiv(pix, a.div_pw);
            const int px   = pix - py * a.PW;
            const int iy = y0 + py, ix = x0 + px;
            const bool img = iy >= 0 && iy < g.IH && ix >= 0 && ix < g.IW;
            ppix[u]        = ok ? pix : -1;
            pdst[u]        = ok ? pix * a.pstride + p_cc16 : -1;
            psrc[u]        = !ok ? kNone : (img ? (uint32_t)(iy * g.IW + ix) * (uint32_t)row_bytes + (uint32_t)p_cc16 : kFill);
        }
        if (w_contig)
            return;
#pragma unroll
        for (int u = 0; u < WU; u++)
        {
            const int j   = w_part + (round * WU + u) * LPR;    // (tap, chunk) pair inside the row
            const bool ok = j < n_pairs;
            const int jc  = ok ? j : 0;
            wdst[u]       = ok ? w_row * a.wstride + j * 16 : -1;
            wsrc[u]       = (ok && w_oc_ok)
                                ? w_src_row + (uint32_t)((jc >> ch_shift) * row_bytes + (jc & (a.CH - 1)) * 16)
                                : kNone;
        }
    };
    // chunk column (byte offset inside the channel block) of weight work item u of a round
    auto w_cc16 = [&](int round, int u) { return ((w_part + (round * WU + u) * LPR) & (a.CH - 1)) * 16; };
    // Per slot and wave: `void` if no lane has a destination (the slot is skipped), `plain` if every lane has a
    // source and a destination.  A plain slot of a channel block that lies wholly inside the channel vector
    // needs no per-item test: the load takes a scalar base plus the item's offset and the data goes to LDS as
    // it arrived.  The masks are wave-uniform; they are only known when a block is one round.
    uint32_t p_plain = 0, p_void = 0, w_plain = 0, w_void = 0;
    auto classify = [&]() {
#pragma unroll
        for (int u = 0; u < PU; u++)
        {
            p_plain |= (__all(psrc[u] < kFill) ? 1u : 0u) << u;
            p_void |= (__all(ppix[u] < 0) ? 1u : 0u) << u;
        }
#pragma unroll
        for (int u = 0; u < WU; u++)
        {
            w_plain |= (__all(wsrc[u] != kNone) ? 1u : 0u) << u;
            w_void |= (__all(wdst[u] < 0) ? 1u : 0u) << u;
        }
    };

    // `whole`: the channel block [ic_off, ic_off + blk_bytes) ends inside the channel vector
    auto issue = [&](int round, int ic_off, bool whole) {
        const uint8_t* pb = in_n + ic_off;
        const uint8_t* wb = w_n + ic_off;
#pragma unroll
        for (int u = 0; u < PU; u++)
        {
            if (MULTI && ((p_void >> u) & 1u))
                continue;
            if (MULTI && VEC && whole && ((p_plain >> u) & 1u))
            {
                pv[u] = *reinterpret_cast<const v4i*>(pb + psrc[u]);
                continue;
            }
            const bool in_row = ic_off + p_cc16 < row_bytes;
            if constexpr (VEC)
            {
                const bool ld = psrc[u] < kFill && in_row;
                pv[u]         = *reinterpret_cast<const v4i*>(in_n + (ld ? psrc[u] + (uint32_t)ic_off : 0u));
            }
            else
            {
                pv[u] = v4i{ 0, 0, 0, 0 };
                if (psrc[u] < kFill)
                    pv[u] = a.row_words ? load_chunk_words(in_n + (psrc[u] - p_cc16), ic_off + p_cc16, row_bytes, a.row_words)
                                        : load_chunk_bytes(in_n + (psrc[u] - p_cc16), ic_off + p_cc16, row_bytes);
                else if (psrc[u] == kFill)
                    pv[u] = fill_chunk(ic_off + p_cc16, row_bytes, M::is_int ? a.za : 0);
            }
        }
        if (w_contig)
            return;    // requested before anything else, see below
#pragma unroll
        for (int u = 0; u < WU; u++)
        {
            if (MULTI && ((w_void >> u) & 1u))
                continue;
            if (MULTI && VEC && whole && ((w_plain >> u) & 1u))
            {
                wv[u] = *reinterpret_cast<const v4i*>(wb + wsrc[u]);
                continue;
            }
            const int cc16 = w_cc16(round, u);
            if constexpr (VEC)
            {
                const bool ld = wsrc[u] != kNone && ic_off + cc16 < row_bytes;
                wv[u]         = *reinterpret_cast<const v4i*>(w_n + (ld ? wsrc[u] + (uint32_t)ic_off : 0u));
            }
            else
            {
                wv[u] = v4i{ 0, 0, 0, 0 };
                if (wsrc[u] != kNone)
                    wv[u] = a.row_words ? load_chunk_words(w_n + (wsrc[u] - cc16), ic_off + cc16, row_bytes, a.row_words)
                                        : load_chunk_bytes(w_n + (wsrc[u] - cc16), ic_off + cc16, row_bytes);
            }
        }
    };

    // Writes a round to LDS.  Work items without a destination write to the dump area, so a slot has no
    // divergent branch.  The byte sums for the zero-point correction are taken here, from the registers: sum(w)
    // of the lane's share of its weight row goes to wacc; with a non-zero weight zero point the byte sum of
    // every patch chunk goes to pacc (`defer`: one round per block, flushed to psum once after the last block)
    // or, when the slots change from round to round, straight to psum: the CH lanes that hold a pixel's chunks
    // add them up and the first of them owns the pixel's entry.
    auto commit = [&](int round, int ic_off, uint8_t* wl, uint8_t* pl, bool first_block, bool whole, bool defer) {
#pragma unroll
        for (int u = 0; u < PU; u++)
        {
            if (MULTI && ((p_void >> u) & 1u))
                continue;
            v4i v = pv[u];
            uint8_t* dst = pl + pdst[u];
            if (!(MULTI && whole && ((p_plain >> u) & 1u)))
            {
                if constexpr (VEC)
                {
                    const bool in_row = ic_off + p_cc16 < row_bytes;
                    const bool ld     = psrc[u] < kFill && in_row;
                    const int fw      = (psrc[u] == kFill && in_row) ? fill_word : 0;    // whole chunks only here
                    v                 = ld ? v : v4i{ fw, fw, fw, fw };
                }
                dst = pdst[u] >= 0 ? dst : dump;
            }
            *reinterpret_cast<v4i*>(dst) = v;
            if constexpr (M::is_int)
                if (a.zw != 0)
                {
                    int sum = dot4_ones(v);
                    if (defer)
                        pacc[u] += sum;
                    else
                    {
                        for (int m = 1; m < a.CH; m <<= 1)
                            sum += __shfl_xor(sum, m);
                        if (p_cc16 == 0 && ppix[u] >= 0)
                            psum[ppix[u]] = first_block ? sum : psum[ppix[u]] + sum;
                    }
                }
        }
        if (w_contig)
        {
            commit_weights_contig(wl);
            return;
        }
#pragma unroll
        for (int u = 0; u < WU; u++)
        {
            if (MULTI && ((w_void >> u) & 1u))
                continue;
            v4i v = wv[u];
            uint8_t* dst = wl + wdst[u];
            if (!(MULTI && whole && ((w_plain >> u) & 1u)))
            {
                if constexpr (VEC)
                {
                    const bool ld = wsrc[u] != kNone && ic_off + w_cc16(round, u) < row_bytes;
                    v             = ld ? v : v4i{ 0, 0, 0, 0 };
                }
                dst = wdst[u] >= 0 ? dst : dump;
            }
            *reinterpret_cast<v4i*>(dst) = v;
            if constexpr (M::is_int)
                if (a.za != 0)
                    wacc += dot4_ones(v);    // work items without a source hold zeros
        }
    };

    // The channel blocks are taken in an order rotated by the workgroup's position: workgroups that run side
    // by side would otherwise all read the same 16*CH-byte column of every row at the same time, which lands
    // on a fraction of the memory channels when the row length is a power of two.  (Integer sums do not depend
    // on the order; the floating-point bound holds for any order.)
    const int rot = MULTI ? (int)((tile + ocb) % (uint32_t)a.n_icb) : 0;
    auto block_offset = [&](int icb) {
        if constexpr (!MULTI)
            return 0;
        const int b = icb + rot;
        return (b >= a.n_icb ? b - a.n_icb : b) * blk_bytes;
    };

    // With one round per block the first block's loads are started before anything else, so that the table
    // set-up below (which has global loads of its own) runs in their shadow.
    const bool one_round = a.rounds == 1;
    // a block is whole when it ends inside the channel vector; only the last one in memory order may not be
    auto block_is_whole = [&](int off) { return off + blk_bytes <= row_bytes; };
    if (w_contig)
        issue_weights_contig();    // needs no per-slot arithmetic: in flight while the patch slots are worked out
    if (one_round)
    {
        describe(0);
        if constexpr (MULTI)
            classify();
        issue(0, block_offset(0), block_is_whole(block_offset(0)));
    }

    // ---- tables ----------------------------------------------------------------------------------------
    uint32_t flags = 0;
    if (tid < 4)
        reinterpret_cast<int*>(zero_chunk)[tid] = 0;
    // An odd pair count leaves the upper K half of the last step empty: the spare chunk behind every weight
    // row is zero, so that half contributes nothing whatever the pixel operand holds.
    if ((n_pairs & 1) && tid < OCB)
    {
        *reinterpret_cast<v4i*>(buf0 + tid * a.wstride + n_pairs * 16) = v4i{ 0, 0, 0, 0 };
        if (a.pipelined)
            *reinterpret_cast<v4i*>(buf0 + a.buf_bytes + tid * a.wstride + n_pairs * 16) = v4i{ 0, 0, 0, 0 };
    }
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
    if (tid < 128)    // the first two waves; OCB <= 128
    {
        const int oc  = oc0 + tid;
        const bool ok = oc < g.OC && tid < OCB;
        const int occ = ok ? oc : 0;    // clamped: the loads below are unconditional and issued together
        if constexpr (M::is_int)
        {
            const int32_t b_raw = reinterpret_cast<const int32_t*>(a.bias)[g.bias_len == 1 ? 0 : occ];
            ChanEntry e;
            e.m = 0, e.s = 32, e.lim = 0x80000000u, e.rnd_pos = e.rnd_neg = 0;
            if constexpr (EPI == EPI_FAST)
            {
                // the fast path has 32-bit multipliers; channels past OC get neutral constants (0, 32): every
                // value legal, nothing raised
                const int sc          = a.rp.per_channel ? occ : 0;
                const int32_t m_raw   = reinterpret_cast<const int32_t*>(a.rp.multiplier)[sc];
                const int32_t s_raw   = (int32_t)a.rp.shift[sc];
                // channels past OC take the shift of the wave's first channel, so that they do not break a block
                // whose channels all share one shift
                const int32_t s_first = __builtin_amdgcn_readfirstlane(ok ? s_raw : 32);
                const ChannelScale cs =
                    make_channel_scale(ok ? m_raw : 0, ok ? s_raw : s_first, a.rp.double_round, flags);
                // The output zero point rides in the rounding term where that cannot overflow (see
                // zp_fold_max_shift); if some channel of the wave has too large a shift for it, none of the wave's
                // channels folds and the epilogue adds output_zp after the shift.
                const int s_max       = zp_fold_max_shift(a.rp.out_zp);
                const int nofold      = __any(cs.s > s_max);
                const int64_t zp_term = nofold ? 0 : ((int64_t)a.rp.out_zp << cs.s);
                e.m = cs.m, e.s = cs.s, e.lim = cs.lim, e.rnd_pos = cs.rnd_pos + zp_term, e.rnd_neg = cs.rnd_neg + zp_term;
                // a shift below 32 somewhere: apply_scale_32's value range can be violated and must be checked.
                // One ballot per table wave; each wave's first lane writes that wave's word.
                const int any_check = __any(cs.lim != 0x80000000u);
                // One shift (of at least 32) for the whole wave: the epilogue then keeps the rounding terms in scalar
                // registers and reads 8 bytes per channel instead of 32.
                const int uni = __all(cs.s == s_first) && s_first >= 32 && s_first <= s_max;
                if (lane == 0)
                {
                    need_check[wave]     = any_check;
                    need_check[2 + wave] = uni ? s_first : -1;
                    need_check[4 + wave] = nofold;
                }
            }
            e.bias = ok ? b_raw : 0;
            if (tid < OCB)
            {
                ctab[tid]  = e;
                mbtab[tid] = int2{ e.m, e.bias };
            }
        }
        else if (tid < OCB)
            ftab[tid] = ok ? load_as_float<T>(a.bias, g.bias_len == 1 ? 0 : occ) : 0.0f;
    }

    const int n_icb = MULTI ? a.n_icb : 1;
    for (int icb = 0; icb < n_icb; icb++)
    {
        const int ic_off   = block_offset(icb);
        const bool whole   = block_is_whole(ic_off);
        uint8_t* wl        = buf0 + ((a.pipelined && (icb & 1)) ? a.buf_bytes : 0);
        uint8_t* pl        = wl + w_bytes;
        if (MULTI && a.pipelined)
        {
            // this block's chunks were requested one block ago; its buffer was last read two blocks ago, and
            // every wave has passed a barrier since
            commit(0, ic_off, wl, pl, icb == 0, whole, true);
        }
        else
        {
            if (icb)
                __syncthreads();    // every wave is done reading the buffer
            for (int round = 0; round < a.rounds; round++)
            {
                if (!one_round)
                    describe(round);
                if (!one_round || icb)
                    issue(round, ic_off, whole);
                commit(round, ic_off, wl, pl, icb == 0, whole, one_round);
            }
        }
        __syncthreads();

        if (MULTI && a.pipelined && icb + 1 < n_icb)
        {
            const int next = block_offset(icb + 1);
            issue(0, next, block_is_whole(next));
        }

        // ---- MFMA over the (tap, chunk) pairs of this channel block -----------------------------------
        if (wave_active)
        {
            // Double buffered in groups of G steps: at the top of a round the fragments of the next group are
            // requested (their patch offsets were read from the table one round earlier), then the current
            // group's MFMAs issue, so the wait in front of an MFMA only meets loads that have had a whole
            // group of matrix instructions to complete.  The main loop runs on whole pairs of groups and has no
            // branch in its body; what is left (fewer than 2G steps) goes through the checked tail.  Loads past
            // the last step are clamped to it and never used.  Nothing but loads and MFMAs is in the loop: the
            // zero-point sums are taken while staging.
            constexpr int G     = TT::G;
            const uint8_t* wrow = wl + (woc * OCT * 32 + li) * a.wstride + lh * 16;
            const int* tab      = pairoff + lh;
            const int last_step = a.ksteps - 1;
            const int wtile     = 32 * a.wstride;
            const uint8_t* prow[PXT];
#pragma unroll
            for (int i = 0; i < PXT; i++)
                prow[i] = pl + pidx[i] * a.pstride;
            v4i fa[2][G][OCT], fb[2][G][PXT];
            int po[G];
            auto load_group = [&](int s0, v4i(&ga)[G][OCT], v4i(&gb)[G][PXT]) {
#pragma unroll
                for (int u = 0; u < G; u++)
                {
                    const int sc = s0 + u < last_step ? s0 + u : last_step;
#pragma unroll
                    for (int t = 0; t < OCT; t++)
                        ga[u][t] = *reinterpret_cast<const v4i*>(wrow + t * wtile + sc * 32);
#pragma unroll
                    for (int i = 0; i < PXT; i++)
                        gb[u][i] = *reinterpret_cast<const v4i*>(prow[i] + po[u]);
                }
#pragma unroll
                for (int u = 0; u < G; u++)
                    po[u] = tab[2 * (s0 + G + u)];    // offsets of the group after that one
            };
            auto compute = [&](const v4i(&ga)[OCT], const v4i(&gb)[PXT]) {
#pragma unroll
                for (int i = 0; i < PXT; i++)
#pragma unroll
                    for (int t = 0; t < OCT; t++)
                        acc[i][t] = M::mma(ga[t], gb[i], acc[i][t]);
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
                    compute(fa[0][u], fb[0][u]);
                load_group(s + 2 * G, fa[0], fb[0]);
#pragma unroll
                for (int u = 0; u < G; u++)
                    compute(fa[1][u], fb[1][u]);
            }
            if (s < a.ksteps)
            {
                load_group(s + G, fa[1], fb[1]);
#pragma unroll
                for (int u = 0; u < G; u++)
                    if (s + u < a.ksteps)
                        compute(fa[0][u], fb[0][u]);
#pragma unroll
                for (int u = 0; u < G; u++)
                    if (s + G + u < a.ksteps)
                        compute(fa[1][u], fb[1][u]);
            }
        }
    }

    // ---- zero-point sums ---------------------------------------------------------------------------------
    // sum(w) per output channel: the LPR lanes that share a weight row finish its byte sum with a butterfly and
    // -za*sum(w) goes into the channel table's bias (one LDS atomic per row, all rows distinct; the table was
    // written before the first barrier).  sum(a) per patch pixel, when it was kept in registers: the CH lanes
    // that hold a pixel's chunks add up and the first writes the pixel's entry.  The barrier in the epilogue
    // makes both visible.
    if constexpr (M::is_int)
    {
        if (a.za != 0)
        {
            int sum = wacc;
#pragma unroll
            for (int m = 1; m < LPR; m <<= 1)
                sum += __shfl_xor(sum, m);
            if (w_part == 0)
            {
                atomicAdd(&ctab[w_ocl].bias, -a.za * sum);
                atomicAdd(&mbtab[w_ocl].y, -a.za * sum);
            }
        }
        if (a.zw != 0 && one_round)
        {
#pragma unroll
            for (int u = 0; u < PU; u++)
            {
                int sum = pacc[u];
                for (int m = 1; m < a.CH; m <<= 1)
                    sum += __shfl_xor(sum, m);
                if (p_cc16 == 0 && ppix[u] >= 0)
                    psum[ppix[u]] = sum;
            }
        }
    }

    // ---- epilogue -------------------------------------------------------------------------------------
    // per pixel tile: validity and output offset of this lane's pixel; in channel tile t the lane owns
    // channels [ocl0 + 32t, ocl0 + 32t + 16) of the block
    bool pix_ok[PXT];
    size_t obase[PXT];
    const int ocl0 = woc * OCT * 32 + 16 * lh;
#pragma unroll
    for (int i = 0; i < PXT; i++)
    {
        const int p  = (wpx * PXT + i) * 32 + li;
        const int ty = fdiv(p, a.div_tw);
        const int oy = oy0 + ty, ox = ox0 + (p - ty * a.TW);
        pix_ok[i]    = wave_active && p < P && oy < g.OH && ox < g.OW;
        obase[i]     = (((size_t)n * g.OH + oy) * g.OW + ox) * g.OC + oc0 + ocl0;
    }

    if constexpr (!M::is_int)
    {
        // floating point: out = bias + acc, rounded to the output type (16 channels = 32 bytes per pixel), or
        // kept in fp32 (MATMUL: 64 bytes per pixel)
#pragma unroll
        for (int t = 0; t < OCT; t++)
        {
            const int oclt     = ocl0 + 32 * t;
            const bool full    = (oc0 + oclt + 16 <= g.OC);
            const bool vec_out = full && (g.OC & 7) == 0 && ((uintptr_t)a.out & 15) == 0;
#pragma unroll
            for (int i = 0; i < PXT; i++)
            {
                if (a.out_dtype == TMI_FP32)
                {
                    float* o = reinterpret_cast<float*>(a.out) + obase[i] + 32 * t;
#pragma unroll
                    for (int q = 0; q < 4; q++)
                    {
                        const v4f b = *reinterpret_cast<const v4f*>(ftab + oclt + 4 * q);
                        v4f r;
#pragma unroll
                        for (int j = 0; j < 4; j++)
                            r[j] = b[j] + acc[i][t][4 * q + j];
                        if (!pix_ok[i])
                            continue;
                        if (vec_out)
                            *reinterpret_cast<v4f*>(o + 4 * q) = r;
                        else
#pragma unroll
                            for (int j = 0; j < 4; j++)
                                if (oc0 + oclt + 4 * q + j < g.OC)
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
                    const v4f b = *reinterpret_cast<const v4f*>(ftab + oclt + 4 * q);
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        store_from_float(&u.e[4 * q + r], b[r] + acc[i][t][4 * q + r]);
                }
                if (!pix_ok[i])
                    continue;
                T* o = reinterpret_cast<T*>(a.out) + obase[i] + 32 * t;
                if (vec_out)
                {
                    reinterpret_cast<v4i*>(o)[0] = u.v[0];
                    reinterpret_cast<v4i*>(o)[1] = u.v[1];
                }
                else
                {
#pragma unroll
                    for (int j = 0; j < 16; j++)
                        if (oc0 + oclt + j < g.OC)
                            o[j] = u.e[j];
                }
            }
        }
    }
    else
    {
        // the zero-point sums were written after the last block: make them visible to every wave
        if (a.za != 0 || a.zw != 0)
            __syncthreads();
        const int kzz = g.KH * g.KW * g.IC * a.za * a.zw;
        int pcorr[PXT];    // the zero-point terms that depend on the pixel only: K*za*zw - zw*sum(a)
#pragma unroll
        for (int i = 0; i < PXT; i++)
        {
            int sa = 0;
            if (a.zw != 0)    // sum(a) over the window of this pixel from the per-pixel byte sums
                for (int ky = 0; ky < g.KH; ky++)
                    for (int kx = 0; kx < g.KW; kx++)
                        sa += psum[pidx[i] + ky * g.dil_y * a.PW + kx * g.dil_x];
            pcorr[i] = kzz - a.zw * sa;
        }
        if constexpr (EPI == EPI_GENERIC)
            __syncthreads();    // every wave is done reading the operands: LDS becomes the staging area
        int32_t* stage = reinterpret_cast<int32_t*>(lds + kCtab);    // [pixel of the tile][channel of the block]
        bool check     = false;
        int s_uni      = -1;    // the block's common shift (>= 32), or -1
        if constexpr (EPI == EPI_FAST)
        {
            check        = (need_check[0] | need_check[1]) != 0;
            const int s0 = need_check[2], s1 = need_check[3];
            s_uni        = __builtin_amdgcn_readfirstlane((s0 >= 0 && (OCB <= 64 || s1 == s0)) ? s0 : -1);
        }
        // output_zp where the table wave of this wave's channels did not fold it into the rounding terms
        auto zp_after_shift = [&](int oclt) {
            if constexpr (EPI != EPI_FAST)
                return 0;
            return __builtin_amdgcn_readfirstlane(need_check[4 + (oclt >= 64 ? 1 : 0)] ? a.rp.out_zp : 0);
        };

#pragma unroll
        for (int t = 0; t < OCT; t++)
        {
            const int oclt  = ocl0 + 32 * t;
            const bool full = (oc0 + oclt + 16 <= g.OC);
            // int32 rows of four channels can be stored as one vector; int8 rows of 16 channels likewise
            const bool vec4  = full && (g.OC & 3) == 0 && ((uintptr_t)a.out & 15) == 0;
            const bool vec16 = full && (g.OC & 15) == 0 && ((uintptr_t)a.out & 15) == 0;
            int packed[PXT][4];    // int8 results, four channels per word

            // The common case -- RESCALE to int8, whole aligned 16-channel rows -- as straight-line code: about
            // ten vector instructions per element and no branch; `checked` adds apply_scale_32's value-range
            // test and is only taken when some channel's shift is below 32.
            const bool fast_i8 = EPI == EPI_FAST && a.out_dtype == TMI_INT8 && vec16;
            if constexpr (EPI == EPI_FAST)
            {
                if (fast_i8)
                {
                    auto rows = [&](auto checked_tag, auto pcorr_tag) {
                        const int zp_post      = zp_after_shift(oclt);
                        constexpr bool CHECKED = decltype(checked_tag)::value;
                        constexpr bool PCORR   = decltype(pcorr_tag)::value;    // weight_zp != 0
#pragma unroll
                        for (int q = 0; q < 4; q++)
                        {
                            ChanEntry ce[4];
#pragma unroll
                            for (int r = 0; r < 4; r++)
                                ce[r] = ctab[oclt + 4 * q + r];
#pragma unroll
                            for (int i = 0; i < PXT; i++)
                            {
                                int32_t res[4];
#pragma unroll
                                for (int r = 0; r < 4; r++)
                                {
                                    int32_t v = acc[i][t][4 * q + r] + ce[r].bias;
                                    if constexpr (PCORR)
                                        v += pcorr[i];
                                    if constexpr (CHECKED)
                                        if ((uint32_t)v + ce[r].lim > 2u * ce[r].lim - 1u && pix_ok[i])
                                            flags |= TMI_FLAG_SCALE_VALUE;    // pixels outside the image raise nothing
                                    const int64_t pr =
                                        (int64_t)v * (int64_t)ce[r].m + (v >= 0 ? ce[r].rnd_pos : ce[r].rnd_neg);
                                    res[r] = clamp_med3((int32_t)(pr >> ce[r].s) + zp_post, a.rp.lo, a.rp.hi);
                                }
                                // the low bytes of four clamped values into one word
                                const int lo2 = __builtin_amdgcn_perm(res[1], res[0], 0x0c0c0400);
                                const int hi2 = __builtin_amdgcn_perm(res[3], res[2], 0x04000c0c);
                                packed[i][q]  = lo2 | hi2;
                            }
                        }
                    };
                    // every channel of the block has the same shift s >= 32: the rounding terms are scalars, the
                    // result is the high word of the product shifted by s - 32, and no value-range test applies
                    auto rows_uni = [&](auto pcorr_tag) {
                        constexpr bool PCORR = decltype(pcorr_tag)::value;
                        const int64_t dr     = a.rp.double_round ? (int64_t(1) << 30) : 0;
                        const int64_t rp     = (int64_t(1) << (s_uni - 1)) + dr + ((int64_t)a.rp.out_zp << s_uni);
                        const int64_t rn     = rp - 2 * dr;
                        const int sh         = s_uni - 32;
#pragma unroll
                        for (int q = 0; q < 4; q++)
                        {
                            int2 mb[4];
#pragma unroll
                            for (int r = 0; r < 4; r++)
                                mb[r] = mbtab[oclt + 4 * q + r];
#pragma unroll
                            for (int i = 0; i < PXT; i++)
                            {
                                int32_t res[4];
#pragma unroll
                                for (int r = 0; r < 4; r++)
                                {
                                    int32_t v = acc[i][t][4 * q + r] + mb[r].y;
                                    if constexpr (PCORR)
                                        v += pcorr[i];
                                    const int64_t pr = (int64_t)v * (int64_t)mb[r].x + (v >= 0 ? rp : rn);
                                    res[r]           = clamp_med3((int32_t)(pr >> 32) >> sh, a.rp.lo, a.rp.hi);
                                }
                                const int lo2 = __builtin_amdgcn_perm(res[1], res[0], 0x0c0c0400);
                                const int hi2 = __builtin_amdgcn_perm(res[3], res[2], 0x04000c0c);
                                packed[i][q]  = lo2 | hi2;
                            }
                        }
                    };
                    if (s_uni >= 0 && a.zw != 0)
                        rows_uni(std::true_type{});
                    else if (s_uni >= 0)
                        rows_uni(std::false_type{});
                    else if (check && a.zw != 0)
                        rows(std::true_type{}, std::true_type{});
                    else if (check)
                        rows(std::true_type{}, std::false_type{});
                    else if (a.zw != 0)
                        rows(std::false_type{}, std::true_type{});
                    else
                        rows(std::false_type{}, std::false_type{});
                }
            }

            // every other combination: four channels at a time, constants fetched once and used for every pixel
            if (!fast_i8)
#pragma unroll
                for (int q = 0; q < 4; q++)
                {
                    const int c0 = oc0 + oclt + 4 * q;
                    ChanEntry ce[4];
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        ce[r] = ctab[oclt + 4 * q + r];
#pragma unroll
                    for (int i = 0; i < PXT; i++)
                    {
                        int32_t res[4];
#pragma unroll
                        for (int r = 0; r < 4; r++)
                        {
                            int32_t v = acc[i][t][4 * q + r] + pcorr[i] + ce[r].bias;    // bias minus za*sum(w)
                            if constexpr (EPI == EPI_FAST)
                            {
                                if ((uint32_t)v + ce[r].lim > 2u * ce[r].lim - 1u && pix_ok[i])
                                    flags |= TMI_FLAG_SCALE_VALUE;    // pixels outside the image raise nothing
                                const int64_t pr =
                                    (int64_t)v * (int64_t)ce[r].m + (v >= 0 ? ce[r].rnd_pos : ce[r].rnd_neg);
                                v = (int32_t)(pr >> ce[r].s) + zp_after_shift(oclt);    // output_zp: in the rounding term, or here
                                v = v < a.rp.lo ? a.rp.lo : v;
                                v = v > a.rp.hi ? a.rp.hi : v;
                            }
                            res[r] = v;
                        }
                        if constexpr (EPI == EPI_GENERIC)
                        {
                            const int p = (wpx * PXT + i) * 32 + li;
                            if (wave_active && p < P)
                                *reinterpret_cast<v4i*>(stage + (size_t)p * OCB + oclt + 4 * q) =
                                    v4i{ res[0], res[1], res[2], res[3] };
                            continue;
                        }
                        if (!pix_ok[i])
                            continue;
                        if (EPI == EPI_PLAIN || a.out_dtype == TMI_INT32)
                        {
                            int32_t* o = reinterpret_cast<int32_t*>(a.out) + obase[i] + 32 * t + 4 * q;
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
                                int8_t* o = reinterpret_cast<int8_t*>(a.out) + obase[i] + 32 * t + 4 * q;
#pragma unroll
                                for (int r = 0; r < 4; r++)
                                    if (c0 + r < g.OC)
                                        o[r] = (int8_t)res[r];
                            }
                        }
                        else
                        {
                            int16_t* o = reinterpret_cast<int16_t*>(a.out) + obase[i] + 32 * t + 4 * q;
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
                            *reinterpret_cast<v4i*>(reinterpret_cast<int8_t*>(a.out) + obase[i] + 32 * t) =
                                v4i{ packed[i][0], packed[i][1], packed[i][2], packed[i][3] };
                }
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
static constexpr int kCUs    = 256;

template <typename T, int WOC, int OCT, int PXT, int EPI, bool VEC, bool MULTI>
static bool launch_patch(hipStream_t st, PatchArgs& a, size_t lds_bytes, int blocks)
{
    auto kern                = conv2d_patch_kernel<T, WOC, OCT, PXT, EPI, VEC, MULTI>;
    static LdsLimit granted{};
    if (!ensure_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, granted))
        return false;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(512), lds_bytes, st, a);
    return true;
}

static int ceil_div(int a, int b)
{
    return (a + b - 1) / b;
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
    const int taps = g.KH * g.KW;
    // the staging addresses one image and one image's weights with 32-bit byte offsets
    if ((int64_t)g.IH * g.IW * row_bytes >= 0xfffffff0ll || (int64_t)g.OC * taps * row_bytes >= 0xfffffff0ll)
        return nullptr;

    PatchArgs a{};
    a.g = g, a.in = (const uint8_t*)in, a.w = (const uint8_t*)w, a.bias = bias, a.out = out;
    a.flag_word = flag_word, a.rp = rp, a.za = in_zp, a.zw = w_zp, a.out_dtype = out_dtype;
    a.w_batch_stride = w_batch_stride;

    // channel vectors made of whole, aligned 16-byte chunks take the branch-free staging path
    const bool vec = (row_bytes & 15) == 0 && (((uintptr_t)in | (uintptr_t)w) & 15) == 0;
    const uintptr_t align = (uintptr_t)row_bytes | (uintptr_t)in | (uintptr_t)w | (uintptr_t)w_batch_stride;
    a.row_words           = vec ? 0 : ((align & 7) == 0 ? 8 : ((align & 3) == 0 ? 4 : 0));

    // ---- workgroup shape: WOC x OCT channel tiles, PXT pixel tiles per wave -------------------------------
    // Each candidate is priced in SIMD cycles: rounds of workgroups over the CUs times (MFMA time of one
    // workgroup + the cost of staging its operands + a fixed start-up); the cheapest wins.  The pixel tile
    // prefers full output rows and spreads the rows evenly over the tiles.
    const int WOC = g.OC > 32 ? 2 : 1;
    auto tile_for = [&](int max_px, int& TH, int& TW) {
        TW = g.OW < max_px ? g.OW : max_px;
        TW = ceil_div(g.OW, ceil_div(g.OW, TW));
        TH = max_px / TW;
        if (TH > g.OH)
            TH = g.OH;
        if (TH < 1)
            TH = 1;
        TH = ceil_div(g.OH, ceil_div(g.OH, TH));
    };
    int OCT = 1, PXT = 1;
    if (vec)
    {
        static const int cand[4][2] = { { 1, 1 }, { 1, 2 }, { 2, 2 }, { 2, 4 } };
        double best = 0;
        for (int c = 0; c < 4; c++)
        {
            const int oct = cand[c][0], pxt = cand[c][1];
            if (oct == 2 && g.OC <= 64)
                continue;
            // with the fused fast RESCALE the four- and eight-tile shapes do not fit the register file (320 and 576
            // bytes of scratch per lane, and a kernel with a scratch segment ran 2.4 times as long as the plain one)
            if (oct == 2 && rp.enabled && rp.fast)
                continue;
            const int ocb = 32 * oct * WOC, max_px = 32 * (8 / WOC) * pxt;
            int th, tw;
            tile_for(max_px, th, tw);
            const double wgs    = (double)g.N * ceil_div(g.OH, th) * ceil_div(g.OW, tw) * ceil_div(g.OC, ocb);
            const double rounds = (double)(int64_t)((wgs + kCUs - 1) / kCUs);
            const double ksteps = (double)taps * ceil_div(row_bytes, 32);             // 32 bytes of K per MFMA and lane half
            const double mfma   = 2.0 * oct * pxt * ksteps * 32;                      // two waves per SIMD
            const double stage  = (double)(ocb + max_px) * taps * row_bytes / 16 / 512 * 2 * 40;
            const double cost   = rounds * (mfma + stage + 3000);
            if (c == 0 || cost < best)
                best = cost, OCT = oct, PXT = pxt;
        }
    }
    const int OCB           = 32 * OCT * WOC;
    const int64_t oc_blocks = (g.OC + OCB - 1) / OCB;
    const int max_px        = 32 * (8 / WOC) * PXT;
    const int WU = OCT * PXT >= 8 ? 2 : 5;              // the values of TileTraits<OCT, PXT, n_icb > 1>
    auto PU_for  = [&](int n_icb) { return OCT * PXT >= 8 ? 4 : ((OCT * PXT >= 4) ? 8 : (n_icb > 1 ? 4 : 2)); };
    const int LPR = 512 / OCB;
    int TH, TW;
    tile_for(max_px, TH, TW);

    // ---- channel block ------------------------------------------------------------------------------------
    // Candidates from the largest block down.  A single block that covers the whole channel vector is staged
    // in rounds into one buffer; several blocks are software pipelined over two LDS buffers when a block fits
    // one staging round per lane.  If no candidate qualifies, blocks of at most 64 bytes go through a single
    // buffer one after the other, with the tile shrunk until it fits.
    const int ch_needed = row_bytes <= 16 ? 1 : (row_bytes <= 32 ? 2 : (row_bytes <= 64 ? 4 : (row_bytes <= 128 ? 8 : 16)));
    auto set_block = [&](int CH) {
        a.CH       = CH;
        a.ch_shift = CH == 16 ? 4 : (CH == 8 ? 3 : (CH == 4 ? 2 : (CH == 2 ? 1 : 0)));
        a.pstride  = CH == 1 ? 16 : CH * 16 + 16;    // all = 16 (mod 32)
        a.n_icb    = ceil_div(row_bytes, CH * 16);
        const int rch = taps * CH;                   // chunks per weight row
        a.wstride  = (rch + (rch & 1)) * 16 + 16;    // room for a spare zero chunk; = 16 (mod 32)
        a.ksteps   = (rch + 1) / 2;
    };
    auto fixed_bytes = [&]() {    // channel table, zero chunk, check words, (multiplier, bias) table, dump area, pair
                                  // table, patch byte sums
        return (size_t)OCB * 32 + 48 + (size_t)OCB * 8 + 1024 + ((((size_t)taps * a.CH + 32) * 4 + 15) & ~(size_t)15) +
               (Mma<T>::is_int ? (((size_t)a.PH * a.PW * 4 + 15) & ~(size_t)15) : 0);
    };
    auto buf_bytes   = [&]() { return (size_t)OCB * a.wstride + (size_t)a.PH * a.PW * a.pstride; };
    auto set_patch   = [&]() {
        a.PH = (TH - 1) * g.stride_y + (g.KH - 1) * g.dil_y + 1;
        a.PW = (TW - 1) * g.stride_x + (g.KW - 1) * g.dil_x + 1;
    };
    auto set_rounds = [&]() {
        const int w_rounds = ceil_div(ceil_div(taps * a.CH, LPR), WU);
        const int p_rounds = ceil_div(ceil_div(a.PH * a.PW * a.CH, 512), PU_for(a.n_icb));
        a.rounds           = w_rounds > p_rounds ? w_rounds : p_rounds;
    };
    set_patch();
    size_t lds_bytes = 0;
    bool chosen      = false;
    if (vec)
        for (int CH = ch_needed; CH >= 1 && !chosen; CH >>= 1)
        {
            set_block(CH);
            set_rounds();
            if (a.n_icb == 1)
            {
                lds_bytes = fixed_bytes() + buf_bytes();
                if (lds_bytes <= (size_t)kMaxLds)
                    a.pipelined = 0, chosen = true;
                continue;
            }
            if (a.rounds > 1)
                continue;
            lds_bytes = fixed_bytes() + 2 * buf_bytes();
            if (lds_bytes <= (size_t)kMaxLds)
                a.pipelined = 1, chosen = true;
        }
    if (!chosen)
    {
        set_block(ch_needed > 4 ? 4 : ch_needed);
        for (;;)
        {
            set_patch();
            lds_bytes = fixed_bytes() + buf_bytes();
            if (lds_bytes <= (size_t)kMaxLds)
                break;
            if (TH > 1)
                TH = (TH + 1) / 2;
            else if (TW > 16)
                TW = (TW + 1) / 2;
            else
                return nullptr;    // the weight slab alone does not fit: not eligible
        }
        a.pipelined = 0;
        set_rounds();
    }
    a.buf_bytes = (int)buf_bytes();
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
    a.div_tiles_x = make_fastdiv(a.tiles_x);
    a.div_tiles_y = make_fastdiv(a.tiles_y);
    a.n_ocb       = (int)oc_blocks;
    a.div_group   = make_fastdiv(4 * a.n_ocb);    // kGroup of the kernel
    a.div_kw      = make_fastdiv(g.KW);
    // fdiv is exact for n*d < 2^32: every dividend but the block index is bounded by the LDS capacity;
    // guard the products that involve the block index
    if ((uint64_t)blocks * (uint64_t)(4 * oc_blocks) >= (uint64_t(1) << 32) ||
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
#define TMI_PATCH_CASE(O, C, P, E)                                                                                   \
    if (WOC == O && OCT == C && PXT == P && epi == E)                                                                \
        ok = a.n_icb > 1 ? launch_patch<T, O, C, P, E, true, true>(st, a, lds_bytes, (int)blocks)                      \
                         : launch_patch<T, O, C, P, E, true, false>(st, a, lds_bytes, (int)blocks);
#define TMI_PATCH_CASE_BYTES(O, E)                                                                                   \
    if (WOC == O && epi == E)                                                                                        \
        ok = a.n_icb > 1 ? launch_patch<T, O, 1, 1, E, false, true>(st, a, lds_bytes, (int)blocks)                     \
                         : launch_patch<T, O, 1, 1, E, false, false>(st, a, lds_bytes, (int)blocks);
#define TMI_PATCH_SHAPES(E)                                                                                          \
    TMI_PATCH_CASE(1, 1, 1, E)                                                                                       \
    TMI_PATCH_CASE(1, 1, 2, E)                                                                                       \
    TMI_PATCH_CASE(2, 1, 1, E)                                                                                       \
    TMI_PATCH_CASE(2, 1, 2, E)                                                                                       \
    TMI_PATCH_CASE(2, 2, 2, E)                                                                                       \
    TMI_PATCH_CASE(2, 2, 4, E)
    if (vec)
    {
        TMI_PATCH_SHAPES(EPI_PLAIN)
        if constexpr (Mma<T>::is_int)
        {
            TMI_PATCH_CASE(1, 1, 1, EPI_FAST)
            TMI_PATCH_CASE(1, 1, 2, EPI_FAST)
            TMI_PATCH_CASE(2, 1, 1, EPI_FAST)
            TMI_PATCH_CASE(2, 1, 2, EPI_FAST)
            TMI_PATCH_SHAPES(EPI_GENERIC)
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
#undef TMI_PATCH_SHAPES
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
