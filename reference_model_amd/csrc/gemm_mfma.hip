// CONV2D as a GEMM over (ky, kx, ic) and MATMUL on the matrix cores, for work large enough that operand
// delivery, not set-up, decides the time.
//
//   out[b][p][oc] = sum_k (a[b][p][k] - za) * (w[b][oc][k] - zw) + bias[oc]
//
// (tensor_ops.cpp:843-882 with one tap; tensor_ops.cpp:1463-1500 for MATMUL, whose second operand arrives
// with K contiguous.)  Both operands are rows of kb = K * sizeof(element) bytes, kb a multiple of 64.
//
// A workgroup of 8 waves (2 along the output channels x 4 along the pixels) owns a tile of 64*OCT channels x
// 128*PXT pixels; a wave owns OCT x PXT accumulator tiles of 32x32.  K is walked in blocks of 64 bytes per
// row.  The operands of a block go from global memory straight into LDS (global_load_lds_dwordx4: no
// staging registers, no LDS store instructions), into a ring of stage buffers, so the loads of the next blocks
// are in flight while one is multiplied; one barrier per block both publishes a stage and frees the one the
// next loads will overwrite.  Where the ring can be six or eight stages long and K is deep, the blocks are
// requested two at a time - the two 64-byte halves of a row's 128-byte line back to back, which the L1 merges
// into one request to L2 - with one barrier per pair.
//
// LDS layout of a stage: row r (weight rows first, then pixel rows) occupies bytes [64r, 64r + 64); its four
// 16-byte chunks are stored permuted, chunk c at position c ^ swz(r), so that the 16 lanes the LDS serves in
// one cycle, which read the same chunk of 16 different rows, hit 16 different bank groups.  A direct load writes
// LDS at base + 16 * lane, so lane l of a load serves row l / 4 of a 16-row group and position l % 4, and
// fetches chunk (l % 4) ^ swz(row) from global memory: the permutation costs nothing.
//
// Accumulator rows are assigned to channels as in the patch kernel: row 8q + 4h' + j of a channel tile is
// channel 16h' + 4q + j, which makes every lane own 16 consecutive channels of one pixel.
//
// Zero points (int8): sum(a*w) - zw*sum(a) - za*sum(w) + K*za*zw.  The sums are taken with v_dot4 from the
// fragments as they pass through registers on their way to the matrix core (only in the ZP instantiation).
#include "tmi_mfma.h"
#include <type_traits>

namespace tmi
{

struct GemmArgs
{
    const uint8_t* a;    // pixel operand, rows of kb bytes
    const uint8_t* w;    // weight operand, rows of kb bytes
    const void* bias;
    void* out;
    int64_t a_batch, w_batch, o_batch;    // bytes between batches
    int32_t M, N;                         // pixel rows per batch, weight rows
    int32_t kb;                           // bytes per row
    int32_t n_blocks;                     // kb / 64
    int32_t tiles_n, tiles_per_batch, tiles_total, per_xcd;
    int32_t bias_len, za, zw, K;
    int32_t out_is_wide;    // floating point: 1 = fp32 output, 0 = output of the input type
    RescaleParams rp;       // int8: the fused RESCALE (+ CLAMP) when enabled, through fast_rescale()
    uint32_t* flag_word;    // where its REQUIRE conditions are latched
    int32_t out_bytes;      // fused RESCALE: 1 (int8 results) or 2 (int16)
    int32_t ldw;            // K-major weights: bytes between consecutive K rows (rows of N elements)
    // implicit GEMM of a KH x KW convolution: the K axis is (ky, kx, ic), a 64-byte block lies inside one tap
    const uint8_t* pad_page;    // 64 bytes of input_zp (zeros for floating point): what a tap outside the image reads
    int32_t IH, IW, OH, OW, KW, taps;
    int32_t icb;                 // bytes of one input pixel (IC * sizeof(element)), a multiple of 64
    int32_t bpt;                 // blocks per tap = icb / 64
    int32_t sy, sx, dy, dx, pad_top, pad_left;
    FastDiv div_bpt, div_kw;
    FastDiv div_batch, div_tn;
    // patch mode: a tile is rows_per_tile whole output rows of one image; its input patch stays in LDS
    int32_t rows_per_tile, tiles_per_image;
    int32_t patch_w, patch_pixels;    // patch width in pixels, pixels of the patch
    int32_t patch_units;              // 64-byte units of the patch = bpt * patch_pixels
    int32_t patch_bytes;              // LDS the patch takes
    FastDiv div_tpi, div_pw, div_ppix, div_ow;
};


// Bank-group permutation of a stage row.  A ds_read_b128 is served 16 lanes a cycle, and the 16 are not
// consecutive: within each half wave the quads (4 lanes) {0,3,5,6} go together and the quads {1,2,4,7}
// (measured with two active lanes reading one bank group at different addresses).  Lane rho of a half reads
// row rho (pixels) or channel_of_row(rho) (weights) of a 32-row tile, so the four rows of a quad already
// differ in row % 4, i.e. in which 64 of the 256 bank bytes they use; (row / 8) % 4 separates the four quads
// of either set for both row assignments.
__device__ __forceinline__ int swz(int r)
{
    return (r >> 3) & 3;
}

// accumulator row -> channel of its tile
__device__ __forceinline__ int channel_of_row(int rho)
{
    return 16 * ((rho >> 2) & 1) + 4 * (rho >> 3) + (rho & 3);
}

// Stage buffers of a workgroup: four 64-byte blocks per row.  The 256x256 shape fills the LDS with them; two
// workgroups of a smaller shape with three stages each were measured and are slower (the operand traffic per
// matrix instruction, not the barrier, is what the smaller shapes wait for).
static constexpr int kStagesDefault = 4;

// K-major weights (KM): the weight operand lies in memory as [K][N] (MATMUL's second operand as the operator
// defines it).  Its part of a stage is then 64 / sizeof(T) rows of K with the tile's 64*OCT channels side by
// side, loaded as it lies (whole 16-byte pieces of a K row per lane), and the fragments come out of LDS through
// the transposing reads ds_read_b64_tr_b16 / _b8: a block of 16 lanes hands in 16 addresses of 8 bytes and
// gets back, per lane, the elements of one column - 4 consecutive K of one channel (2-byte types) or 8 (int8) -
// so two reads make the 16 bytes of K a lane feeds the matrix instruction.  A transposing read serves 32
// lanes a cycle; their addresses are 4 (8) consecutive K rows x 64 (32) bytes, which the row stride alone
// would put on the same banks, so the 64-byte (32-byte) segments of a row are permuted by the row number.
// With int8 the 8 lanes that share a source address get 8 consecutive channels, so the accumulator rows of
// the int8 K-major variant are assigned to channels in order (row r is channel r) and a lane stores four
// groups of 4 channels instead of 16 consecutive ones.
//
// Convolutions with taps (MODE 2): the pixel operand's row p of K block b is the 64-byte piece b % bpt of input
// pixel (oy*sy - pad + ky*dy, ox*sx - pad + kx*dx) for tap (ky, kx) = b / bpt of output pixel p: the same
// direct load with a per-lane pixel offset worked out once, a per-block tap offset in scalar registers, and
// the 64-byte zero page as the source where the tap falls outside the image (a bit per tap and lane).
enum
{
    GEMM_KCONTIG = 0,
    GEMM_KMAJOR  = 1,
    GEMM_TAPS    = 2,
    GEMM_PATCH   = 3
};

enum
{
    PIPE_SINGLE     = 0,    // a ring of kStages stages, one 64-byte block requested per block period
    PIPE_PAIRS      = 1,    // a ring of six or eight stages, two blocks requested every second period
    PIPE_PIXEL_PAIRS = 2    // K-major weights: four stages of weight rows, three slots of two blocks of pixel rows
};

template <typename T, int OCT, int PXT, bool ZP, int MODE, int kStages, int PIPE>
__global__ __launch_bounds__(512) void gemm_lds_kernel(GemmArgs a)
{
    constexpr bool PAIR    = PIPE == PIPE_PAIRS;
    constexpr bool APAIR   = PIPE == PIPE_PIXEL_PAIRS;
    static_assert(!PAIR || (kStages >= 6 && kStages % 2 == 0), "pairs of blocks need an even ring of six stages or more");
    static_assert(!APAIR || (MODE == GEMM_KMAJOR && kStages == 4), "pixel pairs: K-major weights in a ring of four");
    constexpr bool KM      = MODE == GEMM_KMAJOR;
    constexpr bool TAPS    = MODE == GEMM_TAPS;
    // PATCH: a convolution with taps whose tile is whole output rows of one image.  The input patch under the tile
    // (with its halo; pixels outside the image come from the page of input_zp bytes) is fetched once, as planes of
    // 64-byte pieces, and stays in LDS behind the ring; the ring holds weight rows only, and the pixel fragments of
    // block (tap, piece) are read from plane `piece` at the tap's offset.
    constexpr bool PATCH   = MODE == GEMM_PATCH;
    static_assert(!PATCH || (PIPE == PIPE_PAIRS && PXT == 1), "the patch form: pairs of weight blocks, 128 pixel rows");
    using M                = Mma<T>;
    constexpr int EB       = (int)sizeof(T);
    constexpr bool IDENT   = KM && EB == 1;    // accumulator row r of a channel tile is channel r
    constexpr int RB       = 64 * OCT * EB;    // KM: bytes of a K row in LDS
    constexpr int KSTEP    = 32 / EB;          // K rows per matrix instruction
    // KM: units of 16 bytes a row's pieces are moved by, as a function of the K row
    auto km_swizzle = [](int k) {
        if constexpr (EB == 2)
            return (k & 3) << 2;
        else if constexpr (RB >= 256)
            return (k & 7) << 1;
        else
            return ((k >> 1) & 3) << 1;
    };
    auto row_channel = [](int r) { return IDENT ? r : channel_of_row(r); };
    using acc_t            = typename M::acc_t;
    constexpr int WROWS    = 64 * OCT;
    constexpr int PROWS    = 128 * PXT;
    constexpr int ROWS     = PATCH ? WROWS : WROWS + PROWS;    // rows of a ring stage
    constexpr int STAGE    = ROWS * 64;
    constexpr int LOADS    = ROWS / 128;    // direct loads per wave and block (16 rows each)
    constexpr int WLOADS   = WROWS / 128;   // of which carry weight rows
    constexpr int PLOADS   = LOADS - WLOADS;
    static_assert(ROWS % 128 == 0, "a block must split evenly over the 8 waves");
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rho  = lane & 31;
    const int h    = lane >> 5;
    const int wo   = wave & 1;
    const int wp   = wave >> 1;

    // Workgroups are dealt round-robin to the 8 XCDs; each XCD takes a contiguous range of the tile list
    // (tiles with the same pixel rows are neighbours) so that its L2 sees every operand row few times.
    const int xcd  = blockIdx.x & 7;
    const int slot = blockIdx.x >> 3;
    const int L    = xcd * a.per_xcd + slot;
    if (L >= a.tiles_total)
        return;
    const int batch = (int)fdiv((uint32_t)L, a.div_batch);
    const int rem   = L - batch * a.tiles_per_batch;
    const int tm    = (int)fdiv((uint32_t)rem, a.div_tn);
    const int tn    = rem - tm * a.tiles_n;
    int p0          = tm * PROWS;
    int m_end       = a.M;    // pixel rows of the tile end here
    int patch_n = 0, patch_oy0 = 0;
    if constexpr (PATCH)
    {
        patch_n             = (int)fdiv((uint32_t)tm, a.div_tpi);
        patch_oy0           = (tm - patch_n * a.tiles_per_image) * a.rows_per_tile;
        const int rows_here = a.OH - patch_oy0 < a.rows_per_tile ? a.OH - patch_oy0 : a.rows_per_tile;
        p0                  = (patch_n * a.OH + patch_oy0) * a.OW;
        m_end               = p0 + rows_here * a.OW;
    }
    const int oc0   = tn * WROWS;

    const uint8_t* a_base = a.a + batch * a.a_batch;
    const uint8_t* w_base = a.w + batch * a.w_batch;

    // ---- direct loads: per lane one byte offset per load, constant over the blocks ------------------------
    uint32_t voff[LOADS];
    const uint8_t* gbase[LOADS];
    uint32_t ldst[LOADS];
    uint32_t gstep[LOADS];    // bytes a load's source advances per block
#pragma unroll
    for (int j = 0; j < LOADS; j++)
    {
        const int grp   = j * 8 + wave;    // 16-row group of the stage
        const int r     = grp * 16 + (lane >> 2);
        const bool is_w = grp * 16 < WROWS;
        int row         = is_w ? oc0 + r : p0 + r - WROWS;
        const int last  = (is_w ? a.N : a.M) - 1;
        row             = row < last ? row : last;    // rows past the end repeat the last one; never stored
        voff[j]         = (uint32_t)row * (uint32_t)a.kb + (uint32_t)(((lane & 3) ^ swz(r)) * 16);
        gbase[j]        = is_w ? w_base : a_base;
        gstep[j]        = 64;
        if (KM && is_w)
        {
            // 16-byte unit of the weight part -> K row of the block and piece of that row
            const int unit = grp * 64 + lane;
            const int k    = unit / (RB / 16);
            const int pc   = (unit % (RB / 16)) ^ km_swizzle(k);
            int col        = oc0 * EB + pc * 16;
            col            = col < a.N * EB - 16 ? col : a.N * EB - 16;    // pieces past the row end: never used
            voff[j]        = (uint32_t)k * (uint32_t)a.ldw + (uint32_t)col;
            gstep[j]       = (uint32_t)(64 / EB) * (uint32_t)a.ldw;
        }
        ldst[j]         = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds + grp * 1024;
    }
    // TAPS: byte offset of the window's first tap of the lane's pixel (may lie before the tensor) and the taps
    // of the window that fall inside the image.  Loads j < OCT / 2 carry weight rows, the others pixel rows.
    int32_t coff[LOADS];
    uint32_t cmask[LOADS];
    if constexpr (TAPS)
    {
#pragma unroll
        for (int j = WLOADS; j < LOADS; j++)
        {
            const int r = (j * 8 + wave) * 16 + (lane >> 2);
            int p       = p0 + r - WROWS;
            p           = p < a.M - 1 ? p : a.M - 1;
            const int ox = p % a.OW, t2 = p / a.OW;
            const int oy = t2 % a.OH, n = t2 / a.OH;
            const int iy0 = oy * a.sy - a.pad_top, ix0 = ox * a.sx - a.pad_left;
            coff[j]       = ((n * a.IH + iy0) * a.IW + ix0) * a.icb + (((lane & 3) ^ swz(r)) * 16);
            uint32_t m    = 0;
            for (int t = 0; t < a.taps; t++)
            {
                const int ky = t / a.KW, kx = t - ky * a.KW;
                const int y = iy0 + ky * a.dy, x = ix0 + kx * a.dx;
                m |= (y >= 0 && y < a.IH && x >= 0 && x < a.IW ? 1u : 0u) << t;
            }
            cmask[j] = m;
        }
    }
    const int nb = a.n_blocks;
    // Every block period issues one block's loads, also past the end (the last block again, into a stage nobody
    // reads any more): the count of loads in flight is then the same in every iteration and the wait for a
    // block is one instruction with an immediate.
    auto issue_at = [&](int block, uint32_t dst, int j) {
        const int blk      = block < nb ? block : nb - 1;
        if (TAPS && j >= WLOADS)
        {
            // tap of the block (scalar), then per lane: the pixel under that tap, or the zero page
            const int t       = (int)fdiv((uint32_t)blk, a.div_bpt);
            const int piece   = blk - t * a.bpt;
            const int ky      = (int)fdiv((uint32_t)t, a.div_kw);
            const int kx      = t - ky * a.KW;
            const int tap_off = (ky * a.dy * a.IW + kx * a.dx) * a.icb + piece * 64;
            const bool inside = (cmask[j] >> t) & 1u;
            const uint8_t* src =
                inside ? a_base + (ptrdiff_t)(coff[j] + tap_off) : a.pad_page + (lane & 3) * 16;
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(dst) : "memory");
            return;
        }
        const uint8_t* src = gbase[j] + (size_t)blk * gstep[j];
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :
                     : "v"(voff[j]), "s"(src), "s"(dst)
                     : "memory");
    };
    // PAIR: the two 64-byte blocks that share a 128-byte line are requested back to back (the second request
    // then finds the line on its way into the L1 instead of fetching it from L2 again), a pair every two blocks
    auto issue_one = [&](int block, int stage, int j) { issue_at(block, ldst[j] + stage * STAGE, j); };
    // PIXEL_PAIRS: the weight rows (whole lines already, K-major) keep a ring of four single blocks at the start
    // of the LDS; the pixel rows are requested in pairs into three slots of two blocks behind it
    constexpr int WB    = WROWS * 64;
    constexpr int PB    = PROWS * 64;
    constexpr int PBASE = 4 * WB;
    auto issue_w = [&](int block, int j) { issue_at(block, ldst[j] + (block & 3) * WB, j); };
    auto issue_p = [&](int block, int slot, int q) {    // q-th load of the pair that starts at the even `block`
        const int j = WLOADS + (q >> 1);
        issue_at(block + (q & 1), ldst[j] - WB + PBASE + slot * 2 * PB + (q & 1) * PB, j);
    };
    auto issue_pair = [&](int block, int q) {
        issue_one(block + (q & 1), block + (q & 1), q >> 1);    // prologue: stage = block
    };
    // PATCH: the patch first (loads complete in the order they were issued, so the wait for the first weight blocks
    // covers it).  Unit u = plane (u / patch_pixels), pixel (u % patch_pixels); a wave instruction moves 16 units.
    constexpr int PATCH_OFF = kStages * STAGE;
    if constexpr (PATCH)
    {
        const int iy0 = patch_oy0 * a.sy - a.pad_top;
        const uint32_t dst0 =
            (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds + PATCH_OFF + wave * 1024;
#pragma unroll 1
        for (int u0 = 0; u0 < a.patch_units; u0 += 128)
        {
            const int u       = u0 + wave * 16 + (lane >> 2);
            const int plane   = (int)fdiv((uint32_t)u, a.div_ppix);
            const int pix     = u - plane * a.patch_pixels;
            const int r       = (int)fdiv((uint32_t)pix, a.div_pw);
            const int c       = pix - r * a.patch_w;
            const int iy      = iy0 + r, ix = c - a.pad_left;
            const bool inside = iy >= 0 && iy < a.IH && ix >= 0 && ix < a.IW;
            const uint8_t* src =
                inside ? a_base + (ptrdiff_t)(((patch_n * a.IH + iy) * a.IW + ix) * a.icb + plane * 64 +
                                              (((lane & 3) ^ swz(pix)) * 16))
                       : a.pad_page + (lane & 3) * 16;
            const uint32_t dst = dst0 + (uint32_t)u0 * 64;
            if (u < a.patch_units)    // (lanes past the last unit write nothing)
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(dst) : "memory");
        }
    }
    if constexpr (PAIR)
    {
#pragma unroll
        for (int s = 0; s < kStages - 2; s += 2)
#pragma unroll
            for (int q = 0; q < 2 * LOADS; q++)
                issue_pair(s, q);
    }
    else if constexpr (APAIR)
    {
        // in the order the loop continues: pixel pair 0, weights 0, weights 1, pixel pair 1, weights 2
#pragma unroll
        for (int q = 0; q < 2 * PLOADS; q++)
            issue_p(0, 0, q);
#pragma unroll
        for (int j = 0; j < 2 * WLOADS; j++)
            issue_w(j / WLOADS, j % WLOADS);
#pragma unroll
        for (int q = 0; q < 2 * PLOADS; q++)
            issue_p(2, 1, q);
#pragma unroll
        for (int j = 0; j < WLOADS; j++)
            issue_w(2, j);
    }
    else
    {
#pragma unroll
        for (int s = 0; s < kStages - 1; s++)
#pragma unroll
            for (int j = 0; j < LOADS; j++)
                issue_one(s, s, j);
    }

    // ---- tables: bias per channel of the tile (in the shadow of the first loads) ---------------------------
    // (PIXEL_PAIRS fills the LDS with operands: its bias table is written after the loop, into a free stage)
    uint8_t* tables = lds + kStages * STAGE + (PATCH ? a.patch_bytes : 0);
    int* tab_bias   = reinterpret_cast<int*>(APAIR ? lds + 4096 : tables);    // WROWS words
    auto write_bias_table = [&]() {
        if (tid >= WROWS)
            return;
        const int oc = oc0 + tid;
        int v        = 0;
        if (oc < a.N)
        {
            if constexpr (M::is_int)
                v = reinterpret_cast<const int32_t*>(a.bias)[a.bias_len == 1 ? 0 : oc];
            else
                v = __float_as_int(load_as_float<T>(a.bias, a.bias_len == 1 ? 0 : oc));
        }
        tab_bias[tid] = v;
    };
    if constexpr (!APAIR)
        write_bias_table();

    // per-channel constants of the fused RESCALE, derived once per workgroup (WROWS entries of 32 bytes)
    ChannelScale* tab_cs = reinterpret_cast<ChannelScale*>(tables + WROWS * 4);
    uint32_t flags       = 0;
    if constexpr (M::is_int && !APAIR)
    {
        if (a.rp.enabled && tid < WROWS)
        {
            const int oc  = oc0 + tid;
            const bool ok = oc < a.N;    // channels past the end get neutral constants: nothing raised
            const int occ = ok ? oc : 0;
            const int32_t m_raw = load_multiplier(a.rp, occ), s_raw = load_shift(a.rp, occ);
            tab_cs[tid] = make_channel_scale(ok ? m_raw : 0, ok ? s_raw : 32, a.rp.double_round != 0, flags);
        }
    }

    // ---- fragment addresses -----------------------------------------------------------------------------
    const int wrow = wo * 32 * OCT + row_channel(rho);
    const int prow = WROWS + wp * 32 * PXT + rho;
    uint32_t aw[2], ap[2];
#pragma unroll
    for (int s = 0; s < 2; s++)
    {
        aw[s] = wrow * 64 + (((2 * s + h) ^ swz(wrow)) * 16);
        ap[s] = prow * 64 + (((2 * s + h) ^ swz(prow)) * 16);
    }

    // PATCH: the lane's pixel fragments of block (tap, piece) lie in plane `piece` at the patch pixel under that tap
    int pbase = 0;    // patch pixel under the first tap of the lane's output pixel
    if constexpr (PATCH)
    {
        int r_out = wp * 32 + rho;
        r_out     = r_out < m_end - p0 ? r_out : 0;    // rows past the tile's end: any pixel, never stored
        const int py = (int)fdiv((uint32_t)r_out, a.div_ow);
        pbase        = py * a.sy * a.patch_w + (r_out - py * a.OW) * a.sx;
    }
    // Per block: the plane of the piece (a scalar) plus the lane's part, which changes with the tap only.
    uint32_t patch_lane = 0;
    auto patch_block = [&](int block) {
        if constexpr (PATCH)
        {
            const int blk   = block < nb ? block : nb - 1;
            const int t     = (int)fdiv((uint32_t)blk, a.div_bpt);
            const int piece = blk - t * a.bpt;
            if (piece == 0 || block == 0)
            {
                const int ky = (int)fdiv((uint32_t)t, a.div_kw);
                const int kx = t - ky * a.KW;
                const int pp = pbase + ky * a.dy * a.patch_w + kx * a.dx;
                patch_lane   = (uint32_t)PATCH_OFF + ((uint32_t)pp << 6) + (uint32_t)((h ^ swz(pp)) << 4);
            }
            ap[0] = patch_lane + (uint32_t)(piece * a.patch_pixels) * 64u;
            ap[1] = ap[0] ^ 32u;    // K-step 1: pieces 2 + h of the permuted four
        }
    };
    patch_block(0);

    // KM: per channel tile, the address this lane hands to the transposing reads of K-step 0, first read
    uint32_t akm[OCT];
    if constexpr (KM)
    {
        const int sl   = lane & 15;           // position in the 16-lane block of a transposing read
        const int brho = (lane >> 4) & 1;     // which 16 accumulator rows of the tile the block serves
#pragma unroll
        for (int t = 0; t < OCT; t++)
        {
            const int tile = wo * OCT + t;
            if constexpr (EB == 2)
            {
                // source lane sl: K row sl / 4 of the four, channels cb .. cb+3 (lanes 4a .. 4a+3 receive them)
                const int m  = sl >> 2;
                const int a4 = sl & 3;
                const int cb = 16 * (a4 & 1) + 4 * (2 * brho + (a4 >> 1));
                akm[t]       = (8 * h + m) * RB + ((((tile ^ m) << 2) + (cb >> 3)) << 4) + ((cb * 2) & 15);
            }
            else
            {
                // source lane sl: K row sl / 2 of the eight, channels 16*brho + 8*(sl % 2) .. +7
                const int m8 = sl >> 1;
                const int m  = RB >= 256 ? m8 : (m8 >> 1);
                akm[t]       = (16 * h + m8) * RB + ((((tile ^ m) << 1) + brho) << 4) + 8 * (sl & 1);
            }
        }
    }

    acc_t acc[PXT][OCT];
#pragma unroll
    for (int i = 0; i < PXT; i++)
#pragma unroll
        for (int t = 0; t < OCT; t++)
#pragma unroll
            for (int e = 0; e < 16; e++)
                acc[i][t][e] = 0;
    int wsum[OCT], psum[PXT];
#pragma unroll
    for (int t = 0; t < OCT; t++)
        wsum[t] = 0;
#pragma unroll
    for (int i = 0; i < PXT; i++)
        psum[i] = 0;

    // ---- main loop ----------------------------------------------------------------------------------------
    // A block is two K-steps.  The fragments of a step are requested one step ahead of their matrix
    // instructions: step 1 of block n is read while step 0 multiplies, and step 0 of block n+1 while step 1
    // multiplies.  The barrier that publishes block n+1 therefore sits between the two steps of block n; past
    // it every wave has consumed block n-1, whose stage the loads of block n+3 may now overwrite.
    //
    // Every LDS read and every direct load is placed behind a matrix instruction (and kept there with
    // scheduling barriers), so that the time those instructions spend waiting for a slot in the LDS and
    // address queues - all eight waves come out of the barrier together - passes while the matrix core works.
    constexpr int NM = OCT * PXT;    // matrix instructions per step
    constexpr int NW = KM ? 2 * OCT : OCT;    // weight fragment reads per step
    constexpr int NR = NW + PXT;              // fragment reads per step
    v4i fa[2][OCT], fb[2][PXT];
    // reads in the order the matrix instructions want them: pixel tile 0, the channel tiles, the other pixel tiles
    // wb: the stage's weight rows; pb: its pixel rows minus their offset in a whole stage (ap[] includes it)
    auto read_one = [&](const uint8_t* wb, const uint8_t* pb, int s, int j) {
        const uint8_t* sb = wb;
        if (j == 0)
            fb[s][0] = *reinterpret_cast<const v4i*>(pb + ap[s]);
        else if (j <= NW)
        {
            if constexpr (KM)
            {
                const int t = (j - 1) >> 1, r = (j - 1) & 1;
                const uint8_t* src = sb + akm[t] + (KSTEP * s + (KSTEP / 4) * r) * RB;
                v2i half;
                if constexpr (EB == 2)
                    half = __builtin_bit_cast(v2i, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                                       (__attribute__((address_space(3))) v4s*)src));
                else
                    half = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i*)src);
                fa[s][t][2 * r]     = half.x;
                fa[s][t][2 * r + 1] = half.y;
            }
            else
                fa[s][j - 1] = *reinterpret_cast<const v4i*>(sb + aw[s] + (j - 1) * 2048);
        }
        else
            fb[s][j - NW] = *reinterpret_cast<const v4i*>(pb + ap[s] + (j - NW) * 2048);
    };
    auto sums = [&](int s) {
        if constexpr (ZP)
        {
#pragma unroll
            for (int t = 0; t < OCT; t++)
                wsum[t] += dot4_ones(fa[s][t]);
#pragma unroll
            for (int i = 0; i < PXT; i++)
                psum[i] += dot4_ones(fb[s][i]);
        }
    };
    auto mma_one = [&](int s, int k) {
        const int i = k / OCT, t = k % OCT;
        acc[i][t]   = M::mma(fa[s][t], fb[s][i], acc[i][t]);
    };
    // A bare s_barrier: __syncthreads() would also drain this wave's LDS reads (the fragments of the step
    // about to be multiplied), which nothing here needs.  What the barrier orders is the direct loads (waited
    // for by hand just before it) against the reads that follow it, and the reads of two steps ago against the
    // loads that follow it; the fragments of block n-1 were consumed before this wave got here.
    auto publish = [&]() {
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((kStages - 3) * LOADS) : "memory");
    };
    // PAIR: a pair lands as a whole (its loads alternate between the two blocks), so one barrier per pair, in
    // the second block, publishes the next pair; another pair may still be on its way behind it.
    auto publish_pair = [&]() {
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(PAIR ? (kStages / 2 - 3) * 2 * LOADS : 0) : "memory");
    };
    if constexpr (PAIR)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PAIR ? (kStages / 2 - 2) * 2 * LOADS : 0) : "memory");
    else if constexpr (APAIR)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * PLOADS + 2 * WLOADS) : "memory");
    else
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kStages - 2) * LOADS) : "memory");
    __syncthreads();    // block 0 and the bias table are in LDS for every wave
#pragma unroll
    for (int j = 0; j < NR; j++)
        read_one(lds, APAIR ? lds + PBASE - WB : lds, 0, j);
    __builtin_amdgcn_sched_barrier(0);
    // first K-step of a block: its matrix instructions, and the requests for the fragments of the second step;
    // two requests behind each of the first matrix instructions, so that the last ones of a step cover the
    // latency of the fragments the next step starts with
    auto first_step = [&](const uint8_t* cur, const uint8_t* curp) {
        constexpr int PA = NR > 2 * NM ? (NR + NM - 1) / NM : 2;
        sums(0);
#pragma unroll
        for (int k = 0; k < NM; k++)
        {
            mma_one(0, k);
#pragma unroll
            for (int j = k * PA; j < (k + 1) * PA && j < NR; j++)
                read_one(cur, curp, 1, j);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // second K-step: its matrix instructions, NL direct loads (they have the longest way to go, so they come
    // first) and the requests for the first fragments of the next block
    auto second_step = [&](const uint8_t* next, const uint8_t* nextp, auto NL_tag, auto&& load) {
        constexpr int NL = decltype(NL_tag)::value;
        constexpr int NO = NL + NR;
        constexpr int PB = NO > 2 * NM ? (NO + NM - 1) / NM : 2;
        sums(1);
#pragma unroll
        for (int k = 0; k < NM; k++)
        {
            mma_one(1, k);
#pragma unroll
            for (int q = k * PB; q < (k + 1) * PB && q < NO; q++)
            {
                if (q < NL)
                    load(q);
                else
                    read_one(next, nextp, 0, q - NL);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    if constexpr (PAIR)
    {
        // Where every operand row is K-contiguous (no taps to decode per load), a trip round the ring needs no
        // arithmetic per load: the sources of its blocks are one scalar pointer per load, advanced once per trip, plus
        // an offset field, and the destination stage is a constant added to the wave's LDS base on its way into M0.
        // Such a trip only requests blocks that exist; the last trips, whose requests run past the last block and
        // repeat it, take the general form.
        constexpr bool FASTABLE = !TAPS && !KM;    // (K-major weight rows advance by their own stride)
        // (The offset field of a direct load moves the LDS destination as well as the source, so the constant that
        // goes into M0 takes it off again; offsets are counted from the trip's third request, the one into stage 0,
        // which keeps every M0 value at or above the wave's LDS base.)
        const uint8_t* fptr[LOADS];    // per load: source of block n + kStages of the current trip
#pragma unroll
        for (int j = 0; j < LOADS; j++)
            fptr[j] = gbase[j] + (size_t)kStages * gstep[j];
        auto issue_fast = [&](int rel, int j) {
#define TMI_FAST_LOAD(R)                                                                                               \
    case R:                                                                                                            \
        asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%4"                    \
                     :                                                                                                 \
                     : "v"(voff[j]), "s"(fptr[j]), "s"(ldst[j]),                                                       \
                       "n"(((R + kStages - 2) % kStages) * STAGE - (R - 2) * 64), "n"((R - 2) * 64)                    \
                     : "memory", "scc");                                                                               \
        break;
            switch (rel)
            {
                TMI_FAST_LOAD(0)
                TMI_FAST_LOAD(1)
                TMI_FAST_LOAD(2)
                TMI_FAST_LOAD(3)
                TMI_FAST_LOAD(4)
                TMI_FAST_LOAD(5)
                TMI_FAST_LOAD(6)
                TMI_FAST_LOAD(7)
            }
#undef TMI_FAST_LOAD
        };
        // PATCH, pieces per tap a multiple of the ring length: the blocks of a trip lie under one tap, in consecutive
        // planes, so their fragment addresses are the trip's first plus k planes (scalars set up here)
        uint32_t plane_k[kStages];
        uint32_t trip_ap = 0;
        if constexpr (PATCH)
        {
#pragma unroll
            for (int k = 0; k < kStages; k++)
                plane_k[k] = (uint32_t)(k * a.patch_pixels) * 64u;
        }
        // (FAST: 0 the general form, 1 a trip under one tap, 2 a trip whose halves lie under two taps)
        const int fast_patch = !PATCH || a.bpt % kStages == 0 ? 1 : (a.bpt * 2 == kStages ? 2 : 0);
        uint32_t half_ap = 0;    // FAST 2: fragment address of the trip's block kStages / 2
        // one pair of blocks, n and n + 1, in stages sc and sc + 1
        auto pair = [&](int n, int sc, auto FAST) {
            constexpr int fast_form = decltype(FAST)::value;
            constexpr bool fast     = fast_form != 0;
            const int sn        = sc + 2 < kStages ? sc + 2 : 0;
            const int sfree     = sc >= 2 ? sc - 2 : kStages - 2;    // the pair consumed before this one
            const uint8_t* cur0 = lds + sc * STAGE;
            // (PATCH: pixel fragments are addressed from the start of the LDS, and the addresses of the next block's
            // are set before the step that requests its first fragments)
            auto next_patch = [&](int k) {    // block k of the trip (fast) or block n - sc + k
                if constexpr (PATCH)
                {
                    if (fast_form == 1 && k < kStages)
                        ap[0] = trip_ap + plane_k[k], ap[1] = ap[0] ^ 32u;
                    else if (fast_form == 2 && k < kStages && k != kStages / 2)
                        ap[0] = (k < kStages / 2 ? trip_ap : half_ap) + plane_k[k % (kStages / 2)], ap[1] = ap[0] ^ 32u;
                    else
                    {
                        patch_block(n - sc + k);
                        if (fast_form == 2 && k == kStages / 2)
                            half_ap = ap[0];
                    }
                }
            };
            first_step(cur0, PATCH ? lds : cur0);
            next_patch(sc + 1);
            second_step(cur0 + STAGE, PATCH ? lds : cur0 + STAGE, std::integral_constant<int, 0>{}, [](int) {});
            first_step(cur0 + STAGE, PATCH ? lds : cur0 + STAGE);
            publish_pair();    // the next pair is in LDS for every wave, and every wave is past the pair before
            next_patch(sc + 2);
            second_step(lds + sn * STAGE, PATCH ? lds : lds + sn * STAGE, std::integral_constant<int, 2 * LOADS>{},
                        [&](int q) {
                            if constexpr (fast)
                                issue_fast(sc + (q & 1), q >> 1);
                            else
                                issue_one(n + kStages - 2 + (q & 1), sfree + (q & 1), q >> 1);
                        });
        };
        // Once round the ring per iteration, so that every stage address is a constant of its instruction (an offset
        // field instead of an addition per fragment read and per load); the pairs left over follow one by one.
        int n = 0;
        if constexpr (FASTABLE)
        {
            if (fast_patch == 1)
            {
#pragma unroll 1
                for (; n + 2 * kStages - 2 <= nb; n += kStages)
                {
                    trip_ap = ap[0];    // block n: set by the trip before, or by the prologue
#pragma unroll
                    for (int sc = 0; sc < kStages; sc += 2)
                        pair(n + sc, sc, std::integral_constant<int, 1>{});
#pragma unroll
                    for (int j = 0; j < LOADS; j++)
                        fptr[j] += kStages * 64;
                }
            }
            if constexpr (PATCH)
            {
                if (fast_patch == 2)
                {
#pragma unroll 1
                    for (; n + 2 * kStages - 2 <= nb; n += kStages)
                    {
                        trip_ap = ap[0];
#pragma unroll
                        for (int sc = 0; sc < kStages; sc += 2)
                            pair(n + sc, sc, std::integral_constant<int, 2>{});
#pragma unroll
                        for (int j = 0; j < LOADS; j++)
                            fptr[j] += kStages * 64;
                    }
                }
            }
        }
        // (not with taps: the unrolled trip with the tap decode of every pixel load does not fit the register file)
        if constexpr (!TAPS)
        {
#pragma unroll 1
            for (; n + kStages - 1 < nb; n += kStages)
            {
#pragma unroll
                for (int sc = 0; sc < kStages; sc += 2)
                    pair(n + sc, sc, std::integral_constant<int, 0>{});
            }
        }
        int sc = 0;    // stage of the pair's first block
#pragma unroll 1
        for (; n + 1 < nb; n += 2)
        {
            pair(n, sc, std::integral_constant<int, 0>{});
            sc = sc + 2 < kStages ? sc + 2 : 0;
        }
        if (nb & 1)
        {
            // the last block of an odd count: the first half of a pair whose second half is a repeat
            const uint8_t* cur = lds + sc * STAGE;
            first_step(cur, PATCH ? lds : cur);
            second_step(cur + STAGE, PATCH ? lds : cur + STAGE, std::integral_constant<int, 0>{}, [](int) {});
        }
    }
    else if constexpr (APAIR)
    {
        // Loads are waited for in the order they were issued.  Behind the weights of block n+1 (needed at the
        // barrier of an even block n) come a pixel pair and a block of weights; behind the pixel pair and the
        // weights of block n+2 (needed at the barrier of the odd block n+1) a block of weights.
        int slot = 0;    // pixel slot of the pair (n, n+1)
#pragma unroll 1
        for (int n = 0; n + 1 < nb; n += 2)
        {
            const int slot_next = slot == 2 ? 0 : slot + 1;
            const int slot_free = slot == 0 ? 2 : slot - 1;    // held the pair before this one
            const uint8_t* wb0  = lds + (n & 3) * WB;
            const uint8_t* wb1  = lds + ((n + 1) & 3) * WB;
            const uint8_t* wb2  = lds + ((n + 2) & 3) * WB;
            const uint8_t* pb0  = lds + PBASE - WB + slot * 2 * PB;
            const uint8_t* pb2  = lds + PBASE - WB + slot_next * 2 * PB;
            first_step(wb0, pb0);
            asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * PLOADS + WLOADS) : "memory");
            second_step(wb1, pb0 + PB, std::integral_constant<int, WLOADS>{}, [&](int q) { issue_w(n + 3, q); });
            first_step(wb1, pb0 + PB);
            asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(WLOADS) : "memory");
            second_step(wb2, pb2, std::integral_constant<int, 2 * PLOADS + WLOADS>{}, [&](int q) {
                if (q < 2 * PLOADS)
                    issue_p(n + 4, slot_free, q);
                else
                    issue_w(n + 4, q - 2 * PLOADS);
            });
            slot = slot_next;
        }
        if (nb & 1)
        {
            // the last block of an odd count: published by the barrier before it, nothing left to request
            const uint8_t* wb = lds + ((nb - 1) & 3) * WB;
            const uint8_t* pb = lds + PBASE - WB + slot * 2 * PB;
            first_step(wb, pb);
            second_step(wb, pb, std::integral_constant<int, 0>{}, [](int) {});
        }
    }
    else
    {
        int n = 0;
        // Whole trips round the ring first, as in the pair form: stage addresses are constants, a K-contiguous row's
        // block is the trip's pointer plus an offset field (taken off the LDS side again in M0, counted from the
        // request that goes into stage 0), a K-major weight block has one running pointer per stage.  A trip only
        // requests blocks that exist; the rest of the loop is the general form.
        if constexpr (!TAPS && kStages == 4)
        {
            const uint8_t* fptr[LOADS];            // K-contiguous: source of block n + kStages
            const uint8_t* kptr[LOADS][kStages];    // K-major: source of block n + kStages - 1 + r
#pragma unroll
            for (int j = 0; j < LOADS; j++)
            {
                fptr[j] = gbase[j] + (size_t)kStages * gstep[j];
#pragma unroll
                for (int r = 0; r < kStages; r++)
                    kptr[j][r] = gbase[j] + (size_t)(kStages - 1 + r) * gstep[j];
            }
            auto issue_trip = [&](int r, int j) {
                if (KM && j < WLOADS)
                {
                    const uint32_t dst = ldst[j] + ((r + kStages - 1) % kStages) * STAGE;
                    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                                 :
                                 : "v"(voff[j]), "s"(kptr[j][r]), "s"(dst)
                                 : "memory");
                    return;
                }
#define TMI_TRIP_LOAD(R)                                                                                               \
    case R:                                                                                                            \
        asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%4"                    \
                     :                                                                                                 \
                     : "v"(voff[j]), "s"(fptr[j]), "s"(ldst[j]),                                                       \
                       "n"(((R + kStages - 1) % kStages) * STAGE - (R - 1) * 64), "n"((R - 1) * 64)                    \
                     : "memory", "scc");                                                                               \
        break;
                switch (r)
                {
                    TMI_TRIP_LOAD(0)
                    TMI_TRIP_LOAD(1)
                    TMI_TRIP_LOAD(2)
                    TMI_TRIP_LOAD(3)
                }
#undef TMI_TRIP_LOAD
            };
#pragma unroll 1
            for (; n + 2 * kStages - 1 <= nb; n += kStages)
            {
#pragma unroll
                for (int r = 0; r < kStages; r++)
                {
                    const uint8_t* cur  = lds + r * STAGE;
                    const uint8_t* next = lds + ((r + 1) % kStages) * STAGE;
                    first_step(cur, cur);
                    publish();
                    second_step(next, next, std::integral_constant<int, LOADS>{}, [&](int q) { issue_trip(r, q); });
                }
#pragma unroll
                for (int j = 0; j < LOADS; j++)
                {
                    fptr[j] += (size_t)kStages * gstep[j];
#pragma unroll
                    for (int r = 0; r < kStages; r++)
                        kptr[j][r] += (size_t)kStages * gstep[j];
                }
            }
        }
#pragma unroll 1
        for (; n < nb; n++)
        {
            const uint8_t* cur  = lds + (n % kStages) * STAGE;
            const uint8_t* next = lds + ((n + 1) % kStages) * STAGE;
            first_step(cur, cur);
            publish();    // block n+1 (after the last block: its repeat) is in LDS for every wave
            second_step(next, next, std::integral_constant<int, LOADS>{}, [&](int q) {
                issue_one(n + kStages - 1, (n + kStages - 1) % kStages, q);
            });
        }
    }

    // ---- epilogue -----------------------------------------------------------------------------------------
    // The loads issued past the last block are still on their way into LDS: let them land before a stage is
    // given another use.  The stage buffers are then free: the channel sums go through the first one.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    int* tab_wsum = reinterpret_cast<int*>(lds);    // WROWS words
    if constexpr (ZP || APAIR)
    {
        __syncthreads();    // every wave has read its last fragments and seen its last loads land
        if constexpr (APAIR)
            write_bias_table();
        if constexpr (ZP)
        {
#pragma unroll
            for (int t = 0; t < OCT; t++)
            {
                const int sum = wsum[t] + __shfl_xor(wsum[t], 32);
                if (wp == 0 && h == 0)
                    tab_wsum[wo * 32 * OCT + t * 32 + row_channel(rho)] = sum;
            }
#pragma unroll
            for (int i = 0; i < PXT; i++)
                psum[i] += __shfl_xor(psum[i], 32);
        }
        __syncthreads();
    }
    // Four-byte results (int32, fp32) whose rows are whole 128-byte lines per channel tile leave through LDS: a lane
    // holds 64 bytes of one pixel's row, so a store instruction straight from the accumulators is 64 separate
    // 16-byte requests to the L2 (4.2 M of them for the named bf16 MATMUL, which kept its 256 workgroups storing
    // for 22 us at the end); transposed through a per-wave 4.5 KB buffer, an instruction writes 8 whole lines.
    // (The buffer lies in the stage memory: every wave must be done with its fragments first.)
    const bool wide_out = M::is_int ? !(!APAIR && a.rp.enabled) : a.out_is_wide != 0;
    const bool lines    = wide_out && (a.N & 31) == 0;
    // Floating-point results of the input type (2 bytes): a pixel's OCT x 32 channels are 128 or 256 bytes, gathered
    // from all the wave's channel tiles before they leave.
    constexpr int HROW   = OCT * 64;    // bytes of a pixel's channels held by this wave
    constexpr int HPITCH = HROW + 16;
    const bool half_lines = !M::is_int && !wide_out && (a.N & 63) == 0 && oc0 + (wo + 1) * 32 * OCT <= a.N;
    const bool any_half_lines = !M::is_int && !wide_out && (a.N & 63) == 0;    // the same for every wave
    if constexpr (!(ZP || APAIR))
        if (lines || any_half_lines)
            __syncthreads();
    constexpr int TPITCH = 144;    // bytes per pixel row in the buffer: 128 + 16, so that rows spread over the banks
    uint8_t* tbuf        = lds + 8192 + wave * (32 * (HPITCH > TPITCH ? HPITCH : TPITCH));

    // A lane's 16 accumulator registers of a tile are four groups of 4 consecutive channels: group q starts at
    // channel 16h + 4q (all 16 consecutive), or 8q + 4h with the in-order row assignment.
    auto group_channel = [&](int q) { return IDENT ? 8 * q + 4 * h : 16 * h + 4 * q; };
    const bool rows16 = (a.N & 15) == 0;    // every lane's 16 channels are inside the tensor or all outside
    const bool rows4  = (a.N & 3) == 0;     // the same for a group of 4
    uint8_t* out_b    = reinterpret_cast<uint8_t*>(a.out) + batch * a.o_batch;
    if constexpr (!M::is_int)
    {
        if (half_lines)
        {
#pragma unroll
            for (int i = 0; i < PXT; i++)
            {
                const int pt0 = p0 + wp * 32 * PXT + i * 32;    // the tile's first pixel row
                if (pt0 >= m_end)
                    continue;
#pragma unroll
                for (int t = 0; t < OCT; t++)
                {
                    const int tl = wo * 32 * OCT + t * 32;
                    alignas(16) T packed[16];
#pragma unroll
                    for (int q = 0; q < 4; q++)
                    {
                        const v4i b = *reinterpret_cast<const v4i*>(tab_bias + tl + 16 * h + 4 * q);
                        store_from_float(packed + 4 * q, acc[i][t][4 * q] + __int_as_float(b.x));
                        store_from_float(packed + 4 * q + 1, acc[i][t][4 * q + 1] + __int_as_float(b.y));
                        store_from_float(packed + 4 * q + 2, acc[i][t][4 * q + 2] + __int_as_float(b.z));
                        store_from_float(packed + 4 * q + 3, acc[i][t][4 * q + 3] + __int_as_float(b.w));
                    }
                    uint8_t* d = tbuf + rho * HPITCH + t * 64 + h * 32;
                    reinterpret_cast<v4i*>(d)[0] = reinterpret_cast<const v4i*>(packed)[0];
                    reinterpret_cast<v4i*>(d)[1] = reinterpret_cast<const v4i*>(packed)[1];
                }
                constexpr int PIECES = HROW / 16;      // 16-byte pieces per pixel row: 8 or 16
                constexpr int RPI    = 64 / PIECES;    // rows per store instruction
#pragma unroll
                for (int j = 0; j < 32 / RPI; j++)
                {
                    const int row = lane / PIECES + RPI * j, piece = lane % PIECES;
                    const v4i d   = *reinterpret_cast<const v4i*>(tbuf + row * HPITCH + piece * 16);
                    if (pt0 + row < m_end)
                        *reinterpret_cast<v4i*>(out_b + ((size_t)(pt0 + row) * a.N + oc0 + wo * 32 * OCT) * 2 + piece * 16) = d;
                }
            }
            return;
        }
    }
#pragma unroll
    for (int t = 0; t < OCT; t++)
    {
        const int tl = wo * 32 * OCT + t * 32;    // first channel of the tile within the workgroup's channels
        int cb[16];
#pragma unroll
        for (int q = 0; q < 4; q++)
        {
            const v4i b = *reinterpret_cast<const v4i*>(tab_bias + tl + group_channel(q));
            cb[4 * q] = b.x, cb[4 * q + 1] = b.y, cb[4 * q + 2] = b.z, cb[4 * q + 3] = b.w;
        }
        if constexpr (ZP)
        {
            const int kzz = a.K * a.za * a.zw;
#pragma unroll
            for (int q = 0; q < 4; q++)
            {
                const v4i sw = *reinterpret_cast<const v4i*>(tab_wsum + tl + group_channel(q));
                cb[4 * q] += kzz - a.za * sw.x, cb[4 * q + 1] += kzz - a.za * sw.y;
                cb[4 * q + 2] += kzz - a.za * sw.z, cb[4 * q + 3] += kzz - a.za * sw.w;
            }
        }
#pragma unroll
        for (int i = 0; i < PXT; i++)
        {
            const int p = p0 + wp * 32 * PXT + i * 32 + rho;
            if (lines)
            {
                const int pt0 = p0 + wp * 32 * PXT + i * 32;    // the tile's first pixel row
                if (pt0 >= m_end || oc0 + tl >= a.N)
                    continue;
                int w4[16];
                if constexpr (M::is_int)
                {
                    const int pcorr = ZP ? a.zw * psum[i] : 0;
#pragma unroll
                    for (int e = 0; e < 16; e++)
                        w4[e] = acc[i][t][e] + cb[e] - pcorr;
                }
                else
                {
#pragma unroll
                    for (int e = 0; e < 16; e++)
                        w4[e] = __float_as_int(acc[i][t][e] + __int_as_float(cb[e]));
                }
#pragma unroll
                for (int q = 0; q < 4; q++)
                    *reinterpret_cast<v4i*>(tbuf + rho * TPITCH + group_channel(q) * 4) =
                        v4i{ w4[4 * q], w4[4 * q + 1], w4[4 * q + 2], w4[4 * q + 3] };
#pragma unroll
                for (int j = 0; j < 4; j++)
                {
                    const int row = (lane >> 3) + 8 * j, piece = lane & 7;
                    const v4i d   = *reinterpret_cast<const v4i*>(tbuf + row * TPITCH + piece * 16);
                    if (pt0 + row < m_end)
                        *reinterpret_cast<v4i*>(out_b + ((size_t)(pt0 + row) * a.N + oc0 + tl) * 4 + piece * 16) = d;
                }
                continue;
            }
            if (p >= m_end || oc0 + tl >= a.N)
                continue;
            if constexpr (M::is_int)
            {
                const int pcorr = ZP ? a.zw * psum[i] : 0;
                if (!APAIR && a.rp.enabled)
                {
                    // fused RESCALE (+ CLAMP): the lane's 16 consecutive channels leave as 16 (32) bytes
                    const int ocl = tl + 16 * h;
                    const int oc  = oc0 + ocl;
                    if (oc >= a.N)
                        continue;
                    int r[16];
#pragma unroll
                    for (int e = 0; e < 16; e++)
                    {
                        const ChannelScale cs = tab_cs[ocl + e];
                        r[e] = fast_rescale(acc[i][t][e] + cb[e] - pcorr, cs, a.rp.out_zp, a.rp.lo, a.rp.hi, flags);
                    }
                    uint8_t* dst = out_b + ((size_t)p * a.N + oc) * a.out_bytes;
                    if (a.out_bytes == 1)
                    {
                        if (rows16)
                        {
                            v4i packed;
#pragma unroll
                            for (int q = 0; q < 4; q++)
                                packed[q] = (r[4 * q] & 0xff) | ((r[4 * q + 1] & 0xff) << 8) |
                                            ((r[4 * q + 2] & 0xff) << 16) | ((r[4 * q + 3] & 0xff) << 24);
                            *reinterpret_cast<v4i*>(dst) = packed;
                        }
                        else
                        {
#pragma unroll
                            for (int e = 0; e < 16; e++)
                                if (oc + e < a.N)
                                    dst[e] = (uint8_t)r[e];
                        }
                    }
                    else
                    {
                        if (rows16)
                        {
#pragma unroll
                            for (int hq = 0; hq < 2; hq++)
                            {
                                v4i packed;
#pragma unroll
                                for (int q = 0; q < 4; q++)
                                    packed[q] = (r[8 * hq + 2 * q] & 0xffff) | ((r[8 * hq + 2 * q + 1] & 0xffff) << 16);
                                reinterpret_cast<v4i*>(dst)[hq] = packed;
                            }
                        }
                        else
                        {
#pragma unroll
                            for (int e = 0; e < 16; e++)
                                if (oc + e < a.N)
                                    reinterpret_cast<int16_t*>(dst)[e] = (int16_t)r[e];
                        }
                    }
                    continue;
                }
                int32_t* row    = reinterpret_cast<int32_t*>(out_b) + (size_t)p * a.N;
#pragma unroll
                for (int q = 0; q < 4; q++)
                {
                    const int oc = oc0 + tl + group_channel(q);
                    int v[4];
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        v[e] = acc[i][t][4 * q + e] + cb[4 * q + e] - pcorr;
                    if (rows4)
                    {
                        if (oc < a.N)
                            *reinterpret_cast<v4i*>(row + oc) = v4i{ v[0], v[1], v[2], v[3] };
                    }
                    else
                    {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (oc + e < a.N)
                                row[oc + e] = v[e];
                    }
                }
            }
            else
            {
                const int oc = oc0 + tl + 16 * h;    // floating point: always 16 consecutive channels
                if (oc >= a.N)
                    continue;
                float v[16];
#pragma unroll
                for (int e = 0; e < 16; e++)
                    v[e] = acc[i][t][e] + __int_as_float(cb[e]);
                if (a.out_is_wide)
                {
                    float* dst = reinterpret_cast<float*>(out_b) + (size_t)p * a.N + oc;
                    if (rows16)
                    {
#pragma unroll
                        for (int q = 0; q < 4; q++)
                            reinterpret_cast<v4f*>(dst)[q] = v4f{ v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3] };
                    }
                    else
                    {
#pragma unroll
                        for (int e = 0; e < 16; e++)
                            if (oc + e < a.N)
                                dst[e] = v[e];
                    }
                }
                else
                {
                    T* dst = reinterpret_cast<T*>(out_b) + (size_t)p * a.N + oc;
                    if (rows16)
                    {
                        alignas(16) T packed[16];
#pragma unroll
                        for (int e = 0; e < 16; e++)
                            store_from_float(packed + e, v[e]);
                        reinterpret_cast<v4i*>(dst)[0] = reinterpret_cast<const v4i*>(packed)[0];
                        reinterpret_cast<v4i*>(dst)[1] = reinterpret_cast<const v4i*>(packed)[1];
                    }
                    else
                    {
#pragma unroll
                        for (int e = 0; e < 16; e++)
                            if (oc + e < a.N)
                                store_from_float(dst + e, v[e]);
                    }
                }
            }
        }
    }
    if constexpr (M::is_int && !APAIR)
        if (a.rp.enabled)
            raise_flags(a.flag_word, flags);
}

template <typename T, int OCT, int PXT, bool ZP, int MODE, int STAGES, int PIPE>
static bool launch_gemm_pipe(hipStream_t st, const GemmArgs& a, int blocks)
{
    // stages, bias table, per-channel RESCALE constants; PIXEL_PAIRS: four stages of weight rows and three slots
    // of two blocks of pixel rows, the bias table goes through a stage after the loop
    const size_t lds_bytes = PIPE == PIPE_PIXEL_PAIRS
                                 ? (size_t)4 * 64 * OCT * 64 + (size_t)6 * 128 * PXT * 64
                                 : (MODE == GEMM_PATCH
                                        ? (size_t)STAGES * 64 * OCT * 64 + (size_t)a.patch_bytes
                                        : (size_t)STAGES * (64 * OCT + 128 * PXT) * 64) +
                                       64 * OCT * 4 + 64 * OCT * 32;
    auto kern                  = gemm_lds_kernel<T, OCT, PXT, ZP, MODE, STAGES, PIPE>;
    static LdsLimit granted{};
    if (!ensure_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, granted))
        return false;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(512), lds_bytes, st, a);
    return true;
}

template <typename T, int OCT, int PXT, bool ZP, int MODE>
static bool launch_gemm_shape(hipStream_t st, const GemmArgs& a, int blocks)
{
    // The two smaller shapes have LDS to spare for a ring of 8 x 16 KB or 6 x 24 KB, which lets them request
    // the blocks in pairs (both halves of every 128-byte line together).  Measured on MI355X, us without /
    // with: 3x3 layers fp16 [16,28,28,256]->256 24.8 / 23.4, [8,28,28,512]->512 51.1 / 48.1, int8 42.1 / 38.9;
    // with few blocks the longer prologue costs more than the pairs return (pointwise [8,56,56,256]->64 fp16
    // 5.0 / 5.6, int8 7.1 / 7.5; 32 blocks: 12.1 / 12.4), and the deeper ring without pairs is slower everywhere.
    if constexpr (OCT * PXT <= 4)
    {
        constexpr int DEEP = OCT * PXT == 2 ? 8 : 6;
        if (a.n_blocks > 32)
            return launch_gemm_pipe<T, OCT, PXT, ZP, MODE, DEEP, PIPE_PAIRS>(st, a, blocks);
    }
    // MATMUL on the two larger shapes: the second operand lies K-major and is fetched in whole lines already; the
    // first one's rows are requested in pairs (a third fewer read requests at the L2 for the named bf16 MATMUL,
    // 8.8 M instead of 12.8 M).  Measured, us without / with: bf16 [4,2048,4096]x[4,4096,2048] 127.3 / 124.7 and
    // 123.7 / 120.3 on two boxes, [1,4096,2048]x[1,2048,4096] 71.9 / 70.6, int8 [1,4096,4096]x[1,4096,4096]
    // 65.1 / 64.1; below some 48 blocks of K nothing or the other way (int8 [8,1024,512] 13.8 / 14.0,
    // [16,1024,768] 23.2 / 23.6).  The layout needs the whole LDS for the 256x256 shape: if the device does not
    // grant it, the plain ring runs.
    if constexpr (MODE == GEMM_KMAJOR && OCT * PXT >= 4)
    {
        if (a.n_blocks >= 48 && !a.rp.enabled &&
            launch_gemm_pipe<T, OCT, PXT, ZP, MODE, 4, PIPE_PIXEL_PAIRS>(st, a, blocks))
            return true;
    }
    return launch_gemm_pipe<T, OCT, PXT, ZP, MODE, kStagesDefault, PIPE_SINGLE>(st, a, blocks);
}

// The patch form of a convolution with taps (stride 1): tiles of whole output rows, 128 x 128 results, the input patch
// resident in LDS behind a ring of eight weight stages.  False when the layer does not fit the form.
// Geometry of the patch form, or false: output rows per tile, patch height and width in pixels.
static bool patch_form_geometry(int OH, int OW, int KH, int KW, int sy, int sx, int dy, int dx, int64_t icb, int OC,
                                int& rows, int& patch_h, int& patch_w)
{
    constexpr int kRing = 8 * 128 * 64, kTables = 128 * 4 + 128 * 32, kLds = 160 * 1024;
    if (sy != 1 || sx != 1 || OW > 128 || OC < 128 || icb % 64 != 0 || (int64_t)KH * KW * icb / 64 < 8)
        return false;
    rows = 128 / OW < OH ? 128 / OW : OH;
    // the tiles must not leave much of their 128 pixel rows, or of the image's last tile, unused
    if (rows * OW < 96 || (int64_t)OH * 4 < (int64_t)((OH + rows - 1) / rows) * rows * 3)
        return false;
    patch_h              = (rows - 1) * sy + (KH - 1) * dy + 1;
    patch_w              = (OW - 1) * sx + (KW - 1) * dx + 1;
    const int64_t bytes  = ((int64_t)patch_h * patch_w * icb + 1023) / 1024 * 1024;
    return kRing + bytes + kTables <= kLds;
}

template <typename T>
static bool launch_gemm_patch(hipStream_t st, GemmArgs& a)
{
    int rows = 0, patch_h = 0, patch_w = 0;
    if (!patch_form_geometry(a.OH, a.OW, a.taps / a.KW, a.KW, a.sy, a.sx, a.dy, a.dx, a.icb, a.N, rows, patch_h, patch_w))
        return false;
    const int64_t pixels  = (int64_t)patch_h * patch_w;
    const int64_t units   = pixels * a.bpt;
    const int64_t bytes   = (units * 64 + 1023) / 1024 * 1024;
    const int images      = a.M / (a.OH * a.OW);
    a.rows_per_tile       = rows;
    a.tiles_per_image     = (a.OH + rows - 1) / rows;
    a.patch_w             = patch_w;
    a.patch_pixels        = (int32_t)pixels;
    a.patch_units         = (int32_t)units;
    a.patch_bytes         = (int32_t)bytes;
    a.div_tpi             = make_fastdiv((uint32_t)a.tiles_per_image);
    a.div_pw              = make_fastdiv((uint32_t)patch_w);
    a.div_ppix            = make_fastdiv((uint32_t)pixels);
    a.div_ow              = make_fastdiv((uint32_t)a.OW);
    a.tiles_n             = (a.N + 127) / 128;
    const int64_t tiles_m = (int64_t)images * a.tiles_per_image;
    const int64_t tiles   = tiles_m * a.tiles_n;
    // A workgroup has a CU to itself, so the time hardly depends on how many there are; from some 48 tiles on this
    // form is faster than the patch kernel (us patch kernel / this form, host clock: fp16 3x3 [4,28,28,256]->256
    // 21.3 / 16.5, [16,14,14,256]->256 21.5 / 16.5, [8,28,28,128]->128 13.0 / 10.5; int8 14.8 / 11.1, 14.6 / 11.1).
    if (tiles < 48)
        return false;
    // the divisions of the tile decode and of the patch loads are exact in these ranges
    if (tiles > (1 << 22) || !fastdiv_exact_up_to((uint64_t)tiles - 1, (uint32_t)tiles) ||
        !fastdiv_exact_up_to((uint64_t)tiles - 1, (uint32_t)a.tiles_n) ||
        !fastdiv_exact_up_to((uint64_t)tiles_m, (uint32_t)a.tiles_per_image) ||
        !fastdiv_exact_up_to((uint64_t)units + 128, (uint32_t)pixels) ||
        !fastdiv_exact_up_to((uint64_t)pixels, (uint32_t)patch_w) || !fastdiv_exact_up_to(128, (uint32_t)a.OW))
        return false;
    a.tiles_per_batch = (int32_t)tiles;
    a.tiles_total     = (int32_t)tiles;
    a.per_xcd         = (a.tiles_total + 7) / 8;
    a.div_batch       = make_fastdiv((uint32_t)a.tiles_per_batch);
    a.div_tn          = make_fastdiv((uint32_t)a.tiles_n);
    const bool zp     = Mma<T>::is_int && (a.za != 0 || a.zw != 0);
    if (zp)
        return launch_gemm_pipe<T, 2, 1, Mma<T>::is_int, GEMM_PATCH, 8, PIPE_PAIRS>(st, a, a.per_xcd * 8);
    return launch_gemm_pipe<T, 2, 1, false, GEMM_PATCH, 8, PIPE_PAIRS>(st, a, a.per_xcd * 8);
}

template <typename T>
static const char* launch_gemm_t(hipStream_t st, GemmArgs& a, int batches, bool tapped, const char* label,
                                 const char* patch_label = nullptr)
{
    // Floating-point convolutions with taps whose patch fits the LDS take the patch form.  Measured on MI355X, us
    // taps form / patch form (host clock, launch included): fp16 3x3 [16,28,28,256]->256 25.0 / 22.0,
    // [16,28,28,192]->256 20.6 / 18.4, [16,20,20,256]->384 23.2 / 20.5, [16,56,56,128]->128 26.1 / 25.7, dilation 2
    // [16,28,28,256]->256 25.3 / 25.6.
    if (tapped && batches == 1 && patch_label && launch_gemm_patch<T>(st, a))
        return patch_label;
    // Enough work for this kernel to be the faster one, in tiles of the smallest shape.  MATMUL and pointwise
    // convolutions: almost any (us patch kernel / this kernel, host clock: MATMUL int8 [1,512,512]x[1,512,512], 16
    // tiles, 10.1 / 5.4; [8,256,256]x[8,256,256] 9.3 / 5.0; bf16 12.6 / 6.3, 10.5 / 5.4; fp16 [1,14,14,1024]->1024,
    // 16 tiles, 15.1 / 7.2; [4,7,7,2048]->512, 8 tiles, 23.4 / 13.4; [2,28,28,512]->128 9.5 / 5.4; int8 11.1 / 6.0,
    // 15.5 / 7.6, 7.9 / 5.0).  A convolution with taps: from some 96 tiles (fp16 3x3 [64,7,7,512]->512, 100 tiles,
    // 64.8 / 40.0; [16,14,14,512]->512 41.4 / 40.0; [32,7,7,512]->512, 52 tiles, 34.5 / 39.7).
    const int64_t min_tiles = a.taps > 1 ? 96 : 4;
    if ((((int64_t)a.M + 127) / 128) * ((a.N + 127) / 128) * batches < min_tiles)
        return nullptr;
    // Tile shapes, largest first; the cost of a shape is the number of passes its tiles take over the 256
    // CUs times the matrix work of one tile.  Work too small to fill the CUs with the smallest shape is left
    // to the patch kernel.
    static const int shapes[3][2] = { { 4, 2 }, { 2, 2 }, { 2, 1 } };
    int best = -1;
    double best_cost = 0;
    for (int c = 0; c < 3; c++)
    {
        const int64_t tn = (a.N + 64 * shapes[c][0] - 1) / (64 * shapes[c][0]);
        const int64_t tm = (a.M + 128 * shapes[c][1] - 1) / (128 * shapes[c][1]);
        const int64_t tiles = tn * tm * batches;
        // the tile index is split by two FastDiv divisions, exact while dividend * divisor < 2^32
        if (tiles > (1 << 22) || !fastdiv_exact_up_to((uint64_t)tiles - 1, (uint32_t)(tn * tm)) ||
            !fastdiv_exact_up_to((uint64_t)(tn * tm) - 1, (uint32_t)tn))
            continue;
        const double passes = (double)((tiles + 255) / 256);
        const double cost   = passes * shapes[c][0] * shapes[c][1];
        if (best < 0 || cost < best_cost * 0.999)
            best = c, best_cost = cost;
    }
    if (best < 0)
        return nullptr;
    const int OCT = shapes[best][0], PXT = shapes[best][1];
    a.tiles_n         = (a.N + 64 * OCT - 1) / (64 * OCT);
    const int tiles_m = (a.M + 128 * PXT - 1) / (128 * PXT);
    a.tiles_per_batch = a.tiles_n * tiles_m;
    a.tiles_total     = a.tiles_per_batch * batches;
    a.per_xcd         = (a.tiles_total + 7) / 8;
    a.div_batch       = make_fastdiv((uint32_t)a.tiles_per_batch);
    a.div_tn          = make_fastdiv((uint32_t)a.tiles_n);
    const int blocks  = a.per_xcd * 8;
    const bool zp     = Mma<T>::is_int && (a.za != 0 || a.zw != 0);
    bool ok           = false;
#define TMI_GEMM_MODE(O, P, MODE)                                                                                      \
    ok = zp ? launch_gemm_shape<T, O, P, Mma<T>::is_int, MODE>(st, a, blocks)                                          \
            : launch_gemm_shape<T, O, P, false, MODE>(st, a, blocks)
#define TMI_GEMM_SHAPE(O, P)                                                                                           \
    if (OCT == O && PXT == P)                                                                                          \
    {                                                                                                                  \
        if (a.ldw)                                                                                                     \
            TMI_GEMM_MODE(O, P, GEMM_KMAJOR);                                                                          \
        else if (tapped)                                                                                               \
            TMI_GEMM_MODE(O, P, GEMM_TAPS);                                                                            \
        else                                                                                                           \
            TMI_GEMM_MODE(O, P, GEMM_KCONTIG);                                                                         \
    }
    TMI_GEMM_SHAPE(4, 2);
    TMI_GEMM_SHAPE(2, 2);
    TMI_GEMM_SHAPE(2, 1);
#undef TMI_GEMM_MODE
#undef TMI_GEMM_SHAPE
    return ok ? label : nullptr;
}

// Which of the two MFMA kernels a CONV2D tries first when the caller leaves the choice open.  The patch kernel
// stages an input patch with its halo once and serves every tap from LDS; this kernel reads each tap's operand
// block through L2 again, and wins where that does not matter or K is deep.  Measured on MI355X over ResNet-like
// layers (us, patch kernel / this kernel): pointwise layers int8 8.6 / 7.1, 21.3 / 14.8, 28.4 / 26.4 and
// fp16 7.5 / 5.3, 26.4 / 11.8, 21.7 / 15.8; 3x3 layers fp16 with IC 256 and 512: 31.7 / 28.2, 56.8 / 50.4,
// IC 128: 17.9 / 17.4, IC 64: 7.8 / 10.4; 3x3 layers int8: 7.5 / 11.0 (IC 64), 15.7 / 18.1 (IC 128),
// 23.7 / 25.9 (IC 256), 36.4 / 39.8 (IC 512).
bool gemm_mfma_preferred(int32_t in_dtype, const ConvGeom& g)
{
    if (g.KH * g.KW == 1)
        return true;
    // fp16 / bf16 layers with taps and 128 channels or more are this kernel's, except those that leave half of its
    // 128-channel tile empty: 3x3 stride 1, us patch kernel / this kernel: [32,56,56,256]->64 57.7 / 75.2,
    // [8,112,112,128]->64 33.6 / 45.7, [16,56,56,128]->64 18.1 / 24.8 (a tie from 512 channels on:
    // [32,28,28,512]->64 40.6 / 40.4; with a stride this kernel again: [32,56,56,256]->64 stride 2 35.5 / 24.4;
    // and from 80 output channels: [64,28,28,512]->80 93.3 / 79.7, [16,56,56,256]->96 53.4 / 40.3).
    if (in_dtype != TMI_INT8 && g.IC >= 128 && !(g.OC <= 64 && g.IC < 512 && g.stride_y * g.stride_x == 1))
        return true;
    // int8 layers with taps: where this kernel can keep the input patch in LDS it is the faster one.  us patch
    // kernel / this kernel (host clock): 3x3 [16,28,28,256]->256 25.3 / 19.8, [8,28,28,512]->512 37.3 / 28.4,
    // [16,56,56,128]->128 29.0 / 22.6, [32,28,28,256]->256 39.8 / 33.6; with the fused RESCALE 19.4 / 18.7,
    // 31.7 / 28.3, (slab kernel 15.3) / 24.8, 41 / 36.9.  The same for fp16 / bf16 layers with fewer than 128
    // channels, which the form without the patch loses: fp16 3x3 [8,56,56,64]->128 11.0 / 9.3, ->256 20.1 / 16.6,
    // [16,28,28,64]->256 11.3 / 8.9, [8,56,56,96]->192 26.0 / 20.1, [8,56,56,32]->128 8.3 / 6.6
    // (without the patch, [32,56,56,64]->64: 20.3 / 30.6).
    // int8 layers with taps and a stride: the patch kernel's patch grows with the stride, this kernel's loads do
    // not.  us patch kernel / this kernel, 3x3 stride 2: [64,28,28,256]->256 (196 tiles) 34.6 / 22.3,
    // [32,56,56,192]->192 45.2 / 26.8, [128,14,14,512]->512 89.1 / 33.8, [32,28,28,256]->512 34.4 / 21.8; with the
    // fused RESCALE 30.3 / 22.1, 49.4 / 28.2, 88.2 / 34.4, 29.9 / 22.0.  Around 100 tiles the two tie
    // ([32,28,28,512]->256 32.4 / 33.1, [32,28,28,192]->256 17.6 / 17.9, fused 15.5 / 19.0), so from 128 on.
    // Without a stride the patch kernel is the faster one on the mid-sized layers the rule was first measured on
    // (100 - 200 tiles: [16,28,28,256]->256 23.7 / 25.9, [16,14,14,512]->512 36.4 / 39.8) and loses beyond: 3x3
    // [16,28,28,1024]->256 (196 tiles) 63.0 / 60.3, [20,28,28,1024]->256 (246) 101.3 / 64.7, [32,28,28,1024]->256
    // 109.4 / 93.3, [12,56,56,512]->128 59.3 / 51.2, [16,56,56,512]->128 64.2 / 52.6; with the fused RESCALE 58.9 / 60.5,
    // 121.3 / 65.3, 113.4 / 94.2, 68.6 / 52.2, 61.4 / 53.2.  On images smaller than a tile it loses from this kernel's
    // minimum on: [32,7,7,1024]->1024 (104 tiles) 74.0 / 58.8, [64,7,7,512]->512 42.4 / 32.8, [128,7,7,1024]->1024
    // 288.4 / 93.8.  With 64 output channels half of this kernel's tile is empty and the patch kernel stays ahead
    // ([32,56,56,256]->64 45.4 / 59.2).
    const int64_t tiles = ((int64_t)g.N * g.OH * g.OW + 127) / 128 * ((g.OC + 127) / 128);
    if (in_dtype == TMI_INT8 && g.OC >= 96)
    {
        if (tiles >= (g.stride_y * g.stride_x > 1 ? 128 : 200) || (g.OH * g.OW <= 64 && tiles >= 96))
            return true;
    }
    // fp16 / bf16 layers with taps and 64 or 96 channels outside the patch form (a stride, rows wider than a tile): what
    // the patch kernel wins there are the layers with 64 output channels.  fp16 3x3, us patch kernel / this kernel:
    // stride 2 [32,56,56,64]->128 (196 tiles) 16.6 / 11.5, [64,28,28,96]->192 21.5 / 13.4, [64,56,56,64]->128
    // 29.9 / 17.5, [32,56,56,64]->256 29.5 / 17.6; stride 1 [2,160,160,64]->128 30.9 / 17.5, [8,160,160,64]->96
    // 66.2 / 49.5; with 32 channels the two tie ([16,112,112,32]->128 stride 2 13.2 / 13.4).
    if (in_dtype != TMI_INT8 && g.IC >= 64 && g.OC >= 96 && tiles >= 196)
        return true;
    // int8 layers below 120 tiles: the patch kernel, whose set-up is the shorter one (us patch kernel / this kernel's patch
    // form, 3x3, fused RESCALE: [4,28,28,256]->256 (50 tiles) 14.5 / 17.3, [8,28,28,256]->256 (98) 15.0 / 17.3,
    // [32,14,14,256]->256 15.2 / 17.3, [16,14,14,512]->512 (100) 23.6 / 26.7, [8,14,14,384]->384 18.8 / 24.1; int32 results
    // [8,28,28,256]->256 15.8 / 16.3; from 147 tiles on the other way: [12,28,28,256]->256 18.1 / 17.5, [16,..] 19.7 / 18.1).
    if (in_dtype == TMI_INT8 && tiles < 120)
        return false;
    int rows, patch_h, patch_w;
    const int icb = g.IC * (in_dtype == TMI_INT8 ? 1 : 2);
    return patch_form_geometry(g.OH, g.OW, g.KH, g.KW, g.stride_y, g.stride_x, g.dil_y, g.dil_x, icb, g.OC, rows,
                               patch_h, patch_w);
}

// nullptr when the operation is not a GEMM this kernel takes; the caller then goes to the patch kernel.
const char* launch_gemm_mfma(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                             const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                             void* out, int64_t w_batch_stride, int64_t w_kmajor_stride, const void* pad_page,
                             uint32_t* flag_word)
{
    // a fused RESCALE: the fast form only (32-bit scale, SINGLE / DOUBLE rounding), on int8 convolutions
    if (rp.enabled && (!rp.fast || in_dtype != TMI_INT8 || (out_dtype != TMI_INT8 && out_dtype != TMI_INT16) ||
                       w_batch_stride || w_kmajor_stride || !flag_word))
        return nullptr;
    const int taps    = g.KH * g.KW;
    const bool plain  = taps == 1 && g.stride_y == 1 && g.stride_x == 1 && g.pad_top == 0 && g.pad_left == 0 &&
                       g.OH == g.IH && g.OW == g.IW;
    if (in_dtype != TMI_INT8 && in_dtype != TMI_FP16 && in_dtype != TMI_BF16)
        return nullptr;
    const int eb = in_dtype == TMI_INT8 ? 1 : 2;
    if (!plain)
    {
        // a convolution with taps, strides or padding: per-image weights and K-major weights are MATMUL's; a tap
        // outside the image reads the page of input_zp bytes
        if (w_batch_stride || w_kmajor_stride || !pad_page || taps > 32)
            return nullptr;
        if ((int64_t)g.N * g.IH * g.IW * g.IC * eb >= (int64_t(1) << 31))
            return nullptr;
    }
    const bool wide = in_dtype == TMI_INT8 ? out_dtype == TMI_INT32 : out_dtype == TMI_FP32;
    if (!wide && !rp.enabled && (in_dtype == TMI_INT8 || out_dtype != in_dtype))
        return nullptr;
    if (rp.enabled && wide)
        return nullptr;
    const int64_t icb = (int64_t)g.IC * eb;
    const int64_t kb  = icb * taps;
    if (icb % 64 != 0)
        return nullptr;
    // MATMUL: one GEMM per image with its own weights; CONV2D: all images are rows of one GEMM
    const bool per_image  = w_batch_stride != 0;
    const int batches     = per_image ? g.N : 1;
    const int64_t M       = (int64_t)g.OH * g.OW * (per_image ? 1 : g.N);
    const int64_t out_eb  = rp.enabled ? (out_dtype == TMI_INT8 ? 1 : 2) : (wide ? 4 : eb);
    if (M < 128 || g.OC < 64 || M * kb >= (int64_t(1) << 32) || (int64_t)g.OC * kb >= (int64_t(1) << 32))
        return nullptr;
    // K-major weights: whole 16-byte pieces per K row
    if (w_kmajor_stride && ((w_kmajor_stride & 15) || w_kmajor_stride != (int64_t)g.OC * eb))
        return nullptr;
    // rows are multiples of 64 bytes, so 16-byte aligned bases keep every operand chunk aligned; the 16-byte
    // stores are only used when OC is a multiple of 16, which keeps every output row and batch aligned too
    if ((((uintptr_t)in | (uintptr_t)w | (uintptr_t)out | (uintptr_t)pad_page) & 15) || (w_batch_stride & 15))
        return nullptr;
    // (enough work to fill the CUs: checked by the launcher of the form that takes the layer)

    GemmArgs a{};
    a.a = (const uint8_t*)in, a.w = (const uint8_t*)w, a.bias = bias, a.out = out;
    a.a_batch = per_image ? M * kb : 0, a.w_batch = per_image ? w_batch_stride : 0;
    a.o_batch = per_image ? M * g.OC * out_eb : 0;
    a.M = (int32_t)M, a.N = g.OC, a.kb = (int32_t)kb, a.n_blocks = (int32_t)(kb / 64);
    a.bias_len = g.bias_len, a.za = in_zp, a.zw = w_zp, a.K = g.IC * taps;
    a.out_is_wide = wide ? 1 : 0;
    a.rp = rp, a.flag_word = flag_word, a.out_bytes = (int32_t)out_eb;
    a.ldw         = (int32_t)w_kmajor_stride;
    a.taps        = 1;
    if (!plain)
    {
        a.taps      = taps;
        a.pad_page = (const uint8_t*)pad_page;
        a.IH = g.IH, a.IW = g.IW, a.OH = g.OH, a.OW = g.OW, a.KW = g.KW;
        a.icb = (int32_t)icb, a.bpt = (int32_t)(icb / 64);
        a.sy = g.stride_y, a.sx = g.stride_x, a.dy = g.dil_y, a.dx = g.dil_x;
        a.pad_top = g.pad_top, a.pad_left = g.pad_left;
        a.div_bpt = make_fastdiv((uint32_t)a.bpt), a.div_kw = make_fastdiv((uint32_t)a.KW);
    }
    const bool tapped = !plain;
    switch (in_dtype)
    {
        case TMI_INT8:
            return launch_gemm_t<int8_t>(st, a, batches, tapped, rp.enabled ? "gemm_mfma_i8_rescale" : "gemm_mfma_i8",
                                         rp.enabled ? "gemm_mfma_i8_rescale_patch" : "gemm_mfma_i8_patch");
        case TMI_FP16: return launch_gemm_t<_Float16>(st, a, batches, tapped, "gemm_mfma_f16", "gemm_mfma_f16_patch");
        default: return launch_gemm_t<bf16_t>(st, a, batches, tapped, "gemm_mfma_bf16", "gemm_mfma_bf16_patch");
    }
}

}    // namespace tmi
