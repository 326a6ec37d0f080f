// Operand re-layouts that turn TRANSPOSE_CONV2D and CONV3D into the CONV2D the matrix-core kernel computes.
//
// TRANSPOSE_CONV2D (tensor_ops.cpp:2138-2187): out[oy,ox] takes tap (ky,kx) from input position
// ((oy - out_pad_top - ky) / sy, (ox - out_pad_left - kx) / sx) when both divisions are exact and in range.
// With ky' = KH-1-ky this is a stride-1 CONV2D with the taps flipped, pads KH-1+out_pad, over the input with
// sy-1 (sx-1) holes between its rows (columns).  A hole contributes nothing in the reference; a hole that
// holds input_zp contributes (zp - zp) * (w - w_zp) = 0 as well, so the holes are filled with input_zp.
//
// CONV3D (tensor_ops.cpp:1058-1108): the depth taps become channels.  Output slice (n, od) is a CONV2D over
// the KD input slices it touches, laid side by side along the channel axis (slices outside the volume hold
// input_zp), with the weights permuted from [OC,KD,KH,KW,IC] to [OC,KH,KW,KD*IC].
//
// All four are copies of whole channel vectors ("rows"); a lane moves one 16-byte piece when the row length
// and the pointers allow it, else one byte.
#include "tmi_kernels.h"

namespace tmi
{

typedef int rl_v4i __attribute__((ext_vector_type(4)));

enum
{
    RL_FLIP_TAPS    = 0,
    RL_UPSAMPLE     = 1,
    RL_GATHER_DEPTH = 2,
    RL_PERMUTE_W3D  = 3
};

struct RelayoutArgs
{
    const uint8_t* src;
    uint8_t* dst;
    int64_t n_rows;       // destination rows
    int32_t row_bytes;    // bytes of one channel vector
    int32_t pieces;       // pieces per row (row_bytes / 16 or row_bytes)
    int32_t fill;         // byte stored where the source has no row (input_zp)
    int32_t mode;
    int32_t d[10];        // mode-specific dimensions, see source_row()
};

// Source row of a destination row, or -1 when the destination is a fill row.
__device__ __forceinline__ int64_t source_row(const RelayoutArgs& a, int64_t r)
{
    const int32_t* d = a.d;
    switch (a.mode)
    {
        case RL_FLIP_TAPS:
        {    // d: KH, KW; rows [OC][KH][KW]
            const int64_t taps = (int64_t)d[0] * d[1];
            const int64_t oc   = r / taps;
            const int t        = (int)(r - oc * taps);
            return oc * taps + (taps - 1 - t);    // (KH-1-ky)*KW + (KW-1-kx) = taps-1 - (ky*KW+kx)
        }
        case RL_UPSAMPLE:
        {    // d: IH, IW, UH, UW, sy, sx; rows [N][UH][UW]
            const int64_t x = r % d[3];
            const int64_t t = r / d[3];
            const int64_t y = t % d[2];
            const int64_t n = t / d[2];
            if ((y % d[4]) != 0 || (x % d[5]) != 0)
                return -1;
            return (n * d[0] + y / d[4]) * d[1] + x / d[5];
        }
        case RL_GATHER_DEPTH:
        {    // d: ID, OD, KD, HW (= IH*IW), sd, dd, pd0; rows [N][OD][HW][KD]
            const int64_t kd = r % d[2];
            int64_t t        = r / d[2];
            const int64_t p  = t % d[3];
            t /= d[3];
            const int64_t od = t % d[1];
            const int64_t n  = t / d[1];
            const int64_t z  = od * d[4] + kd * d[5] - d[6];
            if (z < 0 || z >= d[0])
                return -1;
            return (n * d[0] + z) * d[3] + p;
        }
        default:
        {    // RL_PERMUTE_W3D  d: KD, KHW (= KH*KW); rows [OC][KHW][KD] <- [OC][KD][KHW]
            const int64_t kd = r % d[0];
            const int64_t t  = r / d[0];
            const int64_t k  = t % d[1];
            const int64_t oc = t / d[1];
            return (oc * d[0] + kd) * d[1] + k;
        }
    }
}

template <bool VEC>
__device__ __forceinline__ void relayout_rows(const RelayoutArgs& a, int64_t block, int64_t n_blocks)
{
    const int64_t total  = a.n_rows * a.pieces;
    const int64_t stride = n_blocks * blockDim.x;
    const int fill_word  = (a.fill & 0xff) * 0x01010101;
    for (int64_t i = block * blockDim.x + threadIdx.x; i < total; i += stride)
    {
        const int64_t r   = i / a.pieces;
        const int piece   = (int)(i - r * a.pieces);
        const int64_t src = source_row(a, r);
        if constexpr (VEC)
        {
            rl_v4i v = rl_v4i{ fill_word, fill_word, fill_word, fill_word };
            if (src >= 0)
                v = *reinterpret_cast<const rl_v4i*>(a.src + src * a.row_bytes + piece * 16);
            *reinterpret_cast<rl_v4i*>(a.dst + r * a.row_bytes + piece * 16) = v;
        }
        else
            a.dst[r * a.row_bytes + piece] = src >= 0 ? a.src[src * a.row_bytes + piece] : (uint8_t)a.fill;
    }
}

template <bool VEC>
__global__ __launch_bounds__(256) void relayout_kernel(RelayoutArgs a)
{
    relayout_rows<VEC>(a, blockIdx.x, gridDim.x);
}

// Two re-layouts (an operator's weights and its input) in one launch: the first blocks_a workgroups take the first.
struct RelayoutPair
{
    RelayoutArgs a, b;
    int32_t blocks_a;
};

__global__ __launch_bounds__(256) void relayout_pair_kernel(RelayoutPair p)
{
    if ((int)blockIdx.x < p.blocks_a)
        relayout_rows<true>(p.a, blockIdx.x, p.blocks_a);
    else
        relayout_rows<true>(p.b, (int)blockIdx.x - p.blocks_a, (int)gridDim.x - p.blocks_a);
}

static bool relayout_vec(RelayoutArgs& a)
{
    const bool vec = (a.row_bytes & 15) == 0 && (((uintptr_t)a.src | (uintptr_t)a.dst) & 15) == 0;
    a.pieces       = vec ? a.row_bytes / 16 : a.row_bytes;
    return vec;
}

static int64_t relayout_blocks(const RelayoutArgs& a)
{
    const int64_t blocks = (a.n_rows * a.pieces + 255) / 256;
    return blocks > 256 * 64 ? 256 * 64 : blocks;
}

static const char* launch_relayout(hipStream_t st, RelayoutArgs& a)
{
    if (a.n_rows <= 0 || a.row_bytes <= 0)
        return "relayout_empty";
    const bool vec       = relayout_vec(a);
    const int64_t blocks = relayout_blocks(a);
    if (vec)
        hipLaunchKernelGGL(relayout_kernel<true>, dim3((int)blocks), dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL(relayout_kernel<false>, dim3((int)blocks), dim3(256), 0, st, a);
    return "relayout";
}

// One launch when both re-layouts move 16-byte pieces, else one each.
static const char* launch_relayout_pair(hipStream_t st, RelayoutArgs& a, RelayoutArgs& b)
{
    if (a.n_rows > 0 && b.n_rows > 0 && a.row_bytes > 0 && b.row_bytes > 0 && relayout_vec(a) && relayout_vec(b))
    {
        RelayoutPair p{ a, b, (int32_t)relayout_blocks(a) };
        hipLaunchKernelGGL(relayout_pair_kernel, dim3(p.blocks_a + (int)relayout_blocks(b)), dim3(256), 0, st, p);
        return "relayout_pair";
    }
    launch_relayout(st, a);
    return launch_relayout(st, b);
}

static RelayoutArgs flip_taps_args(int32_t row_bytes, int32_t OC, int32_t KH, int32_t KW, const void* src, void* dst)
{
    RelayoutArgs a{};
    a.src = (const uint8_t*)src, a.dst = (uint8_t*)dst, a.row_bytes = row_bytes, a.mode = RL_FLIP_TAPS;
    a.n_rows = (int64_t)OC * KH * KW;
    a.d[0] = KH, a.d[1] = KW;
    return a;
}

static RelayoutArgs upsample_args(int32_t row_bytes, int32_t N, int32_t IH, int32_t IW, int32_t sy, int32_t sx,
                                  int32_t fill, const void* src, void* dst)
{
    RelayoutArgs a{};
    a.src = (const uint8_t*)src, a.dst = (uint8_t*)dst, a.row_bytes = row_bytes, a.mode = RL_UPSAMPLE, a.fill = fill;
    const int32_t UH = (IH - 1) * sy + 1, UW = (IW - 1) * sx + 1;
    a.n_rows = (int64_t)N * UH * UW;
    a.d[0] = IH, a.d[1] = IW, a.d[2] = UH, a.d[3] = UW, a.d[4] = sy, a.d[5] = sx;
    return a;
}

static RelayoutArgs gather_depth_args(int32_t row_bytes, int32_t N, int32_t ID, int32_t OD, int32_t KD, int32_t HW,
                                      int32_t stride_d, int32_t dilation_d, int32_t pad_d0, int32_t fill,
                                      const void* src, void* dst)
{
    RelayoutArgs a{};
    a.src = (const uint8_t*)src, a.dst = (uint8_t*)dst, a.row_bytes = row_bytes, a.mode = RL_GATHER_DEPTH;
    a.fill   = fill;
    a.n_rows = (int64_t)N * OD * HW * KD;
    a.d[0] = ID, a.d[1] = OD, a.d[2] = KD, a.d[3] = HW, a.d[4] = stride_d, a.d[5] = dilation_d, a.d[6] = pad_d0;
    return a;
}

static RelayoutArgs permute_w3d_args(int32_t row_bytes, int32_t OC, int32_t KD, int32_t KHW, const void* src, void* dst)
{
    RelayoutArgs a{};
    a.src = (const uint8_t*)src, a.dst = (uint8_t*)dst, a.row_bytes = row_bytes, a.mode = RL_PERMUTE_W3D;
    a.n_rows = (int64_t)OC * KD * KHW;
    a.d[0] = KD, a.d[1] = KHW;
    return a;
}

const char* launch_flip_taps(hipStream_t st, int32_t row_bytes, int32_t OC, int32_t KH, int32_t KW, const void* src,
                             void* dst)
{
    RelayoutArgs a = flip_taps_args(row_bytes, OC, KH, KW, src, dst);
    return launch_relayout(st, a);
}

const char* launch_upsample(hipStream_t st, int32_t row_bytes, int32_t N, int32_t IH, int32_t IW, int32_t sy,
                            int32_t sx, int32_t fill, const void* src, void* dst)
{
    RelayoutArgs a = upsample_args(row_bytes, N, IH, IW, sy, sx, fill, src, dst);
    return launch_relayout(st, a);
}

const char* launch_gather_depth(hipStream_t st, int32_t row_bytes, int32_t N, int32_t ID, int32_t OD, int32_t KD,
                                int32_t HW, int32_t stride_d, int32_t dilation_d, int32_t pad_d0, int32_t fill,
                                const void* src, void* dst)
{
    RelayoutArgs a = gather_depth_args(row_bytes, N, ID, OD, KD, HW, stride_d, dilation_d, pad_d0, fill, src, dst);
    return launch_relayout(st, a);
}

const char* launch_permute_w3d(hipStream_t st, int32_t row_bytes, int32_t OC, int32_t KD, int32_t KHW,
                               const void* src, void* dst)
{
    RelayoutArgs a = permute_w3d_args(row_bytes, OC, KD, KHW, src, dst);
    return launch_relayout(st, a);
}

// TRANSPOSE_CONV2D's two operands (flipped taps; input with holes) in one launch where possible.
const char* launch_tconv_operands(hipStream_t st, int32_t row_bytes, int32_t OC, int32_t KH, int32_t KW, const void* w_src,
                                  void* w_dst, int32_t N, int32_t IH, int32_t IW, int32_t sy, int32_t sx, int32_t fill,
                                  const void* in_src, void* in_dst)
{
    RelayoutArgs a = flip_taps_args(row_bytes, OC, KH, KW, w_src, w_dst);
    RelayoutArgs b = upsample_args(row_bytes, N, IH, IW, sy, sx, fill, in_src, in_dst);
    return launch_relayout_pair(st, a, b);
}

// CONV3D's two operands (weights with the depth taps as channels; input slices gathered along the channels).
const char* launch_conv3d_operands(hipStream_t st, int32_t row_bytes, int32_t OC, int32_t KD, int32_t KHW, const void* w_src,
                                   void* w_dst, int32_t N, int32_t ID, int32_t OD, int32_t HW, int32_t stride_d,
                                   int32_t dilation_d, int32_t pad_d0, int32_t fill, const void* in_src, void* in_dst)
{
    RelayoutArgs a = permute_w3d_args(row_bytes, OC, KD, KHW, w_src, w_dst);
    RelayoutArgs b = gather_depth_args(row_bytes, N, ID, OD, KD, HW, stride_d, dilation_d, pad_d0, fill, in_src, in_dst);
    return launch_relayout_pair(st, a, b);
}

}    // namespace tmi
