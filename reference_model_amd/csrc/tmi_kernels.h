// Host-callable launchers of every kernel family.  Each returns the name of the kernel variant it
// enqueued (nullptr if the combination is not implemented) and never synchronises.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "tmi_device.h"

namespace tmi
{

// A kernel's dynamic LDS limit is a per-device attribute of the function.  `done` holds, per device, the largest
// size already granted to one kernel instantiation; the attribute is set again only when a launch needs more.
// Safe for contexts used from different host threads.
constexpr int kMaxDevices = 16;
struct LdsLimit
{
    std::atomic<size_t> done[kMaxDevices];
};
inline bool ensure_dynamic_lds(const void* kernel, size_t bytes, LdsLimit& lim)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return false;
    if (bytes <= lim.done[dev].load(std::memory_order_acquire))
        return true;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
    {
        (void)hipGetLastError();    // the caller goes on to another kernel, whose launch must not inherit this error
        return false;
    }
    lim.done[dev].store(bytes, std::memory_order_release);
    return true;
}

// Validated geometry of a CONV2D / DEPTHWISE_CONV2D call.
struct ConvGeom
{
    int32_t N, IH, IW, IC, OC, KH, KW, OH, OW;
    int32_t pad_top, pad_left, stride_y, stride_x, dil_y, dil_x;
    int32_t bias_len;
    int32_t M;    // depthwise channel multiplier (unused by CONV2D)
};

// bf16 carried as its bit pattern
struct bf16_t
{
    uint16_t bits;
};

__host__ __device__ inline float bf16_to_float(bf16_t v)
{
    union
    {
        uint32_t u;
        float f;
    } x;
    x.u = (uint32_t)v.bits << 16;
    return x.f;
}

__host__ __device__ inline bf16_t float_to_bf16(float f)
{
    union
    {
        uint32_t u;
        float f;
    } x;
    x.f = f;
    bf16_t r;
    if ((x.u & 0x7fffffffu) > 0x7f800000u)    // NaN: keep it quiet
        r.bits = (uint16_t)((x.u >> 16) | 0x0040u);
    else
        r.bits = (uint16_t)((x.u + 0x7fffu + ((x.u >> 16) & 1u)) >> 16);    // round to nearest even
    return r;
}

// elementwise.hip
const char* launch_rescale(hipStream_t st, const RescaleParams& p, int32_t in_dtype, int32_t out_dtype,
                           const void* in, void* out, int64_t n, int32_t C, uint32_t* flag_word);
const char* launch_clamp(hipStream_t st, int32_t dtype, const void* in, void* out, int64_t n, int32_t lo,
                         int32_t hi);
const char* launch_clamp_fp(hipStream_t st, int32_t dtype, const void* in, void* out, int64_t n, float lo, float hi,
                            int32_t nan_mode);
// copy (mode 0), read-only (1) or write-only (2) pass over `bytes` bytes: what the memory system sustains
const char* launch_stream_probe(hipStream_t st, int32_t mode, const void* src, void* dst, int64_t bytes);
// grid, block and dynamic LDS bytes of this thread's latest launch of the kernel that loads a CONV2D layer's
// operands straight into LDS (zeros before the first)
extern thread_local int32_t last_launch_shape[3];
// a kernel without work: the cost of one launch of this grid, block and dynamic LDS size
const char* launch_empty(hipStream_t st, int32_t grid, int32_t block, int32_t lds_bytes);

// pointwise.hip: int8 CONV2D 1x1 (unit stride, no padding) with 16 ... 2048 input channels in multiples of 8 and
// weight_zp 0; a wave per tile of 32 output channels (from 168 input channels on: four waves that split K), operands
// straight from global memory into registers
const char* launch_conv2d_pointwise(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                                    const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                                    void* out, uint32_t* flag_word);

// pointwise.hip, first layers: int8 CONV2D with 3 x 3 ... 7 x 7 taps over at most 4 channels (KW * IC <= 32, dilation_x 1,
// weight_zp 0) as a pre-pass into `scratch` (padding materialised, weights as 32 bytes per tap row) plus the pointwise
// kernel with a K step per tap row.  conv2d_stem_scratch_bytes() is 0 for a layer the form does not take.
size_t conv2d_stem_scratch_bytes(int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, int32_t w_zp, const RescaleParams& rp);
const char* launch_conv2d_stem(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                               const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp, void* out,
                               void* scratch, uint32_t* flag_word);

// conv_ksplit.hip: small int8 CONV2D layers with taps and a long reduction (IC a multiple of 32, weight_zp 0): a workgroup
// per tile of 32 x 32 results, K split over its waves, operands straight from global memory into registers
const char* launch_conv2d_ksplit(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                                 const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                                 void* out, const void* pad_page, uint32_t* flag_word);

// direct.hip: one output element per lane, any legal shape.  out_dtype is the stored output type
// (INT32 without rescale; the rescale output type with it; FP16/BF16/FP32 for floating point).
const char* launch_conv2d_direct(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g,
                                 const void* in, const void* w, const void* bias, int32_t in_zp, int32_t w_zp,
                                 const RescaleParams& rp, void* out, uint32_t* flag_word);
const char* launch_depthwise_direct(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g,
                                    const void* in, const void* w, const void* bias, int32_t in_zp, int32_t w_zp,
                                    const RescaleParams& rp, void* out, uint32_t* flag_word);
// precise.hip: fp64 precise-mode / bounds-mode passes (abs_mode != 0: sums over absolute values) of CONV2D,
// DEPTHWISE_CONV2D and MATMUL on fp16 / bf16 / fp32 operands, and the DOT_PRODUCT check as a reduction
// (results: 3 doubles, counts: 1 word, both zero before the launch).  nullptr for another operand type.
// abs_max_slot: device scratch of one double; when given together with abs_mode, every input element is replaced by
// the input tensor's largest magnitude (the bounds pass of an operator whose local_bound attribute is false).
const char* launch_conv_precise(hipStream_t st, int32_t in_dtype, bool depthwise, const ConvGeom& g, const void* in,
                                const void* w, const void* bias, int32_t abs_mode, double* abs_max_slot, double* out);
const char* launch_matmul_precise(hipStream_t st, int32_t in_dtype, int32_t N, int32_t H, int32_t C, int32_t W,
                                  const void* a, const void* b, int32_t abs_mode, double* out);
const char* launch_dp_check(hipStream_t st, int32_t out_dtype, int64_t n, const void* imp, const double* ref,
                            const double* bnd, int32_t abs_bound, double* results, unsigned long long* counts);

// pool.hip: AVG_POOL2D (avg) / MAX_POOL2D; nullptr for a dtype without a kernel or 2^32 work items or more.
const char* launch_pool(hipStream_t st, bool avg, int32_t dtype, int32_t N, int32_t IH, int32_t IW, int32_t C,
                        int32_t OH, int32_t OW, int32_t kernel_y, int32_t kernel_x, int32_t stride_y, int32_t stride_x,
                        int32_t pad_top, int32_t pad_left, int32_t in_zp, int32_t out_zp, int32_t nan_mode,
                        const void* in, void* out, uint32_t* flag_word);

// conv2d_slab.hip: int8 CONV2D with IC = 64, 96 or 128, 3x3 or 1x1 taps and weight_zp = 0 (int32 result, or the fast form of a fused
// RESCALE to int8 / int16): weight slab and input patch loaded straight into LDS; nullptr for anything else.
// pad_page: 64 bytes of input_zp in device memory.
// TRANSPOSE_CONV2D through the slab kernel: the CONV2D geometry handed over describes the stride-1 convolution over the
// input with up_y - 1 (up_x - 1) holes between its rows (columns); IH x IW are those of the tensor in memory, and
// the weights are in TRANSPOSE_CONV2D's own tap order.
struct SlabHoles
{
    int32_t up_y, up_x, IH, IW;
};
// CONV3D through the slab kernel: the CONV2D geometry handed over has N * OD images and KD * IC channels; the input
// tensor [N, ID, IH, IW, IC] and the weights [OC, KD, KH, KW, IC] are read where they lie.
struct SlabDepth
{
    int32_t KD, ID, OD, stride_d, dilation_d, pad_d0;
};
const char* launch_conv2d_slab(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                               const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                               void* out, const void* pad_page, uint32_t* flag_word, const SlabHoles* tc = nullptr,
                               const SlabDepth* c3d = nullptr);

// depthwise_slab.hip: int8 DEPTHWISE_CONV2D with multiplier 1, 3x3 taps, weight_zp = 0 and 32..512 channels in
// multiples of 16 on the matrix cores (one MFMA per tap against a diagonal weight tile); nullptr for anything else.
const char* launch_depthwise_slab(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                                  const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                                  void* out, const void* pad_page, uint32_t* flag_word);

// depthwise_stream.hip: the same layers with the pixel operand loaded straight from global memory into the matrix
// instruction's registers (no patch in LDS; a wave keeps a group of channel blocks and walks pixel tiles with the next
// tile's loads in flight); nullptr for anything else.
const char* launch_depthwise_stream(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                                    const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                                    void* out, uint32_t* flag_word);

// gemm_mfma.hip: whether a CONV2D left to automatic choice tries the GEMM kernel before the patch kernel.
bool gemm_mfma_preferred(int32_t in_dtype, const ConvGeom& g);

// gemm_mfma.hip: CONV2D as a GEMM over (ky, kx, ic), with a fused RESCALE (+ CLAMP) when rp is enabled and of the
// fast form, and MATMUL (w_batch_stride != 0: per-image weights), with operands loaded straight into LDS; nullptr
// when the operation is not such a GEMM or too small to gain.  w_kmajor_stride != 0: the weights are [K][OC] with
// that many bytes per K row (MATMUL's second operand as it lies in memory) instead of [OC][K].  pad_page: 64
// bytes of input_zp (zeros for floating point) in device memory, read where a tap falls outside the image;
// without it only 1x1 / stride 1 / unpadded convolutions are taken.  flag_word: needed for a fused RESCALE.
const char* launch_gemm_mfma(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                             const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                             void* out, int64_t w_batch_stride, int64_t w_kmajor_stride = 0,
                             const void* pad_page = nullptr, uint32_t* flag_word = nullptr);

// fp16 / bf16 DEPTHWISE_CONV2D, 8 channels per lane (depthwise_fp.hip); nullptr when the layer is not eligible.
const char* launch_depthwise_fp_vec(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                                    const void* w, const void* bias, void* out);

// conv2d_mfma.hip: implicit GEMM on the matrix cores with the fused epilogue; nullptr when not eligible.
const char* launch_conv2d_mfma(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g, const void* in,
                               const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                               void* out, uint32_t* flag_word, int64_t w_batch_stride = 0);
// elementwise.hip: [N, R, C] -> [N, C, R] for 1- or 2-byte elements (MATMUL's second operand becomes K-contiguous).
const char* launch_transpose(hipStream_t st, int32_t elem_bytes, int32_t N, int32_t R, int32_t C, const void* in,
                             void* out);
// relayout.hip: whole-channel-vector copies that turn TRANSPOSE_CONV2D / CONV3D operands into CONV2D operands.
const char* launch_flip_taps(hipStream_t st, int32_t row_bytes, int32_t OC, int32_t KH, int32_t KW, const void* src,
                             void* dst);
const char* launch_upsample(hipStream_t st, int32_t row_bytes, int32_t N, int32_t IH, int32_t IW, int32_t sy,
                            int32_t sx, int32_t fill, const void* src, void* dst);
const char* launch_gather_depth(hipStream_t st, int32_t row_bytes, int32_t N, int32_t ID, int32_t OD, int32_t KD,
                                int32_t HW, int32_t stride_d, int32_t dilation_d, int32_t pad_d0, int32_t fill,
                                const void* src, void* dst);
const char* launch_permute_w3d(hipStream_t st, int32_t row_bytes, int32_t OC, int32_t KD, int32_t KHW,
                               const void* src, void* dst);
const char* launch_tconv_operands(hipStream_t st, int32_t row_bytes, int32_t OC, int32_t KH, int32_t KW, const void* w_src,
                                  void* w_dst, int32_t N, int32_t IH, int32_t IW, int32_t sy, int32_t sx, int32_t fill,
                                  const void* in_src, void* in_dst);
const char* launch_conv3d_operands(hipStream_t st, int32_t row_bytes, int32_t OC, int32_t KD, int32_t KHW, const void* w_src,
                                   void* w_dst, int32_t N, int32_t ID, int32_t OD, int32_t HW, int32_t stride_d,
                                   int32_t dilation_d, int32_t pad_d0, int32_t fill, const void* in_src, void* in_dst);
// depthwise.hip: 4 channels per lane, dot4 across taps, fused epilogue; nullptr when not eligible.
const char* launch_depthwise_vec(hipStream_t st, int32_t in_dtype, int32_t out_dtype, const ConvGeom& g,
                                 const void* in, const void* w, const void* bias, int32_t in_zp, int32_t w_zp,
                                 const RescaleParams& rp, void* out, uint32_t* flag_word);
// INT16 x INT8 -> INT48 CONV2D / DEPTHWISE_CONV2D and INT16 x INT16 -> INT48 MATMUL (int64 bias and results)
const char* launch_conv_i16_direct(hipStream_t st, bool depthwise, const ConvGeom& g, const void* in, const void* w,
                                   const void* bias, int32_t w_zp, void* out);
const char* launch_matmul_i16_direct(hipStream_t st, int32_t N, int32_t H, int32_t C, int32_t W, const void* a, const void* b,
                                     void* out);
const char* launch_matmul_direct(hipStream_t st, int32_t in_dtype, int32_t N, int32_t H, int32_t C, int32_t W,
                                 const void* a, const void* b, int32_t a_zp, int32_t b_zp, void* out);

}    // namespace tmi
