// C ABI of the library: context, device memory, operand validation and kernel selection.
// Validation follows the reference operator's checkTensorAttributes()/eval() checks so that the same
// malformed node is rejected with the same status; arithmetic lives in the kernel files.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "tmi_kernels.h"

// Scratch memory of tmi_transpose_conv2d_noalloc, the one entry point that may not allocate: it lives in the
// library's device image, so every GPU the library runs on holds its own copy (at its own address) from the
// moment the code object is loaded until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; the per-device address obtained from it at context creation is what kernels receive.
static __device__ __align__(256) unsigned char scratch[TMI_NOALLOC_SCRATCH_BYTES];

namespace
{
using tmi::kMaxDevices;
std::mutex g_scratch_mutex;
unsigned char* g_scratch_ptr[kMaxDevices] = {};    // device address of `scratch` on each device, once known

// Looks up this device's copy of `scratch` (the device must be current).  No allocation happens here: the
// array is part of the loaded code object.
hipError_t scratch_address(int device, unsigned char** out)
{
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device])
    {
        unsigned char* p = nullptr;
        hipError_t e     = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess)
            return e;
        if (!p)
            return hipErrorInvalidSymbol;
        g_scratch_ptr[device] = p;
    }
    *out = g_scratch_ptr[device];
    return hipSuccess;
}
}    // namespace

struct tmi_ctx
{
    int device            = 0;
    hipStream_t stream    = nullptr;
    bool owns_stream      = false;
    uint32_t* flags_dev   = nullptr;    // latched REQUIRE conditions
    uint8_t* pages_dev    = nullptr;    // 256 pages of 64 bytes, page v filled with byte v: what padding reads
    uint32_t* flags_host  = nullptr;    // pinned staging word
    void* workspace       = nullptr;    // scratch for operand re-layout (MATMUL's transposed B)
    size_t workspace_size = 0;
    std::vector<void*> retired;         // outgrown scratch blocks: captured graphs may still name them
    size_t retired_bytes  = 0;          // their sizes, summed
    unsigned char* static_scratch = nullptr;    // this device's copy of the library's static scratch array
    uint32_t last_flags   = 0;
    uint32_t host_flags   = 0;          // conditions found on the host since the last sync (TMI_FLAG_LEVEL)
    tmi_level_t level     = { 0, 0, 0, 0, 0 };    // all zero: no level configured (func_config_t::NONE)
    int32_t inexact_mode  = 1;          // how INEXACT_ROUND is evaluated: RescaleParams::inexact_round
    int32_t kernel_choice = 0;
    std::string last_error;
    const char* last_kernel = "";
};

namespace
{

using namespace tmi;

int fail(tmi_ctx* ctx, const char* fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    if (ctx)
        ctx->last_error = buf;
    return TMI_ERROR;
}

int hip_fail(tmi_ctx* ctx, hipError_t e, const char* what)
{
    return fail(ctx, "%s: %s", what, hipGetErrorString(e));
}

// LEVEL_CHECK (func_debug.h:132-141): with a level configured, a violated limit makes the graph UNPREDICTABLE and
// evaluation goes on.  The condition is latched on the host and reported by the next tmi_ctx_sync().
bool level_on(const tmi_ctx* ctx)
{
    const tmi_level_t& l = ctx->level;
    return l.max_rank || l.max_kernel || l.max_stride || l.max_scale || l.max_tensor_list_size;
}

void level_check(tmi_ctx* ctx, bool cond, const char* op, const char* what)
{
    if (cond || !level_on(ctx))
        return;
    ctx->host_flags |= TMI_FLAG_LEVEL;
    ctx->last_error = std::string(op) + ": LEVEL_CHECK: " + what;
}

// the LEVEL_CHECKs at the head of OpConv2d / OpDepthwiseConv2d::eval (tensor_ops.cpp:761-771, 1210-1220)
void level_check_conv(tmi_ctx* ctx, const char* op, const tmi_conv_desc_t* d)
{
    if (!level_on(ctx))
        return;
    const tmi_level_t& l = ctx->level;
    level_check(ctx, (int64_t)d->dilation[0] * d->KH <= l.max_kernel, op, "dilation_y * KH should be smaller than or equal to MAX_KERNEL");
    level_check(ctx, (int64_t)d->dilation[1] * d->KW <= l.max_kernel, op, "dilation_x * KW should be smaller than or equal to MAX_KERNEL");
    static const char* const pad_msg[4] = { "pad_top should be smaller than or equal to MAX_KERNEL",
                                            "pad_bottom should be smaller than or equal to MAX_KERNEL",
                                            "pad_left should be smaller than or equal to MAX_KERNEL",
                                            "pad_right should be smaller than or equal to MAX_KERNEL" };
    for (int i = 0; i < 4; i++)
        level_check(ctx, d->pad[i] <= l.max_kernel, op, pad_msg[i]);
    level_check(ctx, d->stride[0] <= l.max_stride, op, "stride_y should be smaller than or equal to MAX_STRIDE");
    level_check(ctx, d->stride[1] <= l.max_stride, op, "stride_x should be smaller than or equal to MAX_STRIDE");
}

#define TMI_HIP(ctx, call)                                                                                          \
    do                                                                                                              \
    {                                                                                                               \
        hipError_t e_ = (call);                                                                                     \
        if (e_ != hipSuccess)                                                                                       \
            return hip_fail(ctx, e_, #call);                                                                        \
    } while (0)

int after_launch(tmi_ctx* ctx, const char* kernel_name)
{
    if (!kernel_name)
        return fail(ctx, "no kernel implements this operand type combination");
    ctx->last_kernel = kernel_name;
    hipError_t e     = hipGetLastError();
    if (e != hipSuccess)
        return hip_fail(ctx, e, kernel_name);
    return TMI_VALID;
}

// Grows the context's scratch buffer.  An outgrown block is kept until tmi_ctx_destroy: launches already
// enqueued, and HIP graphs captured from earlier calls, still name it.  Growing is refused while the stream is
// being captured (an allocation cannot be part of a graph): the caller sizes the buffer with an eager call of
// the same operator first, or uses tmi_ctx_reserve_workspace().
int ensure_workspace(tmi_ctx* ctx, size_t bytes, bool exact = false)
{
    if (bytes <= ctx->workspace_size)
        return TMI_VALID;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(ctx->stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
        return fail(ctx, "the context's scratch buffer would have to grow to %zu bytes during stream capture: "
                         "call tmi_ctx_reserve_workspace first", bytes);
    // An operator that outgrows the block gets at least twice the old size, so the blocks kept for launches and graphs
    // that may still name them sum to less than the live block (a request of its own size, from
    // tmi_ctx_reserve_workspace, is taken as it is).
    size_t want = exact || bytes >= 2 * ctx->workspace_size ? bytes : 2 * ctx->workspace_size;
    void* block = nullptr;
    if (hipMalloc(&block, want) != hipSuccess)
    {
        (void)hipGetLastError();
        want = bytes;    // no room for the doubled block: the request itself
        TMI_HIP(ctx, hipMalloc(&block, want));
    }
    if (ctx->workspace)
    {
        ctx->retired.push_back(ctx->workspace);
        ctx->retired_bytes += ctx->workspace_size;
    }
    ctx->workspace      = block;
    ctx->workspace_size = want;
    return TMI_VALID;
}

int dtype_bits(int32_t dt)
{
    switch (dt)
    {
        case TMI_INT8:
            return 8;
        case TMI_INT16:
        case TMI_FP16:
        case TMI_BF16:
            return 16;
        case TMI_INT32:
        case TMI_FP32:
            return 32;
        case TMI_INT48:
            return 48;
        default:
            return 0;
    }
}

bool is_int_dtype(int32_t dt)
{
    return dt == TMI_INT8 || dt == TMI_INT16 || dt == TMI_INT32;
}

// check_conv_attribute (tensor_ops.cpp:120-226) and the ERROR_IFs of eval (:742-748, :805, :811;
// depthwise :1191-1197, :1237, :1241).
int validate_conv(tmi_ctx* ctx, const char* op, const tmi_conv_desc_t* d, bool depthwise, int32_t in_zp,
                  int32_t w_zp, ConvGeom& g)
{
    if (!d)
        return fail(ctx, "%s: null descriptor", op);
    if (d->in_dtype != TMI_INT8 && d->in_dtype != TMI_INT16 && d->in_dtype != TMI_FP16 && d->in_dtype != TMI_BF16 &&
        d->in_dtype != TMI_FP32)
        return fail(ctx, "%s: input data type not supported for this configuration of operator", op);
    // INT16 inputs come with INT8 weights and INT48 accumulator, bias and result (tensor_ops.cpp:2225, 2247)
    const int32_t want_out = d->in_dtype == TMI_INT8 ? TMI_INT32 : (d->in_dtype == TMI_INT16 ? TMI_INT48 : d->in_dtype);
    if (d->out_dtype != want_out)
        return fail(ctx, "%s: Output data type not supported for this configuration of operator", op);
    // the accumulator type is part of the operator's type signature (op_factory.h:97-118, tensor_ops.cpp:2219-2251):
    // INT32 for INT8 operands, INT48 for INT16, FP32 for floating point; FP16 accumulation of FP16 operands exists in the
    // reference and is not built here
    const int32_t want_acc = d->in_dtype == TMI_INT8 ? TMI_INT32 : (d->in_dtype == TMI_INT16 ? TMI_INT48 : TMI_FP32);
    if (d->acc_dtype != 0 && d->acc_dtype != want_acc)    // 0: the operand type's default
        return fail(ctx, "%s: accumulator type %d not supported for this configuration of operator", op, d->acc_dtype);
    if (d->N < 0 || d->IH < 0 || d->IW < 0 || d->IC < 0 || d->OC < 0 || d->KH < 1 || d->KW < 1 || d->OH < 0 ||
        d->OW < 0)
        return fail(ctx, "%s: negative tensor dimension", op);
    for (int i = 0; i < 4; i++)
        if (d->pad[i] < 0)
            return fail(ctx, "%s: At least one pad is smaller than zero", op);
    for (int i = 0; i < 2; i++)
        if (d->stride[i] < 1)
            return fail(ctx, "%s: At least one stride dimension is smaller than one", op);
    for (int i = 0; i < 2; i++)
        if (d->dilation[i] < 1)
            return fail(ctx, "%s: At least one dilation dimension is smaller than one", op);

    const int64_t full_h = (int64_t)d->IH - 1 + d->pad[0] + d->pad[1] - (int64_t)(d->KH - 1) * d->dilation[0];
    const int64_t full_w = (int64_t)d->IW - 1 + d->pad[2] + d->pad[3] - (int64_t)(d->KW - 1) * d->dilation[1];
    if ((full_h % d->stride[0]) != 0 || (full_w % d->stride[1]) != 0)
        return fail(ctx, "%s: Parameters must yield exact integer output dimensions", op);
    if (d->OH != full_h / d->stride[0] + 1 || d->OW != full_w / d->stride[1] + 1)
        return fail(ctx, "%s: Mismatch between output shape provided and expected output shape (%lld,%lld)", op,
                    (long long)(full_h / d->stride[0] + 1), (long long)(full_w / d->stride[1] + 1));

    int32_t M = 1;
    if (depthwise)
    {
        if (d->IC == 0 || d->OC % d->IC != 0)
            return fail(ctx, "%s: tensor output channel mismatch %d != %d", op, d->IC, d->OC);
        M = d->OC / d->IC;
        if (M < 1)
            return fail(ctx, "%s: tensor output channel mismatch %d != %d", op, d->IC, d->OC);
    }
    if (d->bias_len != d->OC && d->bias_len != 1)
        return fail(ctx, "%s: bias channel mismatch %d != %d", op, d->bias_len, d->OC);
    if (d->in_dtype != TMI_INT8 && in_zp != 0)
        return fail(ctx, "%s: Input zero point must be zero for non int8_t data", op);
    if (d->in_dtype != TMI_INT8 && d->in_dtype != TMI_INT16 && w_zp != 0)    // INT16 inputs have INT8 weights
        return fail(ctx, "%s: Weight zero point must be zero for non int8_t data", op);
    if (in_zp < -128 || in_zp > 127 || w_zp < -128 || w_zp > 127)
        return fail(ctx, "%s: zero point outside the int8 range", op);

    g.N = d->N, g.IH = d->IH, g.IW = d->IW, g.IC = d->IC, g.OC = d->OC, g.KH = d->KH, g.KW = d->KW;
    g.OH = d->OH, g.OW = d->OW;
    g.pad_top = d->pad[0], g.pad_left = d->pad[2];
    g.stride_y = d->stride[0], g.stride_x = d->stride[1], g.dil_y = d->dilation[0], g.dil_x = d->dilation[1];
    g.bias_len = d->bias_len;
    g.M        = M;
    return TMI_VALID;
}

int64_t extend(int32_t v, int bits, bool is_unsigned)
{
    if (bits == 8)
        return is_unsigned ? (int64_t)(uint8_t)v : (int64_t)(int8_t)v;
    if (bits == 16)
        return is_unsigned ? (int64_t)(uint16_t)v : (int64_t)(int16_t)v;
    return is_unsigned ? (int64_t)(uint32_t)v : (int64_t)v;
}

// Decides whether the kernels may use fast_rescale(): signed INT32 input, no input zero point, 32-bit scale
// with SINGLE or DOUBLE rounding, and an output clip / CLAMP pair that merges into one range.
void set_fast_path(RescaleParams& p)
{
    p.lo = p.qmin, p.hi = p.qmax;
    bool merged = true;
    if (p.has_clamp)
    {
        p.lo   = p.qmin > p.clamp_min ? p.qmin : p.clamp_min;
        p.hi   = p.qmax < p.clamp_max ? p.qmax : p.clamp_max;
        merged = p.lo <= p.hi;
    }
    p.fast = merged && p.scale32 && !p.inexact_round && p.in_bits == 32 && !p.in_unsigned && p.in_zp == 0;
}

// OpRescale::checkTensorAttributes (type_conversion.cpp:111-151) and the zero-point ERROR_IFs of eval
// (:242-255).  Fills the kernel parameters.
int validate_rescale(tmi_ctx* ctx, const tmi_rescale_desc_t* r, int32_t rank, int32_t C, const void* mult,
                     const void* shift, RescaleParams& p)
{
    if (!r)
        return fail(ctx, "OpRescale: null descriptor");
    const bool i48in = r->in_dtype == TMI_INT48;
    if ((!is_int_dtype(r->in_dtype) && !i48in) || !is_int_dtype(r->out_dtype))
        return fail(ctx, "OpRescale: unsupported data type");
    const bool i32in = r->in_dtype == TMI_INT32, i32out = r->out_dtype == TMI_INT32;
    const bool i8in = r->in_dtype == TMI_INT8, i8out = r->out_dtype == TMI_INT8;
    const bool i16in = r->in_dtype == TMI_INT16, i16out = r->out_dtype == TMI_INT16;
    const bool in_u = r->input_unsigned != 0, out_u = r->output_unsigned != 0;

    if (r->rounding_mode != TMI_ROUND_SINGLE && r->rounding_mode != TMI_ROUND_DOUBLE &&
        r->rounding_mode != TMI_ROUND_INEXACT)
        return fail(ctx, "OpRescale: Unsupported rounding mode");
    if (!r->scale32 && r->rounding_mode == TMI_ROUND_DOUBLE)
        return fail(ctx, "OpRescale: Scale set to false but rounding mode set to double round");
    if (in_u && out_u)
        return fail(ctx, "OpRescale: input_unsigned and output_unsigned set to true");
    if (i32out && in_u)
        return fail(ctx, "OpRescale: Output signed int32 and input_unsigned set to true");
    if (i32in && out_u)
        return fail(ctx, "OpRescale: Input signed int32 and output_unsigned set to true");
    if (i32in && in_u)
        return fail(ctx, "OpRescale: Input unsigned int32");
    if (i32out && out_u)
        return fail(ctx, "OpRescale: Output unsigned int32");
    if (r->scale32 && i48in)
        return fail(ctx, "OpRescale: Scale set to true but input type is INT48");
    if (i48in && out_u)
        return fail(ctx, "OpRescale: Input signed int48 and output_unsigned set to true");
    if (i48in && in_u)
        return fail(ctx, "OpRescale: Input unsigned int48");
    if (r->per_channel)
    {
        if (rank < 1)
            return fail(ctx, "OpRescale: per_channel set to true and rank of input < 1");
        if (r->n_multiplier != C)
            return fail(ctx, "OpRescale: wrong size multiplier array for per_channel=true");
        if (r->n_shift != C)
            return fail(ctx, "OpRescale: wrong size shift array for per_channel=true");
    }
    else
    {
        if (r->n_multiplier != 1)
            return fail(ctx, "OpRescale: wrong size multiplier array for per_channel=false");
        if (r->n_shift != 1)
            return fail(ctx, "OpRescale: wrong size shift array for per_channel=false");
    }

    const int64_t out_zp = extend(r->out_zp, dtype_bits(r->out_dtype), out_u);
    const int64_t in_zp  = extend(r->in_zp, dtype_bits(r->in_dtype), in_u);
    if (!i8in && !(i16in && in_u) && in_zp != 0)
        return fail(ctx, "OpRescale: Input TOSA_REF_TYPE not INT8/UINT8/UINT16 and zero point not 0");
    if (!i8out && !(i16out && out_u) && out_zp != 0)
        return fail(ctx, "OpRescale: Output TOSA_REF_TYPE not INT8/UINT8/UINT16 and zero point not 0");
    if (i16in && in_u && in_zp != 0 && in_zp != 32768)
        return fail(ctx, "OpRescale: Input unsigned int16 and zero point (%lld) not 0 or 32768", (long long)in_zp);
    if (i16out && out_u && out_zp != 0 && out_zp != 32768)
        return fail(ctx, "OpRescale: Output unsigned int16 and zero point (%lld) not 0 or 32768",
                    (long long)out_zp);
    if (!mult || !shift)
        return fail(ctx, "OpRescale: null multiplier or shift tensor");

    p               = RescaleParams{};
    p.multiplier    = mult;
    p.shift         = reinterpret_cast<const int8_t*>(shift);
    p.in_zp         = (int32_t)in_zp;
    p.out_zp        = (int32_t)out_zp;
    p.qmin          = out_u ? 0 : (i8out ? -128 : (i16out ? -32768 : INT32_MIN));
    p.qmax          = out_u ? (i8out ? 255 : 65535) : (i8out ? 127 : (i16out ? 32767 : INT32_MAX));
    p.scale32       = r->scale32 != 0;
    p.double_round  = r->rounding_mode == TMI_ROUND_DOUBLE;
    p.inexact_round = r->rounding_mode == TMI_ROUND_INEXACT ? (uint8_t)ctx->inexact_mode : 0;
    p.per_channel   = r->per_channel != 0;
    p.in_bits       = (uint8_t)dtype_bits(r->in_dtype);
    p.in_unsigned   = in_u;
    p.has_clamp     = 0;
    p.enabled       = 1;
    set_fast_path(p);
    return TMI_VALID;
}

int validate_fused_rescale(tmi_ctx* ctx, const char* op, const tmi_conv_desc_t* d, const tmi_rescale_desc_t* r,
                           const void* mult, const void* shift, int32_t has_clamp, int32_t clamp_min,
                           int32_t clamp_max, RescaleParams& p)
{
    if (!r)
        return fail(ctx, "%s: null rescale descriptor", op);
    if (d->in_dtype != TMI_INT8)
        return fail(ctx, "%s: the fused rescale needs an INT8 convolution", op);
    if (r->in_dtype != TMI_INT32)
        return fail(ctx, "%s: the fused rescale consumes the INT32 convolution output", op);
    int rc = validate_rescale(ctx, r, 4, d->OC, mult, shift, p);
    if (rc != TMI_VALID)
        return rc;
    if (has_clamp)
    {
        // OpClamp::register_fcn: ERROR_IF(max < min) (activation_funcs.cpp:91)
        if (clamp_max < clamp_min)
            return fail(ctx, "OpClamp: max smaller than min");
        p.has_clamp = 1;
        p.clamp_min = clamp_min;
        p.clamp_max = clamp_max;
        set_fast_path(p);
    }
    return TMI_VALID;
}

// check_level: false for the CONV2D that TRANSPOSE_CONV2D / CONV3D are evaluated as (their own limits were checked).
// own_scratch: false when the caller holds operands of its own in a scratch buffer (the context's or the static one of
// the entry point that allocates nothing): then no kernel that would grow or write the context's buffer is chosen.
int run_conv(tmi_ctx* ctx, const char* op, bool depthwise, const tmi_conv_desc_t* d, const void* in, const void* w,
             const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp, int32_t out_dtype, void* out,
             bool check_level = true, bool own_scratch = true)
{
    ConvGeom g;
    int rc = validate_conv(ctx, op, d, depthwise, in_zp, w_zp, g);
    if (rc != TMI_VALID)
        return rc;
    if (check_level)
        level_check_conv(ctx, op, d);
    const int64_t total = (int64_t)g.N * g.OH * g.OW * g.OC;
    if (total > 0 && (!in || !w || !bias || !out))
        return fail(ctx, "%s: null tensor pointer", op);
    TMI_HIP(ctx, hipSetDevice(ctx->device));

    const char* name = nullptr;
    if (total == 0)
    {
        ctx->last_kernel = "empty";
        return TMI_VALID;
    }
    if (d->in_dtype == TMI_INT16)
    {
        if (rp.enabled)
            return fail(ctx, "%s: the fused rescale needs an INT8 convolution", op);
        return after_launch(ctx, launch_conv_i16_direct(ctx->stream, depthwise, g, in, w, bias, w_zp, out));
    }
    // Small depthwise layers: the vector kernel (a lane per four channels of a pixel, no LDS, no barrier) costs 3.15 us plus
    // 4.4 us per million results, the matrix-core kernel 3.3 us plus 3.7 ns per channel (its per-channel tables) and next
    // to nothing per result.  us matrix-core / vector kernel, 3x3, fused RESCALE: [8,14,14,384] stride 2 4.3 / 3.3,
    // [8,7,7,512] 4.9 / 3.4, [8,7,7,960] 6.8 / 4.1, [2,14,14,576] 5.1 / 3.8, [4,14,14,576] 5.3 / 4.8, [1,28,28,192] 3.8 / 3.4,
    // [8,10,10,672] 5.6 / 5.0; the other way: [1,56,56,144] 3.9 / 4.3, [8,14,14,576] 5.3 / 7.2, [8,14,14,1024] 7.1 / 7.5,
    // [8,28,28,384] 4.8 / 9.5, [32,14,14,576] 5.8 / 14.7.
    // fp16 / bf16 depthwise layers with channels in multiples of 8: the vector kernel (us one-result-per-lane kernel / this
    // one, fp16 3x3: [8,112,112,96] stride 2 25.6 / 8.1, [8,112,112,32] 31.0 / 8.6, [8,56,56,144] 31.6 / 10.7, [8,28,28,192]
    // 11.4 / 5.6, [8,14,14,576] 9.4 / 5.2, [64,112,112,96] stride 2 182 / 38.5)
    if (depthwise && ctx->kernel_choice != 1 && !rp.enabled && (d->in_dtype == TMI_FP16 || d->in_dtype == TMI_BF16))
        name = launch_depthwise_fp_vec(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, out);
    if (depthwise && !name && ctx->kernel_choice == 0 && total < 34000 + 850 * (int64_t)g.IC)
        name = launch_depthwise_vec(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out,
                                    ctx->flags_dev);
    // Layers with at most 48 channels and 1.6 M results or more: the kernel whose waves load the pixel operand straight from
    // global memory (a pixel is one or two 32-byte pieces, neighbouring lanes read neighbouring memory; us LDS-patch kernel /
    // this one, fused RESCALE: [8,112,112,32] 6.5 / 5.3, [32,...] 16.8 / 11.9, [64,...] 29.9 / 20.8, stride 2 11.9 / 8.6,
    // [64,56,56,32] 10.8 / 7.8, [64,56,56,48] 13.4 / 11.7, [8,150,150,32] 9.9 / 6.4; the other way: [4,112,112,32] 4.2 / 4.1
    // is the border, [8,56,56,32] 3.6 / 3.9, [8,56,56,48] 3.9 / 4.1).  With 64 channels and more a load instruction takes 32
    // bytes out of every pixel and the L1 looks up a line per lane: [64,112,112,64] 40.8 / 43.4, [64,112,112,96] stride 2
    // 23.0 / 28.7, [32,28,28,384] 10.1 / 20.4.
    if (depthwise && !name && (ctx->kernel_choice == 6 || (ctx->kernel_choice == 0 && g.IC <= 48 && total >= 1600000)))
        name = launch_depthwise_stream(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out,
                                       ctx->flags_dev);
    if (depthwise && !name && (ctx->kernel_choice == 0 || ctx->kernel_choice == 4))
        name = launch_depthwise_slab(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out,
                                     ctx->pages_dev + (in_zp & 255) * 64, ctx->flags_dev);
    if (depthwise && !name && ctx->kernel_choice != 1 && ctx->kernel_choice != 4 && ctx->kernel_choice != 6)
        name = launch_depthwise_vec(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out,
                                    ctx->flags_dev);
    if (!depthwise && ctx->kernel_choice != 1)
    {
        // kernel choice 2 / 3 name one kernel; left open, the likely faster one is tried first
        const void* pad_page = ctx->pages_dev + (d->in_dtype == TMI_INT8 ? (in_zp & 255) * 64 : 0);
        const bool gemm_ok   = ctx->kernel_choice == 0 || ctx->kernel_choice == 3;
        const bool patch_ok  = ctx->kernel_choice == 0 || ctx->kernel_choice == 2;
        const bool gemm_1st  = gemm_ok && (!patch_ok || gemm_mfma_preferred(d->in_dtype, g));
        // A pointwise layer with int32 results and more than 2 M of them: the GEMM kernel, whose results leave as
        // whole lines, before the slab kernel (us slab / GEMM, host clock: [8,56,56,64]->256 12.8 / 8.8,
        // [32,56,56,64]->256 35.9 / 21.6, [8,28,28,128]->512 8.3 / 6.6, [32,28,28,128]->512 24.0 / 14.5; smaller ones
        // and every layer with the fused RESCALE are the slab kernel's: 5.3 / 5.5, fused 6.9 / 10.1, 19.6 / 28.3).
        if (ctx->kernel_choice == 0 && !rp.enabled && g.KH * g.KW == 1 && total > (int64_t(1) << 21) && g.IC <= 128)
            name = launch_gemm_mfma(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out, 0, 0,
                                    pad_page, ctx->flags_dev);
        // Pointwise int8 layers with up to 112 input channels: the kernel that keeps a wave on one tile of 32 output channels
        // and takes both operands straight from global memory, before every other (us slab or patch kernel / pointwise
        // kernel, graph replays, fused RESCALE: [8,112,112,16]->96 16.6 / 6.4, [8,112,112,32]->16 9.0 / 3.4, [8,56,56,96]->24
        // 7.5 / 2.8, [8,28,28,32]->192 4.9 / 2.9, [8,56,56,80]->80 10.0 / 3.8, [8,28,28,112]->224 6.3 / 3.7, [8,56,56,64]->64
        // 3.5 / 3.3, [8,56,56,64]->256 6.4 / 5.5, [32,56,56,64]->256 18.0 / 12.6, [32,56,56,96]->192 16.4 / 11.3, [8,14,14,64]->384
        // 3.3 / 2.8, [1,32,32,16]->16 3.7 (one result per lane) / 2.5; int32 results [8,56,56,96]->24 7.6 / 2.8, [8,112,112,16]->96
        // 21.0 / 15.9, [8,56,56,64]->64 4.9 / 4.6).  With 128 input channels the slab kernel leads ([8,28,28,128]->512
        // 4.9 / 6.0, [8,56,56,128]->128 5.1 / 6.1) and this kernel takes what that one declines; with 144 and 160 there is
        // only the patch kernel to beat ([8,56,56,144]->24 10.2 / 3.1, [8,7,7,160]->960 5.4 / 3.2).  Large int32 results
        // stay with the GEMM kernel above ([8,56,56,64]->256 8.1 / 11.8, [8,28,28,128]->512 6.3 / 8.9).
        // With more than 160 input channels the pointwise kernel splits K over the four waves of a workgroup, a workgroup
        // per tile of 32 x 32 results (or per few of them): the better form while the layer is small, up to 500 M
        // multiply-adds on at most 1600 such tiles, or up to 900 M where the GEMM kernel would have at most 64 tiles of
        // 128 x 128 for the chip.  us GEMM kernel / this form, fused RESCALE: [8,28,28,192]->32 9.2 / 3.3, [8,14,14,384]->64
        // 7.4 / 3.8, [8,7,7,960]->320 9.7 / 4.3, [8,7,7,320]->1280 7.4 / 4.2, [8,14,14,1024]->256 10.0 / 6.9, [8,7,7,2048]->512
        // 14.2 / 7.5, [8,28,28,512]->128 8.1 / 6.5, [8,7,7,512]->2048 8.0 / 6.4, [8,14,14,256]->1024 7.2 / 6.7, [8,56,56,256]->64
        // 7.1 / 7.0, [8,28,28,256]->256 7.1 / 6.7, [32,14,14,384]->96 7.6 / 5.3, [8,28,28,256]->128 7.0 / 5.3, [32,7,7,960]->320
        // 9.7 / 5.7; 500 - 900 M: [8,14,14,1024]->512 (52 tiles) 10.0 / 8.6, [8,28,28,1024]->128 (49) 10.1 / 8.7, [8,14,14,2048]->256
        // (26) 14.2 / 11.0; the other way: [8,28,28,192]->384 (2352 small tiles) 7.0 / 7.6, [8,28,28,512]->256 (98 tiles of
        // 128 x 128) 8.2 / 8.8, [8,14,14,768]->768 (78) 9.1 / 10.1, [8,56,56,256]->128 7.4 / 10.5.
        const int64_t pixels   = (int64_t)g.N * g.OH * g.OW;
        const int64_t tiles128 = ((pixels + 127) / 128) * ((g.OC + 127) / 128);
        const int64_t tiles32  = ((pixels + 31) / 32) * ((g.OC + 31) / 32);
        const int64_t macs     = total * g.IC * g.KH * g.KW;
        const bool deep_first  = g.IC > 160 && ((macs <= 500000000ll && tiles32 <= 1600) || (macs <= 900000000ll && tiles128 <= 64));
        // Pointwise layers with 160 ... 1024 input channels (the counts the slab kernel is instantiated for): its weight slab,
        // 64 rows of up to 1 KB, and a patch of 62 ... 124 pixels fit the LDS as those of 3 x 3 taps on 64 channels do, so it
        // comes before all of these - up to 256 channels at every size, beyond while the layer fits one round of
        // workgroups (900 M multiply-adds): a workgroup then takes 75 ... 135 KB of LDS, one fits a CU, and from the second
        // round on the GEMM kernel leads.  us slab / K-split pointwise / GEMM kernel, fused RESCALE:
        // [8,56,56,256]->64 4.2 / 7.0 / 7.2, [32,..] 7.7 / 17.6 / 19.9, [8,56,56,256]->128 5.7 / 10.6 / 7.4, [32,..] 16.7 / 30.0 / 21.7,
        // [8,56,56,256]->512 16.8 / 28.7 / 19.2, [8,14,14,256]->1024 4.1 / 6.8 / 7.1, [32,..] 7.6 / 16.0 / 11.1, [1,14,14,256]->1024
        // 3.4 / 3.5 / 6.9; [8,28,28,512]->128 4.2 / 6.6 / 8.1, [16,..] 4.9 / 9.5 / 8.2, [8,28,28,512]->256 4.9 / 8.9 / 8.2,
        // [8,7,7,512]->2048 4.2 / 6.6 / 8.1, [1,7,7,512]->512 3.6 / 4.0 / -, [8,14,14,1024]->256 4.7 / 6.8 / 10.0, [8,14,14,1024]->512
        // 5.1 / 8.7 / 10.0, [8,28,28,192]->64 3.3 / 3.7 / 6.6, [8,56,56,192]->64 3.8 / 6.3 / 6.9, [8,28,28,384]->192 4.3 / 7.0 / 7.7,
        // [8,28,28,192]->384 5.1 / 7.8 / 7.0, [32,14,14,384]->96 4.0 / 5.4 / 7.5; the other way: [32,28,28,512]->128 (1.6 G)
        // 10.8 / 15.8 / 8.5, [16,28,28,512]->256 10.8 / 15.8 / 8.5, [32,7,7,512]->2048 10.7 / 13.0 / 8.5, [8,28,28,512]->1024
        // 20.1 / 22.7 / 12.9, [32,14,14,1024]->256 11.9 / 16.1 / 10.2.  int32 results: [32,56,56,256]->64 15.0 / 17.3 / 17.3,
        // [8,14,14,256]->1024 5.6 / 6.1 / 6.0, [8,14,14,1024]->256 4.4 / 6.3 / 8.3.
        const bool slab_deep = d->in_dtype == TMI_INT8 && g.KH * g.KW == 1 && g.IC > 128 && g.IC <= 1024 && (g.IC <= 256 || macs <= 900000000ll);
        if (!name && ctx->kernel_choice == 0 && slab_deep)
            name = launch_conv2d_slab(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out, pad_page,
                                      ctx->flags_dev);
        // fp16 / bf16 on the slab kernel (channel vectors of 64 ... 128 bytes under 3 x 3 taps, up to 1024 bytes under 1 x 1):
        // every 3 x 3 layer it takes, and the pointwise ones up to 1.6 M results - beyond, the GEMM kernel's whole-line stores
        // win.  us patch or GEMM kernel / slab kernel, fp16: 3x3 [8,56,56,64]->64 7.2 / 4.8, ->128 8.4 / 6.9, stride 2 10.3 / 4.1,
        // [32,56,56,64]->64 18.7 / 12.7, [8,56,56,32]->64 4.8 / 3.8, [8,28,28,48]->96 7.0 / 3.7; 1x1 [8,28,28,256]->128 4.2 / 3.6,
        // [8,14,14,512]->256 5.0 / 4.0, [1,14,14,512]->512 4.9 / 3.5, [8,28,28,96]->192 3.7 / 3.2, [8,56,56,256]->64 4.6 / 4.4,
        // [8,14,14,256]->1024 4.5 / 4.4; the other way: [8,28,28,128]->512 (3.2 M results) 4.7 / 5.3, [8,56,56,64]->256 6.2 / 6.7,
        // [32,28,28,256]->128 5.4 / 7.7, [32,56,56,64]->256 15.8 / 20.4.  Large 3 x 3 layers: stride 1 [2,160,160,64]->128 17.2 / 13.9,
        // [8,160,160,64]->96 50.9 / 47.7, [8,56,56,64]->256 16.6 / 13.9, [16,28,28,64]->256 8.5 / 7.5; with a stride the patch grows
        // with the tile, and from 160 tiles of 128 x 128 on the GEMM kernel leads: [16,56,56,64]->128 stride 2 (98 tiles) 9.5 / 7.7,
        // [32,..] (196) 10.3 / 13.2, [64,..] 17.3 / 25.0, [32,56,56,64]->256 17.0 / 24.8.
        const bool fp16b = d->in_dtype == TMI_FP16 || d->in_dtype == TMI_BF16;
        const bool fp_slab33 = g.KH * g.KW == 9 && !(g.stride_y * g.stride_x > 1 && tiles128 >= 160);
        if (!name && ctx->kernel_choice == 0 && fp16b && (fp_slab33 || (g.KH * g.KW == 1 && total <= 1600000)))
            name = launch_conv2d_slab(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out, pad_page,
                                      ctx->flags_dev);
        if (!name && ctx->kernel_choice == 0 && (g.IC <= 112 || deep_first))
            name = launch_conv2d_pointwise(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out,
                                           ctx->flags_dev);
        // Tiny int8 layers: the patch kernel's set-up (4.4 us for a layer of a few workgroups, 1.8 more with the fused
        // RESCALE, 0.5 more when the channel vector is staged by 4- or 8-byte words and 1.8 when by bytes) exceeds what
        // the one-result-per-lane kernel takes, 2.6 us plus the longer of a lane's chain of K multiply-adds (90 ns each)
        // and the whole layer at 1000 multiply-adds per ns.  us patch kernel / direct kernel (graph replays, fused):
        // [1,32,32,8]->16 1x1 6.6 / 3.1, [1,64,64,8]->16 6.7 / 3.2, [8,32,32,8]->32 5.1 / 4.2, [1,32,32,16]->16 6.2 / 3.7,
        // [4,16,16,24]->48 6.5 / 4.2, 3x3 [1,32,32,3]->16 7.7 / 5.1, [1,112,112,3]->32 stride 2 6.9 / 5.8, int32 results
        // [2,32,32,8]->16 4.7 / 2.8, [1,32,32,16]->16 4.4 / 3.4; the other way: 3x3 [1,14,14,8]->16 6.7 / 8.5,
        // [1,28,28,12]->32 5.3 / 11.5, [1,224,224,3]->32 stride 2 7.7 / 11.9, 1x1 [8,56,56,8]->64 5.4 / 12.8,
        // [1,56,56,24]->144 6.3 / 9.9.
        if (!name && ctx->kernel_choice == 0 && d->in_dtype == TMI_INT8)
        {
            const double k      = (double)g.KH * g.KW * g.IC;
            const double chain  = 0.09 * k, whole = (double)total * k * 1e-6;
            const double direct = 2.6 + (chain > whole ? chain : whole);
            const double patch  = 4.4 + ((g.IC & 15) == 0 ? 0.0 : ((g.IC & 3) == 0 ? 0.5 : 1.8)) + (rp.enabled ? 1.8 : 0.0);
            if (direct + 0.3 < patch)
                name = launch_conv2d_direct(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out,
                                            ctx->flags_dev);
        }
        // (left open, the slab kernel's layers with more than 128 input channels are the ones tried above)
        if (!name && (ctx->kernel_choice == 4 || (ctx->kernel_choice == 0 && g.IC <= 128 && d->in_dtype == TMI_INT8)))
            name = launch_conv2d_slab(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out, pad_page,
                                      ctx->flags_dev);
        // Layers with taps that are small and deep (at most 2.4 G multiply-adds on at most 64 tiles of 128 x 128 results, or
        // on at most 100 from 160 input channels on) and not the slab kernel's: workgroups that own tiles of 32 x 32 results
        // with K split over their waves, before the patch and GEMM kernels, which would keep a fraction of the chip busy.
        // us patch kernel / this kernel, 3x3, fused RESCALE: [8,14,14,256]->256 14.3 / 9.0, [8,28,28,256]->256 stride 2
        // 16.2 / 9.1, [8,7,7,512]->512 21.1 / 10.8, [8,14,14,512]->512 stride 2 22.5 / 10.8, [8,14,14,160]->160 13.6 / 4.5,
        // [1,14,14,256]->256 14.2 / 6.9, [16,14,14,256]->256 (50 tiles) 14.4 / 12.8, [20,14,14,256]->256 (62) 14.5 / 12.8,
        // [8,14,14,384]->384 18.8 / 15.2, [8,14,14,256]->512 14.5 / 12.8, [8,14,14,512]->256 23.2 / 15.7, [16,7,7,512]->512
        // 21.2 / 15.1, [8,14,14,320]->320 16.6 / 8.8, [8,28,28,160]->160 (98) 13.8 / 9.2, [8,28,28,192]->192 (98) 12.1 / 11.4,
        // 5x5 [8,14,14,192]->192 31.1 / 11.1, [8,56,56,32]->32 stride 2 6.8 / 3.9; ties at [24,14,14,256]->256 (74 tiles, 2.8 G)
        // 14.6 / 15.0 and [32,7,7,512]->512 21.2 / 21.8; the other way: [32,14,14,256]->256 (98, 3.7 G) 15.2 / 18.7,
        // [16,14,14,512]->512 23.6 / 34.2, [8,56,56,32]->64 (196) 5.3 / 11.9, [8,112,112,32]->32 8.1 / 19.5.
        const bool split_first = g.KH * g.KW > 1 && macs <= 2400000000ll && (tiles128 <= 64 || (g.IC >= 160 && tiles128 <= 100));
        if (!name && g.KH * g.KW > 1 && (ctx->kernel_choice == 5 || (ctx->kernel_choice == 0 && split_first)))
            name = launch_conv2d_ksplit(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out, pad_page,
                                        ctx->flags_dev);
        // First layers (at most 4 input channels, 3 x 3 ... 7 x 7 taps): a pre-pass into the scratch buffer and the pointwise
        // kernel with a K step per row of taps, unless an operand of this call lies in that buffer already.
        if (!name && own_scratch && (ctx->kernel_choice == 5 || ctx->kernel_choice == 0))
        {
            const size_t need = conv2d_stem_scratch_bytes(d->in_dtype, out_dtype, g, w_zp, rp);
            auto in_scratch   = [&](const void* p) {
                return ctx->workspace && (const uint8_t*)p >= (const uint8_t*)ctx->workspace &&
                       (const uint8_t*)p < (const uint8_t*)ctx->workspace + ctx->workspace_size;
            };
            if (need && !in_scratch(in) && !in_scratch(w) && !in_scratch(out) && !in_scratch(bias))
            {
                rc = ensure_workspace(ctx, need);
                if (rc != TMI_VALID)
                    return rc;
                name = launch_conv2d_stem(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out,
                                          ctx->workspace, ctx->flags_dev);
            }
        }
        if (!name && (ctx->kernel_choice == 5 || (ctx->kernel_choice == 0 && g.IC <= 160)))    // (the layers it leads on were tried above)
            name = launch_conv2d_pointwise(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out,
                                           ctx->flags_dev);
        if (!name && gemm_1st)
            name = launch_gemm_mfma(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out, 0, 0,
                                    pad_page, ctx->flags_dev);
        if (!name && patch_ok)
            name = launch_conv2d_mfma(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out,
                                      ctx->flags_dev);
        if (!name && gemm_ok && !gemm_1st)
            name = launch_gemm_mfma(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out, 0, 0,
                                    pad_page, ctx->flags_dev);
    }
    if (!name && ctx->kernel_choice >= 2)
        return fail(ctx, "%s: no MFMA / vector kernel is eligible for this shape", op);
    if (!name && depthwise)
        name = launch_depthwise_direct(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out,
                                       ctx->flags_dev);
    else if (!name)
        name = launch_conv2d_direct(ctx->stream, d->in_dtype, out_dtype, g, in, w, bias, in_zp, w_zp, rp, out,
                                    ctx->flags_dev);
    return after_launch(ctx, name);
}

}    // namespace

extern "C" {

const char* tmi_version(void)
{
    return "tosa_mi355 0.1 gfx950";
}

int tmi_ctx_create(tmi_ctx_t** out_ctx, int device)
{
    if (!out_ctx)
        return TMI_ERROR;
    *out_ctx = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count || device >= kMaxDevices)
        return TMI_ERROR;
    tmi_ctx* ctx = new tmi_ctx();
    ctx->device  = device;
    if (hipSetDevice(device) != hipSuccess || hipStreamCreate(&ctx->stream) != hipSuccess)
    {
        delete ctx;
        return TMI_ERROR;
    }
    ctx->owns_stream = true;
    if (scratch_address(device, &ctx->static_scratch) != hipSuccess)
    {
        tmi_ctx_destroy(ctx);
        return TMI_ERROR;
    }
    if (hipMalloc((void**)&ctx->flags_dev, 256) != hipSuccess ||
        hipHostMalloc((void**)&ctx->flags_host, 256, hipHostMallocDefault) != hipSuccess ||
        hipMemset(ctx->flags_dev, 0, 256) != hipSuccess)
    {
        tmi_ctx_destroy(ctx);
        return TMI_ERROR;
    }
    *ctx->flags_host = 0;
    {
        std::string pages(256 * 64, '\0');
        for (int v = 0; v < 256; v++)
            memset(&pages[(size_t)v * 64], v, 64);
        if (hipMalloc((void**)&ctx->pages_dev, pages.size()) != hipSuccess ||
            hipMemcpy(ctx->pages_dev, pages.data(), pages.size(), hipMemcpyHostToDevice) != hipSuccess)
        {
            tmi_ctx_destroy(ctx);
            return TMI_ERROR;
        }
    }
    *out_ctx = ctx;
    return TMI_VALID;
}

int tmi_ctx_destroy(tmi_ctx_t* ctx)
{
    if (!ctx)
        return TMI_VALID;
    // teardown is best effort: there is nobody left to report a failure to
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->workspace)
        (void)hipFree(ctx->workspace);
    for (void* block : ctx->retired)
        (void)hipFree(block);
    if (ctx->flags_dev)
        (void)hipFree(ctx->flags_dev);
    if (ctx->pages_dev)
        (void)hipFree(ctx->pages_dev);
    if (ctx->flags_host)
        (void)hipHostFree(ctx->flags_host);
    if (ctx->owns_stream && ctx->stream)
        (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return TMI_VALID;
}

int tmi_ctx_set_stream(tmi_ctx_t* ctx, void* hip_stream)
{
    if (!ctx)
        return TMI_ERROR;
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    TMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (ctx->owns_stream && ctx->stream)
        TMI_HIP(ctx, hipStreamDestroy(ctx->stream));
    ctx->stream      = (hipStream_t)hip_stream;
    ctx->owns_stream = false;
    return TMI_VALID;
}

int tmi_ctx_sync(tmi_ctx_t* ctx)
{
    if (!ctx)
        return TMI_ERROR;
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    TMI_HIP(ctx, hipMemcpyAsync(ctx->flags_host, ctx->flags_dev, sizeof(uint32_t), hipMemcpyDeviceToHost,
                                ctx->stream));
    TMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
    const uint32_t dev_flags = *ctx->flags_host;
    ctx->last_flags          = dev_flags | ctx->host_flags;
    ctx->host_flags          = 0;
    if (dev_flags)
    {
        // cleared with a plain stream-ordered memset: nothing captures this path into a graph
        TMI_HIP(ctx, hipMemsetAsync(ctx->flags_dev, 0, sizeof(uint32_t), ctx->stream));
        TMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
    }
    return ctx->last_flags ? TMI_UNPREDICTABLE : TMI_VALID;
}

uint32_t tmi_ctx_flags(const tmi_ctx_t* ctx)
{
    return ctx ? ctx->last_flags : 0;
}

const char* tmi_last_error(const tmi_ctx_t* ctx)
{
    return ctx ? ctx->last_error.c_str() : "null context";
}

const char* tmi_last_kernel(const tmi_ctx_t* ctx)
{
    return ctx ? ctx->last_kernel : "";
}

int tmi_ctx_set_level(tmi_ctx_t* ctx, const tmi_level_t* level)
{
    if (!ctx)
        return TMI_ERROR;
    ctx->level = level ? *level : tmi_level_t{ 0, 0, 0, 0, 0 };
    return TMI_VALID;
}

int tmi_ctx_set_precise_mode(tmi_ctx_t* ctx, int32_t precise_mode, int32_t compliance_mode, int32_t bounds_mode)
{
    if (!ctx)
        return TMI_ERROR;
    ctx->inexact_mode = !precise_mode ? 1 : (!compliance_mode ? 2 : (bounds_mode ? 4 : 3));
    return TMI_VALID;
}

int tmi_ctx_set_kernel_choice(tmi_ctx_t* ctx, int32_t choice)
{
    if (!ctx || choice < 0 || choice > 6)
        return TMI_ERROR;
    ctx->kernel_choice = choice;
    return TMI_VALID;
}

int tmi_debug_launch_empty(tmi_ctx_t* ctx, int32_t grid, int32_t block, int32_t lds_bytes)
{
    if (!ctx)
        return TMI_ERROR;
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    const char* name = launch_empty(ctx->stream, grid, block, lds_bytes);
    if (!name)
        return fail(ctx, "tmi_debug_launch_empty: grid %d, block %d, LDS %d bytes cannot be launched", grid, block, lds_bytes);
    return after_launch(ctx, name);
}

int tmi_debug_stream(tmi_ctx_t* ctx, int32_t mode, const void* src_dev, void* dst_dev, int64_t bytes)
{
    if (!ctx)
        return TMI_ERROR;
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    const char* name = launch_stream_probe(ctx->stream, mode, src_dev, dst_dev, bytes);
    if (!name)
        return fail(ctx, "tmi_debug_stream: mode %d with %lld bytes: the mode is 0..3, the buffers are 16-byte aligned and "
                         "the size is a positive multiple of 16", mode, (long long)bytes);
    return after_launch(ctx, name);
}

void tmi_debug_last_launch_shape(int32_t* out3)
{
    if (out3)
        out3[0] = last_launch_shape[0], out3[1] = last_launch_shape[1], out3[2] = last_launch_shape[2];
}

int tmi_debug_tile_decode(int64_t grid, uint32_t n_ocb, uint32_t tiles_x, uint32_t tiles_y, uint32_t block,
                          int32_t* out4)
{
    const int exact = tile_decode_is_exact(grid, n_ocb, tiles_x, tiles_y) ? 1 : 0;
    if (out4 && n_ocb && tiles_x && tiles_y)
    {
        const uint32_t tile = fdiv_host(block, make_fastdiv(n_ocb));
        const uint32_t trow = fdiv_host(tile, make_fastdiv(tiles_x));
        const uint32_t n    = fdiv_host(trow, make_fastdiv(tiles_y));
        out4[0] = (int32_t)(block - tile * n_ocb), out4[1] = (int32_t)(tile - trow * tiles_x);
        out4[2] = (int32_t)(trow - n * tiles_y), out4[3] = (int32_t)n;
    }
    return exact;
}

int tmi_ctx_reserve_workspace(tmi_ctx_t* ctx, size_t bytes)
{
    if (!ctx)
        return TMI_ERROR;
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    return ensure_workspace(ctx, bytes, true);
}

int tmi_ctx_workspace_bytes(const tmi_ctx_t* ctx, size_t* live, size_t* retired)
{
    if (!ctx)
        return TMI_ERROR;
    if (live)
        *live = ctx->workspace_size;
    if (retired)
        *retired = ctx->retired_bytes;
    return TMI_VALID;
}

int tmi_ctx_trim_workspace(tmi_ctx_t* ctx)
{
    if (!ctx)
        return TMI_ERROR;
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    TMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
    for (void* b : ctx->retired)
        (void)hipFree(b);
    ctx->retired.clear();
    ctx->retired_bytes = 0;
    return TMI_VALID;
}

int tmi_buf_alloc(tmi_ctx_t* ctx, size_t bytes, void** out_dev)
{
    if (!ctx || !out_dev)
        return TMI_ERROR;
    *out_dev = nullptr;
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    TMI_HIP(ctx, hipMalloc(out_dev, bytes ? bytes : 16));
    return TMI_VALID;
}

int tmi_buf_free(tmi_ctx_t* ctx, void* dev)
{
    if (!ctx)
        return TMI_ERROR;
    if (!dev)
        return TMI_VALID;
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    TMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
    TMI_HIP(ctx, hipFree(dev));
    return TMI_VALID;
}

int tmi_upload(tmi_ctx_t* ctx, void* dst_dev, const void* src_host, size_t bytes)
{
    if (!ctx || (bytes && (!dst_dev || !src_host)))
        return fail(ctx, "tmi_upload: null pointer");
    if (!bytes)
        return TMI_VALID;
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    TMI_HIP(ctx, hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    TMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return TMI_VALID;
}

int tmi_download(tmi_ctx_t* ctx, void* dst_host, const void* src_dev, size_t bytes)
{
    if (!ctx || (bytes && (!dst_host || !src_dev)))
        return fail(ctx, "tmi_download: null pointer");
    if (!bytes)
        return TMI_VALID;
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    TMI_HIP(ctx, hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    TMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return TMI_VALID;
}

int tmi_conv2d_check(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, int32_t depthwise)
{
    if (!ctx)
        return TMI_ERROR;
    ConvGeom g;
    return validate_conv(ctx, depthwise ? "OpDepthwiseConv2d" : "OpConv2d", d, depthwise != 0, 0, 0, g);
}

int tmi_rescale_check(tmi_ctx_t* ctx, const tmi_rescale_desc_t* r, int32_t rank, int32_t C)
{
    if (!ctx)
        return TMI_ERROR;
    if (rank < 0 || rank > 6)
        return fail(ctx, "OpRescale: rank outside [0,6]");
    RescaleParams p;
    static const int8_t dummy = 0;    // only the pointers' presence is checked here
    return validate_rescale(ctx, r, rank, C, &dummy, &dummy, p);
}

int tmi_conv2d(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev, const void* weight_dev,
               const void* bias_dev, int32_t in_zp, int32_t w_zp, void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    RescaleParams none{};
    return run_conv(ctx, "OpConv2d", false, d, in_dev, weight_dev, bias_dev, in_zp, w_zp, none,
                    d ? d->out_dtype : 0, out_dev);
}

static size_t align256(size_t v)
{
    return (v + 255) & ~(size_t)255;
}

// OpTransposeConv2d::checkTensorAttributes and the head of eval() (tensor_ops.cpp:1982-2056, :2083-2091, :2123-2129)
static int validate_tconv(tmi_ctx* ctx, const char* op, const tmi_tconv_desc_t* d, int32_t in_zp, int32_t w_zp)
{
    if (!d)
        return fail(ctx, "%s: null descriptor", op);
    // INT8 x INT8 -> INT32, INT16 x INT8 -> INT48, FP16 / BF16 / FP32 with fp32 accumulation (tensor_ops.cpp:2286-2291)
    if (d->in_dtype != TMI_INT8 && d->in_dtype != TMI_INT16 && d->in_dtype != TMI_FP16 && d->in_dtype != TMI_BF16 &&
        d->in_dtype != TMI_FP32)
        return fail(ctx, "%s: input data type not supported for this configuration of operator", op);
    if (d->out_dtype != (d->in_dtype == TMI_INT8 ? TMI_INT32 : (d->in_dtype == TMI_INT16 ? TMI_INT48 : d->in_dtype)))
        return fail(ctx, "%s: Output data type not supported for this configuration of operator", op);
    if (d->acc_dtype != 0 &&
        d->acc_dtype != (d->in_dtype == TMI_INT8 ? TMI_INT32 : (d->in_dtype == TMI_INT16 ? TMI_INT48 : TMI_FP32)))    // 0: the operand type's default
        return fail(ctx, "%s: accumulator type %d not supported for this configuration of operator", op, d->acc_dtype);
    if (d->N < 0 || d->IH < 0 || d->IW < 0 || d->IC < 0 || d->OC < 0 || d->KH < 1 || d->KW < 1)
        return fail(ctx, "%s: negative tensor dimension", op);
    // checkTensorAttributes (tensor_ops.cpp:2017-2053)
    for (int i = 0; i < 2; i++)
        if (d->stride[i] < 1)
            return fail(ctx, "%s: At least one stride is smaller than one", op);
    for (int i = 0; i < 4; i++)
        if (d->out_pad[i] <= -(i < 2 ? d->KH : d->KW))
            return fail(ctx, "%s: At least one out_pad value is larger than kernel size", op);
    const int64_t H = (int64_t)(d->IH - 1) * d->stride[0] + d->out_pad[0] + d->out_pad[1] + d->KH;
    const int64_t W = (int64_t)(d->IW - 1) * d->stride[1] + d->out_pad[2] + d->out_pad[3] + d->KW;
    if (d->OH != H || d->OW != W)
        return fail(ctx, "%s: Mismatch between output shape provided and expected output shape (%lld,%lld)", op,
                    (long long)H, (long long)W);
    if (d->bias_len != d->OC && d->bias_len != 1)
        return fail(ctx, "%s: bias channels mismatch %d != %d", op, d->bias_len, d->OC);
    // tensor_ops.cpp:2115-2119; INT16 inputs come with INT8 weights, which keep their zero point
    if (d->in_dtype != TMI_INT8 && in_zp != 0)
        return fail(ctx, "%s: Input zero point must be zero for non int8_t data", op);
    if (d->in_dtype != TMI_INT8 && d->in_dtype != TMI_INT16 && w_zp != 0)
        return fail(ctx, "%s: Weight zero point must be zero for non int8_t data", op);
    return TMI_VALID;
}

int tmi_transpose_conv2d_check(tmi_ctx_t* ctx, const tmi_tconv_desc_t* d)
{
    if (!ctx)
        return TMI_ERROR;
    return validate_tconv(ctx, "OpTransposeConv2d", d, 0, 0);
}

// TRANSPOSE_CONV2D on either scratch memory: the context's buffer, grown on demand (static_only = false), or the
// library's static array, which is never grown (static_only = true: nothing on this path allocates or frees).
static int run_transpose_conv2d(tmi_ctx* ctx, bool static_only, const tmi_tconv_desc_t* d, const void* in_dev,
                                const void* weight_dev, const void* bias_dev, int32_t in_zp, int32_t w_zp, void* out_dev)
{
    const char* op = "OpTransposeConv2d";
    int rc = validate_tconv(ctx, op, d, in_zp, w_zp);
    if (rc != TMI_VALID)
        return rc;
    if (level_on(ctx))
    {
        // tensor_ops.cpp:2096-2104
        const tmi_level_t& l = ctx->level;
        level_check(ctx, d->KH <= l.max_kernel, op, "KH should be smaller than or equal to MAX_KERNEL");
        level_check(ctx, d->KW <= l.max_kernel, op, "KW should be smaller than or equal to MAX_KERNEL");
        for (int i = 0; i < 4; i++)
            level_check(ctx, d->out_pad[i] <= l.max_kernel, op, "out_pad should be smaller than or equal to MAX_KERNEL");
        level_check(ctx, d->stride[0] <= l.max_stride, op, "stride_y should be smaller than or equal to MAX_STRIDE");
        level_check(ctx, d->stride[1] <= l.max_stride, op, "stride_x should be smaller than or equal to MAX_STRIDE");
    }
    const int64_t total = (int64_t)d->N * d->OH * d->OW * d->OC;
    if (total == 0)
    {
        ctx->last_kernel = "empty";
        return TMI_VALID;
    }
    if (!in_dev || !weight_dev || !bias_dev || !out_dev)
        return fail(ctx, "%s: null tensor pointer", op);
    if (d->IH == 0 || d->IW == 0 || d->IC == 0)
        return fail(ctx, "%s: empty input with a non-empty output", op);
    TMI_HIP(ctx, hipSetDevice(ctx->device));

    // the equivalent CONV2D: flipped taps, stride 1, pads KH-1+out_pad, input with holes between its pixels
    const int eb         = dtype_bits(d->in_dtype) / 8;
    const int row_bytes  = d->IC * eb;
    const int w_row_bytes = d->in_dtype == TMI_INT16 ? d->IC : row_bytes;    // INT16 inputs come with INT8 weights
    const bool holes     = d->stride[0] > 1 || d->stride[1] > 1;
    const int32_t UH     = (d->IH - 1) * d->stride[0] + 1, UW = (d->IW - 1) * d->stride[1] + 1;
    tmi_conv_desc_t c{};
    c.in_dtype = d->in_dtype, c.out_dtype = d->out_dtype;
    c.N = d->N, c.IH = UH, c.IW = UW, c.IC = d->IC, c.OC = d->OC, c.KH = d->KH, c.KW = d->KW, c.OH = d->OH, c.OW = d->OW;
    c.pad[0] = d->KH - 1 + d->out_pad[0], c.pad[1] = d->KH - 1 + d->out_pad[1];
    c.pad[2] = d->KW - 1 + d->out_pad[2], c.pad[3] = d->KW - 1 + d->out_pad[3];
    c.stride[0] = c.stride[1] = 1, c.dilation[0] = c.dilation[1] = 1;
    c.bias_len = d->bias_len, c.acc_dtype = d->acc_dtype;
    RescaleParams none{};
    // the slab kernel reads both operands where they lie (holes and flip are part of its addressing)
    if ((ctx->kernel_choice == 0 || ctx->kernel_choice == 4) && d->in_dtype == TMI_INT8)
    {
        ConvGeom g;
        rc = validate_conv(ctx, op, &c, false, in_zp, w_zp, g);
        if (rc != TMI_VALID)
            return rc;
        const SlabHoles h{ d->stride[0], d->stride[1], d->IH, d->IW };
        const char* name = launch_conv2d_slab(ctx->stream, d->in_dtype, d->out_dtype, g, in_dev, weight_dev, bias_dev, in_zp,
                                              w_zp, none, out_dev, ctx->pages_dev + (in_zp & 255) * 64, ctx->flags_dev, &h);
        if (name)
            return after_launch(ctx, name);
    }
    const size_t w_bytes = align256((size_t)d->OC * d->KH * d->KW * w_row_bytes);
    const size_t u_bytes = holes ? align256((size_t)d->N * UH * UW * row_bytes) : 0;
    uint8_t* w_flip = nullptr;
    if (static_only)
    {
        if (w_bytes + u_bytes > (size_t)TMI_NOALLOC_SCRATCH_BYTES)
            return fail(ctx, "%s: the re-laid-out operands need %zu bytes of scratch memory, more than the %zu bytes "
                             "of the static scratch array (TMI_NOALLOC_SCRATCH_BYTES)", op, w_bytes + u_bytes,
                        (size_t)TMI_NOALLOC_SCRATCH_BYTES);
        w_flip = ctx->static_scratch;
    }
    else
    {
        rc = ensure_workspace(ctx, w_bytes + u_bytes);
        if (rc != TMI_VALID)
            return rc;
        w_flip = (uint8_t*)ctx->workspace;
    }
    uint8_t* u      = w_flip + w_bytes;
    if (w_row_bytes != row_bytes)
    {
        // operands of different element sizes: one launch each (the input zero point of INT16 data is 0)
        if (!launch_flip_taps(ctx->stream, w_row_bytes, d->OC, d->KH, d->KW, weight_dev, w_flip) ||
            (holes && !launch_upsample(ctx->stream, row_bytes, d->N, d->IH, d->IW, d->stride[0], d->stride[1], 0, in_dev, u)))
            return fail(ctx, "%s: operand re-layout launch failed", op);
    }
    else if (!(holes ? launch_tconv_operands(ctx->stream, row_bytes, d->OC, d->KH, d->KW, weight_dev, w_flip, d->N, d->IH, d->IW,
                                             d->stride[0], d->stride[1], in_zp, in_dev, u)
                     : launch_flip_taps(ctx->stream, row_bytes, d->OC, d->KH, d->KW, weight_dev, w_flip)))
        return fail(ctx, "%s: operand re-layout launch failed", op);
    return run_conv(ctx, op, false, &c, holes ? (const void*)u : in_dev, w_flip, bias_dev, in_zp, w_zp, none,
                    d->out_dtype, out_dev, false, false);
}

int tmi_transpose_conv2d(tmi_ctx_t* ctx, const tmi_tconv_desc_t* d, const void* in_dev, const void* weight_dev,
                         const void* bias_dev, int32_t in_zp, int32_t w_zp, void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    return run_transpose_conv2d(ctx, false, d, in_dev, weight_dev, bias_dev, in_zp, w_zp, out_dev);
}

int tmi_transpose_conv2d_noalloc(tmi_ctx_t* ctx, const tmi_tconv_desc_t* d, const void* in_dev, const void* weight_dev,
                                 const void* bias_dev, int32_t in_zp, int32_t w_zp, void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    return run_transpose_conv2d(ctx, true, d, in_dev, weight_dev, bias_dev, in_zp, w_zp, out_dev);
}

// OpConv3d::checkTensorAttributes and the head of eval() (tensor_ops.cpp:901-933, :120-226, :963-970, :1024-1033)
static int validate_conv3d(tmi_ctx* ctx, const char* op, const tmi_conv3d_desc_t* d, int32_t in_zp, int32_t w_zp)
{
    if (!d)
        return fail(ctx, "%s: null descriptor", op);
    // INT8 x INT8 -> INT32, INT16 x INT8 -> INT48, FP16 / BF16 / FP32 with fp32 accumulation (tensor_ops.cpp:2232-2237)
    if (d->in_dtype != TMI_INT8 && d->in_dtype != TMI_INT16 && d->in_dtype != TMI_FP16 && d->in_dtype != TMI_BF16 &&
        d->in_dtype != TMI_FP32)
        return fail(ctx, "%s: input data type not supported for this configuration of operator", op);
    if (d->out_dtype != (d->in_dtype == TMI_INT8 ? TMI_INT32 : (d->in_dtype == TMI_INT16 ? TMI_INT48 : d->in_dtype)))
        return fail(ctx, "%s: Output data type not supported for this configuration of operator", op);
    if (d->acc_dtype != 0 &&
        d->acc_dtype != (d->in_dtype == TMI_INT8 ? TMI_INT32 : (d->in_dtype == TMI_INT16 ? TMI_INT48 : TMI_FP32)))    // 0: the operand type's default
        return fail(ctx, "%s: accumulator type %d not supported for this configuration of operator", op, d->acc_dtype);
    if (d->N < 0 || d->ID < 0 || d->IH < 0 || d->IW < 0 || d->IC < 0 || d->OC < 0 || d->KD < 1 || d->KH < 1 ||
        d->KW < 1)
        return fail(ctx, "%s: negative tensor dimension", op);
    // check_conv_attribute with three dimensions (tensor_ops.cpp:120-226)
    for (int i = 0; i < 6; i++)
        if (d->pad[i] < 0)
            return fail(ctx, "%s: At least one pad is smaller than zero", op);
    for (int i = 0; i < 3; i++)
        if (d->stride[i] < 1)
            return fail(ctx, "%s: At least one stride dimension is smaller than one", op);
    for (int i = 0; i < 3; i++)
        if (d->dilation[i] < 1)
            return fail(ctx, "%s: At least one dilation dimension is smaller than one", op);
    const int64_t full_d = (int64_t)d->ID - 1 + d->pad[0] + d->pad[1] - (int64_t)(d->KD - 1) * d->dilation[0];
    const int64_t full_h = (int64_t)d->IH - 1 + d->pad[2] + d->pad[3] - (int64_t)(d->KH - 1) * d->dilation[1];
    const int64_t full_w = (int64_t)d->IW - 1 + d->pad[4] + d->pad[5] - (int64_t)(d->KW - 1) * d->dilation[2];
    if ((full_d % d->stride[0]) != 0 || (full_h % d->stride[1]) != 0 || (full_w % d->stride[2]) != 0)
        return fail(ctx, "%s: Parameters must yield exact integer output dimensions", op);
    if (d->OD != full_d / d->stride[0] + 1 || d->OH != full_h / d->stride[1] + 1 ||
        d->OW != full_w / d->stride[2] + 1)
        return fail(ctx, "%s: Mismatch between output shape provided and expected output shape (%lld,%lld,%lld)", op,
                    (long long)(full_d / d->stride[0] + 1), (long long)(full_h / d->stride[1] + 1),
                    (long long)(full_w / d->stride[2] + 1));
    if (d->bias_len != d->OC && d->bias_len != 1)
        return fail(ctx, "%s: bias channel mismatch %d != %d", op, d->bias_len, d->OC);
    // tensor_ops.cpp:1031-1037; INT16 inputs come with INT8 weights, which keep their zero point
    if (d->in_dtype != TMI_INT8 && in_zp != 0)
        return fail(ctx, "%s: Input zero point must be zero for non int8_t data", op);
    if (d->in_dtype != TMI_INT8 && d->in_dtype != TMI_INT16 && w_zp != 0)
        return fail(ctx, "%s: Weight zero point must be zero for non int8_t data", op);
    return TMI_VALID;
}

int tmi_conv3d_check(tmi_ctx_t* ctx, const tmi_conv3d_desc_t* d)
{
    if (!ctx)
        return TMI_ERROR;
    return validate_conv3d(ctx, "OpConv3d", d, 0, 0);
}

int tmi_conv3d(tmi_ctx_t* ctx, const tmi_conv3d_desc_t* d, const void* in_dev, const void* weight_dev,
               const void* bias_dev, int32_t in_zp, int32_t w_zp, void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    const char* op = "OpConv3d";
    int rc = validate_conv3d(ctx, op, d, in_zp, w_zp);
    if (rc != TMI_VALID)
        return rc;
    if (level_on(ctx))
    {
        // tensor_ops.cpp:981-995
        const tmi_level_t& l = ctx->level;
        level_check(ctx, (int64_t)d->dilation[0] * d->KD <= l.max_kernel, op, "dilation_d * KD should be smaller than or equal to MAX_KERNEL");
        level_check(ctx, (int64_t)d->dilation[1] * d->KH <= l.max_kernel, op, "dilation_y * KH should be smaller than or equal to MAX_KERNEL");
        level_check(ctx, (int64_t)d->dilation[2] * d->KW <= l.max_kernel, op, "dilation_x * KW should be smaller than or equal to MAX_KERNEL");
        for (int i = 0; i < 6; i++)
            level_check(ctx, d->pad[i] <= l.max_kernel, op, "pad should be smaller than or equal to MAX_KERNEL");
        for (int i = 0; i < 3; i++)
            level_check(ctx, d->stride[i] <= l.max_stride, op, "stride should be smaller than or equal to MAX_STRIDE");
    }
    const int64_t total = (int64_t)d->N * d->OD * d->OH * d->OW * d->OC;
    if (total == 0)
    {
        ctx->last_kernel = "empty";
        return TMI_VALID;
    }
    if (!in_dev || !weight_dev || !bias_dev || !out_dev)
        return fail(ctx, "%s: null tensor pointer", op);
    if ((int64_t)d->N * d->OD > INT32_MAX || (int64_t)d->KD * d->IC > INT32_MAX)
        return fail(ctx, "%s: shape too large", op);
    TMI_HIP(ctx, hipSetDevice(ctx->device));

    const int eb         = dtype_bits(d->in_dtype) / 8;
    const int row_bytes  = d->IC * eb;
    tmi_conv_desc_t c{};
    c.in_dtype = d->in_dtype, c.out_dtype = d->out_dtype;
    c.N = d->N * d->OD, c.IH = d->IH, c.IW = d->IW, c.IC = d->KD * d->IC, c.OC = d->OC, c.KH = d->KH, c.KW = d->KW;
    c.OH = d->OH, c.OW = d->OW;
    for (int i = 0; i < 4; i++)
        c.pad[i] = d->pad[2 + i];
    c.stride[0] = d->stride[1], c.stride[1] = d->stride[2];
    c.dilation[0] = d->dilation[1], c.dilation[1] = d->dilation[2];
    c.bias_len = d->bias_len, c.acc_dtype = d->acc_dtype;
    RescaleParams none{};
    // the slab kernel reads both operands where they lie (the depth taps are part of its addressing)
    if ((ctx->kernel_choice == 0 || ctx->kernel_choice == 4) && d->in_dtype == TMI_INT8 && d->KD > 1)
    {
        ConvGeom g;
        rc = validate_conv(ctx, op, &c, false, in_zp, w_zp, g);
        if (rc != TMI_VALID)
            return rc;
        const SlabDepth dep{ d->KD, d->ID, d->OD, d->stride[0], d->dilation[0], d->pad[0] };
        const char* name = launch_conv2d_slab(ctx->stream, d->in_dtype, d->out_dtype, g, in_dev, weight_dev, bias_dev, in_zp,
                                              w_zp, none, out_dev, ctx->pages_dev + (in_zp & 255) * 64, ctx->flags_dev,
                                              nullptr, &dep);
        if (name)
            return after_launch(ctx, name);
    }
    const int w_row_bytes = d->in_dtype == TMI_INT16 ? d->IC : row_bytes;    // INT16 inputs come with INT8 weights
    const size_t w_bytes = align256((size_t)d->OC * d->KD * d->KH * d->KW * w_row_bytes);
    const size_t g_bytes = align256((size_t)d->N * d->OD * d->IH * d->IW * d->KD * row_bytes);
    rc                   = ensure_workspace(ctx, w_bytes + g_bytes);
    if (rc != TMI_VALID)
        return rc;
    uint8_t* w_perm = (uint8_t*)ctx->workspace;
    uint8_t* gath   = w_perm + w_bytes;
    if (w_row_bytes != row_bytes)
    {
        // operands of different element sizes: one launch each (the input zero point of INT16 data is 0)
        if (!launch_permute_w3d(ctx->stream, w_row_bytes, d->OC, d->KD, d->KH * d->KW, weight_dev, w_perm) ||
            !launch_gather_depth(ctx->stream, row_bytes, d->N, d->ID, d->OD, d->KD, d->IH * d->IW, d->stride[0], d->dilation[0],
                                 d->pad[0], 0, in_dev, gath))
            return fail(ctx, "%s: operand re-layout launch failed", op);
    }
    else if (!launch_conv3d_operands(ctx->stream, row_bytes, d->OC, d->KD, d->KH * d->KW, weight_dev, w_perm, d->N, d->ID,
                                     d->OD, d->IH * d->IW, d->stride[0], d->dilation[0], d->pad[0], in_zp, in_dev, gath))
        return fail(ctx, "%s: operand re-layout launch failed", op);
    return run_conv(ctx, op, false, &c, gath, w_perm, bias_dev, in_zp, w_zp, none, d->out_dtype, out_dev, false,
                    false);
}

// The fused operators under INEXACT_ROUND in precise mode: the convolution's INT32 results go to the scratch buffer and
// the stand-alone RESCALE kernel, the only one that holds the FP64 forms, converts them.  (The convolution kernels keep
// their epilogues free of FP64 code; precise mode is the reference's checking mode, not a path to be fast on.)
static int run_conv_then_rescale(tmi_ctx* ctx, const char* op, bool depthwise, const tmi_conv_desc_t* d, const void* in,
                                 const void* w, const void* bias, int32_t in_zp, int32_t w_zp, const RescaleParams& rp,
                                 int32_t out_dtype, void* out)
{
    ConvGeom g;
    int rc = validate_conv(ctx, op, d, depthwise, in_zp, w_zp, g);
    if (rc != TMI_VALID)
        return rc;
    const int64_t total = (int64_t)g.N * g.OH * g.OW * g.OC;
    if (total > 0 && !out)
        return fail(ctx, "%s: null tensor pointer", op);
    rc = ensure_workspace(ctx, (size_t)(total > 0 ? total : 1) * sizeof(int32_t));
    if (rc != TMI_VALID)
        return rc;
    RescaleParams none{};
    rc = run_conv(ctx, op, depthwise, d, in, w, bias, in_zp, w_zp, none, TMI_INT32, ctx->workspace);
    if (rc != TMI_VALID || total == 0)
        return rc;
    const char* name = launch_rescale(ctx->stream, rp, TMI_INT32, out_dtype, ctx->workspace, out, total, g.OC, ctx->flags_dev);
    return after_launch(ctx, name);
}

int tmi_depthwise_conv2d(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev, const void* weight_dev,
                         const void* bias_dev, int32_t in_zp, int32_t w_zp, void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    RescaleParams none{};
    return run_conv(ctx, "OpDepthwiseConv2d", true, d, in_dev, weight_dev, bias_dev, in_zp, w_zp, none,
                    d ? d->out_dtype : 0, out_dev);
}

int tmi_conv2d_rescale_clamp(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev, const void* weight_dev,
                             const void* bias_dev, int32_t in_zp, int32_t w_zp, const tmi_rescale_desc_t* r,
                             const void* multiplier_dev, const void* shift_dev, int32_t has_clamp,
                             int32_t clamp_min, int32_t clamp_max, void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    if (!d)
        return fail(ctx, "OpConv2d: null descriptor");
    RescaleParams rp;
    int rc = validate_fused_rescale(ctx, "OpConv2d+OpRescale", d, r, multiplier_dev, shift_dev, has_clamp,
                                    clamp_min, clamp_max, rp);
    if (rc != TMI_VALID)
        return rc;
    if (rp.inexact_round >= 2)
        return run_conv_then_rescale(ctx, "OpConv2d", false, d, in_dev, weight_dev, bias_dev, in_zp, w_zp, rp,
                                     r->out_dtype, out_dev);
    return run_conv(ctx, "OpConv2d", false, d, in_dev, weight_dev, bias_dev, in_zp, w_zp, rp, r->out_dtype, out_dev);
}

int tmi_depthwise_conv2d_rescale_clamp(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev,
                                       const void* weight_dev, const void* bias_dev, int32_t in_zp, int32_t w_zp,
                                       const tmi_rescale_desc_t* r, const void* multiplier_dev,
                                       const void* shift_dev, int32_t has_clamp, int32_t clamp_min,
                                       int32_t clamp_max, void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    if (!d)
        return fail(ctx, "OpDepthwiseConv2d: null descriptor");
    RescaleParams rp;
    int rc = validate_fused_rescale(ctx, "OpDepthwiseConv2d+OpRescale", d, r, multiplier_dev, shift_dev, has_clamp,
                                    clamp_min, clamp_max, rp);
    if (rc != TMI_VALID)
        return rc;
    if (rp.inexact_round >= 2)
        return run_conv_then_rescale(ctx, "OpDepthwiseConv2d", true, d, in_dev, weight_dev, bias_dev, in_zp, w_zp, rp,
                                     r->out_dtype, out_dev);
    return run_conv(ctx, "OpDepthwiseConv2d", true, d, in_dev, weight_dev, bias_dev, in_zp, w_zp, rp, r->out_dtype,
                    out_dev);
}

int tmi_matmul(tmi_ctx_t* ctx, int32_t in_dtype, int32_t N, int32_t H, int32_t C, int32_t W, const void* a_dev,
               const void* b_dev, int32_t a_zp, int32_t b_zp, void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    if (in_dtype != TMI_INT8 && in_dtype != TMI_INT16 && in_dtype != TMI_FP16 && in_dtype != TMI_BF16 && in_dtype != TMI_FP32)
        return fail(ctx, "OpMatMul: input data type not supported for this configuration of operator");
    if (N < 0 || H < 0 || C < 0 || W < 0)
        return fail(ctx, "OpMatMul: negative tensor dimension");
    // tensor_ops.cpp:1433-1434
    if (in_dtype != TMI_INT8 && a_zp != 0)
        return fail(ctx, "OpMatMul: A zeropoint must be zero for non int8_t data");
    if (in_dtype != TMI_INT8 && b_zp != 0)
        return fail(ctx, "OpMatMul: B zeropoint must be zero for non int8_t data");
    if (a_zp < -128 || a_zp > 127 || b_zp < -128 || b_zp > 127)
        return fail(ctx, "OpMatMul: zero point outside the int8 range");
    const int64_t total = (int64_t)N * H * W;
    if (total > 0 && (!out_dev || ((int64_t)C > 0 && (!a_dev || !b_dev))))
        return fail(ctx, "OpMatMul: null tensor pointer");
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    if (total == 0)
    {
        ctx->last_kernel = "empty";
        return TMI_VALID;
    }
    if (in_dtype == TMI_INT16)    // INT16 x INT16 -> INT48 (tensor_ops.cpp:2257): int64 results
        return after_launch(ctx, launch_matmul_i16_direct(ctx->stream, N, H, C, W, a_dev, b_dev, out_dev));
    const char* name = nullptr;
    if (ctx->kernel_choice != 1 && C > 0 && in_dtype != TMI_FP32)
    {
        // MFMA paths: one "image" per batch, pixels = rows of A, output channels = columns of B, 1x1 taps,
        // per-image weights.  The bias operand is the permanently zero word kept after the flags.  The GEMM
        // kernel takes B as it lies in memory ([C][W], transposed on its way out of LDS); what it does not
        // take that way (rows of B that are not whole 16-byte pieces) is first made K-contiguous ([N,C,W] ->
        // [N,W,C]) in the context's scratch buffer and offered to the GEMM kernel again, then to the
        // implicit-GEMM kernel.
        const int eb = in_dtype == TMI_INT8 ? 1 : 2;
        ConvGeom g{};
        g.N = N, g.IH = H, g.IW = 1, g.IC = C, g.OC = W, g.KH = 1, g.KW = 1, g.OH = H, g.OW = 1;
        g.stride_y = g.stride_x = g.dil_y = g.dil_x = 1;
        g.bias_len = 1, g.M = 1;
        RescaleParams none{};
        const int32_t out_dtype = in_dtype == TMI_INT8 ? TMI_INT32 : TMI_FP32;
        if (ctx->kernel_choice != 2)
            name = launch_gemm_mfma(ctx->stream, in_dtype, out_dtype, g, a_dev, b_dev, ctx->flags_dev + 16, a_zp, b_zp,
                                    none, out_dev, (int64_t)W * C * eb, (int64_t)W * eb);
        const bool direct = name != nullptr;    // B read as it lies, no transposed copy
        if (!name)
        {
            const size_t bytes = (size_t)N * C * W * eb;
            int rc             = ensure_workspace(ctx, bytes);
            if (rc != TMI_VALID)
                return rc;
            if (!launch_transpose(ctx->stream, eb, N, C, W, b_dev, ctx->workspace))
                return fail(ctx, "OpMatMul: transpose launch failed");
            if (ctx->kernel_choice != 2)
                name = launch_gemm_mfma(ctx->stream, in_dtype, out_dtype, g, a_dev, ctx->workspace, ctx->flags_dev + 16,
                                        a_zp, b_zp, none, out_dev, (int64_t)W * C * eb);
        }
        if (name && direct)
            name = in_dtype == TMI_INT8 ? "matmul_gemm_i8" : (in_dtype == TMI_FP16 ? "matmul_gemm_f16" : "matmul_gemm_bf16");
        else if (name)
            name = in_dtype == TMI_INT8 ? "matmul_tgemm_i8"
                                        : (in_dtype == TMI_FP16 ? "matmul_tgemm_f16" : "matmul_tgemm_bf16");
        else if (ctx->kernel_choice != 3)
        {
            name = launch_conv2d_mfma(ctx->stream, in_dtype, out_dtype, g, a_dev, ctx->workspace, ctx->flags_dev + 16,
                                      a_zp, b_zp, none, out_dev, ctx->flags_dev, (int64_t)W * C * eb);
            if (name)
                name = in_dtype == TMI_INT8 ? "matmul_mfma_i8"
                                            : (in_dtype == TMI_FP16 ? "matmul_mfma_f16" : "matmul_mfma_bf16");
        }
    }
    if (!name && ctx->kernel_choice >= 2)
        return fail(ctx, "OpMatMul: no MFMA kernel is eligible for this shape");
    if (!name)
        name = launch_matmul_direct(ctx->stream, in_dtype, N, H, C, W, a_dev, b_dev, a_zp, b_zp, out_dev);
    return after_launch(ctx, name);
}

// ---- floating-point compliance passes (precise.hip) -------------------------------------------------------
static int run_conv_precise(tmi_ctx* ctx, const char* op, bool depthwise, const tmi_conv_desc_t* d, const void* in,
                            const void* w, const void* bias, int32_t bounds_mode, int32_t local_bound, double* out)
{
    ConvGeom g;
    int rc = validate_conv(ctx, op, d, depthwise, 0, 0, g);
    if (rc != TMI_VALID)
        return rc;
    if (d->in_dtype != TMI_FP16 && d->in_dtype != TMI_BF16 && d->in_dtype != TMI_FP32)
        return fail(ctx, "%s: the precise / bounds passes take floating-point operands", op);
    const int64_t total = (int64_t)g.N * g.OH * g.OW * g.OC;
    if (total > 0 && (!in || !w || !bias || !out))
        return fail(ctx, "%s: null tensor pointer", op);
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    if (total == 0)
    {
        ctx->last_kernel = "empty";
        return TMI_VALID;
    }
    // one double of the context's 256-byte block (bytes 160..167) holds the input's largest magnitude
    double* abs_max_slot = (bounds_mode && !local_bound) ? reinterpret_cast<double*>(reinterpret_cast<uint8_t*>(ctx->flags_dev) + 160)
                                                         : nullptr;
    const char* name = launch_conv_precise(ctx->stream, d->in_dtype, depthwise, g, in, w, bias, bounds_mode, abs_max_slot, out);
    if (!name)
        return fail(ctx, "%s: operand type without a precise-mode kernel", op);
    return after_launch(ctx, name);
}

int tmi_conv2d_precise(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev, const void* weight_dev,
                       const void* bias_dev, int32_t bounds_mode, int32_t local_bound, double* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    return run_conv_precise(ctx, "OpConv2d", false, d, in_dev, weight_dev, bias_dev, bounds_mode, local_bound, out_dev);
}

int tmi_depthwise_conv2d_precise(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev, const void* weight_dev,
                                 const void* bias_dev, int32_t bounds_mode, int32_t local_bound, double* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    return run_conv_precise(ctx, "OpDepthwiseConv2d", true, d, in_dev, weight_dev, bias_dev, bounds_mode, local_bound,
                            out_dev);
}

int tmi_matmul_precise(tmi_ctx_t* ctx, int32_t in_dtype, int32_t N, int32_t H, int32_t C, int32_t W, const void* a_dev,
                       const void* b_dev, int32_t bounds_mode, double* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    if (in_dtype != TMI_FP16 && in_dtype != TMI_BF16 && in_dtype != TMI_FP32)
        return fail(ctx, "OpMatMul: the precise / bounds passes take floating-point operands");
    if (N < 0 || H < 0 || C < 0 || W < 0)
        return fail(ctx, "OpMatMul: negative tensor dimension");
    const int64_t total = (int64_t)N * H * W;
    if (total > 0 && (!out_dev || (C > 0 && (!a_dev || !b_dev))))
        return fail(ctx, "OpMatMul: null tensor pointer");
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    if (total == 0)
    {
        ctx->last_kernel = "empty";
        return TMI_VALID;
    }
    const char* name = launch_matmul_precise(ctx->stream, in_dtype, N, H, C, W, a_dev, b_dev, bounds_mode, out_dev);
    if (!name)
        return fail(ctx, "OpMatMul: operand type without a precise-mode kernel");
    return after_launch(ctx, name);
}

int tmi_dot_product_check(tmi_ctx_t* ctx, int32_t out_dtype, int64_t n, const void* imp_dev, const double* ref_dev,
                          const double* bnd_dev, int32_t ksb, int32_t set_number, tmi_dp_result_t* result)
{
    if (!ctx)
        return TMI_ERROR;
    if (!result || n <= 0 || !imp_dev || !ref_dev || !bnd_dev || ksb <= 0)
        return fail(ctx, "dot product check: bad argument");
    if (out_dtype != TMI_FP16 && out_dtype != TMI_BF16 && out_dtype != TMI_FP32)
        return fail(ctx, "dot product check: result type must be FP16, BF16 or FP32");
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    // accumulators: 3 doubles + 1 word in the upper half of the context's 256-byte flag block
    uint8_t* acc = reinterpret_cast<uint8_t*>(ctx->flags_dev) + 128;
    TMI_HIP(ctx, hipMemsetAsync(acc, 0, 32, ctx->stream));
    const int32_t abs_bound = 2 * ksb;
    if (!launch_dp_check(ctx->stream, out_dtype, n, imp_dev, ref_dev, bnd_dev, abs_bound,
                         reinterpret_cast<double*>(acc), reinterpret_cast<unsigned long long*>(acc + 24)))
        return fail(ctx, "dot product check: launch failed");
    ctx->last_kernel = "dot_product_check";
    struct
    {
        double v[3];
        unsigned long long bad;
    } host;
    TMI_HIP(ctx, hipMemcpyAsync(&host, acc, 32, hipMemcpyDeviceToHost, ctx->stream));
    TMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
    result->err_sum = host.v[0], result->err_sumsq = host.v[1], result->max_abs_err = host.v[2];
    result->failed_elements = (int64_t)host.bad, result->elements = n;
    result->abs_bound = abs_bound, result->variance_bound = 4.0 * 0.4 * ksb;
    // validateDataDP: every element within its bound; for sets 3..5 |sum| <= sqrt(10 * var * T); sumsq <= var * T
    bool ok = host.bad == 0 && result->err_sumsq <= result->variance_bound * (double)n;
    if (set_number >= 3 && set_number <= 5)
        ok = ok && fabs(result->err_sum) <= sqrt(10.0 * result->variance_bound * (double)n);
    result->compliant = ok ? 1 : 0;
    return TMI_VALID;
}

// check_pool2d_attribute (tensor_ops.cpp:29-117) with the reference's messages, plus the type rules.
static int validate_pool(tmi_ctx* ctx, const char* op, const tmi_pool_desc_t* d, bool avg, int32_t in_zp,
                         int32_t out_zp)
{
    if (!d)
        return fail(ctx, "%s: null descriptor", op);
    const bool is_int = d->dtype == TMI_INT8 || d->dtype == TMI_INT16;
    const bool is_fp  = d->dtype == TMI_FP16 || d->dtype == TMI_BF16 || d->dtype == TMI_FP32;
    if (!is_int && !is_fp)
        return fail(ctx, "%s: input data type not supported for this configuration of operator", op);
    if (avg && d->acc_dtype != 0 && d->acc_dtype != (is_int ? TMI_INT32 : TMI_FP32))
        return fail(ctx, "%s: accumulator type not supported for this configuration of operator", op);
    if (d->N < 0 || d->IH < 0 || d->IW < 0 || d->C < 0)
        return fail(ctx, "%s: negative tensor dimension", op);
    for (int i = 0; i < 4; i++)
        if (d->pad[i] < 0)
            return fail(ctx, "%s: At least one pad is smaller than zero", op);
    for (int i = 0; i < 2; i++)
        if (d->kernel[i] < 1)
            return fail(ctx, "%s: At least one kernel dimension is smaller than one", op);
    for (int i = 0; i < 2; i++)
        if (d->stride[i] < 1)
            return fail(ctx, "%s: At least one stride dimension is smaller than one", op);
    if (d->pad[0] >= d->kernel[0] || d->pad[1] >= d->kernel[0] || d->pad[2] >= d->kernel[1] ||
        d->pad[3] >= d->kernel[1])
        return fail(ctx, "%s: At least one pad is >= kernel dimension", op);
    const int32_t full_h = d->IH + d->pad[0] + d->pad[1] - d->kernel[0];
    const int32_t full_w = d->IW + d->pad[2] + d->pad[3] - d->kernel[1];
    if (full_h % d->stride[0] != 0 || full_w % d->stride[1] != 0)
        return fail(ctx, "%s: Parameters must yield exact integer output dimensions", op);
    if (d->OH != full_h / d->stride[0] + 1 || d->OW != full_w / d->stride[1] + 1)
        return fail(ctx, "%s: Mismatch between output shape provided and expected output shape (%d,%d)", op,
                    full_h / d->stride[0] + 1, full_w / d->stride[1] + 1);
    if (avg && d->dtype != TMI_INT8 && in_zp != 0)
        return fail(ctx, "%s: Input zeropoint must be zero for non int8_t data", op);
    if (avg && d->dtype != TMI_INT8 && out_zp != 0)
        return fail(ctx, "%s: Output zeropoint must be zero for non int8_t data", op);
    if (!avg && is_fp && d->nan_mode != 1 && d->nan_mode != 2)
        return fail(ctx, "%s: invalid NaN propagation mode", op);
    return TMI_VALID;
}

int tmi_pool2d_check(tmi_ctx_t* ctx, const tmi_pool_desc_t* d, int32_t avg)
{
    if (!ctx)
        return TMI_ERROR;
    return validate_pool(ctx, avg ? "OpAvgPool2d" : "OpMaxPool2d", d, avg != 0, 0, 0);
}

static int run_pool(tmi_ctx* ctx, const char* op, bool avg, const tmi_pool_desc_t* d, const void* in_dev, int32_t in_zp,
                    int32_t out_zp, void* out_dev)
{
    int rc = validate_pool(ctx, op, d, avg, in_zp, out_zp);
    if (rc != TMI_VALID)
        return rc;
    if (level_on(ctx))
    {
        // tensor_ops.cpp:575-582, 1572-1579
        const tmi_level_t& l = ctx->level;
        level_check(ctx, d->kernel[0] <= l.max_kernel, op, "kernel_y should be smaller than or equal to MAX_KERNEL");
        level_check(ctx, d->kernel[1] <= l.max_kernel, op, "kernel_x should be smaller than or equal to MAX_KERNEL");
        level_check(ctx, d->stride[0] <= l.max_stride, op, "stride_y should be smaller than or equal to MAX_STRIDE");
        level_check(ctx, d->stride[1] <= l.max_stride, op, "stride_x should be smaller than or equal to MAX_STRIDE");
        for (int i = 0; i < 4; i++)
            level_check(ctx, d->pad[i] <= l.max_kernel, op, "pad should be smaller than or equal to MAX_KERNEL");
    }
    const int64_t total = (int64_t)d->N * d->OH * d->OW * d->C;
    if (total > 0 && (!in_dev || !out_dev))
        return fail(ctx, "%s: null tensor pointer", op);
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    if (total == 0)
    {
        ctx->last_kernel = "empty";
        return TMI_VALID;
    }
    const char* name = launch_pool(ctx->stream, avg, d->dtype, d->N, d->IH, d->IW, d->C, d->OH, d->OW, d->kernel[0],
                                   d->kernel[1], d->stride[0], d->stride[1], d->pad[0], d->pad[2], in_zp, out_zp,
                                   d->nan_mode, in_dev, out_dev, ctx->flags_dev);
    if (!name)
        return fail(ctx, "%s: tensor too large for the pooling kernel", op);
    return after_launch(ctx, name);
}

int tmi_avg_pool2d(tmi_ctx_t* ctx, const tmi_pool_desc_t* d, const void* in_dev, int32_t in_zp, int32_t out_zp,
                   void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    return run_pool(ctx, "OpAvgPool2d", true, d, in_dev, in_zp, out_zp, out_dev);
}

int tmi_max_pool2d(tmi_ctx_t* ctx, const tmi_pool_desc_t* d, const void* in_dev, void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    return run_pool(ctx, "OpMaxPool2d", false, d, in_dev, 0, 0, out_dev);
}

int tmi_rescale(tmi_ctx_t* ctx, const tmi_rescale_desc_t* r, int32_t rank, int64_t rows, int32_t C,
                const void* in_dev, const void* multiplier_dev, const void* shift_dev, void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    if (rank < 0 || rank > 6)
        return fail(ctx, "OpRescale: rank outside [0,6]");
    if (rows < 0 || C < 0)
        return fail(ctx, "OpRescale: negative tensor dimension");
    RescaleParams p;
    int rc = validate_rescale(ctx, r, rank, C, multiplier_dev, shift_dev, p);
    if (rc != TMI_VALID)
        return rc;
    // type_conversion.cpp:76
    level_check(ctx, rank <= ctx->level.max_rank, "OpRescale", "Rank should be smaller than or equal to MAX_RANK");
    const int64_t n = rows * (int64_t)C;
    if (n > 0 && (!in_dev || !out_dev))
        return fail(ctx, "OpRescale: null tensor pointer");
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    const char* name = launch_rescale(ctx->stream, p, r->in_dtype, r->out_dtype, in_dev, out_dev, n, C > 0 ? C : 1,
                                      ctx->flags_dev);
    return after_launch(ctx, name);
}

int tmi_clamp(tmi_ctx_t* ctx, int32_t dtype, int64_t n, const void* in_dev, int32_t min_val, int32_t max_val,
              void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    if (dtype != TMI_INT8 && dtype != TMI_INT16)
        return fail(ctx, "OpClamp: unsupported TOSA_REF_TYPE");
    if (max_val < min_val)
        return fail(ctx, "OpClamp: max smaller than min");
    if (n < 0 || (n > 0 && (!in_dev || !out_dev)))
        return fail(ctx, "OpClamp: bad tensor");
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    return after_launch(ctx, launch_clamp(ctx->stream, dtype, in_dev, out_dev, n, min_val, max_val));
}

int tmi_clamp_fp(tmi_ctx_t* ctx, int32_t dtype, int64_t n, const void* in_dev, float min_val, float max_val,
                 int32_t nan_mode, void* out_dev)
{
    if (!ctx)
        return TMI_ERROR;
    if (dtype != TMI_FP16 && dtype != TMI_BF16 && dtype != TMI_FP32)
        return fail(ctx, "OpClamp: unsupported TOSA_REF_TYPE");
    if (max_val < min_val)
        return fail(ctx, "OpClamp: max smaller than min");
    if (min_val != min_val || max_val != max_val)
        return fail(ctx, "OpClamp: min/max cannot be NaN");
    if (nan_mode != 1 && nan_mode != 2)
        return fail(ctx, "OpClamp: invalid NaN propagation mode");
    if (n < 0 || (n > 0 && (!in_dev || !out_dev)))
        return fail(ctx, "OpClamp: bad tensor");
    TMI_HIP(ctx, hipSetDevice(ctx->device));
    return after_launch(ctx, launch_clamp_fp(ctx->stream, dtype, in_dev, out_dev, n, min_val, max_val, nan_mode));
}

}    // extern "C"
