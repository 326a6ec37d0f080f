/*
 * tosa_mi355.h -- C ABI of the MI355X (gfx950) implementation of the TOSA reference model's tensor-op
 * hot path: CONV2D, DEPTHWISE_CONV2D, MATMUL, RESCALE, CLAMP and their fused forms.
 *
 * The TOSA reference model has no C ABI for built-in operators: each operator is a C++ GraphNode
 * subclass whose virtual eval() is called by SubgraphTraverser::evaluateNextNode()
 * (reference_model/src/graph_node.h:176-179, reference_model/src/subgraph_traverser.cpp:856).  The entry
 * points below are what a GraphNode adapter for these operators binds: one call per eval(), operands
 * given as device pointers to packed row-major tensors, attributes as plain structs, and the
 * reference's GraphStatus integer (reference_model/include/graph_status.h:18-23) as the return value.
 *
 * Conventions
 *   - Every function returns TMI_VALID (0), TMI_UNPREDICTABLE (1) or TMI_ERROR (2); none throws.
 *     TMI_ERROR corresponds to the reference's ERROR_IF / validation failures and is detected on the
 *     host before anything is launched; tmi_last_error() then holds the message.
 *   - Kernels are enqueued on the context's stream and the call returns without waiting.  The
 *     conditions that the reference turns into REQUIRE failures while evaluating RESCALE
 *     (reference_model/src/quant_util.h:48-82, reference_model/src/ops/type_conversion.cpp:348-360) are
 *     detected on the device and latched in a per-context flag word; tmi_ctx_sync() waits for the
 *     stream and returns TMI_UNPREDICTABLE if any was raised since the previous sync.
 *   - Tensors are packed: INT8 1 byte, INT16/FP16/BF16 2 bytes, INT32/FP32 4 bytes per element
 *     (the reference widens INT8 to int32 and FP16/BF16 to float in host memory:
 *     reference_model/src/ops/template_types.h:67-163).  Layouts are those of the TOSA operators:
 *     input/output NHWC, CONV2D weight OHWI, DEPTHWISE_CONV2D weight [KH,KW,C,M], MATMUL [N,H,C]x[N,C,W].
 *   - Pointers named *_dev must be device memory (from tmi_buf_alloc or any other HIP allocation on the
 *     context's device), 16-byte aligned for whole tensors.
 *   - One context serves one host thread at a time (the reference is single threaded and keeps its
 *     configuration in process globals: reference_model/src/model_runner.cpp:22-23).
 */
#ifndef TOSA_MI355_H
#define TOSA_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GraphStatus values: reference_model/include/graph_status.h:18-23 */
enum
{
    TMI_VALID         = 0,
    TMI_UNPREDICTABLE = 1,
    TMI_ERROR         = 2
};

/* Element types; the numbers are those of the serialized TOSA DType enum so that a graph loader can
 * pass them through (INT8 = 3 and INT32 = 5 as found in the reference's example graphs). */
enum
{
    TMI_INT8  = 3,
    TMI_INT16 = 4,
    TMI_INT32 = 5,
    TMI_INT48 = 6, /* one int64 per element, as the reference stores it: RESCALE input, and the bias, accumulator and
                      output of the INT16 convolutions and MATMUL */
    TMI_FP32  = 7,
    TMI_FP16  = 8,
    TMI_BF16  = 9
};

/* RescaleAttribute.rounding_mode as serialized (reference_model/src/ops/type_conversion.cpp:118-120) */
enum
{
    TMI_ROUND_SINGLE  = 1,
    TMI_ROUND_INEXACT = 2,
    TMI_ROUND_DOUBLE  = 3
};

/* Bits of the device flag word reported by tmi_ctx_flags(): which REQUIRE condition fired. */
enum
{
    TMI_FLAG_SCALE_MULTIPLIER = 1u << 0, /* multiplier < 0                      quant_util.h:48-52  */
    TMI_FLAG_SCALE_SHIFT      = 1u << 1, /* shift outside [2,62]                quant_util.h:53-58  */
    TMI_FLAG_SCALE_VALUE      = 1u << 2, /* value outside [-2^(s-1), 2^(s-1))   quant_util.h:59-67  */
    TMI_FLAG_SCALE_RESULT     = 1u << 3, /* scaled result exceeds int32         quant_util.h:78-82  */
    TMI_FLAG_ZP_RESULT        = 1u << 4, /* result + output_zp exceeds int32    type_conversion.cpp:352-360 */
    TMI_FLAG_LEVEL            = 1u << 5  /* a LEVEL_CHECK of the configured level failed (found on the host)  */
};

/* tosa_level_t of the reference (reference_model/include/func_config.h:23-36); all zero = no level
 * (func_config_t::NONE), { 6, 8192, 8192, 256, 64 } = EIGHTK (:65). */
typedef struct
{
    int32_t max_rank, max_kernel, max_stride, max_scale, max_tensor_list_size;
} tmi_level_t;

typedef struct tmi_ctx tmi_ctx_t;

/* ---- context -------------------------------------------------------------------------------------- */

/* Creates a context on HIP device `device` with its own stream.  Replaces nothing in the reference
 * (which has no device); plays the role of SubgraphTraverser as owner of per-graph state
 * (reference_model/src/subgraph_traverser.cpp:56-80). */
int tmi_ctx_create(tmi_ctx_t** out_ctx, int device);
int tmi_ctx_destroy(tmi_ctx_t* ctx);

/* Makes the context enqueue on a stream owned by the caller (a hipStream_t passed as void*; NULL selects
 * the device's default stream).  The context never destroys a borrowed stream. */
int tmi_ctx_set_stream(tmi_ctx_t* ctx, void* hip_stream);

/* Waits for all enqueued work.  Returns TMI_UNPREDICTABLE if a device-side REQUIRE condition was latched
 * since the last sync (and clears the latch), TMI_ERROR on a HIP failure, else TMI_VALID.
 * Counterpart of reading SubgraphTraverser::getGraphStatus() after evaluateAll()
 * (reference_model/src/model_runner_impl.cpp:56-126). */
int tmi_ctx_sync(tmi_ctx_t* ctx);

/* g_func_config.tosa_level (--tosa_level, reference_model/src/command_line_utils.h:62).  With a level set, every
 * operator call evaluates the reference's LEVEL_CHECKs for it (e.g. reference_model/src/ops/tensor_ops.cpp:761-771 for
 * CONV2D: dilation * kernel and pads against MAX_KERNEL, strides against MAX_STRIDE; RESCALE: rank against MAX_RANK).
 * As in the reference (include/func_debug.h:132-141) a violated limit does not stop evaluation: the operator runs,
 * TMI_FLAG_LEVEL is latched, the next tmi_ctx_sync() returns TMI_UNPREDICTABLE and tmi_last_error() names the limit.
 * NULL or an all-zero level switches the checks off.  tmi_clamp takes no rank, so CLAMP's rank check
 * (activation_funcs.cpp:32) stays with the caller. */
int tmi_ctx_set_level(tmi_ctx_t* ctx, const tmi_level_t* level);

/* g_func_config.precise_mode / compliance_mode / bounds_mode as far as RESCALE reads them
 * (reference_model/src/ops/type_conversion.cpp:318-346): with precise_mode an INEXACT_ROUND RESCALE computes the scaled
 * value in FP64 and truncates it; with compliance_mode as well it first moves the value to the edge of the error bound
 * the specification grants an FP32 implementation, ceil(x - bound) in the normal pass and floor(x + bound) in the
 * bounds pass.  All zero (the default): FP32 maths, rounded to nearest.  The floating-point operators take their
 * precise and bounds passes through the tmi_*_precise entry points and do not read this setting. */
int tmi_ctx_set_precise_mode(tmi_ctx_t* ctx, int32_t precise_mode, int32_t compliance_mode, int32_t bounds_mode);

/* Flag bits (TMI_FLAG_*) seen by the most recent tmi_ctx_sync(). */
uint32_t tmi_ctx_flags(const tmi_ctx_t* ctx);

/* Message of the most recent TMI_ERROR on this context ("" if none).  The reference prints these with
 * printNodeValidationError / ERROR_IF (reference_model/include/func_debug.h:143-158). */
const char* tmi_last_error(const tmi_ctx_t* ctx);

/* Name of the kernel variant chosen by the most recent operator call (for tests and profiling). */
const char* tmi_last_kernel(const tmi_ctx_t* ctx);

/* Grows the context's scratch buffer (the re-laid-out operands of TRANSPOSE_CONV2D / CONV3D layers that are not
 * read in place, MATMUL's transposed second operand) to at least `bytes`.  Lifetime rule of that buffer: an operator
 * call that needs more than the buffer holds allocates a larger block and keeps the old one until
 * tmi_ctx_destroy(), so launches already enqueued and HIP graphs captured earlier stay valid; while the context's
 * stream is being captured such a call returns TMI_ERROR instead of allocating -- size the buffer beforehand with
 * this function or with one eager call of the same operator.  Has no counterpart in the reference. */
int tmi_ctx_reserve_workspace(tmi_ctx_t* ctx, size_t bytes);

/* Size of the scratch buffer in use (`live`) and of the outgrown blocks still held (`retired`); either pointer may be
 * NULL.  An operator call that outgrows the buffer at least doubles it, so `retired` stays below `live` unless
 * tmi_ctx_reserve_workspace() was called with sizes of the caller's own choosing.  Has no counterpart in the reference. */
int tmi_ctx_workspace_bytes(const tmi_ctx_t* ctx, size_t* live, size_t* retired);

/* Frees the outgrown blocks after waiting for the context's stream.  Only for callers that hold no captured HIP graph
 * from before the last growth: such a graph may still name a block freed here.  Has no counterpart in the reference. */
int tmi_ctx_trim_workspace(tmi_ctx_t* ctx);

/* ---- device memory (replaces Tensor::allocate / deallocate and the element-wise host copies of
 *      reference_model/src/tensor.cpp:993-1015, 4722-4736) -------------------------------------------- */
int tmi_buf_alloc(tmi_ctx_t* ctx, size_t bytes, void** out_dev);
int tmi_buf_free(tmi_ctx_t* ctx, void* dev);
int tmi_upload(tmi_ctx_t* ctx, void* dst_dev, const void* src_host, size_t bytes);   /* synchronous */
int tmi_download(tmi_ctx_t* ctx, void* dst_host, const void* src_dev, size_t bytes); /* synchronous */

/* ---- operator descriptors ----------------------------------------------------------------------- */

/* Shapes and Conv2dAttribute / DepthwiseConv2dAttribute fields as read at the top of
 * OpConv2d::eval / OpDepthwiseConv2d::eval (reference_model/src/ops/tensor_ops.cpp:725-758, 1174-1207). */
typedef struct
{
    int32_t in_dtype;    /* TMI_INT8, TMI_FP16, TMI_BF16 or TMI_FP32 (weight has the same type)     */
    int32_t out_dtype;   /* TMI_INT32 for INT8 input; the input type otherwise                       */
    int32_t N, IH, IW, IC;
    int32_t OC;          /* CONV2D: weight dim 0.  DEPTHWISE: IC * M (output channels)               */
    int32_t KH, KW;
    int32_t OH, OW;      /* declared output shape; checked against the reference's shape rule        */
    int32_t pad[4];      /* top, bottom, left, right */
    int32_t stride[2];   /* y, x */
    int32_t dilation[2]; /* y, x */
    int32_t bias_len;    /* 1 (broadcast) or OC */
    int32_t acc_dtype;   /* the attribute's acc_type: TMI_INT32 for INT8 operands, TMI_INT48 for INT16 operands,
                            TMI_FP32 for floating point; 0 (a descriptor zeroed by a caller that predates the field)
                            means that default.  The reference
                            also instantiates FP16 accumulation of FP16 operands (op_factory.h:97-118), which is not
                            built: TMI_ERROR */
} tmi_conv_desc_t;

/* TransposeConv2dAttribute plus operand shapes (reference_model/src/ops/tensor_ops.cpp:1982-2056).
 * input NHWC, weight OHWI, output [N,OH,OW,OC] with OH = (IH-1)*stride_y + out_pad_top + out_pad_bottom + KH. */
typedef struct
{
    int32_t in_dtype;    /* TMI_INT8 / TMI_FP16 / TMI_BF16 */
    int32_t out_dtype;   /* TMI_INT32 for INT8, else the input type */
    int32_t N, IH, IW, IC;
    int32_t OC, KH, KW;
    int32_t OH, OW;
    int32_t out_pad[4];  /* top, bottom, left, right; each > -kernel size */
    int32_t stride[2];   /* y, x */
    int32_t bias_len;    /* 1 (broadcast) or OC */
    int32_t acc_dtype;   /* as in tmi_conv_desc_t */
} tmi_tconv_desc_t;

/* Conv3dAttribute plus operand shapes (reference_model/src/ops/tensor_ops.cpp:901-933, check :120-226).
 * input [N,ID,IH,IW,IC], weight [OC,KD,KH,KW,IC], output [N,OD,OH,OW,OC]. */
typedef struct
{
    int32_t in_dtype, out_dtype;
    int32_t N, ID, IH, IW, IC;
    int32_t OC, KD, KH, KW;
    int32_t OD, OH, OW;
    int32_t pad[6];      /* d0, d1, top, bottom, left, right */
    int32_t stride[3];   /* d, y, x */
    int32_t dilation[3]; /* d, y, x */
    int32_t bias_len;
    int32_t acc_dtype;   /* as in tmi_conv_desc_t */
} tmi_conv3d_desc_t;

/* AvgPool2dAttribute / MaxPool2dAttribute plus operand shapes (reference_model/src/ops/tensor_ops.cpp:29-117
 * check_pool2d_attribute, :472-537, :1508-1543).  input [N,IH,IW,C], output [N,OH,OW,C] of the same type. */
typedef struct
{
    int32_t dtype;       /* TMI_INT8 / TMI_INT16 / TMI_FP16 / TMI_BF16 / TMI_FP32 */
    int32_t acc_dtype;   /* AVG_POOL2D: TMI_INT32 for integers, TMI_FP32 for floating point; ignored by MAX_POOL2D */
    int32_t N, IH, IW, C;
    int32_t OH, OW;
    int32_t kernel[2];   /* y, x */
    int32_t stride[2];   /* y, x */
    int32_t pad[4];      /* top, bottom, left, right; each < kernel size */
    int32_t nan_mode;    /* MAX_POOL2D on floating point: 1 = PROPAGATE, 2 = IGNORE */
} tmi_pool_desc_t;

/* RescaleAttribute plus the operand facts OpRescale::checkTensorAttributes / eval read
 * (reference_model/src/ops/type_conversion.cpp:111-151, 226-255). */
typedef struct
{
    int32_t in_dtype;        /* TMI_INT8 / TMI_INT16 / TMI_INT32 (bit pattern width; signedness below) */
    int32_t out_dtype;       /* TMI_INT8 / TMI_INT16 / TMI_INT32 */
    int32_t scale32;         /* 1: multiplier tensor is INT32; 0: INT16 */
    int32_t rounding_mode;   /* TMI_ROUND_* */
    int32_t per_channel;
    int32_t input_unsigned;
    int32_t output_unsigned;
    int32_t in_zp;           /* stored value of the input_zp tensor  (sign-interpreted, as the reference holds it) */
    int32_t out_zp;          /* stored value of the output_zp tensor */
    int32_t n_multiplier;    /* element count of the multiplier tensor */
    int32_t n_shift;         /* element count of the shift tensor      */
} tmi_rescale_desc_t;

/* ---- operators --------------------------------------------------------------------------------- */

/* OpConv2d<In,W,Acc,Out>::eval, reference_model/src/ops/tensor_ops.cpp:723-882 (checks :120-226, :690-720).
 * INT8 x INT8 -> INT32 with int32 accumulation, or FP16 / BF16 / FP32 with fp32 accumulation and an output
 * of the input type (the instantiations at :2220-2229; FP32 runs on the one-element-per-lane kernels, in the
 * reference's summation order).  INT16 x INT8 -> INT48 (:2225; d->in_dtype TMI_INT16, weights INT8, bias and
 * output one int64 per element, the sum kept in 64 bits and REQUIREd to lie within 48 bits, :875-879) runs on a
 * one-element-per-lane kernel.  INT8 x INT4 -> INT32 (:2224) is the INT8 call with the weights handed over as one
 * int8 value of -8 ... 7 per element and w_zp = 0, which the caller checks (the library cannot tell such weights from INT8
 * ones).  in_zp / w_zp are the values of operands 3 and 4: in_zp must be 0 unless the input is INT8, w_zp unless the
 * weights are (:804-811). */
int tmi_conv2d(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev, const void* weight_dev,
               const void* bias_dev, int32_t in_zp, int32_t w_zp, void* out_dev);

/* OpDepthwiseConv2d::eval, reference_model/src/ops/tensor_ops.cpp:1172-1334.  M = d->OC / d->IC.  The same
 * element types as tmi_conv2d (the instantiations at :2242-2251; INT16 x INT8 -> INT48 at :2247, clip :1325-1329). */
int tmi_depthwise_conv2d(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev, const void* weight_dev,
                         const void* bias_dev, int32_t in_zp, int32_t w_zp, void* out_dev);

/* OpMatMul::eval, reference_model/src/ops/tensor_ops.cpp:1423-1492 (checks :1347-1420).
 * in_dtype TMI_INT8 -> INT32 output; TMI_INT16 -> INT48 output (one int64 per element, zero points must be 0,
 * the 48-bit REQUIRE of :1485-1489; the instantiation at :2257); TMI_FP16 / TMI_BF16 / TMI_FP32 -> FP32 output
 * (fp32 accumulation). */
int tmi_matmul(tmi_ctx_t* ctx, int32_t in_dtype, int32_t N, int32_t H, int32_t C, int32_t W, const void* a_dev,
               const void* b_dev, int32_t a_zp, int32_t b_zp, void* out_dev);

/* OpRescale::eval, reference_model/src/ops/type_conversion.cpp:224-421, on a tensor of `rank` dimensions
 * viewed as [rows, C] (C = last dimension, or 1 for rank 0).  multiplier_dev holds INT32 (scale32) or
 * INT16 values, shift_dev INT8 values.  Input INT8 / INT16 / INT32 / INT48 (the instantiations at :874-903;
 * INT48 needs scale32 = 0, :122), output INT8 / INT16 / INT32. */
int tmi_rescale(tmi_ctx_t* ctx, const tmi_rescale_desc_t* r, int32_t rank, int64_t rows, int32_t C,
                const void* in_dev, const void* multiplier_dev, const void* shift_dev, void* out_dev);

/* OpClamp::eval for INT8 / INT16 (reference_model/src/ops/activation_funcs.cpp:27-125 with applyClip,
 * reference_model/src/arith_util.h:389-413).  TMI_ERROR when max_val < min_val. */
int tmi_clamp(tmi_ctx_t* ctx, int32_t dtype, int64_t n, const void* in_dev, int32_t min_val, int32_t max_val,
              void* out_dev);

/* OpClamp::eval for FP16 / BF16 / FP32 (reference_model/src/ops/activation_funcs.cpp:97-106): applyClip with the
 * attribute's nan_mode (1 = PROPAGATE, 2 = IGNORE; reference_model/src/arith_util.h:341-413), then the rounding to the
 * stored type.  TMI_ERROR when max_val < min_val or either is NaN. */
int tmi_clamp_fp(tmi_ctx_t* ctx, int32_t dtype, int64_t n, const void* in_dev, float min_val, float max_val,
                 int32_t nan_mode, void* out_dev);

/* CONV2D -> RESCALE (-> CLAMP) evaluated as one kernel: the int32 convolution result never reaches HBM.
 * Same results as tmi_conv2d + tmi_rescale (+ tmi_clamp) on the same operands.  The rescale input is the
 * INT32 convolution output (r->in_dtype must be TMI_INT32, r->in_zp 0); per-channel constants have OC
 * entries.  has_clamp = 0 skips the clamp. */
int tmi_conv2d_rescale_clamp(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev, const void* weight_dev,
                             const void* bias_dev, int32_t in_zp, int32_t w_zp, const tmi_rescale_desc_t* r,
                             const void* multiplier_dev, const void* shift_dev, int32_t has_clamp,
                             int32_t clamp_min, int32_t clamp_max, void* out_dev);

/* DEPTHWISE_CONV2D -> RESCALE (-> CLAMP) as one kernel; see tmi_conv2d_rescale_clamp. */
int tmi_depthwise_conv2d_rescale_clamp(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev,
                                       const void* weight_dev, const void* bias_dev, int32_t in_zp, int32_t w_zp,
                                       const tmi_rescale_desc_t* r, const void* multiplier_dev,
                                       const void* shift_dev, int32_t has_clamp, int32_t clamp_min,
                                       int32_t clamp_max, void* out_dev);

/* OpTransposeConv2d<In,W,Acc,Out>::eval, reference_model/src/ops/tensor_ops.cpp:2058-2197 (checks :1982-2056).
 * Evaluated as a stride-1 CONV2D with flipped taps over the input with stride-1 holes filled with input_zp.
 * INT8 with 3x3 taps, 64 / 96 / 128 input channels and w_zp 0 reads both operands in place (holes and flip are
 * part of the kernel's addressing); otherwise the re-laid-out operands live in the context's scratch buffer.
 * Element types as tmi_conv2d: INT8 -> INT32, FP16 / BF16 / FP32 (FP32 on the one-element-per-lane kernel, the sum in
 * the order of the equivalent CONV2D, not the reference's scatter order), INT16 x INT8 -> INT48 (:2291; clip :2190-2194). */
int tmi_transpose_conv2d(tmi_ctx_t* ctx, const tmi_tconv_desc_t* d, const void* in_dev, const void* weight_dev,
                         const void* bias_dev, int32_t in_zp, int32_t w_zp, void* out_dev);

/* Size of the scratch array behind tmi_transpose_conv2d_noalloc: 16 MiB of device memory per GPU the library is
 * used on, part of the library's device image and held until the process ends. */
#define TMI_NOALLOC_SCRATCH_BYTES (16u << 20)

/* tmi_transpose_conv2d for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same operands, results and
 * status as tmi_transpose_conv2d, but the re-laid-out operands (flipped weights: OC*KH*KW*IC elements; the input
 * with its stride holes: N*((IH-1)*sy+1)*((IW-1)*sx+1)*IC elements, each rounded up to 256 bytes) go to a static
 * device array of TMI_NOALLOC_SCRATCH_BYTES instead of the context's growable buffer: the call performs no
 * hipMalloc / hipFree and returns TMI_ERROR, launching nothing, when the operands need more than that.  All
 * contexts on one GPU share that GPU's array: calls that overlap in time on one GPU (different streams or
 * contexts) race; calls on one stream are ordered and each call rewrites every byte it later reads. */
int tmi_transpose_conv2d_noalloc(tmi_ctx_t* ctx, const tmi_tconv_desc_t* d, const void* in_dev, const void* weight_dev,
                                 const void* bias_dev, int32_t in_zp, int32_t w_zp, void* out_dev);

/* OpConv3d<In,W,Acc,Out>::eval, reference_model/src/ops/tensor_ops.cpp:935-1120 (checks :901-933, :120-226).
 * Evaluated as a CONV2D over N*OD images whose channels are the KD depth taps side by side.  INT8 with 3x3 taps in
 * the plane, KD*IC = 64 / 96 / 128 (IC 32 or 64) and w_zp 0 reads both operands in place; otherwise the gathered
 * input and the permuted weights live in the context's scratch buffer.  Element types as tmi_conv2d: INT8 -> INT32,
 * FP16 / BF16 / FP32 (FP32 on the one-element-per-lane kernel, the depth taps innermost in the sum), and INT16 x INT8 ->
 * INT48 (:2237; clip :1113-1117). */
int tmi_conv3d(tmi_ctx_t* ctx, const tmi_conv3d_desc_t* d, const void* in_dev, const void* weight_dev,
               const void* bias_dev, int32_t in_zp, int32_t w_zp, void* out_dev);

/* OpAvgPool2d<Dtype,AccDtype>::eval, reference_model/src/ops/tensor_ops.cpp:542-660: the sum over the taps
 * inside the image, divided by their number (integers: reciprocal_scale + apply_scale_32 with a single rounding,
 * quant_util.h:32-84, then output_zp and the clip to the type).  Zero points must be 0 unless dtype is INT8. */
int tmi_avg_pool2d(tmi_ctx_t* ctx, const tmi_pool_desc_t* d, const void* in_dev, int32_t in_zp, int32_t out_zp,
                   void* out_dev);

/* OpMaxPool2d<Dtype>::eval, reference_model/src/ops/tensor_ops.cpp:1546-1640 (applyMax with the attribute's NaN
 * mode, reference_model/src/arith_util.h:341-373). */
int tmi_max_pool2d(tmi_ctx_t* ctx, const tmi_pool_desc_t* d, const void* in_dev, void* out_dev);

/* ---- floating-point compliance passes -------------------------------------------------------------- */

/* The reference evaluates a floating-point graph twice more to judge an implementation: in precise mode
 * (--precise_mode: all floating-point tensors in fp64, reference_model/src/main.cpp and the FP64 instantiations
 * of op_factory.cpp) and in bounds mode (the same sums over absolute values, tensor_ops.cpp:757-765,
 * 1213-1221, 1436-1443).  These entries compute either pass on the device: operands in their storage type
 * (TMI_FP16 / TMI_BF16 / TMI_FP32), fp64 products and sums in the reference's loop order, fp64 output of the operator's
 * output shape.  bounds_mode != 0 selects the sums of absolute values.  local_bound is the operator's attribute of
 * that name (Conv2dAttribute / DepthwiseConv2dAttribute): when it is 0, the bounds pass replaces every input element
 * by the largest magnitude of the whole input tensor (reference_model/src/ops/tensor_ops.cpp:797-801, 1252-1256), which
 * is the flatbuffer default; it has no effect on the precise pass.  MATMUL has no such attribute
 * (tensor_ops.cpp:1436-1441 takes absolute values only). */
int tmi_conv2d_precise(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev, const void* weight_dev,
                       const void* bias_dev, int32_t bounds_mode, int32_t local_bound, double* out_dev);
int tmi_depthwise_conv2d_precise(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, const void* in_dev,
                                 const void* weight_dev, const void* bias_dev, int32_t bounds_mode, int32_t local_bound,
                                 double* out_dev);
int tmi_matmul_precise(tmi_ctx_t* ctx, int32_t in_dtype, int32_t N, int32_t H, int32_t C, int32_t W,
                       const void* a_dev, const void* b_dev, int32_t bounds_mode, double* out_dev);

/* What validateDataDP reports (reference_model/src/verify/verify_dot_product.cpp:89-139). */
typedef struct
{
    double err_sum;          /* sum over the elements of (imp - ref) / max(bnd * 2^-(1+frac), normal_min) */
    double err_sumsq;        /* sum of their squares */
    double max_abs_err;      /* largest magnitude among them */
    int64_t failed_elements; /* elements outside abs_bound, or breaking the zero-bound / NaN rules */
    int64_t elements;
    int32_t abs_bound;       /* 2 * ksb */
    double variance_bound;   /* 1.6 * ksb */
    int32_t compliant;       /* 1 when every rule of validateDataDP holds */
} tmi_dp_result_t;

/* The DOT_PRODUCT compliance check (verify_dot_product.cpp:30-139) of n device-resident results imp_dev of
 * type out_dtype (TMI_FP16 / TMI_BF16 / TMI_FP32) against the precise-mode results ref_dev and the bounds-mode
 * results bnd_dev.  ksb is the kernel size bound, set_number the test data set (the error-sum rule applies to
 * sets 3..5; pass -1 for data that is not one of the sets).  Synchronises the context's stream.  Returns
 * TMI_VALID with result->compliant 0 or 1; TMI_ERROR only for bad arguments. */
int tmi_dot_product_check(tmi_ctx_t* ctx, int32_t out_dtype, int64_t n, const void* imp_dev, const double* ref_dev,
                          const double* bnd_dev, int32_t ksb, int32_t set_number, tmi_dp_result_t* result);

/* ---- validation only (no launch) ---------------------------------------------------------------- */

/* The checks OpConv2d / OpDepthwiseConv2d::checkTensorAttributes and the head of eval() perform
 * (reference_model/src/ops/tensor_ops.cpp:120-226, 690-720, 742-748, 1139-1169, 1191-1197): attribute sizes
 * and signs, the output-shape rule, channel and bias consistency, supported type combination.  Called from an
 * adapter's checkTensorAttributes() so that SubgraphTraverser::validateGraph() rejects a malformed node before
 * anything is evaluated.  depthwise != 0 selects the DEPTHWISE_CONV2D rules. */
int tmi_conv2d_check(tmi_ctx_t* ctx, const tmi_conv_desc_t* d, int32_t depthwise);

/* The checks of OpTransposeConv2d / OpConv3d::checkTensorAttributes and the heads of their eval()
 * (reference_model/src/ops/tensor_ops.cpp:1982-2056, 2083-2091; 901-933, 963-970), for an adapter's
 * checkTensorAttributes(). */
int tmi_transpose_conv2d_check(tmi_ctx_t* ctx, const tmi_tconv_desc_t* d);
int tmi_conv3d_check(tmi_ctx_t* ctx, const tmi_conv3d_desc_t* d);

/* check_pool2d_attribute and the type rules of OpAvgPool2d / OpMaxPool2d::checkTensorAttributes
 * (reference_model/src/ops/tensor_ops.cpp:29-117, 484-537, 1514-1543); avg != 0 selects AVG_POOL2D. */
int tmi_pool2d_check(tmi_ctx_t* ctx, const tmi_pool_desc_t* d, int32_t avg);

/* OpRescale::checkTensorAttributes and the zero-point rules at the head of eval()
 * (reference_model/src/ops/type_conversion.cpp:72-154, 242-255). */
int tmi_rescale_check(tmi_ctx_t* ctx, const tmi_rescale_desc_t* r, int32_t rank, int32_t C);

/* ---- tuning / test hooks ------------------------------------------------------------------------- */

/* Forces a kernel family for the following operator calls: 0 = automatic choice, 1 = direct (one output
 * element per lane, any shape), 2 = MFMA implicit-GEMM ("patch") kernel, 3 = MFMA GEMM kernel with direct
 * loads into LDS (CONV2D and MATMUL), 4 = the kernels that hold a weight slab and an input patch in LDS (CONV2D 3x3 / 1x1
 * on channel vectors of 64 ... 128 bytes, 1x1 on up to 1024 bytes, int8 / fp16 / bf16; int8 DEPTHWISE_CONV2D 3x3),
 * 5 = the int8 kernels that take both operands straight from global memory (CONV2D 1x1 with 16 ... 2048 input
 * channels; small deep layers with taps; first layers with at most 4 channels), 6 = the int8 DEPTHWISE_CONV2D 3x3
 * kernel whose waves load the pixel operand of the matrix instruction straight from global memory;
 * 2, 3, 4, 5 and 6 return TMI_ERROR if the shape is not eligible.  Used by the parity tests to check every kernel on the
 * same operands. */
int tmi_ctx_set_kernel_choice(tmi_ctx_t* ctx, int32_t choice);

/* Launches a kernel that does nothing - grid workgroups of block threads with lds_bytes of dynamic LDS - on
 * the context's stream: what one launch of that shape costs before any work.  No counterpart in the
 * reference; used by the benchmark's launch-floor configuration. */
int tmi_debug_launch_empty(tmi_ctx_t* ctx, int32_t grid, int32_t block, int32_t lds_bytes);

/* Streams `bytes` bytes (a positive multiple of 16, buffers 16-byte aligned) on the context's stream: mode 0
 * copies src to dst, mode 1 only reads src (dst receives nothing unless every word read is 0xFFFFFFFF; it must
 * still be a valid 16-byte buffer), mode 2 only writes dst, mode 3 reads src with loads that go straight into LDS.  What the memory system sustains, to quote kernel
 * rates against.  No counterpart in the reference. */
int tmi_debug_stream(tmi_ctx_t* ctx, int32_t mode, const void* src_dev, void* dst_dev, int64_t bytes);

/* Grid (workgroups), block (threads) and dynamic LDS bytes of the calling thread's latest launch of the CONV2D
 * kernel that keeps a layer's operands in LDS; zeros before the first.  Feeds tmi_debug_launch_empty. */
void tmi_debug_last_launch_shape(int32_t* out3);

/* Host arithmetic only, no GPU call.  The tiled kernels split a block index into (channel block, tile column,
 * tile row, image) with multiply-high divisions that are exact while dividend * divisor < 2^32; a launcher
 * whose layer is outside that leaves the layer to another kernel.  Returns 1 if a grid of `grid` blocks with
 * these divisors passes that guard, else 0, and writes the decode of `block` by the same arithmetic to out4
 * (if not NULL).  Used by the unit tests of the guard. */
int tmi_debug_tile_decode(int64_t grid, uint32_t n_ocb, uint32_t tiles_x, uint32_t tiles_y, uint32_t block,
                          int32_t* out4);

/* Library build identification, e.g. "tosa_mi355 gfx950". */
const char* tmi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* TOSA_MI355_H */
