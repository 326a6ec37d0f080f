/*
 * CPU oracle for the TOSA tensor-op hot path (CONV2D, DEPTHWISE_CONV2D, MATMUL, RESCALE, CLAMP) and its
 * neighbours CONV3D, TRANSPOSE_CONV2D, AVG_POOL2D and MAX_POOL2D.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the arithmetic of the TOSA reference
 * model, used as the checker in the parity tests, in the smoke test and as the timed CPU baseline.
 * Nothing in the shipped library may call, link or load it.
 *
 * Every function works on flat row-major buffers.  Status codes follow the reference's GraphStatus
 * (reference_model/include/graph_status.h:18-23): 0 = valid, 1 = unpredictable, 2 = error.
 *
 * Parity pins (see tests/test_oracle_*.py):
 *   - conv2d int8 + rescale double-round per-channel: the reference's stored golden of
 *     examples/test_conv2d_1x1_1x32x32x8_qi8_st11_padSAME_dilat11 (bit exact).
 *   - conv2d / depthwise / matmul zero points and bias broadcast: the literal vectors of
 *     reference_model/test/ref_model_tests/tensor_ops_tests.cpp:622-683,736-798.
 *   - rescale: type_conversion_tests.cpp:324-405 literals, Python big-integer brute force of
 *     quant_util.h:45-84 and the boundary operands of generate_int_special.cpp:119-131.
 *   - conv3d / transpose_conv2d: the literal vectors of tensor_ops_tests.cpp:268-446,622-766 (zero points,
 *     bias broadcast) and an independent numpy restatement (correlation of the zero-upsampled input with the
 *     flipped kernel for TRANSPOSE_CONV2D; per-depth-tap sums of 2-D convolutions for CONV3D).
 *   - avg_pool2d / max_pool2d: the two literal cases of tensor_ops_tests.cpp:508-575,800-823 (zero point
 *     subtracted in full precision), reciprocal_scale against exact rational arithmetic for every count up to
 *     4096 (multiplier = floor(((2^30+1) << k) / count)), and an independent numpy restatement over padded
 *     windows for general shapes.  Floating-point AVG_POOL2D sums in tap order in fp32 like the reference's
 *     loop nest (tensor_ops.cpp:613-634), so it is compared bit for bit.
 *   - DOT_PRODUCT data sets S0..S5: the generator's own goldens, reference_model/test/generate_tests.cpp:315-372
 *     (MATMUL fp32, first three values of both operands, all six sets), :444-535 (CONV2D fp32, last three values
 *     of input / weight / bias, all six sets) and :1194-1222 (DEPTHWISE_CONV2D fp16, sets 0 and 1), bit for bit.
 *   - large shapes: independent numpy int64 einsum / float64 convolution.
 *   - fp accumulate order of MATMUL (Eigen contraction order): parity unpinned (tolerance covered).
 */
#ifndef TOSA_ORACLE_H
#define TOSA_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum
{
    ORC_VALID         = 0,
    ORC_UNPREDICTABLE = 1,
    ORC_ERROR         = 2
};

/* rounding_mode values as serialized in RescaleAttribute */
enum
{
    ORC_ROUND_SINGLE  = 1,
    ORC_ROUND_INEXACT = 2,
    ORC_ROUND_DOUBLE  = 3
};

typedef struct
{
    int32_t N, IH, IW, IC; /* input  NHWC */
    int32_t OC, KH, KW;    /* weight OHWI (conv2d) ; depthwise: KH,KW,IC,M with OC = IC*M */
    int32_t OH, OW;        /* declared output height/width */
    int32_t pad[4];        /* top, bottom, left, right */
    int32_t stride[2];     /* y, x */
    int32_t dilation[2];   /* y, x */
    int32_t bias_len;      /* 1 (broadcast) or OC */
} orc_conv_shape_t;

/* check_conv_attribute + the ERROR_IFs at the top of eval().  depthwise_m = 0 for CONV2D, else the
 * channel multiplier M.  Returns ORC_VALID or ORC_ERROR. */
int orc_conv_check(const orc_conv_shape_t* s, int32_t depthwise_m);

/* CONV2D.  Elements are given in the reference's storage type (int32 for INT8, float for FP16/BF16/FP32,
 * double in precise mode); accumulate in the same type as the reference's AccEigenType for that
 * instantiation (int32 wraps; float; double).  abs_mode != 0 selects the bounds pass
 * (|in|, |w|, |bias|, local_bound = true). */
int orc_conv2d_i32(const orc_conv_shape_t* s, const int32_t* in, const int32_t* w, const int32_t* bias,
                   int32_t in_zp, int32_t w_zp, int32_t* out);
int orc_conv2d_f32(const orc_conv_shape_t* s, const float* in, const float* w, const float* bias, float* out);
int orc_conv2d_f64(const orc_conv_shape_t* s, const double* in, const double* w, const double* bias, int abs_mode,
                   double* out);

/* Same arithmetic on packed int8 operands (1 byte per element, as they sit in .npy files and in HBM),
 * widened to the reference's int32 storage inside.  Convenience for tests; identical results. */
int orc_conv2d_i8(const orc_conv_shape_t* s, const int8_t* in, const int8_t* w, const int32_t* bias, int32_t in_zp,
                  int32_t w_zp, int32_t* out);

/* DEPTHWISE_CONV2D, weight [KH,KW,IC,M], out channel = ic*M + m. */
int orc_depthwise_i32(const orc_conv_shape_t* s, int32_t M, const int32_t* in, const int32_t* w,
                      const int32_t* bias, int32_t in_zp, int32_t w_zp, int32_t* out);
/* INT16 x INT8 -> INT48 CONV2D / DEPTHWISE_CONV2D: int64 bias and results, clipped to 48 bits; input_zp must be 0 */
int orc_conv2d_i16(const orc_conv_shape_t* s, const int16_t* in, const int8_t* w, const int64_t* bias, int32_t in_zp,
                   int32_t w_zp, int64_t* out);
int orc_depthwise_i16(const orc_conv_shape_t* s, int32_t M, const int16_t* in, const int8_t* w, const int64_t* bias,
                      int32_t in_zp, int32_t w_zp, int64_t* out);
int orc_depthwise_i8(const orc_conv_shape_t* s, int32_t M, const int8_t* in, const int8_t* w, const int32_t* bias,
                     int32_t in_zp, int32_t w_zp, int32_t* out);
int orc_depthwise_f32(const orc_conv_shape_t* s, int32_t M, const float* in, const float* w, const float* bias,
                      float* out);
int orc_depthwise_f64(const orc_conv_shape_t* s, int32_t M, const double* in, const double* w, const double* bias,
                      int abs_mode, double* out);

/* CONV3D (tensor_ops.cpp:901-1120): input [N,ID,IH,IW,IC], weight [OC,KD,KH,KW,IC], output [N,OD,OH,OW,OC]. */
typedef struct
{
    int32_t N, ID, IH, IW, IC;
    int32_t OC, KD, KH, KW;
    int32_t OD, OH, OW;
    int32_t pad[6];      /* d0, d1, top, bottom, left, right */
    int32_t stride[3];   /* d, y, x */
    int32_t dilation[3]; /* d, y, x */
    int32_t bias_len;
} orc_conv3d_shape_t;
int orc_conv3d_check(const orc_conv3d_shape_t* s);
int orc_conv3d_i32(const orc_conv3d_shape_t* s, const int32_t* in, const int32_t* w, const int32_t* bias,
                   int32_t in_zp, int32_t w_zp, int32_t* out);
int orc_conv3d_i8(const orc_conv3d_shape_t* s, const int8_t* in, const int8_t* w, const int32_t* bias, int32_t in_zp,
                  int32_t w_zp, int32_t* out);
int orc_conv3d_i16(const orc_conv3d_shape_t* s, const int16_t* in, const int8_t* w, const int64_t* bias, int32_t in_zp,
                   int32_t w_zp, int64_t* out);
int orc_conv3d_f32(const orc_conv3d_shape_t* s, const float* in, const float* w, const float* bias, float* out);
int orc_conv3d_f64(const orc_conv3d_shape_t* s, const double* in, const double* w, const double* bias, int abs_mode,
                   double* out);

/* TRANSPOSE_CONV2D (tensor_ops.cpp:1982-2197): input NHWC, weight OHWI, OH = (IH-1)*sy + out_pad_top +
 * out_pad_bottom + KH. */
typedef struct
{
    int32_t N, IH, IW, IC;
    int32_t OC, KH, KW;
    int32_t OH, OW;
    int32_t out_pad[4]; /* top, bottom, left, right; each > -kernel size */
    int32_t stride[2];  /* y, x */
    int32_t bias_len;
} orc_tconv_shape_t;
int orc_tconv_check(const orc_tconv_shape_t* s);
int orc_transpose_conv2d_i32(const orc_tconv_shape_t* s, const int32_t* in, const int32_t* w, const int32_t* bias,
                             int32_t in_zp, int32_t w_zp, int32_t* out);
int orc_transpose_conv2d_i8(const orc_tconv_shape_t* s, const int8_t* in, const int8_t* w, const int32_t* bias,
                            int32_t in_zp, int32_t w_zp, int32_t* out);
int orc_transpose_conv2d_i16(const orc_tconv_shape_t* s, const int16_t* in, const int8_t* w, const int64_t* bias,
                             int32_t in_zp, int32_t w_zp, int64_t* out);
int orc_transpose_conv2d_f32(const orc_tconv_shape_t* s, const float* in, const float* w, const float* bias,
                             float* out);
int orc_transpose_conv2d_f64(const orc_tconv_shape_t* s, const double* in, const double* w, const double* bias,
                             int abs_mode, double* out);

/* MATMUL a[N,H,C] x b[N,C,W] -> out[N,H,W]. */
int orc_matmul_i32(int32_t N, int32_t H, int32_t C, int32_t W, const int32_t* a, const int32_t* b, int32_t a_zp,
                   int32_t b_zp, int32_t* out);
int orc_matmul_i8(int32_t N, int32_t H, int32_t C, int32_t W, const int8_t* a, const int8_t* b, int32_t a_zp,
                  int32_t b_zp, int32_t* out);
/* INT16 x INT16 -> INT48 (int64 results clipped to 48 bits) */
int orc_matmul_i16(int32_t N, int32_t H, int32_t C, int32_t W, const int16_t* a, const int16_t* b, int32_t a_zp,
                   int32_t b_zp, int64_t* out);
int orc_matmul_f32(int32_t N, int32_t H, int32_t C, int32_t W, const float* a, const float* b, float* out);
int orc_matmul_f64(int32_t N, int32_t H, int32_t C, int32_t W, const double* a, const double* b, int abs_mode,
                   double* out);

/* QuantUtil::apply_scale_32 / apply_scale_16.  *status is set to ORC_UNPREDICTABLE where the
 * reference throws (the throw becomes a REQUIRE failure in OpRescale::eval). */
int32_t orc_apply_scale_32(int32_t value, int32_t multiplier, int32_t shift, int double_round, int* status);
int32_t orc_apply_scale_16(int64_t value, int16_t multiplier, int32_t shift, int* status);

typedef struct
{
    int32_t in_bits;  /* 8, 16, 32 or 48: nominal width of the input dtype  */
    int32_t out_bits; /* 8, 16 or 32: nominal width of the output dtype */
    int32_t scale32;
    int32_t rounding_mode;
    int32_t per_channel;
    int32_t input_unsigned;
    int32_t output_unsigned;
    int32_t in_zp;  /* stored value of the input_zp tensor  (storage type int32) */
    int32_t out_zp; /* stored value of the output_zp tensor (storage type int32) */
} orc_rescale_attr_t;

/* RESCALE on a tensor viewed as [rows, C] (C = last dimension, 1 for rank 0).  in/out hold one stored
 * value per element in the reference's int32 storage type.  n_scale = number of multiplier / shift
 * entries supplied.  Returns ORC_ERROR for the attribute/shape violations that the reference rejects,
 * ORC_UNPREDICTABLE when a REQUIRE fires (output contents then unspecified), else ORC_VALID. */
int orc_rescale(const orc_rescale_attr_t* a, int64_t rows, int32_t C, const int32_t* in, const int32_t* multiplier,
                const int32_t* shift, int32_t n_mult, int32_t n_shift, int32_t rank, int32_t* out);
/* How INEXACT_ROUND is evaluated by the calls that follow (g_func_config of the reference, type_conversion.cpp:318-346):
 * 0 FP32 maths (the default); 1 precise mode: FP64 maths, truncated; 2 / 3 precise mode with compliance mode: the FP64
 * value moved to the lower / upper edge of the error bound (normal / bounds pass) before the truncation. */
void orc_set_inexact_mode(int mode);
/* The same for an INT48 input (in_bits = 48), whose storage type is int64 (template_types.h:67-163); a stored
 * value with bit 47 set gets bits 48..63 set (value_extend64_impl, type_conversion.cpp:200-215), which changes
 * nothing for values inside the 48-bit range.  Needs scale32 = 0, hence apply_scale_16 (:122). */
int orc_rescale_i48(const orc_rescale_attr_t* a, int64_t rows, int32_t C, const int64_t* in, const int32_t* multiplier,
                    const int32_t* shift, int32_t n_mult, int32_t n_shift, int32_t rank, int32_t* out);

/* CLAMP for the integer instantiations: min(max(x, lo), hi); ORC_ERROR when hi < lo. */
/* AVG_POOL2D / MAX_POOL2D (reference_model/src/ops/tensor_ops.cpp:29-117 check_pool2d_attribute, :472-660
 * OpAvgPool2d, :1508-1640 OpMaxPool2d).  Input and output NHWC with the same N and C. */
typedef struct
{
    int32_t N, IH, IW, C;
    int32_t OH, OW;
    int32_t kernel[2]; /* y, x */
    int32_t stride[2]; /* y, x */
    int32_t pad[4];    /* top, bottom, left, right */
} orc_pool_shape_t;
int orc_pool_check(const orc_pool_shape_t* s);
/* QuantUtil::reciprocal_scale (reference_model/src/quant_util.h:32-43) */
void orc_reciprocal_scale(int32_t count, int32_t* multiplier, int32_t* shift);
/* integer AVG_POOL2D: values widened to int32 by the caller, qmin/qmax = limits of the in/out type */
int orc_avg_pool2d_i32(const orc_pool_shape_t* s, const int32_t* in, int32_t in_zp, int32_t out_zp, int32_t qmin,
                       int32_t qmax, int32_t* out);
/* floating-point AVG_POOL2D with an fp32 accumulator; the caller narrows the result to the output type */
int orc_avg_pool2d_f32(const orc_pool_shape_t* s, const float* in, float* out);
int orc_max_pool2d_i32(const orc_pool_shape_t* s, const int32_t* in, int32_t lowest, int32_t* out);
/* nan_mode: 1 = PROPAGATE, 2 = IGNORE */
int orc_max_pool2d_f32(const orc_pool_shape_t* s, const float* in, int nan_mode, float* out);

/* DOT_PRODUCT test data sets S0..S5 of the TOSA specification (tosa_mi_data), as the reference's data generator
 * produces them (reference_model/src/generate/generate_dot_product_states.cpp:39-300 generators and bound
 * parameter B, generate_dot_product.cpp:23-50 MATMUL, :113-196 CONV2D, :455-538 DEPTHWISE_CONV2D index maps).
 * op: 0 MATMUL, 1 CONV2D, 2 DEPTHWISE_CONV2D; param: operand position (0 input / A, 1 weight / B, 2 bias);
 * shape: the operand's shape; kernel: {KH, KW}, read for the input operand of the convolutions.
 * Values are produced in fp32; the caller narrows them to the operand's type. */
enum
{
    ORC_DP_MATMUL    = 0,
    ORC_DP_CONV2D    = 1,
    ORC_DP_DEPTHWISE = 2
};
/* bound parameter B for (data type bits 16 = fp16, 17 = bf16, 32 = fp32; accumulator fp32 unless acc16) */
float orc_dp_bound_parameter(int data_kind, int acc16);
int orc_dp_generate(int op, int set, int param, uint32_t ks, float B, const int32_t* shape, int rank,
                    const int32_t* kernel, float* out);

int orc_threads(void);
int orc_clamp_i32(int64_t n, const int32_t* in, int32_t lo, int32_t hi, int32_t* out);
/* CLAMP for float storage; nan_mode 1 = PROPAGATE, 2 = IGNORE. */
int orc_clamp_f32(int64_t n, const float* in, float lo, float hi, int nan_mode, float* out);

#ifdef __cplusplus
}
#endif
#endif
