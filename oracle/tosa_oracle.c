/*
 * CPU oracle for the TOSA tensor-op hot path.  TEST INFRASTRUCTURE ONLY: the checker for the parity
 * tests and the timed CPU baseline; never linked into, loaded by or called from the shipped library.
 *
 * Each function restates one piece of the TOSA reference model on flat row-major buffers, keeping
 * the reference's loop nest, its storage types (int32 per INT8 element, float per FP16/BF16
 * element, double in precise mode) and its accumulator types.  Build with -fno-strict-overflow /
 * -fwrapv: the reference is built with -fno-strict-overflow and its int32 accumulators wrap.
 */
#include "tosa_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------------
 * check_conv_attribute (reference_model/src/ops/tensor_ops.cpp:120-226) and the ERROR_IFs that
 * open OpConv2d::eval / OpDepthwiseConv2d::eval (tensor_ops.cpp:742-748, 1191-1197).
 * ---------------------------------------------------------------------------------------------- */
int orc_conv_check(const orc_conv_shape_t* s, int32_t depthwise_m)
{
    for (int i = 0; i < 4; i++)
        if (s->pad[i] < 0)
            return ORC_ERROR;
    for (int i = 0; i < 2; i++)
        if (s->stride[i] < 1 || s->dilation[i] < 1)
            return ORC_ERROR;

    const int32_t full_h = s->IH - 1 + s->pad[0] + s->pad[1] - (s->KH - 1) * s->dilation[0];
    const int32_t full_w = s->IW - 1 + s->pad[2] + s->pad[3] - (s->KW - 1) * s->dilation[1];
    if ((full_h % s->stride[0]) != 0 || (full_w % s->stride[1]) != 0)
        return ORC_ERROR;
    if (s->OH != full_h / s->stride[0] + 1 || s->OW != full_w / s->stride[1] + 1)
        return ORC_ERROR;

    if (depthwise_m > 0 && s->IC * depthwise_m != s->OC)
        return ORC_ERROR;
    if (s->bias_len != s->OC && s->bias_len != 1)
        return ORC_ERROR;
    return ORC_VALID;
}

/* ------------------------------------------------------------------------------------------------
 * OpConv2d::eval (tensor_ops.cpp:723-882).
 * The reference materialises a copy padded with input_zp (:807-808), initialises the output with the
 * broadcast bias (:814-823), then runs ob,oy,ox,oc x ky,kx x ic, skipping out-of-image taps
 * (:845-852; bounds mode visits them, where the padded value minus input_zp contributes zero) and
 * finally stores bias + acc (:868-869).
 * ---------------------------------------------------------------------------------------------- */
#define ORC_DEFINE_CONV2D(NAME, T, ABS_EXPR)                                                                       \
    static int NAME(const orc_conv_shape_t* s, const T* in, const T* w, const T* bias, T in_zp, T w_zp,          \
                    int abs_mode, T* out)                                                                          \
    {                                                                                                              \
        /* abs_mode 1: bounds mode; 2: bounds mode of an operator without local_bound, whose input is replaced by   \
           its largest magnitude (tensor_ops.cpp:797-801) */                                                       \
        if (orc_conv_check(s, 0) != ORC_VALID)                                                                     \
            return ORC_ERROR;                                                                                      \
        const int N = s->N, IH = s->IH, IW = s->IW, IC = s->IC, OC = s->OC, KH = s->KH, KW = s->KW;                \
        const int OH = s->OH, OW = s->OW;                                                                          \
        const int pt = s->pad[0], pb = s->pad[1], pl = s->pad[2], pr = s->pad[3];                                  \
        const int sy = s->stride[0], sx = s->stride[1], dy = s->dilation[0], dx = s->dilation[1];                  \
        const int PH = IH + pt + pb, PW = IW + pl + pr;                                                            \
        const size_t n_w = (size_t)OC * KH * KW * IC;                                                              \
        T* padded        = (T*)malloc(sizeof(T) * (size_t)N * PH * PW * IC + 1);                                   \
        T* wv            = (T*)malloc(sizeof(T) * n_w + 1);                                                        \
        if (!padded || !wv)                                                                                        \
        {                                                                                                          \
            free(padded);                                                                                          \
            free(wv);                                                                                              \
            return ORC_ERROR;                                                                                      \
        }                                                                                                          \
        for (size_t i = 0; i < n_w; i++)                                                                           \
            wv[i] = abs_mode ? ABS_EXPR(w[i]) : w[i];                                                              \
        T in_abs_max = 0;                                                                                          \
        if (abs_mode == 2)                                                                                         \
            for (size_t i = 0; i < (size_t)N * IH * IW * IC; i++)                                                  \
                if (ABS_EXPR(in[i]) > in_abs_max)                                                                  \
                    in_abs_max = ABS_EXPR(in[i]);                                                                  \
        for (int n = 0; n < N; n++)                                                                                \
            for (int y = 0; y < PH; y++)                                                                           \
                for (int x = 0; x < PW; x++)                                                                       \
                    for (int c = 0; c < IC; c++)                                                                   \
                    {                                                                                              \
                        const int iy = y - pt, ix = x - pl;                                                        \
                        T v = in_zp;                                                                               \
                        if (iy >= 0 && iy < IH && ix >= 0 && ix < IW)                                              \
                        {                                                                                          \
                            v = in[(((size_t)n * IH + iy) * IW + ix) * IC + c];                                    \
                            if (abs_mode)                                                                          \
                                v = abs_mode == 2 ? in_abs_max : ABS_EXPR(v);                                      \
                        }                                                                                          \
                        padded[(((size_t)n * PH + y) * PW + x) * IC + c] = v;                                      \
                    }                                                                                              \
        _Pragma("omp parallel for collapse(2) schedule(static)")                                                   \
        for (int ob = 0; ob < N; ob++)                                                                             \
            for (int oy = 0; oy < OH; oy++)                                                                        \
                for (int ox = 0; ox < OW; ox++)                                                                    \
                    for (int oc = 0; oc < OC; oc++)                                                                \
                    {                                                                                              \
                        T acc = 0;                                                                                 \
                        for (int ky = 0; ky < KH; ky++)                                                            \
                        {                                                                                          \
                            const int iy_pad = oy * sy + ky * dy;                                                  \
                            for (int kx = 0; kx < KW; kx++)                                                        \
                            {                                                                                      \
                                const int ix_pad = ox * sx + kx * dx;                                              \
                                const int y = iy_pad - pt, x = ix_pad - pl;                                        \
                                const int in_scope = (0 <= x && x < IW) && (0 <= y && y < IH);                     \
                                if (!in_scope && !abs_mode)                                                        \
                                    continue;                                                                      \
                                const T* ip = padded + (((size_t)ob * PH + iy_pad) * PW + ix_pad) * IC;            \
                                const T* wp = wv + (((size_t)oc * KH + ky) * KW + kx) * IC;                        \
                                for (int ic = 0; ic < IC; ic++)                                                    \
                                    acc += (ip[ic] - in_zp) * (wp[ic] - w_zp);                                     \
                            }                                                                                      \
                        }                                                                                          \
                        T b = bias[s->bias_len == 1 ? 0 : oc];                                                     \
                        if (abs_mode)                                                                              \
                            b = ABS_EXPR(b);                                                                       \
                        out[(((size_t)ob * OH + oy) * OW + ox) * OC + oc] = b + acc;                               \
                    }                                                                                              \
        free(padded);                                                                                              \
        free(wv);                                                                                                  \
        return ORC_VALID;                                                                                          \
    }

#define ORC_ABS_I32(v) ((v) < 0 ? -(v) : (v))
#define ORC_ABS_F32(v) fabsf(v)
#define ORC_ABS_F64(v) fabs(v)

ORC_DEFINE_CONV2D(conv2d_i32_impl, int32_t, ORC_ABS_I32)
ORC_DEFINE_CONV2D(conv2d_i64_impl, int64_t, ORC_ABS_I32)
ORC_DEFINE_CONV2D(conv2d_f32_impl, float, ORC_ABS_F32)
ORC_DEFINE_CONV2D(conv2d_f64_impl, double, ORC_ABS_F64)

int orc_conv2d_i32(const orc_conv_shape_t* s, const int32_t* in, const int32_t* w, const int32_t* bias,
                   int32_t in_zp, int32_t w_zp, int32_t* out)
{
    return conv2d_i32_impl(s, in, w, bias, in_zp, w_zp, 0, out);
}

int orc_conv2d_f32(const orc_conv_shape_t* s, const float* in, const float* w, const float* bias, float* out)
{
    return conv2d_f32_impl(s, in, w, bias, 0.0f, 0.0f, 0, out);
}

int orc_conv2d_f64(const orc_conv_shape_t* s, const double* in, const double* w, const double* bias, int abs_mode,
                   double* out)
{
    return conv2d_f64_impl(s, in, w, bias, 0.0, 0.0, abs_mode, out);
}

static int32_t* widen_i8(const int8_t* p, size_t n)
{
    int32_t* r = (int32_t*)malloc(sizeof(int32_t) * n + 4);
    if (r)
        for (size_t i = 0; i < n; i++)
            r[i] = (int32_t)p[i];
    return r;
}

int orc_conv2d_i8(const orc_conv_shape_t* s, const int8_t* in, const int8_t* w, const int32_t* bias, int32_t in_zp,
                  int32_t w_zp, int32_t* out)
{
    if (orc_conv_check(s, 0) != ORC_VALID)
        return ORC_ERROR;
    int32_t* in32 = widen_i8(in, (size_t)s->N * s->IH * s->IW * s->IC);
    int32_t* w32  = widen_i8(w, (size_t)s->OC * s->KH * s->KW * s->IC);
    int rc        = (in32 && w32) ? orc_conv2d_i32(s, in32, w32, bias, in_zp, w_zp, out) : ORC_ERROR;
    free(in32);
    free(w32);
    return rc;
}

/* INT16 x INT8 -> INT48 (tensor_ops.cpp:2225): the accumulator type is int64 (template_types.h:109), the input zero
 * point must be zero for a tensor that is not INT8 (:805), the weights keep theirs, and the result is clipped to 48 bits
 * (:875-879).  The same loop nest as above on operands widened to the accumulator type. */
static int64_t* widen_i16_to_i64(const int16_t* p, size_t n)
{
    int64_t* r = (int64_t*)malloc(sizeof(int64_t) * n + 8);
    if (r)
        for (size_t i = 0; i < n; i++)
            r[i] = (int64_t)p[i];
    return r;
}

static int64_t* widen_i8_to_i64(const int8_t* p, size_t n)
{
    int64_t* r = (int64_t*)malloc(sizeof(int64_t) * n + 8);
    if (r)
        for (size_t i = 0; i < n; i++)
            r[i] = (int64_t)p[i];
    return r;
}

static void clip_int48(int64_t* p, size_t n)
{
    const int64_t lo = -((int64_t)1 << 47), hi = ((int64_t)1 << 47) - 1;
    for (size_t i = 0; i < n; i++)
        p[i] = p[i] < lo ? lo : (p[i] > hi ? hi : p[i]);
}

int orc_conv2d_i16(const orc_conv_shape_t* s, const int16_t* in, const int8_t* w, const int64_t* bias, int32_t in_zp,
                   int32_t w_zp, int64_t* out)
{
    if (orc_conv_check(s, 0) != ORC_VALID || in_zp != 0)
        return ORC_ERROR;
    int64_t* in64 = widen_i16_to_i64(in, (size_t)s->N * s->IH * s->IW * s->IC);
    int64_t* w64  = widen_i8_to_i64(w, (size_t)s->OC * s->KH * s->KW * s->IC);
    int rc        = (in64 && w64) ? conv2d_i64_impl(s, in64, w64, bias, 0, (int64_t)w_zp, 0, out) : ORC_ERROR;
    if (rc == ORC_VALID)
        clip_int48(out, (size_t)s->N * s->OH * s->OW * s->OC);
    free(in64);
    free(w64);
    return rc;
}

/* ------------------------------------------------------------------------------------------------
 * OpConv3d (tensor_ops.cpp:901-1120): check_conv_attribute with conv_dimension 3 (:120-226), then
 * ob,od,oy,ox,oc x kd,ky,kx x ic on a copy padded with input_zp, out-of-volume taps skipped
 * (:1079-1087; bounds mode visits them, contributing zero), out = bias + acc (:1104-1105).
 * ---------------------------------------------------------------------------------------------- */
int orc_conv3d_check(const orc_conv3d_shape_t* s)
{
    for (int i = 0; i < 6; i++)
        if (s->pad[i] < 0)
            return ORC_ERROR;
    for (int i = 0; i < 3; i++)
        if (s->stride[i] < 1 || s->dilation[i] < 1)
            return ORC_ERROR;
    const int32_t full_d = s->ID - 1 + s->pad[0] + s->pad[1] - (s->KD - 1) * s->dilation[0];
    const int32_t full_h = s->IH - 1 + s->pad[2] + s->pad[3] - (s->KH - 1) * s->dilation[1];
    const int32_t full_w = s->IW - 1 + s->pad[4] + s->pad[5] - (s->KW - 1) * s->dilation[2];
    if ((full_d % s->stride[0]) != 0 || (full_h % s->stride[1]) != 0 || (full_w % s->stride[2]) != 0)
        return ORC_ERROR;
    if (s->OD != full_d / s->stride[0] + 1 || s->OH != full_h / s->stride[1] + 1 || s->OW != full_w / s->stride[2] + 1)
        return ORC_ERROR;
    if (s->bias_len != s->OC && s->bias_len != 1)
        return ORC_ERROR;
    return ORC_VALID;
}

#define ORC_DEFINE_CONV3D(NAME, T, ABS_EXPR)                                                                       \
    static int NAME(const orc_conv3d_shape_t* s, const T* in, const T* w, const T* bias, T in_zp, T w_zp,        \
                    int abs_mode, T* out)                                                                          \
    {                                                                                                              \
        if (orc_conv3d_check(s) != ORC_VALID)                                                                      \
            return ORC_ERROR;                                                                                      \
        const int N = s->N, ID = s->ID, IH = s->IH, IW = s->IW, IC = s->IC, OC = s->OC;                            \
        const int KD = s->KD, KH = s->KH, KW = s->KW, OD = s->OD, OH = s->OH, OW = s->OW;                          \
        for (int ob = 0; ob < N; ob++)                                                                             \
            for (int od = 0; od < OD; od++)                                                                        \
                for (int oy = 0; oy < OH; oy++)                                                                    \
                    for (int ox = 0; ox < OW; ox++)                                                                \
                        for (int oc = 0; oc < OC; oc++)                                                            \
                        {                                                                                          \
                            T acc = 0;                                                                             \
                            for (int kd = 0; kd < KD; kd++)                                                        \
                                for (int ky = 0; ky < KH; ky++)                                                    \
                                    for (int kx = 0; kx < KW; kx++)                                                \
                                    {                                                                              \
                                        const int d = od * s->stride[0] + kd * s->dilation[0] - s->pad[0];         \
                                        const int y = oy * s->stride[1] + ky * s->dilation[1] - s->pad[2];         \
                                        const int x = ox * s->stride[2] + kx * s->dilation[2] - s->pad[4];         \
                                        const int in_scope =                                                       \
                                            0 <= x && x < IW && 0 <= y && y < IH && 0 <= d && d < ID;              \
                                        if (!in_scope)                                                             \
                                            continue; /* the padded value is input_zp: contributes zero */         \
                                        const T* ip = in + ((((size_t)ob * ID + d) * IH + y) * IW + x) * IC;       \
                                        const T* wp = w + ((((size_t)oc * KD + kd) * KH + ky) * KW + kx) * IC;     \
                                        for (int ic = 0; ic < IC; ic++)                                            \
                                        {                                                                          \
                                            T a = ip[ic], b = wp[ic];                                              \
                                            if (abs_mode)                                                          \
                                                a = ABS_EXPR(a), b = ABS_EXPR(b);                                  \
                                            acc += (a - in_zp) * (b - w_zp);                                       \
                                        }                                                                          \
                                    }                                                                              \
                            T b = bias[s->bias_len == 1 ? 0 : oc];                                                 \
                            if (abs_mode)                                                                          \
                                b = ABS_EXPR(b);                                                                   \
                            out[((((size_t)ob * OD + od) * OH + oy) * OW + ox) * OC + oc] = b + acc;               \
                        }                                                                                          \
        return ORC_VALID;                                                                                          \
    }

ORC_DEFINE_CONV3D(conv3d_i32_impl, int32_t, ORC_ABS_I32)
ORC_DEFINE_CONV3D(conv3d_f32_impl, float, ORC_ABS_F32)
ORC_DEFINE_CONV3D(conv3d_f64_impl, double, ORC_ABS_F64)

int orc_conv3d_i32(const orc_conv3d_shape_t* s, const int32_t* in, const int32_t* w, const int32_t* bias,
                   int32_t in_zp, int32_t w_zp, int32_t* out)
{
    return conv3d_i32_impl(s, in, w, bias, in_zp, w_zp, 0, out);
}

int orc_conv3d_f32(const orc_conv3d_shape_t* s, const float* in, const float* w, const float* bias, float* out)
{
    return conv3d_f32_impl(s, in, w, bias, 0.0f, 0.0f, 0, out);
}

int orc_conv3d_f64(const orc_conv3d_shape_t* s, const double* in, const double* w, const double* bias, int abs_mode,
                   double* out)
{
    return conv3d_f64_impl(s, in, w, bias, 0.0, 0.0, abs_mode, out);
}

int orc_conv3d_i8(const orc_conv3d_shape_t* s, const int8_t* in, const int8_t* w, const int32_t* bias, int32_t in_zp,
                  int32_t w_zp, int32_t* out)
{
    if (orc_conv3d_check(s) != ORC_VALID)
        return ORC_ERROR;
    int32_t* in32 = widen_i8(in, (size_t)s->N * s->ID * s->IH * s->IW * s->IC);
    int32_t* w32  = widen_i8(w, (size_t)s->OC * s->KD * s->KH * s->KW * s->IC);
    int rc        = (in32 && w32) ? orc_conv3d_i32(s, in32, w32, bias, in_zp, w_zp, out) : ORC_ERROR;
    free(in32);
    free(w32);
    return rc;
}

/* INT16 x INT8 -> INT48 (tensor_ops.cpp:2237): as orc_conv2d_i16; zero-point rule :1031, 48-bit clip :1113-1117 */
ORC_DEFINE_CONV3D(conv3d_i64_impl, int64_t, ORC_ABS_I32)

int orc_conv3d_i16(const orc_conv3d_shape_t* s, const int16_t* in, const int8_t* w, const int64_t* bias, int32_t in_zp,
                   int32_t w_zp, int64_t* out)
{
    if (orc_conv3d_check(s) != ORC_VALID || in_zp != 0)
        return ORC_ERROR;
    int64_t* in64 = widen_i16_to_i64(in, (size_t)s->N * s->ID * s->IH * s->IW * s->IC);
    int64_t* w64  = widen_i8_to_i64(w, (size_t)s->OC * s->KD * s->KH * s->KW * s->IC);
    int rc        = (in64 && w64) ? conv3d_i64_impl(s, in64, w64, bias, 0, (int64_t)w_zp, 0, out) : ORC_ERROR;
    if (rc == ORC_VALID)
        clip_int48(out, (size_t)s->N * s->OD * s->OH * s->OW * s->OC);
    free(in64);
    free(w64);
    return rc;
}

/* ------------------------------------------------------------------------------------------------
 * OpTransposeConv2d (tensor_ops.cpp:1982-2197): out_pad > -kernel (:2037-2041), output size
 * (IH-1)*stride + out_pad + kernel (:2043-2053); eval: for every output element and tap (ky,kx) the
 * input position y = oy - out_pad_top - ky, x = ox - out_pad_left - kx is used when it is inside
 * [0, IH*sy) x [0, IW*sx) and a multiple of the stride (:2155-2165); out = acc + bias (:2183-2184).
 * ---------------------------------------------------------------------------------------------- */
int orc_tconv_check(const orc_tconv_shape_t* s)
{
    if (s->stride[0] < 1 || s->stride[1] < 1)
        return ORC_ERROR;
    /* a tensor with a negative dimension is never allocated (subgraph_traverser.cpp:583-590): no such call */
    if (s->OH < 0 || s->OW < 0)
        return ORC_ERROR;
    if (s->out_pad[0] <= -s->KH || s->out_pad[1] <= -s->KH || s->out_pad[2] <= -s->KW || s->out_pad[3] <= -s->KW)
        return ORC_ERROR;
    if (s->OH != (s->IH - 1) * s->stride[0] + s->out_pad[0] + s->out_pad[1] + s->KH ||
        s->OW != (s->IW - 1) * s->stride[1] + s->out_pad[2] + s->out_pad[3] + s->KW)
        return ORC_ERROR;
    if (s->bias_len != s->OC && s->bias_len != 1)
        return ORC_ERROR;
    return ORC_VALID;
}

#define ORC_DEFINE_TCONV(NAME, T, ABS_EXPR)                                                                        \
    static int NAME(const orc_tconv_shape_t* s, const T* in, const T* w, const T* bias, T in_zp, T w_zp,         \
                    int abs_mode, T* out)                                                                          \
    {                                                                                                              \
        if (orc_tconv_check(s) != ORC_VALID)                                                                       \
            return ORC_ERROR;                                                                                      \
        const int N = s->N, IH = s->IH, IW = s->IW, IC = s->IC, OC = s->OC, KH = s->KH, KW = s->KW;                \
        const int OH = s->OH, OW = s->OW, sy = s->stride[0], sx = s->stride[1];                                    \
        for (int ob = 0; ob < N; ob++)                                                                             \
            for (int oy = 0; oy < OH; oy++)                                                                        \
                for (int ox = 0; ox < OW; ox++)                                                                    \
                    for (int oc = 0; oc < OC; oc++)                                                                \
                    {                                                                                              \
                        const int iy = oy - s->out_pad[0], ix = ox - s->out_pad[2];                                \
                        T acc = 0;                                                                                 \
                        for (int ky = 0; ky < KH; ky++)                                                            \
                            for (int kx = 0; kx < KW; kx++)                                                        \
                            {                                                                                      \
                                const int y = iy - ky, x = ix - kx;                                                \
                                const int in_scope = 0 <= y && y < IH * sy && 0 <= x && x < IW * sx &&             \
                                                     (y % sy) == 0 && (x % sx) == 0;                               \
                                if (!in_scope)                                                                     \
                                    continue; /* extra multiplies would add 0 * weight */                          \
                                const T* ip = in + (((size_t)ob * IH + y / sy) * IW + x / sx) * IC;                \
                                const T* wp = w + (((size_t)oc * KH + ky) * KW + kx) * IC;                         \
                                for (int ic = 0; ic < IC; ic++)                                                    \
                                {                                                                                  \
                                    T a = ip[ic], b = wp[ic];                                                      \
                                    if (abs_mode)                                                                  \
                                        a = ABS_EXPR(a), b = ABS_EXPR(b);                                          \
                                    acc += (a - in_zp) * (b - w_zp);                                               \
                                }                                                                                  \
                            }                                                                                      \
                        T b = bias[s->bias_len == 1 ? 0 : oc];                                                     \
                        if (abs_mode)                                                                              \
                            b = ABS_EXPR(b);                                                                       \
                        out[(((size_t)ob * OH + oy) * OW + ox) * OC + oc] = acc + b;                               \
                    }                                                                                              \
        return ORC_VALID;                                                                                          \
    }

ORC_DEFINE_TCONV(tconv_i32_impl, int32_t, ORC_ABS_I32)
ORC_DEFINE_TCONV(tconv_f32_impl, float, ORC_ABS_F32)
ORC_DEFINE_TCONV(tconv_f64_impl, double, ORC_ABS_F64)

int orc_transpose_conv2d_i32(const orc_tconv_shape_t* s, const int32_t* in, const int32_t* w, const int32_t* bias,
                             int32_t in_zp, int32_t w_zp, int32_t* out)
{
    return tconv_i32_impl(s, in, w, bias, in_zp, w_zp, 0, out);
}

int orc_transpose_conv2d_f32(const orc_tconv_shape_t* s, const float* in, const float* w, const float* bias,
                             float* out)
{
    return tconv_f32_impl(s, in, w, bias, 0.0f, 0.0f, 0, out);
}

int orc_transpose_conv2d_f64(const orc_tconv_shape_t* s, const double* in, const double* w, const double* bias,
                             int abs_mode, double* out)
{
    return tconv_f64_impl(s, in, w, bias, 0.0, 0.0, abs_mode, out);
}

/* INT16 x INT8 -> INT48 (tensor_ops.cpp:2291): as orc_conv2d_i16; zero-point rule :2115, 48-bit clip :2190-2194 */
ORC_DEFINE_TCONV(tconv_i64_impl, int64_t, ORC_ABS_I32)

int orc_transpose_conv2d_i16(const orc_tconv_shape_t* s, const int16_t* in, const int8_t* w, const int64_t* bias,
                             int32_t in_zp, int32_t w_zp, int64_t* out)
{
    if (orc_tconv_check(s) != ORC_VALID || in_zp != 0)
        return ORC_ERROR;
    int64_t* in64 = widen_i16_to_i64(in, (size_t)s->N * s->IH * s->IW * s->IC);
    int64_t* w64  = widen_i8_to_i64(w, (size_t)s->OC * s->KH * s->KW * s->IC);
    int rc        = (in64 && w64) ? tconv_i64_impl(s, in64, w64, bias, 0, (int64_t)w_zp, 0, out) : ORC_ERROR;
    if (rc == ORC_VALID)
        clip_int48(out, (size_t)s->N * s->OH * s->OW * s->OC);
    free(in64);
    free(w64);
    return rc;
}

int orc_transpose_conv2d_i8(const orc_tconv_shape_t* s, const int8_t* in, const int8_t* w, const int32_t* bias,
                            int32_t in_zp, int32_t w_zp, int32_t* out)
{
    if (orc_tconv_check(s) != ORC_VALID)
        return ORC_ERROR;
    int32_t* in32 = widen_i8(in, (size_t)s->N * s->IH * s->IW * s->IC);
    int32_t* w32  = widen_i8(w, (size_t)s->OC * s->KH * s->KW * s->IC);
    int rc        = (in32 && w32) ? orc_transpose_conv2d_i32(s, in32, w32, bias, in_zp, w_zp, out) : ORC_ERROR;
    free(in32);
    free(w32);
    return rc;
}

/* ------------------------------------------------------------------------------------------------
 * OpDepthwiseConv2d::eval (tensor_ops.cpp:1172-1334): ob,oy,ox,ic,km x ky,kx; an out-of-image tap
 * contributes zero (:1302-1313); weight [KH,KW,IC,M]; output channel ic*M+km (:1320).
 * ---------------------------------------------------------------------------------------------- */
#define ORC_DEFINE_DEPTHWISE(NAME, T, ABS_EXPR)                                                                    \
    static int NAME(const orc_conv_shape_t* s, int32_t M, const T* in, const T* w, const T* bias, T in_zp,        \
                    T w_zp, int abs_mode, T* out)                                                                  \
    {                                                                                                              \
        if (M < 1 || orc_conv_check(s, M) != ORC_VALID)                                                            \
            return ORC_ERROR;                                                                                      \
        const int N = s->N, IH = s->IH, IW = s->IW, IC = s->IC, OC = s->OC, KH = s->KH, KW = s->KW;                \
        const int OH = s->OH, OW = s->OW;                                                                          \
        const int pt = s->pad[0], pl = s->pad[2];                                                                  \
        const int sy = s->stride[0], sx = s->stride[1], dy = s->dilation[0], dx = s->dilation[1];                  \
        /* abs_mode 2: bounds mode without local_bound (tensor_ops.cpp:1252-1256) */                               \
        T in_abs_max = 0;                                                                                          \
        if (abs_mode == 2)                                                                                         \
            for (size_t i = 0; i < (size_t)N * IH * IW * IC; i++)                                                  \
                if (ABS_EXPR(in[i]) > in_abs_max)                                                                  \
                    in_abs_max = ABS_EXPR(in[i]);                                                                  \
        _Pragma("omp parallel for collapse(2) schedule(static)")                                                   \
        for (int ob = 0; ob < N; ob++)                                                                             \
            for (int oy = 0; oy < OH; oy++)                                                                        \
                for (int ox = 0; ox < OW; ox++)                                                                    \
                    for (int ic = 0; ic < IC; ic++)                                                                \
                        for (int km = 0; km < M; km++)                                                             \
                        {                                                                                          \
                            T acc        = 0;                                                                      \
                            const int iy = oy * sy - pt, ix = ox * sx - pl;                                        \
                            for (int ky = 0; ky < KH; ky++)                                                        \
                                for (int kx = 0; kx < KW; kx++)                                                    \
                                {                                                                                  \
                                    const int y = iy + ky * dy, x = ix + kx * dx;                                  \
                                    const int in_scope = (0 <= y && y < IH) && (0 <= x && x < IW);                 \
                                    if (!in_scope)                                                                 \
                                        continue;                                                                  \
                                    T a = in[(((size_t)ob * IH + y) * IW + x) * IC + ic];                          \
                                    T b = w[(((size_t)ky * KW + kx) * IC + ic) * M + km];                          \
                                    if (abs_mode)                                                                  \
                                    {                                                                              \
                                        a = abs_mode == 2 ? in_abs_max : ABS_EXPR(a);                              \
                                        b = ABS_EXPR(b);                                                           \
                                    }                                                                              \
                                    acc += (a - in_zp) * (b - w_zp);                                               \
                                }                                                                                  \
                            const int oc = ic * M + km;                                                            \
                            T bv         = bias[s->bias_len == 1 ? 0 : oc];                                        \
                            if (abs_mode)                                                                          \
                                bv = ABS_EXPR(bv);                                                                 \
                            out[(((size_t)ob * OH + oy) * OW + ox) * OC + oc] = bv + acc;                          \
                        }                                                                                          \
        return ORC_VALID;                                                                                          \
    }

ORC_DEFINE_DEPTHWISE(depthwise_i32_impl, int32_t, ORC_ABS_I32)
ORC_DEFINE_DEPTHWISE(depthwise_i64_impl, int64_t, ORC_ABS_I32)
ORC_DEFINE_DEPTHWISE(depthwise_f32_impl, float, ORC_ABS_F32)
ORC_DEFINE_DEPTHWISE(depthwise_f64_impl, double, ORC_ABS_F64)

int orc_depthwise_i32(const orc_conv_shape_t* s, int32_t M, const int32_t* in, const int32_t* w,
                      const int32_t* bias, int32_t in_zp, int32_t w_zp, int32_t* out)
{
    return depthwise_i32_impl(s, M, in, w, bias, in_zp, w_zp, 0, out);
}

int orc_depthwise_i8(const orc_conv_shape_t* s, int32_t M, const int8_t* in, const int8_t* w, const int32_t* bias,
                     int32_t in_zp, int32_t w_zp, int32_t* out)
{
    if (M < 1 || orc_conv_check(s, M) != ORC_VALID)
        return ORC_ERROR;
    int32_t* in32 = widen_i8(in, (size_t)s->N * s->IH * s->IW * s->IC);
    int32_t* w32  = widen_i8(w, (size_t)s->KH * s->KW * s->IC * M);
    int rc        = (in32 && w32) ? orc_depthwise_i32(s, M, in32, w32, bias, in_zp, w_zp, out) : ORC_ERROR;
    free(in32);
    free(w32);
    return rc;
}

/* INT16 x INT8 -> INT48 (tensor_ops.cpp:2247; the clip at :1325-1329) */
int orc_depthwise_i16(const orc_conv_shape_t* s, int32_t M, const int16_t* in, const int8_t* w, const int64_t* bias,
                      int32_t in_zp, int32_t w_zp, int64_t* out)
{
    if (M < 1 || orc_conv_check(s, M) != ORC_VALID || in_zp != 0)
        return ORC_ERROR;
    int64_t* in64 = widen_i16_to_i64(in, (size_t)s->N * s->IH * s->IW * s->IC);
    int64_t* w64  = widen_i8_to_i64(w, (size_t)s->KH * s->KW * s->IC * M);
    int rc        = (in64 && w64) ? depthwise_i64_impl(s, M, in64, w64, bias, 0, (int64_t)w_zp, 0, out) : ORC_ERROR;
    if (rc == ORC_VALID)
        clip_int48(out, (size_t)s->N * s->OH * s->OW * s->OC);
    free(in64);
    free(w64);
    return rc;
}

int orc_depthwise_f32(const orc_conv_shape_t* s, int32_t M, const float* in, const float* w, const float* bias,
                      float* out)
{
    return depthwise_f32_impl(s, M, in, w, bias, 0.0f, 0.0f, 0, out);
}

int orc_depthwise_f64(const orc_conv_shape_t* s, int32_t M, const double* in, const double* w, const double* bias,
                      int abs_mode, double* out)
{
    return depthwise_f64_impl(s, M, in, w, bias, 0.0, 0.0, abs_mode, out);
}

/* ------------------------------------------------------------------------------------------------
 * OpMatMul::eval (tensor_ops.cpp:1423-1492): per batch, widen to the accumulator type, subtract the
 * zero points, contract over C.  Integer sums are order independent modulo 2^32; the floating-point
 * summation order of Eigen's contraction is not restated (sequential in c here).
 * ---------------------------------------------------------------------------------------------- */
#define ORC_DEFINE_MATMUL(NAME, T, ABS_EXPR)                                                                       \
    static int NAME(int32_t N, int32_t H, int32_t C, int32_t W, const T* a, const T* b, T a_zp, T b_zp,           \
                    int abs_mode, T* out)                                                                          \
    {                                                                                                              \
        if (N < 0 || H < 0 || C < 0 || W < 0)                                                                      \
            return ORC_ERROR;                                                                                      \
        int failed = 0;                                                                                            \
        _Pragma("omp parallel")                                                                                    \
        {                                                                                                          \
        T* row = (T*)malloc(sizeof(T) * (size_t)(W > 0 ? W : 1));                                                  \
        if (!row)                                                                                                  \
            failed = 1;                                                                                            \
        _Pragma("omp for collapse(2) schedule(static)")                                                            \
        for (int n = 0; n < N; n++)                                                                                \
            for (int h = 0; h < H; h++)                                                                            \
            {                                                                                                      \
                if (!row)                                                                                          \
                    continue;                                                                                      \
                for (int x = 0; x < W; x++)                                                                        \
                    row[x] = 0;                                                                                    \
                for (int c = 0; c < C; c++)                                                                        \
                {                                                                                                  \
                    T av = a[((size_t)n * H + h) * C + c];                                                         \
                    if (abs_mode)                                                                                  \
                        av = ABS_EXPR(av);                                                                         \
                    av -= a_zp;                                                                                    \
                    const T* bp = b + ((size_t)n * C + c) * W;                                                     \
                    for (int x = 0; x < W; x++)                                                                    \
                    {                                                                                              \
                        T bv = bp[x];                                                                              \
                        if (abs_mode)                                                                              \
                            bv = ABS_EXPR(bv);                                                                     \
                        row[x] += av * (bv - b_zp);                                                                \
                    }                                                                                              \
                }                                                                                                  \
                memcpy(out + ((size_t)n * H + h) * W, row, sizeof(T) * (size_t)W);                                 \
            }                                                                                                      \
        free(row);                                                                                                 \
        }                                                                                                          \
        return failed ? ORC_ERROR : ORC_VALID;                                                                     \
    }

ORC_DEFINE_MATMUL(matmul_i32_impl, int32_t, ORC_ABS_I32)
ORC_DEFINE_MATMUL(matmul_i64_impl, int64_t, ORC_ABS_I32)
ORC_DEFINE_MATMUL(matmul_f32_impl, float, ORC_ABS_F32)
ORC_DEFINE_MATMUL(matmul_f64_impl, double, ORC_ABS_F64)

int orc_matmul_i32(int32_t N, int32_t H, int32_t C, int32_t W, const int32_t* a, const int32_t* b, int32_t a_zp,
                   int32_t b_zp, int32_t* out)
{
    return matmul_i32_impl(N, H, C, W, a, b, a_zp, b_zp, 0, out);
}

int orc_matmul_i8(int32_t N, int32_t H, int32_t C, int32_t W, const int8_t* a, const int8_t* b, int32_t a_zp,
                  int32_t b_zp, int32_t* out)
{
    int32_t* a32 = widen_i8(a, (size_t)N * H * C);
    int32_t* b32 = widen_i8(b, (size_t)N * C * W);
    int rc       = (a32 && b32) ? orc_matmul_i32(N, H, C, W, a32, b32, a_zp, b_zp, out) : ORC_ERROR;
    free(a32);
    free(b32);
    return rc;
}

/* INT16 x INT16 -> INT48 (tensor_ops.cpp:2257): zero points must be zero for tensors that are not INT8 (:1433-1434),
 * int64 accumulation, the result clipped to 48 bits (:1485-1489) */
int orc_matmul_i16(int32_t N, int32_t H, int32_t C, int32_t W, const int16_t* a, const int16_t* b, int32_t a_zp,
                   int32_t b_zp, int64_t* out)
{
    if (a_zp != 0 || b_zp != 0)
        return ORC_ERROR;
    int64_t* a64 = widen_i16_to_i64(a, (size_t)N * H * C);
    int64_t* b64 = widen_i16_to_i64(b, (size_t)N * C * W);
    int rc       = (a64 && b64) ? matmul_i64_impl(N, H, C, W, a64, b64, 0, 0, 0, out) : ORC_ERROR;
    if (rc == ORC_VALID)
        clip_int48(out, (size_t)N * H * W);
    free(a64);
    free(b64);
    return rc;
}

int orc_matmul_f32(int32_t N, int32_t H, int32_t C, int32_t W, const float* a, const float* b, float* out)
{
    return matmul_f32_impl(N, H, C, W, a, b, 0.0f, 0.0f, 0, out);
}

int orc_matmul_f64(int32_t N, int32_t H, int32_t C, int32_t W, const double* a, const double* b, int abs_mode,
                   double* out)
{
    return matmul_f64_impl(N, H, C, W, a, b, 0.0, 0.0, abs_mode, out);
}

/* ------------------------------------------------------------------------------------------------
 * QuantUtil::apply_scale_32 / apply_scale_16 (reference_model/src/quant_util.h:45-108).
 * ---------------------------------------------------------------------------------------------- */
int32_t orc_apply_scale_32(int32_t value, int32_t multiplier, int32_t shift, int double_round, int* status)
{
    if (multiplier < 0 || shift < 2 || shift > 62)
    {
        *status = ORC_UNPREDICTABLE;
        return 0;
    }
    const int64_t low_val  = -(INT64_C(1) << (shift - 1));
    const int64_t high_val = INT64_C(1) << (shift - 1);
    if ((int64_t)value < low_val || (int64_t)value >= high_val)
    {
        *status = ORC_UNPREDICTABLE;
        return 0;
    }
    int64_t round = INT64_C(1) << (shift - 1);
    if (double_round)
    {
        if (shift > 31 && value >= 0)
            round += INT64_C(1) << 30;
        if (shift > 31 && value < 0)
            round -= INT64_C(1) << 30;
    }
    int64_t result = (int64_t)value * (int64_t)multiplier + round;
    result         = result >> shift;
    if (result < -(INT64_C(1) << 31) || result >= (INT64_C(1) << 31))
    {
        *status = ORC_UNPREDICTABLE;
        return 0;
    }
    return (int32_t)result;
}

int32_t orc_apply_scale_16(int64_t value, int16_t multiplier, int32_t shift, int* status)
{
    if (multiplier < 0 || shift < 2 || shift > 62)
    {
        *status = ORC_UNPREDICTABLE;
        return 0;
    }
    const int64_t round = INT64_C(1) << (shift - 1);
    int64_t result      = (int64_t)((uint64_t)value * (uint64_t)(int64_t)multiplier + (uint64_t)round);
    result              = result >> shift;
    if (result < -(INT64_C(1) << 31) || result >= (INT64_C(1) << 31))
    {
        *status = ORC_UNPREDICTABLE;
        return 0;
    }
    return (int32_t)result;
}

/* value_extend64_impl (reference_model/src/ops/type_conversion.cpp:183-221) for 8/16/32-bit types. */
static int64_t value_extend64(int64_t val, int bits, int is_unsigned)
{
    switch (bits)
    {
        case 48: /* int64 storage; bit 47 set: bits 48..63 are set too (:200-215) */
            if (is_unsigned)
                return val & INT64_C(0x0000FFFFFFFFFFFF);
            return (val & INT64_C(0x800000000000)) ? (int64_t)((uint64_t)val | UINT64_C(0xFFFF000000000000)) : val;
        case 8:
            return is_unsigned ? (int64_t)(uint8_t)(int8_t)val : (int64_t)(int8_t)(uint8_t)(val & 0xFF);
        case 16:
            return is_unsigned ? (int64_t)(uint16_t)(int16_t)val : (int64_t)(int16_t)(uint16_t)(val & 0xFFFF);
        case 32:
            return is_unsigned ? (int64_t)(uint32_t)(int32_t)val : (int64_t)(int32_t)val;
        default:
            return val;
    }
}

/* ------------------------------------------------------------------------------------------------
 * OpRescale::checkTensorAttributes + eval (type_conversion.cpp:72-154, 224-421).
 * ---------------------------------------------------------------------------------------------- */
/* g_func_config.precise_mode / compliance_mode / bounds_mode as RESCALE's INEXACT_ROUND reads them (:318-346):
 * 0 FP32 maths; 1 precise mode (FP64, truncated); 2 / 3 precise mode with compliance mode, normal / bounds pass. */
static int g_inexact_mode = 0;
void orc_set_inexact_mode(int mode)
{
    g_inexact_mode = mode;
}

/* in32: the int32 storage of INT8 / INT16 / INT32 tensors; in64: the int64 storage of an INT48 tensor */
static int rescale_impl(const orc_rescale_attr_t* a, int64_t rows, int32_t C, const int32_t* in32, const int64_t* in64,
                        const int32_t* multiplier, const int32_t* shift, int32_t n_mult, int32_t n_shift, int32_t rank,
                        int32_t* out)
{
    const int i8in = a->in_bits == 8, i16in = a->in_bits == 16, i32in = a->in_bits == 32, i48in = a->in_bits == 48;
    const int i8out = a->out_bits == 8, i16out = a->out_bits == 16, i32out = a->out_bits == 32;
    if (!(i8in || i16in || i32in || i48in) || !(i8out || i16out || i32out) || (i48in ? !in64 : !in32))
        return ORC_ERROR;

    /* checkTensorAttributes :118-151 */
    if (a->rounding_mode != ORC_ROUND_SINGLE && a->rounding_mode != ORC_ROUND_DOUBLE &&
        a->rounding_mode != ORC_ROUND_INEXACT)
        return ORC_ERROR;
    if (!a->scale32 && a->rounding_mode == ORC_ROUND_DOUBLE)
        return ORC_ERROR;
    if (a->input_unsigned && a->output_unsigned)
        return ORC_ERROR;
    if (i32out && a->input_unsigned)
        return ORC_ERROR;
    if (i32in && a->output_unsigned)
        return ORC_ERROR;
    if (i32in && a->input_unsigned)
        return ORC_ERROR;
    if (i32out && a->output_unsigned)
        return ORC_ERROR;
    /* :122, :129, :132 */
    if (i48in && (a->scale32 || a->output_unsigned || a->input_unsigned))
        return ORC_ERROR;
    if (a->per_channel)
    {
        if (rank < 1 || n_mult != C || n_shift != C)
            return ORC_ERROR;
    }
    else if (n_mult != 1 || n_shift != 1)
        return ORC_ERROR;

    /* eval :242-255 */
    const int64_t out_zp_ext = value_extend64(a->out_zp, a->out_bits, a->output_unsigned);
    const int64_t in_zp_ext  = value_extend64(a->in_zp, a->in_bits, a->input_unsigned);
    if (!i8in && !(i16in && a->input_unsigned) && in_zp_ext != 0)
        return ORC_ERROR;
    if (!i8out && !(i16out && a->output_unsigned) && out_zp_ext != 0)
        return ORC_ERROR;
    if (i16in && a->input_unsigned && in_zp_ext != 0 && in_zp_ext != 32768)
        return ORC_ERROR;
    if (i16out && a->output_unsigned && out_zp_ext != 0 && out_zp_ext != 32768)
        return ORC_ERROR;

    /* getSigned/UnsignedMinimum/Maximum for the output type (type_conversion.cpp:61-64) */
    int64_t qmin, qmax;
    if (a->output_unsigned)
    {
        qmin = 0;
        qmax = i8out ? 255 : (i16out ? 65535 : (int64_t)INT32_MAX); /* u32 max is capped to int32 max by applyClip */
    }
    else
    {
        qmin = i8out ? -128 : (i16out ? -32768 : (int64_t)INT32_MIN);
        qmax = i8out ? 127 : (i16out ? 32767 : (int64_t)INT32_MAX);
    }

    const int double_round = a->rounding_mode == ORC_ROUND_DOUBLE;
    const int inexact      = a->rounding_mode == ORC_ROUND_INEXACT;
    int status             = ORC_VALID;

    /* The reference walks channel by channel when per_channel is set (:381-394) and stops at the first
     * throw; results after a REQUIRE failure are unspecified, so the element order here is free. */
    for (int64_t r = 0; r < rows && status == ORC_VALID; r++)
        for (int32_t c = 0; c < C; c++)
        {
            const int32_t m  = a->per_channel ? multiplier[c] : multiplier[0];
            const int32_t sh = a->per_channel ? shift[c] : shift[0];
            const int64_t st = i48in ? in64[r * C + c] : (int64_t)in32[r * C + c];
            const int64_t v  = value_extend64(st, a->in_bits, a->input_unsigned) - in_zp_ext;
            int32_t scaled;
            if (!inexact)
            {
                if (a->scale32)
                    scaled = orc_apply_scale_32((int32_t)v, m, sh, double_round, &status);
                else
                    scaled = orc_apply_scale_16(v, (int16_t)m, sh, &status);
            }
            else if (g_inexact_mode)
            {
                /* INEXACT_ROUND in precise mode: FP64 maths (:326-346) */
                volatile double t = (double)v * (double)m;
                volatile double x = t * exp2((double)(-sh));
                if (g_inexact_mode >= 2)
                {
                    const double with_zp  = x + (double)out_zp_ext;
                    const double half_ulp = exp2(-23 - 1);
                    volatile double three = 3 * fabs(x);
                    volatile double sum   = three + fabs(with_zp);
                    volatile double prod  = sum * half_ulp;
                    const double err_bnd  = 0.5 + prod;
                    volatile double moved = g_inexact_mode == 3 ? x + err_bnd : x - err_bnd;
                    x                     = g_inexact_mode == 3 ? floor(moved) : ceil(moved);
                }
                /* the cast of a value outside int32 is undefined in the reference; the convention of the FP32 branch */
                scaled = (x > -2147483649.0 && x < 2147483648.0) ? (int32_t)x : INT32_MIN;
            }
            else
            {
                /* INEXACT_ROUND with FP32 maths (:318-324), round to nearest even */
                volatile float t = (float)v * (float)m;
                volatile float u = t * exp2f((float)(-sh));
                const float ri   = rintf(u);
                /* outside the int32 range the reference's cast is undefined; its x86-64 builds return INT32_MIN
                 * (cvtss2si's "integer indefinite"), stated here instead of left to the compiler */
                scaled = (ri >= -2147483648.0f && ri < 2147483648.0f) ? (int32_t)ri : INT32_MIN;
            }
            if (status != ORC_VALID)
                break;
            const int64_t res = (int64_t)scaled + out_zp_ext;
            if (res > (int64_t)INT32_MAX || res < (int64_t)INT32_MIN)
            {
                status = ORC_UNPREDICTABLE;
                break;
            }
            int64_t clipped = res < qmin ? qmin : res;
            clipped         = clipped > qmax ? qmax : clipped;
            out[r * C + c]  = (int32_t)clipped;
        }
    return status;
}

int orc_rescale(const orc_rescale_attr_t* a, int64_t rows, int32_t C, const int32_t* in, const int32_t* multiplier,
                const int32_t* shift, int32_t n_mult, int32_t n_shift, int32_t rank, int32_t* out)
{
    if (a->in_bits == 48)
        return ORC_ERROR;
    return rescale_impl(a, rows, C, in, NULL, multiplier, shift, n_mult, n_shift, rank, out);
}

int orc_rescale_i48(const orc_rescale_attr_t* a, int64_t rows, int32_t C, const int64_t* in, const int32_t* multiplier,
                    const int32_t* shift, int32_t n_mult, int32_t n_shift, int32_t rank, int32_t* out)
{
    if (a->in_bits != 48)
        return ORC_ERROR;
    return rescale_impl(a, rows, C, NULL, in, multiplier, shift, n_mult, n_shift, rank, out);
}

/* ------------------------------------------------------------------------------------------------
 * AVG_POOL2D / MAX_POOL2D.  check_pool2d_attribute (reference_model/src/ops/tensor_ops.cpp:29-117).
 * ---------------------------------------------------------------------------------------------- */
int orc_pool_check(const orc_pool_shape_t* s)
{
    for (int i = 0; i < 4; i++)
        if (s->pad[i] < 0)
            return ORC_ERROR;
    if (s->kernel[0] < 1 || s->kernel[1] < 1 || s->stride[0] < 1 || s->stride[1] < 1)
        return ORC_ERROR;
    if (s->pad[0] >= s->kernel[0] || s->pad[1] >= s->kernel[0] || s->pad[2] >= s->kernel[1] ||
        s->pad[3] >= s->kernel[1])
        return ORC_ERROR;
    const int32_t full_h = s->IH + s->pad[0] + s->pad[1] - s->kernel[0];
    const int32_t full_w = s->IW + s->pad[2] + s->pad[3] - s->kernel[1];
    if (full_h % s->stride[0] != 0 || full_w % s->stride[1] != 0)
        return ORC_ERROR;
    if (s->OH != full_h / s->stride[0] + 1 || s->OW != full_w / s->stride[1] + 1)
        return ORC_ERROR;
    return ORC_VALID;
}

/* reference_model/src/quant_util.h:32-43 */
void orc_reciprocal_scale(int32_t count, int32_t* multiplier, int32_t* shift)
{
    const uint32_t v = (uint32_t)count - 1u;
    int32_t lz       = 32;
    for (int b = 31; b >= 0; b--)
        if (v >> b)
        {
            lz = 31 - b;
            break;
        }
    const int32_t k         = 32 - lz; /* (1<<k)/2 < count <= (1<<k) */
    const int64_t numerator = ((INT64_C(1) << 30) + 1) << k;
    *multiplier             = (int32_t)(numerator / count);
    *shift                  = 30 + k;
}

/* OpAvgPool2d::eval, integer branch (tensor_ops.cpp:603-650): sum of (in - in_zp) over the taps inside the
 * image, scaled by the reciprocal of their count with a single rounding, plus out_zp, clipped. */
int orc_avg_pool2d_i32(const orc_pool_shape_t* s, const int32_t* in, int32_t in_zp, int32_t out_zp, int32_t qmin,
                       int32_t qmax, int32_t* out)
{
    if (orc_pool_check(s) != ORC_VALID)
        return ORC_ERROR;
    int status = ORC_VALID;
    for (int32_t n = 0; n < s->N; n++)
        for (int32_t oh = 0; oh < s->OH; oh++)
            for (int32_t ow = 0; ow < s->OW; ow++)
                for (int32_t c = 0; c < s->C; c++)
                {
                    int32_t acc = 0, count = 0;
                    const int32_t iy = oh * s->stride[0] - s->pad[0];
                    const int32_t ix = ow * s->stride[1] - s->pad[2];
                    for (int32_t ky = 0; ky < s->kernel[0]; ky++)
                        for (int32_t kx = 0; kx < s->kernel[1]; kx++)
                        {
                            const int32_t y = iy + ky, x = ix + kx;
                            if (y >= 0 && y < s->IH && x >= 0 && x < s->IW)
                            {
                                acc += in[(((int64_t)n * s->IH + y) * s->IW + x) * s->C + c] - in_zp;
                                count++;
                            }
                        }
                    int32_t m, sh;
                    int st = ORC_VALID;
                    orc_reciprocal_scale(count, &m, &sh);
                    int32_t v = orc_apply_scale_32(acc, m, sh, 0, &st) + out_zp;
                    if (st != ORC_VALID)
                        status = ORC_UNPREDICTABLE;
                    v = v > qmin ? v : qmin;
                    v = v < qmax ? v : qmax;
                    out[(((int64_t)n * s->OH + oh) * s->OW + ow) * s->C + c] = v;
                }
    return status;
}

/* floating-point branch (tensor_ops.cpp:652-657): fp32 accumulator, taps in (ky, kx) order, one division */
int orc_avg_pool2d_f32(const orc_pool_shape_t* s, const float* in, float* out)
{
    if (orc_pool_check(s) != ORC_VALID)
        return ORC_ERROR;
    for (int32_t n = 0; n < s->N; n++)
        for (int32_t oh = 0; oh < s->OH; oh++)
            for (int32_t ow = 0; ow < s->OW; ow++)
                for (int32_t c = 0; c < s->C; c++)
                {
                    volatile float acc = 0.0f; /* one rounding per addition, no contraction */
                    int32_t count      = 0;
                    const int32_t iy   = oh * s->stride[0] - s->pad[0];
                    const int32_t ix   = ow * s->stride[1] - s->pad[2];
                    for (int32_t ky = 0; ky < s->kernel[0]; ky++)
                        for (int32_t kx = 0; kx < s->kernel[1]; kx++)
                        {
                            const int32_t y = iy + ky, x = ix + kx;
                            if (y >= 0 && y < s->IH && x >= 0 && x < s->IW)
                            {
                                acc = acc + in[(((int64_t)n * s->IH + y) * s->IW + x) * s->C + c];
                                count++;
                            }
                        }
                    out[(((int64_t)n * s->OH + oh) * s->OW + ow) * s->C + c] = acc / (float)count;
                }
    return ORC_VALID;
}

/* OpMaxPool2d::eval (tensor_ops.cpp:1546-1640): padding is the lowest value of the type */
int orc_max_pool2d_i32(const orc_pool_shape_t* s, const int32_t* in, int32_t lowest, int32_t* out)
{
    if (orc_pool_check(s) != ORC_VALID)
        return ORC_ERROR;
    for (int32_t n = 0; n < s->N; n++)
        for (int32_t oh = 0; oh < s->OH; oh++)
            for (int32_t ow = 0; ow < s->OW; ow++)
                for (int32_t c = 0; c < s->C; c++)
                {
                    int32_t best     = lowest;
                    const int32_t iy = oh * s->stride[0] - s->pad[0];
                    const int32_t ix = ow * s->stride[1] - s->pad[2];
                    for (int32_t ky = 0; ky < s->kernel[0]; ky++)
                        for (int32_t kx = 0; kx < s->kernel[1]; kx++)
                        {
                            const int32_t y = iy + ky, x = ix + kx;
                            if (y >= 0 && y < s->IH && x >= 0 && x < s->IW)
                            {
                                const int32_t v = in[(((int64_t)n * s->IH + y) * s->IW + x) * s->C + c];
                                best            = best >= v ? best : v;
                            }
                        }
                    out[(((int64_t)n * s->OH + oh) * s->OW + ow) * s->C + c] = best;
                }
    return ORC_VALID;
}

/* floating point: applyMax / compareNan (reference_model/src/arith_util.h:341-373); the padding value is
 * -infinity in PROPAGATE mode (low_extreme, reference_model/src/dtype_limits.h:53) and NaN in IGNORE mode
 * (arith_util.h:423-432), i.e. padding never changes the result. */
int orc_max_pool2d_f32(const orc_pool_shape_t* s, const float* in, int nan_mode, float* out)
{
    if (orc_pool_check(s) != ORC_VALID || (nan_mode != 1 && nan_mode != 2))
        return ORC_ERROR;
    for (int32_t n = 0; n < s->N; n++)
        for (int32_t oh = 0; oh < s->OH; oh++)
            for (int32_t ow = 0; ow < s->OW; ow++)
                for (int32_t c = 0; c < s->C; c++)
                {
                    float best       = nan_mode == 2 ? NAN : -INFINITY;
                    const int32_t iy = oh * s->stride[0] - s->pad[0];
                    const int32_t ix = ow * s->stride[1] - s->pad[2];
                    for (int32_t ky = 0; ky < s->kernel[0]; ky++)
                        for (int32_t kx = 0; kx < s->kernel[1]; kx++)
                        {
                            const int32_t y = iy + ky, x = ix + kx;
                            if (y < 0 || y >= s->IH || x < 0 || x >= s->IW)
                                continue;
                            const float v = in[(((int64_t)n * s->IH + y) * s->IW + x) * s->C + c];
                            if (isnan(best) || isnan(v))
                                best = nan_mode == 1 ? NAN : (isnan(best) ? v : best);
                            else
                                best = best >= v ? best : v;
                        }
                    out[(((int64_t)n * s->OH + oh) * s->OW + ow) * s->C + c] = best;
                }
    return ORC_VALID;
}

/* ------------------------------------------------------------------------------------------------
 * OpClamp (reference_model/src/ops/activation_funcs.cpp:27-125) through applyClip
 * (reference_model/src/arith_util.h:389-413).
 * ---------------------------------------------------------------------------------------------- */
/* threads the loops of this build run on: 1 for the scalar build, the OpenMP team size otherwise */
#ifdef _OPENMP
#include <omp.h>
int orc_threads(void)
{
    return omp_get_max_threads();
}
#else
int orc_threads(void)
{
    return 1;
}
#endif

int orc_clamp_i32(int64_t n, const int32_t* in, int32_t lo, int32_t hi, int32_t* out)
{
    if (hi < lo)
        return ORC_ERROR;
    for (int64_t i = 0; i < n; i++)
    {
        int32_t v = in[i] >= lo ? in[i] : lo;
        out[i]    = v < hi ? v : hi;
    }
    return ORC_VALID;
}

int orc_clamp_f32(int64_t n, const float* in, float lo, float hi, int nan_mode, float* out)
{
    if (hi < lo || isnan(lo) || isnan(hi))
        return ORC_ERROR;
    for (int64_t i = 0; i < n; i++)
    {
        float v = in[i];
        if (isnan(v))
            v = (nan_mode == 1) ? NAN : lo; /* IGNORE: max(NaN, lo) -> lo, then min(lo, hi) -> lo */
        else
        {
            v = v >= lo ? v : lo;
            v = v < hi ? v : hi;
        }
        out[i] = v;
    }
    return ORC_VALID;
}

/* ------------------------------------------------------------------------------------------------
 * DOT_PRODUCT test data (TOSA specification tosa_mi_data; reference_model/src/generate/
 * generate_dot_product_states.cpp).  A primitive generator is the sequence r <- r*m + 1 (mod 2^32) with
 * m = (8*S + 1) * 0x705A5E75, mapped to (-1, 1) by sign bit and the low 31 bits; each set draws from
 * generators 3*set + {0, 1, 2}.  The arithmetic types below are the reference's: float unless a double
 * square root enters the expression.
 * ---------------------------------------------------------------------------------------------- */
typedef struct
{
    uint32_t m, r;
} dp_prim_t;

static void dp_prim_init(dp_prim_t* g, uint32_t S)
{
    g->m = (8u * S + 1u) * 0x705A5E75u;
    g->r = g->m + 1u;
}

static float dp_prim_next(dp_prim_t* g)
{
    const float sign   = (g->r >> 31) == 0 ? 1.0f : -1.0f;
    const float pseudo = sign * (float)(g->r & 0x7FFFFFFFu) / (float)0x7FFFFFFF;
    g->r               = g->r * g->m + 1u;
    return pseudo;
}

float orc_dp_bound_parameter(int data_kind, int acc16)
{
    switch (data_kind)
    {
        case 16: return acc16 ? 255.875f : 65504.0f;    /* (1<<8) - 1/8 ; (1<<16) - (1<<5) */
        case 17: return 18374686479671623680.0f;        /* (1<<64) - (1<<56) */
        case 32: return 18446742974197923840.0f;        /* (1<<64) - (1<<40) */
        default: return 0.0f;
    }
}

typedef struct
{
    int set, p;
    uint32_t ks;
    float B;
    dp_prim_t g0, g1;
} dp_gen_t;

static void dp_gen_init(dp_gen_t* g, int set, int p, uint32_t ks, float B)
{
    g->set = set, g->p = p, g->ks = ks, g->B = B;
    if (set == 0 || set == 4)
    {
        dp_prim_init(&g->g0, 3u * (uint32_t)set);
        dp_prim_init(&g->g1, 3u * (uint32_t)set + 1u);
    }
    else
        dp_prim_init(&g->g0, 3u * (uint32_t)set + (uint32_t)p);
}

static float dp_gen_next(dp_gen_t* g, uint32_t k)
{
    const int p = g->p;
    switch (g->set)
    {
        case 0: { /* sums of products with zero give zero */
            const float s0 = dp_prim_next(&g->g0), s1 = dp_prim_next(&g->g1);
            if (p == 0)
                return s0 < 0.0f ? 0.0f : s1;
            if (p == 1)
                return s0 < 0.0f ? s1 : 0.0f;
            return 0.0f;
        }
        case 1: { /* large exponents */
            const float s0 = dp_prim_next(&g->g0), s1 = dp_prim_next(&g->g0);
            float v        = s0 < 0 ? -0.75f : 0.75f;
            v += 0.25f * s1;
            if (p != 2)
                return (float)(((double)g->B / sqrt((double)(g->ks + 1u))) * (double)v);
            return (g->B * g->B / (float)(g->ks + 1u)) * v;
        }
        case 2: { /* small values of similar magnitude onto a large one */
            const float s = dp_prim_next(&g->g0);
            if (p != 2)
                return k == 0 ? 1.0f : (float)((double)s / sqrt((double)g->ks));
            return 0.0f;
        }
        case 3: { /* small values of varying magnitude onto a large one */
            const float s0 = dp_prim_next(&g->g0), s1 = dp_prim_next(&g->g0);
            if (p != 2)
                return k == 0 ? (s0 < 0 ? -16.0f : 16.0f) : expf(2 * s0) * s1;
            return 0.0f;
        }
        case 4: { /* a mixture of zero and non-zero products */
            const float s0 = dp_prim_next(&g->g0), s1 = dp_prim_next(&g->g1);
            const float big = (float)(((double)g->B / sqrt((double)g->ks)) * (double)s1);
            if (p == 0)
                return k == g->ks / 2 ? (s0 < 0 ? -0.5f : 0.5f) : (s0 < 0 ? 0.0f : big);
            if (p == 1)
                return k == g->ks / 2 ? (s0 < 0 ? 0.5f : -0.5f) : (s0 < 0 ? big : 0.0f);
            return 0.0f;
        }
        default: { /* 5: signed inputs of large range */
            const float s = dp_prim_next(&g->g0);
            if (p != 2)
                return (float)(((double)g->B / sqrt((double)(g->ks + 1u))) * (double)s);
            return 0.0f;
        }
    }
}

int orc_dp_generate(int op, int set, int param, uint32_t ks, float B, const int32_t* shape, int rank,
                    const int32_t* kernel, float* out)
{
    if (set < 0 || set > 5 || param < 0 || param > 2 || !(B > 0.0f) || ks == 0)
        return ORC_ERROR;
    dp_gen_t g;
    dp_gen_init(&g, set, param, ks, B);
    uint64_t T = 1;
    for (int i = 0; i < rank; i++)
        T *= (uint64_t)shape[i];
    if (param == 2) /* bias: every element is generator(2) */
    {
        if (op == ORC_DP_MATMUL || rank != 1)
            return ORC_ERROR;
        for (uint64_t t = 0; t < T; t++)
            out[t] = dp_gen_next(&g, 2);
        return ORC_VALID;
    }
    if (op == ORC_DP_MATMUL)
    {
        if (rank != 3)
            return ORC_ERROR;
        const uint32_t C = (uint32_t)(param == 0 ? shape[2] : shape[1]);
        const uint32_t W = (uint32_t)shape[2];
        for (uint64_t t = 0; t < T; t++)
            out[t] = dp_gen_next(&g, param == 0 ? (uint32_t)(t % C) : (uint32_t)((t / W) % C));
        return ORC_VALID;
    }
    if (rank != 4)
        return ORC_ERROR;
    if (param == 0)
    {
        if (!kernel || kernel[0] <= 0 || kernel[1] <= 0)
            return ORC_ERROR;
        const uint32_t IH = (uint32_t)shape[1], IW = (uint32_t)shape[2], IC = (uint32_t)shape[3];
        const uint32_t KH = (uint32_t)kernel[0], KW = (uint32_t)kernel[1];
        for (uint64_t t = 0; t < T; t++)
        {
            const uint32_t ic = (uint32_t)(t % IC), ix = (uint32_t)((t / IC) % IW), iy = (uint32_t)(((t / IC) / IW) % IH);
            const uint32_t tap = (iy % KH) * KW + (ix % KW);
            out[t]             = dp_gen_next(&g, op == ORC_DP_CONV2D ? tap * IC + ic : tap);
        }
        return ORC_VALID;
    }
    if (op == ORC_DP_CONV2D) /* weight [OC, KH, KW, IC] */
    {
        const uint32_t KH = (uint32_t)shape[1], KW = (uint32_t)shape[2], IC = (uint32_t)shape[3];
        for (uint64_t t = 0; t < T; t++)
        {
            const uint32_t ic = (uint32_t)(t % IC), kx = (uint32_t)((t / IC) % KW), ky = (uint32_t)(((t / IC) / KW) % KH);
            out[t]            = dp_gen_next(&g, (ky * KW + kx) * IC + ic);
        }
        return ORC_VALID;
    }
    /* depthwise weight [KH, KW, C, M] */
    const uint32_t KH = (uint32_t)shape[0], KW = (uint32_t)shape[1], C = (uint32_t)shape[2], M = (uint32_t)shape[3];
    for (uint64_t t = 0; t < T; t++)
    {
        const uint32_t kx = (uint32_t)(((t / M) / C) % KW), ky = (uint32_t)((((t / M) / C) / KW) % KH);
        out[t]            = dp_gen_next(&g, ky * KW + kx);
    }
    return ORC_VALID;
}
