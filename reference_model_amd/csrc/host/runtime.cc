// Graph runtime and operator adapters above the C ABI (see tosa_host.h).
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "tosa_host.h"

namespace tmi_host
{

// ---- Tensor ----------------------------------------------------------------------------------------------
Tensor::Tensor(const TensorDesc& d) : name(d.name), shape(d.shape), dtype(d.dtype) {}

int64_t Tensor::getElementCount() const
{
    int64_t n = 1;
    for (int32_t s : shape)
        n *= s;
    return n;
}

bool Tensor::scalar_value(int32_t& v) const
{
    if (!host_valid || host.size() < dtype_size(dtype))
        return false;
    switch (dtype)
    {
        case DType_INT4:
        case DType_INT8:
            v = (int8_t)host[0];
            return true;
        case DType_INT16:
        {
            int16_t t;
            memcpy(&t, host.data(), 2);
            v = t;
            return true;
        }
        case DType_INT32:
            memcpy(&v, host.data(), 4);
            return true;
        case DType_INT48:
        {
            int64_t t;
            memcpy(&t, host.data(), 8);
            v = t < INT32_MIN ? INT32_MIN : (t > INT32_MAX ? INT32_MAX : (int32_t)t);    // only 0 is a legal INT48 zero point
            return true;
        }
        case DType_FP16:
        case DType_BF16:
        {
            uint16_t t;
            memcpy(&t, host.data(), 2);
            v = (t & 0x7fff) ? 1 : 0;    // any non-zero floating-point zero point is illegal anyway
            return true;
        }
        case DType_FP32:
        {
            uint32_t t;
            memcpy(&t, host.data(), 4);
            v = (t & 0x7fffffffu) ? 1 : 0;
            return true;
        }
        default:
            return false;
    }
}

// ---- GraphNode -------------------------------------------------------------------------------------------
GraphNode::GraphNode(SubgraphTraverser* sgt, uint32_t op, uint64_t id) : nodeType(op), nodeId(id), parent_sgt(sgt) {}
GraphNode::~GraphNode() {}

int GraphNode::checkTensorAttributes()
{
    return 0;
}

// GraphNode::eval of the reference marks every output valid (reference_model/src/graph_node.cpp:77-89); here a
// result is valid on the device unless the operator produced host bytes.
int GraphNode::eval()
{
    for (Tensor* t : outputs)
        if (!t->host_valid)
            t->dev_valid = true;
    return 0;
}

int GraphNode::error(const char* fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    parent_sgt->last_message = buf;
    fprintf(stderr, "Validation error: node %llu (%s): %s\n", (unsigned long long)nodeId, op_name(nodeType), buf);
    parent_sgt->setGraphStatus(GraphStatus::TOSA_ERROR);
    return 1;
}

int GraphNode::call(int rc)
{
    if (rc == TMI_ERROR)
        return error("%s", tmi_last_error(parent_sgt->ctx));
    parent_sgt->kernels_launched++;
    return 0;
}

int GraphNode::validateRequiredOperands()
{
    if (requiredInputCount >= 0 && (int)inputs.size() != requiredInputCount)
        return error("expected %d input operands, got %zu", requiredInputCount, inputs.size());
    if (requiredOutputCount >= 0 && (int)outputs.size() != requiredOutputCount)
        return error("expected %d output operands, got %zu", requiredOutputCount, outputs.size());
    return 0;
}

int GraphNode::validateRequiredRank(const Tensor* t, int rank_min, int rank_max)
{
    if (t->getRank() < rank_min || t->getRank() > rank_max)
        return error("tensor %s has rank %d, expected [%d,%d]", t->getName().c_str(), t->getRank(), rank_min, rank_max);
    return 0;
}

namespace
{

int32_t tmi_dtype(DType t)
{
    switch (t)
    {
        case DType_INT8:
            return TMI_INT8;
        case DType_INT16:
            return TMI_INT16;
        case DType_INT32:
            return TMI_INT32;
        case DType_INT48:
            return TMI_INT48;
        case DType_FP32:
            return TMI_FP32;
        case DType_FP16:
            return TMI_FP16;
        case DType_BF16:
            return TMI_BF16;
        default:
            return 0;
    }
}

// CONST: the payload was decoded in initializeGraph (reference: subgraph_traverser.cpp:617-780)
class OpConst : public GraphNode
{
public:
    OpConst(SubgraphTraverser* sgt, uint64_t id) : GraphNode(sgt, Op_CONST, id) {}
    int eval() override
    {
        return 0;
    }
};

class OpRescale;
class OpClamp;

// Shared by CONV2D and DEPTHWISE_CONV2D: operands [input, weight, bias, input_zp, weight_zp] -> [output]
class ConvBase : public GraphNode
{
public:
    ConvBase(SubgraphTraverser* sgt, uint32_t op, uint64_t id, bool depthwise_) : GraphNode(sgt, op, id), depthwise(depthwise_)
    {
        requiredInputCount  = 5;
        requiredOutputCount = 1;
    }
    GraphNode* fused_rescale = nullptr;    // set by the peephole in linkTensorsAndNodes
    GraphNode* fused_clamp   = nullptr;

    int fill_desc(tmi_conv_desc_t& d)
    {
        const Tensor *in = inputs[0], *w = inputs[1], *bias = inputs[2], *out = outputs[0];
        if (attribute.pad.size() != 4)
            return error("Illegal size for attribute pad");
        if (attribute.stride.size() != 2)
            return error("Illegal size for attribute stride");
        if (attribute.dilation.size() != 2)
            return error("Illegal size for attribute dilation");
        memset(&d, 0, sizeof(d));
        d.in_dtype  = tmi_dtype(in->getDtype());
        d.out_dtype = tmi_dtype(out->getDtype());
        d.N = in->shape[0], d.IH = in->shape[1], d.IW = in->shape[2], d.IC = in->shape[3];
        if (depthwise)
        {
            d.KH = w->shape[0], d.KW = w->shape[1];
            d.OC = w->shape[2] * w->shape[3];
            if (w->shape[2] != d.IC)
                return error("tensor input channel mismatch %d != %d", w->shape[2], d.IC);
        }
        else
        {
            d.OC = w->shape[0], d.KH = w->shape[1], d.KW = w->shape[2];
            if (w->shape[3] != d.IC)
                return error("tensor input channel mismatch %d != %d", w->shape[3], d.IC);
        }
        if (out->shape[0] != d.N)
            return error("tensor batch mismatch %d != %d", d.N, out->shape[0]);
        if (out->shape[3] != d.OC)
            return error("tensor output channel mismatch %d != %d", d.OC, out->shape[3]);
        d.OH = out->shape[1], d.OW = out->shape[2];
        for (int i = 0; i < 4; i++)
            d.pad[i] = attribute.pad[i];
        for (int i = 0; i < 2; i++)
            d.stride[i] = attribute.stride[i], d.dilation[i] = attribute.dilation[i];
        d.bias_len  = bias->shape[0];
        d.acc_dtype = tmi_dtype((DType)attribute.acc_type);
        return 0;
    }

    int checkTensorAttributes() override
    {
        if (validateRequiredOperands())
            return 1;
        if (validateRequiredRank(inputs[0], 4, 4) || validateRequiredRank(inputs[1], 4, 4) ||
            validateRequiredRank(inputs[2], 1, 1) || validateRequiredRank(inputs[3], 1, 1) ||
            validateRequiredRank(inputs[4], 1, 1) || validateRequiredRank(outputs[0], 4, 4))
            return 1;
        // the weights have the input's type, except that INT16 inputs come with INT8 weights (tensor_ops.cpp:2225, 2247)
        // and INT8 inputs may come with INT4 weights (:2224, :2246: the same arithmetic on values of -8 ... 7)
        if (inputs[1]->getDtype() != (inputs[0]->getDtype() == DType_INT16 ? DType_INT8 : inputs[0]->getDtype()) &&
            !(inputs[0]->getDtype() == DType_INT8 && inputs[1]->getDtype() == DType_INT4))
            return error("weight data type not supported for this configuration of operator");
        tmi_conv_desc_t d;
        if (fill_desc(d))
            return 1;
        if (tmi_conv2d_check(parent_sgt->ctx, &d, depthwise) != TMI_VALID)
            return error("%s", tmi_last_error(parent_sgt->ctx));
        return 0;
    }

    int eval() override;

protected:
    bool depthwise;
};

// RESCALE: operands [in, multiplier, shift, in_zp, out_zp]
class OpRescale : public GraphNode
{
public:
    OpRescale(SubgraphTraverser* sgt, uint64_t id) : GraphNode(sgt, Op_RESCALE, id)
    {
        requiredInputCount  = 5;
        requiredOutputCount = 1;
    }
    int fill_desc(tmi_rescale_desc_t& r, bool need_zp_values)
    {
        memset(&r, 0, sizeof(r));
        r.in_dtype        = tmi_dtype(inputs[0]->getDtype());
        r.out_dtype       = tmi_dtype(outputs[0]->getDtype());
        r.scale32         = attribute.scale32;
        r.rounding_mode   = (int32_t)attribute.rounding_mode;
        r.per_channel     = attribute.per_channel;
        r.input_unsigned  = attribute.input_unsigned;
        r.output_unsigned = attribute.output_unsigned;
        r.n_multiplier    = inputs[1]->shape.empty() ? 1 : inputs[1]->shape[0];
        r.n_shift         = inputs[2]->shape.empty() ? 1 : inputs[2]->shape[0];
        if (need_zp_values)
        {
            if (!inputs[3]->scalar_value(r.in_zp) || !inputs[4]->scalar_value(r.out_zp))
                return error("OpRescale: zero-point operands must be available on the host");
        }
        return 0;
    }
    int checkTensorAttributes() override
    {
        if (validateRequiredOperands())
            return 1;
        if (validateRequiredRank(inputs[0], 0, 6) || validateRequiredRank(outputs[0], 0, 6))
            return 1;
        if (inputs[0]->shape != outputs[0]->shape)
            return error("OpRescale: input and output rank/size must match");
        const DType mt = inputs[1]->getDtype();
        if ((attribute.scale32 && mt != DType_INT32) || (!attribute.scale32 && mt != DType_INT16))
            return error("OpRescale: multiplier tensor type does not match scale32");
        if (inputs[2]->getDtype() != DType_INT8)
            return error("OpRescale: shift tensor must be INT8");
        tmi_rescale_desc_t r;
        if (fill_desc(r, false))
            return 1;
        const int rank = inputs[0]->getRank();
        const int C    = rank ? inputs[0]->shape[rank - 1] : 1;
        if (tmi_rescale_check(parent_sgt->ctx, &r, rank, C) != TMI_VALID)
            return error("%s", tmi_last_error(parent_sgt->ctx));
        return 0;
    }
    int eval() override
    {
        if (folded)
            return GraphNode::eval();
        tmi_rescale_desc_t r;
        if (fill_desc(r, true))
            return 1;
        const int rank     = inputs[0]->getRank();
        const int C        = rank ? inputs[0]->shape[rank - 1] : 1;
        const int64_t rows = C ? inputs[0]->getElementCount() / C : 0;
        SubgraphTraverser* s = parent_sgt;
        if (call(tmi_rescale(s->ctx, &r, rank, rows, C, s->device(inputs[0]), s->device(inputs[1]), s->device(inputs[2]),
                             s->device_out(outputs[0]))))
            return 1;
        return GraphNode::eval();
    }
};

// CLAMP: operand [in]; min_val / max_val are one serialized element each (activation_funcs.cpp:36-89)
class OpClamp : public GraphNode
{
public:
    OpClamp(SubgraphTraverser* sgt, uint64_t id) : GraphNode(sgt, Op_CLAMP, id)
    {
        requiredInputCount  = 1;
        requiredOutputCount = 1;
    }
    int decode(int32_t& lo, int32_t& hi)
    {
        const DType t   = inputs[0]->getDtype();
        const size_t es = dtype_size(t);
        if ((t != DType_INT8 && t != DType_INT16) || attribute.min_val.size() < es || attribute.max_val.size() < es)
            return error("OpClamp: unsupported TOSA_REF_TYPE or malformed min/max attribute");
        if (t == DType_INT8)
            lo = (int8_t)attribute.min_val[0], hi = (int8_t)attribute.max_val[0];
        else
        {
            int16_t a, b;
            memcpy(&a, attribute.min_val.data(), 2);
            memcpy(&b, attribute.max_val.data(), 2);
            lo = a, hi = b;
        }
        return 0;
    }
    int checkTensorAttributes() override
    {
        if (validateRequiredOperands())
            return 1;
        if (inputs[0]->shape != outputs[0]->shape || inputs[0]->getDtype() != outputs[0]->getDtype())
            return error("OpClamp: input and output must have the same shape and type");
        return 0;
    }
    // min_val / max_val of a floating-point CLAMP: bytes of the tensor's own type (activation_funcs.cpp:36-89)
    int decode_fp(float& lo, float& hi)
    {
        const DType t   = inputs[0]->getDtype();
        const size_t es = dtype_size(t);
        if (attribute.min_val.size() < es || attribute.max_val.size() < es)
            return error("OpClamp: malformed min/max attribute");
        auto one = [&](const std::vector<uint8_t>& b) -> float {
            if (t == DType_FP32)
            {
                float f;
                memcpy(&f, b.data(), 4);
                return f;
            }
            uint16_t h;
            memcpy(&h, b.data(), 2);
            if (t == DType_BF16)
            {
                const uint32_t u = (uint32_t)h << 16;
                float f;
                memcpy(&f, &u, 4);
                return f;
            }
            // IEEE half -> float
            const uint32_t sign = (uint32_t)(h & 0x8000) << 16;
            uint32_t exp = (h >> 10) & 31, man = h & 1023, u;
            if (exp == 0)
            {
                if (man == 0)
                    u = sign;
                else
                {
                    int e = -1;
                    do
                    {
                        man <<= 1;
                        e++;
                    } while (!(man & 1024));
                    u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 1023) << 13);
                }
            }
            else if (exp == 31)
                u = sign | 0x7f800000u | (man << 13);
            else
                u = sign | ((exp + 127 - 15) << 23) | (man << 13);
            float f;
            memcpy(&f, &u, 4);
            return f;
        };
        lo = one(attribute.min_val), hi = one(attribute.max_val);
        return 0;
    }
    int eval() override
    {
        if (folded)
            return GraphNode::eval();
        const DType t = inputs[0]->getDtype();
        if (t == DType_FP16 || t == DType_BF16 || t == DType_FP32)
        {
            if (parent_sgt->precise_mode)
                return error("CLAMP has no precise-mode (fp64) evaluation in this library");
            float lo = 0.0f, hi = 0.0f;
            if (decode_fp(lo, hi))
                return 1;
            SubgraphTraverser* s = parent_sgt;
            // NanPropagationMode: 1 = PROPAGATE (also the default of an absent field), 2 = IGNORE
            const int32_t nan_mode = attribute.nan_mode == 2 ? 2 : 1;
            if (call(tmi_clamp_fp(s->ctx, tmi_dtype(t), inputs[0]->getElementCount(), s->device(inputs[0]), lo, hi, nan_mode,
                                  s->device_out(outputs[0]))))
                return 1;
            return GraphNode::eval();
        }
        int32_t lo = 0, hi = 0;
        if (decode(lo, hi))
            return 1;
        if (hi < lo)
            return error("OpClamp: max smaller than min");
        SubgraphTraverser* s = parent_sgt;
        if (call(tmi_clamp(s->ctx, tmi_dtype(inputs[0]->getDtype()), inputs[0]->getElementCount(), s->device(inputs[0]),
                           lo, hi, s->device_out(outputs[0]))))
            return 1;
        return GraphNode::eval();
    }
};

int ConvBase::eval()
{
    tmi_conv_desc_t d;
    if (fill_desc(d))
        return 1;
    int32_t in_zp = 0, w_zp = 0;
    if (!inputs[3]->scalar_value(in_zp) || !inputs[4]->scalar_value(w_zp))
        return error("zero-point operands must be available on the host");
    if (inputs[1]->getDtype() == DType_INT4 && w_zp != 0)    // tensor_ops.cpp:811, :1241
        return error("Weight zero point must be zero for non int8_t data");
    SubgraphTraverser* s = parent_sgt;
    if (s->precise_mode && inputs[0]->getDtype() != DType_INT8 && inputs[0]->getDtype() != DType_INT16)
    {
        // precise mode (tensor_ops.cpp:790-802, :1245-1257): fp64 accumulation, fp64 result
        outputs[0]->precise = true;
        auto fn             = depthwise ? tmi_depthwise_conv2d_precise : tmi_conv2d_precise;
        if (call(fn(s->ctx, &d, s->device(inputs[0]), s->device(inputs[1]), s->device(inputs[2]), s->bounds_mode ? 1 : 0,
                    attribute.local_bound ? 1 : 0, static_cast<double*>(s->device_out(outputs[0])))))
            return 1;
        return GraphNode::eval();
    }
    if (!fused_rescale)
    {
        auto fn = depthwise ? tmi_depthwise_conv2d : tmi_conv2d;
        if (call(fn(s->ctx, &d, s->device(inputs[0]), s->device(inputs[1]), s->device(inputs[2]), in_zp, w_zp,
                    s->device_out(outputs[0]))))
            return 1;
        return GraphNode::eval();
    }
    // CONV -> RESCALE (-> CLAMP) as one kernel: the result goes straight into the last node's output
    OpRescale* rs = static_cast<OpRescale*>(fused_rescale);
    OpClamp* cl   = static_cast<OpClamp*>(fused_clamp);
    tmi_rescale_desc_t r;
    if (rs->fill_desc(r, true))
        return 1;
    int32_t lo = 0, hi = 0;
    if (cl && (cl->decode(lo, hi) || (hi < lo && error("OpClamp: max smaller than min"))))
        return 1;
    Tensor* final_out = cl ? cl->outputs[0] : rs->outputs[0];
    auto fn           = depthwise ? tmi_depthwise_conv2d_rescale_clamp : tmi_conv2d_rescale_clamp;
    if (call(fn(s->ctx, &d, s->device(inputs[0]), s->device(inputs[1]), s->device(inputs[2]), in_zp, w_zp, &r,
                s->device(rs->inputs[1]), s->device(rs->inputs[2]), cl ? 1 : 0, lo, hi, s->device_out(final_out))))
        return 1;
    s->nodes_folded += cl ? 2 : 1;
    outputs[0]->dev_valid = false;    // the int32 intermediate is never materialised
    outputs[0]->host_valid = false;
    return 0;
}

class OpConv2d : public ConvBase
{
public:
    OpConv2d(SubgraphTraverser* sgt, uint64_t id) : ConvBase(sgt, Op_CONV2D, id, false) {}
};
class OpDepthwiseConv2d : public ConvBase
{
public:
    OpDepthwiseConv2d(SubgraphTraverser* sgt, uint64_t id) : ConvBase(sgt, Op_DEPTHWISE_CONV2D, id, true) {}
};

// TRANSPOSE_CONV2D and CONV3D: operands [input, weight, bias, input_zp, weight_zp] like CONV2D
// (tensor_ops.cpp:1974, :893); the checks are the C ABI's, run on a dry descriptor in checkTensorAttributes.
class OpTransposeConv2d : public GraphNode
{
public:
    OpTransposeConv2d(SubgraphTraverser* sgt, uint64_t id) : GraphNode(sgt, Op_TRANSPOSE_CONV2D, id)
    {
        requiredInputCount  = 5;
        requiredOutputCount = 1;
    }
    int fill_desc(tmi_tconv_desc_t& d)
    {
        const Tensor *in = inputs[0], *w = inputs[1], *bias = inputs[2], *out = outputs[0];
        if (attribute.pad.size() != 4)
            return error("illegal size for attribute out_pad");
        if (attribute.stride.size() != 2)
            return error("illegal size for attribute stride");
        memset(&d, 0, sizeof(d));
        d.in_dtype = tmi_dtype(in->getDtype()), d.out_dtype = tmi_dtype(out->getDtype());
        d.N = in->shape[0], d.IH = in->shape[1], d.IW = in->shape[2], d.IC = in->shape[3];
        d.OC = w->shape[0], d.KH = w->shape[1], d.KW = w->shape[2];
        if (w->shape[3] != d.IC)
            return error("tensor input channel mismatch %d != %d", w->shape[3], d.IC);
        if (out->shape[0] != d.N)
            return error("tensor batch mismatch %d != %d", d.N, out->shape[0]);
        if (out->shape[3] != d.OC)
            return error("tensor output channel mismatch %d != %d", d.OC, out->shape[3]);
        d.OH = out->shape[1], d.OW = out->shape[2];
        for (int i = 0; i < 4; i++)
            d.out_pad[i] = attribute.pad[i];
        d.stride[0] = attribute.stride[0], d.stride[1] = attribute.stride[1];
        d.bias_len  = bias->shape[0];
        d.acc_dtype = tmi_dtype((DType)attribute.acc_type);
        return 0;
    }
    int checkTensorAttributes() override
    {
        if (validateRequiredOperands())
            return 1;
        if (validateRequiredRank(inputs[0], 4, 4) || validateRequiredRank(inputs[1], 4, 4) ||
            validateRequiredRank(inputs[2], 1, 1) || validateRequiredRank(inputs[3], 1, 1) ||
            validateRequiredRank(inputs[4], 1, 1) || validateRequiredRank(outputs[0], 4, 4))
            return 1;
        if (inputs[1]->getDtype() != (inputs[0]->getDtype() == DType_INT16 ? DType_INT8 : inputs[0]->getDtype()) &&    // INT16 x INT8 (:2237, :2291)
            !(inputs[0]->getDtype() == DType_INT8 && inputs[1]->getDtype() == DType_INT4))    // INT8 x INT4 (:2235, :2289)
            return error("weight data type not supported for this configuration of operator");
        tmi_tconv_desc_t d;
        if (fill_desc(d))
            return 1;
        if (tmi_transpose_conv2d_check(parent_sgt->ctx, &d) != TMI_VALID)
            return error("%s", tmi_last_error(parent_sgt->ctx));
        return 0;
    }
    int eval() override
    {
        // precise / bounds mode (the reference evaluates this operator in fp64 and on absolute values then,
        // e.g. tensor_ops.cpp:601-605): no such pass exists here, and the ordinary result must not stand in for it
        if (parent_sgt->precise_mode && inputs[0]->getDtype() != DType_INT8 && inputs[0]->getDtype() != DType_INT16)
            return error("%s has no precise-mode (fp64) evaluation in this library", "TRANSPOSE_CONV2D");
        tmi_tconv_desc_t d;
        if (fill_desc(d))
            return 1;
        int32_t in_zp = 0, w_zp = 0;
        if (!inputs[3]->scalar_value(in_zp) || !inputs[4]->scalar_value(w_zp))
            return error("zero-point operands must be available on the host");
        if (inputs[1]->getDtype() == DType_INT4 && w_zp != 0)    // tensor_ops.cpp:1037, :2119
            return error("Weight zero point must be zero for non int8_t data");
        SubgraphTraverser* s = parent_sgt;
        if (call(tmi_transpose_conv2d(s->ctx, &d, s->device(inputs[0]), s->device(inputs[1]), s->device(inputs[2]),
                                      in_zp, w_zp, s->device_out(outputs[0]))))
            return 1;
        return GraphNode::eval();
    }
};

// AVG_POOL2D: operands [input, input_zp, output_zp] (tensor_ops.cpp:476); MAX_POOL2D: [input] (:1497).
class OpPool2d : public GraphNode
{
public:
    OpPool2d(SubgraphTraverser* sgt, Op op, uint64_t id) : GraphNode(sgt, op, id), avg(op == Op_AVG_POOL2D)
    {
        requiredInputCount  = avg ? 3 : 1;
        requiredOutputCount = 1;
    }
    const bool avg;
    int fill_desc(tmi_pool_desc_t& d)
    {
        const Tensor *in = inputs[0], *out = outputs[0];
        if (attribute.pad.size() != 4)
            return error("illegal size for attribute padding");
        if (attribute.kernel.size() != 2)
            return error("illegal size for attribute kernel");
        if (attribute.stride.size() != 2)
            return error("illegal size for attribute stride");
        memset(&d, 0, sizeof(d));
        d.dtype     = tmi_dtype(in->getDtype());
        d.acc_dtype = tmi_dtype((DType)attribute.acc_type);
        d.N = in->shape[0], d.IH = in->shape[1], d.IW = in->shape[2], d.C = in->shape[3];
        if (out->shape[0] != d.N)
            return error("tensor batch mismatch %d != %d", d.N, out->shape[0]);
        if (out->shape[3] != d.C)
            return error("tensor channel mismatch %d != %d", d.C, out->shape[3]);
        d.OH = out->shape[1], d.OW = out->shape[2];
        for (int i = 0; i < 2; i++)
            d.kernel[i] = attribute.kernel[i], d.stride[i] = attribute.stride[i];
        for (int i = 0; i < 4; i++)
            d.pad[i] = attribute.pad[i];
        d.nan_mode = attribute.nan_mode ? (int32_t)attribute.nan_mode : 1;    // unset = PROPAGATE
        return 0;
    }
    int checkTensorAttributes() override
    {
        if (validateRequiredOperands())
            return 1;
        if (validateRequiredRank(inputs[0], 4, 4) || validateRequiredRank(outputs[0], 4, 4))
            return 1;
        if (avg && (validateRequiredRank(inputs[1], 1, 1) || validateRequiredRank(inputs[2], 1, 1)))
            return error("input and output zero point must be rank 1");
        if (inputs[0]->getDtype() != outputs[0]->getDtype())
            return error("input and output tensor type mismatch");
        tmi_pool_desc_t d;
        if (fill_desc(d))
            return 1;
        if (tmi_pool2d_check(parent_sgt->ctx, &d, avg ? 1 : 0) != TMI_VALID)
            return error("%s", tmi_last_error(parent_sgt->ctx));
        return 0;
    }
    int eval() override
    {
        // precise / bounds mode (the reference evaluates this operator in fp64 and on absolute values then,
        // e.g. tensor_ops.cpp:601-605): no such pass exists here, and the ordinary result must not stand in for it
        if (parent_sgt->precise_mode && inputs[0]->getDtype() != DType_INT8 && inputs[0]->getDtype() != DType_INT16)
            return error("%s has no precise-mode (fp64) evaluation in this library", "AVG_POOL2D / MAX_POOL2D");
        tmi_pool_desc_t d;
        if (fill_desc(d))
            return 1;
        SubgraphTraverser* s = parent_sgt;
        if (avg)
        {
            int32_t in_zp = 0, out_zp = 0;
            if (!inputs[1]->scalar_value(in_zp) || !inputs[2]->scalar_value(out_zp))
                return error("zero-point operands must be available on the host");
            if (call(tmi_avg_pool2d(s->ctx, &d, s->device(inputs[0]), in_zp, out_zp, s->device_out(outputs[0]))))
                return 1;
        }
        else if (call(tmi_max_pool2d(s->ctx, &d, s->device(inputs[0]), s->device_out(outputs[0]))))
            return 1;
        return GraphNode::eval();
    }
};

class OpConv3d : public GraphNode
{
public:
    OpConv3d(SubgraphTraverser* sgt, uint64_t id) : GraphNode(sgt, Op_CONV3D, id)
    {
        requiredInputCount  = 5;
        requiredOutputCount = 1;
    }
    int fill_desc(tmi_conv3d_desc_t& d)
    {
        const Tensor *in = inputs[0], *w = inputs[1], *bias = inputs[2], *out = outputs[0];
        if (attribute.pad.size() != 6)
            return error("Illegal size for attribute pad");
        if (attribute.stride.size() != 3)
            return error("Illegal size for attribute stride");
        if (attribute.dilation.size() != 3)
            return error("Illegal size for attribute dilation");
        memset(&d, 0, sizeof(d));
        d.in_dtype = tmi_dtype(in->getDtype()), d.out_dtype = tmi_dtype(out->getDtype());
        d.N = in->shape[0], d.ID = in->shape[1], d.IH = in->shape[2], d.IW = in->shape[3], d.IC = in->shape[4];
        d.OC = w->shape[0], d.KD = w->shape[1], d.KH = w->shape[2], d.KW = w->shape[3];
        if (w->shape[4] != d.IC)
            return error("tensor input channel mismatch %d != %d", w->shape[4], d.IC);
        if (out->shape[0] != d.N)
            return error("tensor batch mismatch %d != %d", d.N, out->shape[0]);
        if (out->shape[4] != d.OC)
            return error("tensor output channel mismatch %d != %d", d.OC, out->shape[4]);
        d.OD = out->shape[1], d.OH = out->shape[2], d.OW = out->shape[3];
        for (int i = 0; i < 6; i++)
            d.pad[i] = attribute.pad[i];
        for (int i = 0; i < 3; i++)
            d.stride[i] = attribute.stride[i], d.dilation[i] = attribute.dilation[i];
        d.bias_len  = bias->shape[0];
        d.acc_dtype = tmi_dtype((DType)attribute.acc_type);
        return 0;
    }
    int checkTensorAttributes() override
    {
        if (validateRequiredOperands())
            return 1;
        if (validateRequiredRank(inputs[0], 5, 5) || validateRequiredRank(inputs[1], 5, 5) ||
            validateRequiredRank(inputs[2], 1, 1) || validateRequiredRank(inputs[3], 1, 1) ||
            validateRequiredRank(inputs[4], 1, 1) || validateRequiredRank(outputs[0], 5, 5))
            return 1;
        if (inputs[1]->getDtype() != (inputs[0]->getDtype() == DType_INT16 ? DType_INT8 : inputs[0]->getDtype()) &&    // INT16 x INT8 (:2237, :2291)
            !(inputs[0]->getDtype() == DType_INT8 && inputs[1]->getDtype() == DType_INT4))    // INT8 x INT4 (:2235, :2289)
            return error("weight data type not supported for this configuration of operator");
        tmi_conv3d_desc_t d;
        if (fill_desc(d))
            return 1;
        if (tmi_conv3d_check(parent_sgt->ctx, &d) != TMI_VALID)
            return error("%s", tmi_last_error(parent_sgt->ctx));
        return 0;
    }
    int eval() override
    {
        // precise / bounds mode (the reference evaluates this operator in fp64 and on absolute values then,
        // e.g. tensor_ops.cpp:601-605): no such pass exists here, and the ordinary result must not stand in for it
        if (parent_sgt->precise_mode && inputs[0]->getDtype() != DType_INT8 && inputs[0]->getDtype() != DType_INT16)
            return error("%s has no precise-mode (fp64) evaluation in this library", "CONV3D");
        tmi_conv3d_desc_t d;
        if (fill_desc(d))
            return 1;
        int32_t in_zp = 0, w_zp = 0;
        if (!inputs[3]->scalar_value(in_zp) || !inputs[4]->scalar_value(w_zp))
            return error("zero-point operands must be available on the host");
        if (inputs[1]->getDtype() == DType_INT4 && w_zp != 0)    // tensor_ops.cpp:1037, :2119
            return error("Weight zero point must be zero for non int8_t data");
        SubgraphTraverser* s = parent_sgt;
        if (call(tmi_conv3d(s->ctx, &d, s->device(inputs[0]), s->device(inputs[1]), s->device(inputs[2]), in_zp, w_zp,
                            s->device_out(outputs[0]))))
            return 1;
        return GraphNode::eval();
    }
};

// MATMUL: operands [a, b, a_zp, b_zp]
class OpMatMul : public GraphNode
{
public:
    OpMatMul(SubgraphTraverser* sgt, uint64_t id) : GraphNode(sgt, Op_MATMUL, id)
    {
        requiredInputCount  = 4;
        requiredOutputCount = 1;
    }
    int checkTensorAttributes() override
    {
        if (validateRequiredOperands())
            return 1;
        if (validateRequiredRank(inputs[0], 3, 3) || validateRequiredRank(inputs[1], 3, 3) ||
            validateRequiredRank(inputs[2], 1, 1) || validateRequiredRank(inputs[3], 1, 1) ||
            validateRequiredRank(outputs[0], 3, 3))
            return 1;
        const Tensor *a = inputs[0], *b = inputs[1], *o = outputs[0];
        if (a->shape[0] != b->shape[0] || a->shape[0] != o->shape[0])
            return error("OpMatMul operator a.shape[0], b.shape[0] and output.shape[0] should match");
        if (a->shape[2] != b->shape[1])
            return error("OpMatMul operator a.shape[2] should match b.shape[1]");
        if (a->shape[1] != o->shape[1])
            return error("OpMatMul operator a.shape[1] should match output.shape[1]");
        if (b->shape[2] != o->shape[2])
            return error("OpMatMul operator output.shape[2] should match output.shape[2]");
        if (inputs[2]->shape[0] != 1)
            return error("OpMatMul: 'a_zp' zero point shape should be [1]");
        if (inputs[3]->shape[0] != 1)
            return error("OpMatMul: 'b_zp' zero point shape should be [1]");
        const DType in = a->getDtype();
        // the instantiations of tensor_ops.cpp:2256-2261 that the library has: INT8 -> INT32, INT16 -> INT48, floating
        // point -> FP32
        if (b->getDtype() != in ||
            !(in == DType_INT8 || in == DType_INT16 || in == DType_FP16 || in == DType_BF16 || in == DType_FP32))
            return error("OpMatMul: input data type not supported for this configuration of operator");
        if (o->getDtype() != (in == DType_INT8 ? DType_INT32 : (in == DType_INT16 ? DType_INT48 : DType_FP32)))
            return error("OpMatMul: Output data type not supported for this configuration of operator");
        return 0;
    }
    int eval() override
    {
        int32_t a_zp = 0, b_zp = 0;
        if (!inputs[2]->scalar_value(a_zp) || !inputs[3]->scalar_value(b_zp))
            return error("zero-point operands must be available on the host");
        const Tensor *a = inputs[0], *b = inputs[1];
        SubgraphTraverser* s = parent_sgt;
        if (s->precise_mode && a->getDtype() != DType_INT8 && a->getDtype() != DType_INT16)
        {
            // precise mode (tensor_ops.cpp:1436-1443)
            outputs[0]->precise = true;
            if (call(tmi_matmul_precise(s->ctx, tmi_dtype(a->getDtype()), a->shape[0], a->shape[1], a->shape[2],
                                        b->shape[2], s->device(inputs[0]), s->device(inputs[1]), s->bounds_mode ? 1 : 0,
                                        static_cast<double*>(s->device_out(outputs[0])))))
                return 1;
            return GraphNode::eval();
        }
        if (call(tmi_matmul(s->ctx, tmi_dtype(a->getDtype()), a->shape[0], a->shape[1], a->shape[2], b->shape[2],
                            s->device(inputs[0]), s->device(inputs[1]), a_zp, b_zp, s->device_out(outputs[0]))))
            return 1;
        return GraphNode::eval();
    }
};

}    // namespace

// ---- SubgraphTraverser -----------------------------------------------------------------------------------
SubgraphTraverser::SubgraphTraverser(const BasicBlock& b, int device) : block(b), device_id(device)
{
    if (tmi_ctx_create(&ctx, device_id) != TMI_VALID)
    {
        ctx          = nullptr;
        last_message = "no usable MI355X / HIP device: this runtime has no CPU fall-back";
        status       = GraphStatus::TOSA_ERROR;
    }
}

SubgraphTraverser::~SubgraphTraverser()
{
    if (ctx)
    {
        for (auto& t : tensors)
            if (t->dev)
                tmi_buf_free(ctx, t->dev);
        tmi_ctx_destroy(ctx);
    }
}

void SubgraphTraverser::setGraphStatus(GraphStatus s)
{
    // ERROR_IF does not override an earlier UNPREDICTABLE; REQUIRE always sets UNPREDICTABLE
    // (reference_model/include/func_debug.h:112-158)
    if (s == GraphStatus::TOSA_ERROR && status == GraphStatus::TOSA_UNPREDICTABLE)
        return;
    status = s;
}

Tensor* SubgraphTraverser::findTensorByName(const std::string& name) const
{
    auto it = by_name.find(name);
    return it == by_name.end() ? nullptr : it->second;
}

int SubgraphTraverser::initializeGraph()
{
    if (!ctx)
        return 1;
    for (const TensorDesc& d : block.tensors)
    {
        if (dtype_size(d.dtype) == 0)
        {
            last_message = "tensor " + d.name + ": element type outside the accelerated path";
            setGraphStatus(GraphStatus::TOSA_ERROR);
            return 1;
        }
        tensors.emplace_back(new Tensor(d));
        Tensor* t = tensors.back().get();
        if (by_name.count(d.name))
        {
            last_message = "duplicate tensor name " + d.name;
            setGraphStatus(GraphStatus::TOSA_ERROR);
            return 1;
        }
        by_name[d.name] = t;
        if (!d.data.empty())
        {
            // an INT48 element takes 6 bytes in the serialized payload and one int64 in memory
            // (reference: subgraph_traverser.cpp:652-656, ConvertU8toI48)
            // an INT4 element takes half a byte in the payload, the first of a pair in the low half, and one int8 in memory
            // (reference: subgraph_traverser.cpp:625-630, ConvertU8toI4 of the serialization library, whose source the
            // reference does not hold: the pair order is that library's published one, with no stored graph to confirm it)
            const bool i48      = d.dtype == DType_INT48;
            const bool i4       = d.dtype == DType_INT4;
            const size_t stored = i48 ? (size_t)t->getElementCount() * 6 : (i4 ? ((size_t)t->getElementCount() + 1) / 2 : t->bytes());
            if (d.data.size() < stored)
            {
                last_message = "tensor " + d.name + ": constant payload shorter than the tensor";
                setGraphStatus(GraphStatus::TOSA_ERROR);
                return 1;
            }
            if (i48)
            {
                t->host.resize(t->bytes());
                for (size_t e = 0; e < (size_t)t->getElementCount(); e++)
                {
                    uint64_t v = 0;
                    for (int b = 0; b < 6; b++)
                        v |= (uint64_t)d.data[e * 6 + b] << (8 * b);
                    if (v & 0x800000000000ull)
                        v |= 0xFFFF000000000000ull;
                    memcpy(t->host.data() + e * 8, &v, 8);
                }
            }
            else if (i4)
            {
                t->host.resize(t->bytes());
                for (size_t e = 0; e < (size_t)t->getElementCount(); e++)
                {
                    const uint8_t nib = (uint8_t)((d.data[e / 2] >> (4 * (e & 1))) & 0xf);
                    t->host[e]        = (uint8_t)(int8_t)((nib & 8) ? (int)nib - 16 : (int)nib);
                }
            }
            else
                t->host.assign(d.data.begin(), d.data.begin() + (std::ptrdiff_t)t->bytes());
            t->host_valid = true;
            t->is_const   = true;
        }
    }
    uint64_t id = 0;
    for (const OperatorDesc& o : block.operators)
    {
        GraphNode* n = nullptr;
        switch (o.op)
        {
            case Op_CONST:
                n = new OpConst(this, id);
                break;
            case Op_CONV2D:
                n = new OpConv2d(this, id);
                break;
            case Op_DEPTHWISE_CONV2D:
                n = new OpDepthwiseConv2d(this, id);
                break;
            case Op_AVG_POOL2D:
            case Op_MAX_POOL2D:
                n = new OpPool2d(this, (Op)o.op, id);
                break;
            case Op_TRANSPOSE_CONV2D:
                n = new OpTransposeConv2d(this, id);
                break;
            case Op_CONV3D:
                n = new OpConv3d(this, id);
                break;
            case Op_MATMUL:
                n = new OpMatMul(this, id);
                break;
            case Op_RESCALE:
                n = new OpRescale(this, id);
                break;
            case Op_CLAMP:
                n = new OpClamp(this, id);
                break;
            default:
                last_message = "operator " + std::to_string(o.op) + " is outside the accelerated path "
                               "(CONV2D, CONV3D, DEPTHWISE_CONV2D, TRANSPOSE_CONV2D, MATMUL, RESCALE, CLAMP, AVG_POOL2D, MAX_POOL2D)";
                setGraphStatus(GraphStatus::TOSA_ERROR);
                return 1;
        }
        n->attribute   = o.attr;
        n->inputNames  = o.inputs;
        n->outputNames = o.outputs;
        nodes.emplace_back(n);
        id++;
    }
    return 0;
}

int SubgraphTraverser::linkTensorsAndNodes()
{
    for (auto& n : nodes)
    {
        for (const std::string& nm : n->inputNames)
        {
            Tensor* t = findTensorByName(nm);
            if (!t)
            {
                last_message = "input tensor " + nm + " not found";
                setGraphStatus(GraphStatus::TOSA_ERROR);
                return 1;
            }
            n->inputs.push_back(t);
            t->consumers.push_back(n.get());
        }
        for (const std::string& nm : n->outputNames)
        {
            Tensor* t = findTensorByName(nm);
            if (!t)
            {
                last_message = "output tensor " + nm + " not found";
                setGraphStatus(GraphStatus::TOSA_ERROR);
                return 1;
            }
            if (t->producer && t->producer->nodeType != Op_CONST)
            {
                last_message = "tensor " + nm + " has two producers";
                setGraphStatus(GraphStatus::TOSA_ERROR);
                return 1;
            }
            n->outputs.push_back(t);
            t->producer = n.get();
        }
    }
    for (const std::string& nm : block.inputs)
        if (Tensor* t = findTensorByName(nm))
            t->is_graph_io = true;
    for (const std::string& nm : block.outputs)
        if (Tensor* t = findTensorByName(nm))
            t->is_graph_io = true;

    // Peephole: CONV2D / DEPTHWISE_CONV2D (INT8) -> RESCALE [-> CLAMP] where each intermediate has exactly one
    // consumer and is not a graph output becomes one fused kernel; the consumers only mark their outputs valid.
    if (enable_fusion)
    {
        for (auto& n : nodes)
        {
            if (n->nodeType != Op_CONV2D && n->nodeType != Op_DEPTHWISE_CONV2D)
                continue;
            if (n->inputs.size() != 5 || n->outputs.size() != 1 || n->inputs[0]->getDtype() != DType_INT8)
                continue;
            Tensor* acc = n->outputs[0];
            if (acc->is_graph_io || acc->consumers.size() != 1 || acc->consumers[0]->nodeType != Op_RESCALE)
                continue;
            GraphNode* rs = acc->consumers[0];
            if (rs->inputs.size() != 5 || rs->inputs[0] != acc || rs->outputs.size() != 1)
                continue;
            // the fused kernel reads the RESCALE's multiplier / shift / zero points when the convolution runs: they must
            // hold their values by then (constants or graph inputs), which the ready list only guarantees for the
            // convolution's own operands
            bool settled = true;
            for (int i = 1; i < 5; i++)
                settled = settled && (rs->inputs[i]->is_const || rs->inputs[i]->producer == nullptr);
            if (!settled)
                continue;
            ConvBase* conv      = static_cast<ConvBase*>(n.get());
            conv->fused_rescale = rs;
            rs->folded          = true;
            Tensor* q           = rs->outputs[0];
            if (!q->is_graph_io && q->consumers.size() == 1 && q->consumers[0]->nodeType == Op_CLAMP &&
                q->consumers[0]->outputs.size() == 1 &&
                (q->getDtype() == DType_INT8 || q->getDtype() == DType_INT16))
            {
                conv->fused_clamp         = q->consumers[0];
                q->consumers[0]->folded   = true;
            }
        }
    }
    return 0;
}

int SubgraphTraverser::validateGraph()
{
    for (auto& n : nodes)
        if (n->checkTensorAttributes())
        {
            setGraphStatus(GraphStatus::TOSA_ERROR);
            return 1;
        }
    // A tensor that an operator names is never allocated with a dimension of zero or less: the graph is
    // UNPREDICTABLE (reference: subgraph_traverser.cpp:579-590, SubgraphTraverser::allocateTensor).
    for (auto& n : nodes)
        for (const std::vector<Tensor*>* list : { &n->inputs, &n->outputs })
            for (Tensor* t : *list)
                for (int32_t dim : t->getShape())
                    if (dim <= 0)
                    {
                        last_message = "Failed to allocate tensor " + t->getName() + " with invalid dimension of " +
                                       std::to_string(dim);
                        setGraphStatus(GraphStatus::TOSA_UNPREDICTABLE);
                        return 1;
                    }
    return 0;
}

void* SubgraphTraverser::device_out(Tensor* t)
{
    if (!t->dev)
        if (tmi_buf_alloc(ctx, t->bytes(), &t->dev) != TMI_VALID)
            return nullptr;
    t->host_valid = false;
    return t->dev;
}

void* SubgraphTraverser::device(Tensor* t)
{
    if (t->dev_valid && t->dev)
        return t->dev;
    if (!t->host_valid)
    {
        // neither copy holds the tensor's value: an operand that no node has produced yet
        last_message = "tensor " + t->getName() + " is read before it has a value";
        setGraphStatus(GraphStatus::TOSA_ERROR);
        return nullptr;
    }
    if (!t->dev && tmi_buf_alloc(ctx, t->bytes(), &t->dev) != TMI_VALID)
        return nullptr;
    if (t->bytes())
        if (tmi_upload(ctx, t->dev, t->host.data(), t->bytes()) != TMI_VALID)
            return nullptr;
    t->dev_valid = true;
    return t->dev;
}

int SubgraphTraverser::download(Tensor* t)
{
    if (t->host_valid)
        return 0;
    if (!t->dev_valid || !t->dev)
        return 1;
    t->host.resize(t->bytes());
    if (t->bytes() && tmi_download(ctx, t->host.data(), t->dev, t->bytes()) != TMI_VALID)
        return 1;
    t->host_valid = true;
    return 0;
}

int SubgraphTraverser::evaluateAll()
{
    if (!ctx || status == GraphStatus::TOSA_ERROR)
        return 1;
    for (const std::string& nm : block.inputs)
    {
        Tensor* t = findTensorByName(nm);
        if (!t || !t->host_valid)
        {
            last_message = "graph input " + nm + " has not been set";
            setGraphStatus(GraphStatus::TOSA_ERROR);
            return 1;
        }
    }
    // ready-list evaluation (reference: subgraph_traverser.cpp:827-916): a node runs once all its inputs are
    // valid; a folded node's input is "valid" as soon as the producer of the fused chain has run
    std::vector<bool> done(nodes.size(), false);
    std::vector<int> remaining_uses(tensors.size(), 0);
    std::map<Tensor*, size_t> tindex;
    for (size_t i = 0; i < tensors.size(); i++)
    {
        tindex[tensors[i].get()]  = i;
        remaining_uses[i]         = (int)tensors[i]->consumers.size();
    }
    size_t n_done = 0;
    bool progress = true;
    while (n_done < nodes.size() && progress)
    {
        progress = false;
        for (size_t i = 0; i < nodes.size(); i++)
        {
            if (done[i])
                continue;
            GraphNode* n = nodes[i].get();
            bool ready   = true;
            for (Tensor* t : n->inputs)
            {
                const bool produced_by_fused = n->folded && t->producer && t == n->inputs[0];
                bool prod_done = false;
                if (produced_by_fused)
                    for (size_t j = 0; j < nodes.size(); j++)
                        if (nodes[j].get() == t->producer)
                            prod_done = done[j];
                if (!(t->host_valid || t->dev_valid || prod_done))
                    ready = false;
            }
            if (!ready)
                continue;
            // the fp64 passes take operands in their storage type: a chain of floating-point operators in
            // precise mode is outside this path
            for (Tensor* t : n->inputs)
                if (t->precise)
                {
                    last_message = std::string(op_name(n->nodeType)) + ": operand " + t->name +
                                   " is an fp64 precise-mode result; only graph inputs and constants are taken";
                    setGraphStatus(GraphStatus::TOSA_ERROR);
                    return 1;
                }
            if (n->eval())
                return 1;
            done[i]  = true;
            progress = true;
            n_done++;
            // release device memory of inputs that no later node needs (subgraph_traverser.cpp:865-903)
            for (Tensor* t : n->inputs)
            {
                int& uses = remaining_uses[tindex[t]];
                if (--uses == 0 && !t->is_graph_io && !t->is_const && t->dev)
                {
                    tmi_buf_free(ctx, t->dev);
                    t->dev       = nullptr;
                    t->dev_valid = false;
                }
            }
        }
    }
    if (n_done < nodes.size())
    {
        last_message = "graph has nodes whose inputs never become available";
        setGraphStatus(GraphStatus::TOSA_ERROR);
        return 1;
    }
    for (const std::string& nm : block.outputs)
    {
        Tensor* t = findTensorByName(nm);
        if (!t || download(t))
        {
            last_message = "graph output " + nm + " was not produced";
            setGraphStatus(GraphStatus::TOSA_ERROR);
            return 1;
        }
    }
    const int rc = tmi_ctx_sync(ctx);
    if (rc == TMI_UNPREDICTABLE)
    {
        const uint32_t flags = tmi_ctx_flags(ctx);
        if (flags & TMI_FLAG_LEVEL)
            last_message = std::string("LEVEL_CHECK() fails: ") + tmi_last_error(ctx);
        else
            last_message = "OpRescale failure: a REQUIRE condition of apply_scale fired (flags " + std::to_string(flags) + ")";
        setGraphStatus(GraphStatus::TOSA_UNPREDICTABLE);
    }
    else if (rc == TMI_ERROR)
    {
        last_message = tmi_last_error(ctx);
        setGraphStatus(GraphStatus::TOSA_ERROR);
        return 1;
    }
    return 0;
}

// ---- ModelRunner -----------------------------------------------------------------------------------------
GraphStatus ModelRunner::initialize(const BasicBlock& block)
{
    sgt.reset(new SubgraphTraverser(block, device_id));
    sgt->enable_fusion = fusion;
    sgt->precise_mode  = precise_mode;
    sgt->bounds_mode   = bounds_mode;
    if (sgt->ctx)
    {
        tmi_ctx_set_level(sgt->ctx, &level);
        tmi_ctx_set_precise_mode(sgt->ctx, precise_mode, compliance_mode, bounds_mode);
    }
    if (sgt->initializeGraph() || sgt->linkTensorsAndNodes() || sgt->validateGraph())
        return sgt->getGraphStatus() == GraphStatus::TOSA_VALID ? GraphStatus::TOSA_ERROR : sgt->getGraphStatus();
    return sgt->getGraphStatus();
}

int ModelRunner::setInput(const std::string& name, const uint8_t* raw, size_t size)
{
    Tensor* t = sgt ? sgt->findTensorByName(name) : nullptr;
    if (!t || size != t->bytes())
        return 1;
    t->host.assign(raw, raw + size);
    t->host_valid = true;
    t->dev_valid  = false;
    return 0;
}

GraphStatus ModelRunner::run()
{
    if (!sgt)
        return GraphStatus::TOSA_ERROR;
    sgt->evaluateAll();
    return sgt->getGraphStatus();
}

int ModelRunner::getOutput(const std::string& name, uint8_t* raw, size_t size)
{
    Tensor* t = sgt ? sgt->findTensorByName(name) : nullptr;
    if (!t || !t->host_valid || size != t->bytes())
        return 1;
    memcpy(raw, t->host.data(), size);
    return 0;
}

}    // namespace tmi_host
