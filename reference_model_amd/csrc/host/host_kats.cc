// Known-answer tests of the host adapter, written the way the reference's own operator tests are: build a
// one-operator graph in memory, set the inputs, run, read the outputs (RefModelTestBuilder:
// reference_model/test/include/test_utils.h:75-183).  The vectors are the literal ones of
// reference_model/test/ref_model_tests/tensor_ops_tests.cpp:622-683, 736-798 and type_conversion_tests.cpp:324-383.
// Prints one line per case; exit code 0 only if every case passes.  Needs a GPU.
#include <cstdio>
#include <cstring>

#include "tosa_host.h"

using namespace tmi_host;

namespace
{

int failures = 0;

struct Builder
{
    BasicBlock block;
    ModelRunner runner{ 0 };
    OperatorDesc op;
    int n_in = 0;
    void addInput(const std::vector<int32_t>& shape, DType t)
    {
        TensorDesc d;
        d.name  = "in" + std::to_string(n_in++);
        d.shape = shape;
        d.dtype = t;
        block.tensors.push_back(d);
        block.inputs.push_back(d.name);
        op.inputs.push_back(d.name);
    }
    void addOutput(const std::vector<int32_t>& shape, DType t)
    {
        TensorDesc d;
        d.name  = "out0";
        d.shape = shape;
        d.dtype = t;
        block.tensors.push_back(d);
        block.outputs.push_back(d.name);
        op.outputs.push_back(d.name);
    }
    GraphStatus initializeRunner(uint32_t opcode, const Attribute& a)
    {
        op.op   = opcode;
        op.attr = a;
        block.operators.push_back(op);
        return runner.initialize(block);
    }
    template <typename T>
    void setInput(int i, const std::vector<T>& v)
    {
        if (runner.setInput("in" + std::to_string(i), reinterpret_cast<const uint8_t*>(v.data()), v.size() * sizeof(T)))
        {
            printf("  setInput(%d) failed\n", i);
            failures++;
        }
    }
    template <typename T>
    std::vector<T> getOutput(size_t n)
    {
        std::vector<T> v(n);
        if (runner.getOutput("out0", reinterpret_cast<uint8_t*>(v.data()), n * sizeof(T)))
        {
            printf("  getOutput failed\n");
            failures++;
        }
        return v;
    }
};

template <typename T>
void expect(const char* name, const std::vector<T>& got, const std::vector<T>& want)
{
    const bool ok = got == want;
    printf("%s %s\n", ok ? "PASS" : "FAIL", name);
    if (!ok)
    {
        failures++;
        for (size_t i = 0; i < got.size() && i < want.size(); i++)
            printf("   [%zu] got %lld want %lld\n", i, (long long)got[i], (long long)want[i]);
    }
}

Attribute convAttr(std::vector<int32_t> stride)
{
    Attribute a;
    a.pad         = { 0, 0, 0, 0 };
    a.stride      = stride;
    a.dilation    = { 1, 1 };
    a.local_bound = true;
    a.acc_type    = DType_INT32;
    return a;
}

void testConv2d(const char* name, std::vector<int8_t> in, std::vector<int8_t> w, int8_t izp, int8_t wzp, bool depthwise)
{
    Builder tb;
    tb.addInput({ 1, 2, 2, 1 }, DType_INT8);
    tb.addInput(depthwise ? std::vector<int32_t>{ 2, 2, 1, 1 } : std::vector<int32_t>{ 1, 2, 2, 1 }, DType_INT8);
    tb.addInput({ 1 }, DType_INT32);
    tb.addInput({ 1 }, DType_INT8);
    tb.addInput({ 1 }, DType_INT8);
    tb.addOutput({ 1, 1, 1, 1 }, DType_INT32);
    if (tb.initializeRunner(depthwise ? Op_DEPTHWISE_CONV2D : Op_CONV2D, convAttr({ 2, 2 })) != GraphStatus::TOSA_VALID)
    {
        printf("FAIL %s (initialize)\n", name);
        failures++;
        return;
    }
    int32_t want = 0;
    for (size_t i = 0; i < in.size(); i++)
        want += ((int32_t)in[i] - izp) * ((int32_t)w[i] - wzp);
    tb.setInput(0, in);
    tb.setInput(1, w);
    tb.setInput(2, std::vector<int32_t>{ 0 });
    tb.setInput(3, std::vector<int8_t>{ izp });
    tb.setInput(4, std::vector<int8_t>{ wzp });
    const GraphStatus st = tb.runner.run();
    if (st != GraphStatus::TOSA_VALID)
    {
        printf("FAIL %s (run status %d: %s)\n", name, (int)st, tb.runner.traverser()->last_message.c_str());
        failures++;
        return;
    }
    expect(name, tb.getOutput<int32_t>(1), std::vector<int32_t>{ want });
}

void testMatMul(const char* name, std::vector<int8_t> a, std::vector<int8_t> b, int8_t azp, int8_t bzp)
{
    Builder tb;
    tb.addInput({ 1, 2, 2 }, DType_INT8);
    tb.addInput({ 1, 2, 2 }, DType_INT8);
    tb.addInput({ 1 }, DType_INT8);
    tb.addInput({ 1 }, DType_INT8);
    tb.addOutput({ 1, 2, 2 }, DType_INT32);
    if (tb.initializeRunner(Op_MATMUL, Attribute()) != GraphStatus::TOSA_VALID)
    {
        printf("FAIL %s (initialize)\n", name);
        failures++;
        return;
    }
    std::vector<int32_t> want(4, 0);
    for (int r = 0; r < 2; r++)
        for (int c = 0; c < 2; c++)
            for (int k = 0; k < 2; k++)
                want[r * 2 + c] += ((int32_t)a[r * 2 + k] - azp) * ((int32_t)b[k * 2 + c] - bzp);
    tb.setInput(0, a);
    tb.setInput(1, b);
    tb.setInput(2, std::vector<int8_t>{ azp });
    tb.setInput(3, std::vector<int8_t>{ bzp });
    if (tb.runner.run() != GraphStatus::TOSA_VALID)
    {
        printf("FAIL %s (run)\n", name);
        failures++;
        return;
    }
    expect(name, tb.getOutput<int32_t>(4), want);
}

void testConv2dBias(const char* name, std::vector<int32_t> bias, std::vector<int32_t> want, bool depthwise)
{
    Builder tb;
    tb.addInput({ 1, 1, 1, 2 }, DType_INT8);
    tb.addInput(depthwise ? std::vector<int32_t>{ 1, 1, 2, 1 } : std::vector<int32_t>{ 2, 1, 1, 2 }, DType_INT8);
    tb.addInput({ (int32_t)bias.size() }, DType_INT32);
    tb.addInput({ 1 }, DType_INT8);
    tb.addInput({ 1 }, DType_INT8);
    tb.addOutput({ 1, 1, 1, 2 }, DType_INT32);
    if (tb.initializeRunner(depthwise ? Op_DEPTHWISE_CONV2D : Op_CONV2D, convAttr({ 1, 1 })) != GraphStatus::TOSA_VALID)
    {
        printf("FAIL %s (initialize)\n", name);
        failures++;
        return;
    }
    tb.setInput(0, std::vector<int8_t>{ 5, 9 });
    tb.setInput(1, depthwise ? std::vector<int8_t>{ 3, -7 } : std::vector<int8_t>{ 3, -7, -1, 4 });
    tb.setInput(2, bias);
    tb.setInput(3, std::vector<int8_t>{ 0 });
    tb.setInput(4, std::vector<int8_t>{ 0 });
    if (tb.runner.run() != GraphStatus::TOSA_VALID)
    {
        printf("FAIL %s (run)\n", name);
        failures++;
        return;
    }
    expect(name, tb.getOutput<int32_t>(2), want);
}

// type_conversion_tests.cpp:104-164: rank-1 RESCALE; expect_fail means TOSA_ERROR at initialize or run
template <typename IN, typename OUT, typename SCALE>
void testRescale(const char* name, std::vector<IN> in, std::vector<OUT> want, std::vector<SCALE> mult,
                 std::vector<int8_t> shift, Attribute attr, IN izp, OUT ozp, bool expect_fail, DType it, DType ot, DType st)
{
    Builder tb;
    tb.addInput({ (int32_t)in.size() }, it);
    tb.addInput({ (int32_t)mult.size() }, st);
    tb.addInput({ (int32_t)shift.size() }, DType_INT8);
    tb.addInput({ 1 }, it);
    tb.addInput({ 1 }, ot);
    tb.addOutput({ (int32_t)in.size() }, ot);
    GraphStatus s = tb.initializeRunner(Op_RESCALE, attr);
    if (s == GraphStatus::TOSA_ERROR)
    {
        printf("%s %s (rejected at initialize)\n", expect_fail ? "PASS" : "FAIL", name);
        failures += !expect_fail;
        return;
    }
    tb.setInput(0, in);
    tb.setInput(1, mult);
    tb.setInput(2, shift);
    tb.setInput(3, std::vector<IN>{ izp });
    tb.setInput(4, std::vector<OUT>{ ozp });
    s = tb.runner.run();
    if (expect_fail)
    {
        printf("%s %s (run status %d)\n", s == GraphStatus::TOSA_ERROR ? "PASS" : "FAIL", name, (int)s);
        failures += s != GraphStatus::TOSA_ERROR;
        return;
    }
    if (s != GraphStatus::TOSA_VALID)
    {
        printf("FAIL %s (run status %d)\n", name, (int)s);
        failures++;
        return;
    }
    expect(name, tb.getOutput<OUT>(want.size()), want);
}

Attribute rescaleAttr(bool scale32, uint32_t mode, bool per_channel, bool in_u, bool out_u)
{
    Attribute a;
    a.scale32 = scale32, a.rounding_mode = mode, a.per_channel = per_channel;
    a.input_unsigned = in_u, a.output_unsigned = out_u;
    return a;
}

}    // namespace

int main()
{
    struct
    {
        const char* name;
        std::vector<int8_t> in, w;
        int8_t izp, wzp;
    } zp[] = { { "input negative overflow", { 126, -126, -120, 0 }, { 2, 1, 4, -7 }, 4, 15 },
               { "input positive overflow", { 122, -7, -120, 121 }, { 2, 1, 4, -7 }, -10, -5 },
               { "weight negative overflow", { 3, -12, 5, 70 }, { -120, -12, 0, -7 }, 55, 15 },
               { "weight positive overflow", { -5, 65, -1, 32 }, { -2, 125, 4, -1 }, -10, -5 } };
    for (auto& c : zp)
    {
        char nm[128];
        snprintf(nm, sizeof(nm), "CONV2D zero point: %s", c.name);
        testConv2d(nm, c.in, c.w, c.izp, c.wzp, false);
        snprintf(nm, sizeof(nm), "DEPTHWISE_CONV2D zero point: %s", c.name);
        testConv2d(nm, c.in, c.w, c.izp, c.wzp, true);
        snprintf(nm, sizeof(nm), "MATMUL zero point: %s", c.name);
        testMatMul(nm, c.in, c.w, c.izp, c.wzp);
    }
    testConv2dBias("CONV2D bias broadcasted", { -5 }, { -53, 26 }, false);
    testConv2dBias("CONV2D bias not broadcasted", { -5, 14 }, { -53, 45 }, false);
    testConv2dBias("DEPTHWISE_CONV2D bias broadcasted", { -5 }, { 10, -68 }, true);
    testConv2dBias("DEPTHWISE_CONV2D bias not broadcasted", { -5, 14 }, { 10, -49 }, true);

    testRescale<int8_t, uint16_t, int16_t>("RESCALE value_extend64 of output_zp", { 65 }, { 32832 }, { 4 }, { 2 },
                                           rescaleAttr(false, TMI_ROUND_SINGLE, false, false, true), 1, 32768, false,
                                           DType_INT8, DType_INT16, DType_INT16);
    testRescale<int8_t, int32_t, int32_t>("RESCALE per_channel, size(multiplier) != NC", { 20, -5, -16 }, { 0 }, { 4, 2 },
                                          { 16, 5, 9 }, rescaleAttr(true, TMI_ROUND_SINGLE, true, false, false), -19, 0,
                                          true, DType_INT8, DType_INT32, DType_INT32);
    testRescale<int32_t, int8_t, int16_t>("RESCALE per_channel, size(shift) != NC", { 0, -12, 0, 12 }, { 0 },
                                          { 4, 1024, 2048, 115 }, { 12 },
                                          rescaleAttr(false, TMI_ROUND_SINGLE, true, false, false), 0, -12, true,
                                          DType_INT32, DType_INT8, DType_INT16);
    testRescale<int8_t, int32_t, int32_t>("RESCALE per_tensor, size(multipliers) > 1", { 20, -5, -16 }, { 0 }, { 4, 519 },
                                          { 12 }, rescaleAttr(true, TMI_ROUND_SINGLE, false, false, false), -19, 0, true,
                                          DType_INT8, DType_INT32, DType_INT32);
    testRescale<int32_t, int8_t, int16_t>("RESCALE per_tensor, size(shifts) > 1", { 0, -12, 0, 12 }, { 0 }, { 4 }, { 6, 16 },
                                          rescaleAttr(false, TMI_ROUND_SINGLE, false, false, false), 0, -12, true,
                                          DType_INT32, DType_INT8, DType_INT16);
    testRescale<int8_t, uint16_t, int16_t>("RESCALE inexact round, unsigned output", { 65 }, { 32832 }, { 4 }, { 2 },
                                           rescaleAttr(false, TMI_ROUND_INEXACT, false, false, true), 1, 32768, false,
                                           DType_INT8, DType_INT16, DType_INT16);
    testRescale<int8_t, uint8_t, int16_t>("RESCALE inexact round, uint8 output", { 103 }, { 114 }, { 147 }, { 8 },
                                          rescaleAttr(false, TMI_ROUND_INEXACT, false, false, true), -95, 0, false,
                                          DType_INT8, DType_INT8, DType_INT16);
    printf("%d failure(s)\n", failures);
    return failures ? 1 : 0;
}
