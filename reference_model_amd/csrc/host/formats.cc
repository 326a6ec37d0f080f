// Readers/writers for the reference's on-disk formats: TOSA flatbuffer graphs and NumPy .npy tensors.
// No flatbuffers library or schema compiler is used: tables are walked generically (root offset -> vtable ->
// field offsets) with the field numbers of the TOSA 1.0 schema:
//   TosaGraph       0 version, 1 regions[]            TosaRegion   0 name, 1 blocks[]
//   TosaBasicBlock  0 name, 1 operators[], 2 tensors[], 3 inputs[str], 4 outputs[str]
//   TosaTensor      0 name, 1 shape[int32], 2 type(uint32), 3 data[ubyte]
//   TosaOperator    0 op(uint32), 1 attribute_type(ubyte), 2 attribute(table), 3 inputs[str], 4 outputs[str]
//   Conv2dAttribute / DepthwiseConv2dAttribute / Conv3dAttribute  0 pad, 1 stride, 2 dilation, 3 local_bound, 4 acc_type
//   TransposeConv2dAttribute  0 out_pad, 1 stride, 2 local_bound, 3 acc_type
//   AvgPool2dAttribute        0 kernel, 1 stride, 2 pad, 3 acc_type
//   MaxPool2dAttribute        0 kernel, 1 stride, 2 pad, 3 nan_mode
//   RescaleAttribute  0 scale32, 1 rounding_mode, 2 per_channel, 3 input_unsigned, 4 output_unsigned
//   ClampAttribute    0 min_val[ubyte], 1 max_val[ubyte], 2 nan_mode
// The numbers of the Conv2d, Rescale and tensor / operator tables are confirmed by the reference's example graphs.  Those of
// the TransposeConv2d, pooling and Clamp attributes have no stored graph to confirm them; they follow the argument order in
// which the reference's test generator hands the fields to the serializer (verif/generator/tosa_test_gen.py:910, 974,
// 1239, 1522), the correspondence that the confirmed Conv2dAttribute (:1065) and RescaleAttribute (:2290) show.
#include <cstdio>
#include <cstring>
#include <fstream>
#include <sstream>

#include "tosa_host.h"

namespace tmi_host
{

size_t dtype_size(DType t)
{
    switch (t)
    {
        case DType_INT4:    // one value per byte in memory and in .npy files; two per byte in a .tosa payload
        case DType_INT8:
            return 1;
        case DType_INT16:
        case DType_FP16:
        case DType_BF16:
            return 2;
        case DType_INT32:
        case DType_FP32:
            return 4;
        case DType_INT48:
            return 8;    // one int64 per element in memory and in .npy files; 6 bytes in a .tosa payload
        default:
            return 0;
    }
}

const char* op_name(uint32_t op)
{
    switch (op)
    {
        case Op_CONV2D:
            return "CONV2D";
        case Op_CONV3D:
            return "CONV3D";
        case Op_TRANSPOSE_CONV2D:
            return "TRANSPOSE_CONV2D";
        case Op_AVG_POOL2D:
            return "AVG_POOL2D";
        case Op_MAX_POOL2D:
            return "MAX_POOL2D";
        case Op_DEPTHWISE_CONV2D:
            return "DEPTHWISE_CONV2D";
        case Op_MATMUL:
            return "MATMUL";
        case Op_CLAMP:
            return "CLAMP";
        case Op_RESCALE:
            return "RESCALE";
        case Op_CONST:
            return "CONST";
        case Op_IDENTITY:
            return "IDENTITY";
        default:
            return "(operator outside the accelerated path)";
    }
}

namespace
{

// Bounds-checked view of a flatbuffer table.
struct Buf
{
    const uint8_t* p;
    size_t n;
    bool ok = true;
    template <typename T>
    T rd(size_t off)
    {
        T v{};
        if (off + sizeof(T) > n)
        {
            ok = false;
            return v;
        }
        memcpy(&v, p + off, sizeof(T));
        return v;
    }
};

struct Table
{
    Buf* b;
    size_t pos = 0, vt = 0;
    uint16_t vt_len = 0;
    bool valid      = false;
    Table() : b(nullptr) {}
    Table(Buf* b_, size_t pos_) : b(b_), pos(pos_)
    {
        const int32_t so = b->rd<int32_t>(pos);
        vt               = (size_t)((int64_t)pos - so);
        vt_len           = b->rd<uint16_t>(vt);
        valid            = b->ok;
    }
    size_t field(int f)
    {
        const size_t o = 4 + 2 * (size_t)f;
        if (!valid || o + 2 > vt_len)
            return 0;
        const uint16_t fo = b->rd<uint16_t>(vt + o);
        return fo ? pos + fo : 0;
    }
    template <typename T>
    T scalar(int f, T dflt)
    {
        const size_t a = field(f);
        return a ? b->rd<T>(a) : dflt;
    }
    size_t indirect(int f)
    {
        const size_t a = field(f);
        return a ? a + b->rd<uint32_t>(a) : 0;
    }
    Table table(int f)
    {
        const size_t a = indirect(f);
        return a ? Table(b, a) : Table();
    }
    std::string str_at(size_t a)
    {
        const uint32_t len = b->rd<uint32_t>(a);
        if (a + 4 + len > b->n)
        {
            b->ok = false;
            return "";
        }
        return std::string(reinterpret_cast<const char*>(b->p + a + 4), len);
    }
    std::string string(int f)
    {
        const size_t a = indirect(f);
        return a ? str_at(a) : "";
    }
    template <typename T>
    std::vector<T> vec(int f)
    {
        std::vector<T> out;
        const size_t a = indirect(f);
        if (!a)
            return out;
        const uint32_t len = b->rd<uint32_t>(a);
        if (a + 4 + (size_t)len * sizeof(T) > b->n)
        {
            b->ok = false;
            return out;
        }
        out.resize(len);
        if (len)
            memcpy(out.data(), b->p + a + 4, (size_t)len * sizeof(T));
        return out;
    }
    std::vector<Table> tables(int f)
    {
        std::vector<Table> out;
        const size_t a = indirect(f);
        if (!a)
            return out;
        const uint32_t len = b->rd<uint32_t>(a);
        for (uint32_t i = 0; i < len && b->ok; i++)
        {
            const size_t q = a + 4 + 4 * (size_t)i;
            out.emplace_back(b, q + b->rd<uint32_t>(q));
        }
        return out;
    }
    std::vector<std::string> strings(int f)
    {
        std::vector<std::string> out;
        const size_t a = indirect(f);
        if (!a)
            return out;
        const uint32_t len = b->rd<uint32_t>(a);
        for (uint32_t i = 0; i < len && b->ok; i++)
        {
            const size_t q = a + 4 + 4 * (size_t)i;
            out.push_back(str_at(q + b->rd<uint32_t>(q)));
        }
        return out;
    }
};

}    // namespace

bool load_tosa_file(const std::string& path, BasicBlock& block, std::string& err)
{
    std::ifstream f(path, std::ios::binary);
    if (!f)
    {
        err = "cannot open " + path;
        return false;
    }
    std::vector<uint8_t> bytes((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    if (bytes.size() < 8 || memcmp(bytes.data() + 4, "TOSA", 4) != 0)
    {
        err = path + ": not a TOSA flatbuffer (file identifier missing)";
        return false;
    }
    Buf b{ bytes.data(), bytes.size() };
    Table root(&b, b.rd<uint32_t>(0));
    auto regions = root.tables(1);
    if (regions.empty())
    {
        err = path + ": no region";
        return false;
    }
    auto blocks = regions[0].tables(1);
    if (blocks.empty())
    {
        err = path + ": no basic block";
        return false;
    }
    Table blk  = blocks[0];
    block      = BasicBlock();
    block.name = blk.string(0);
    for (Table& t : blk.tables(2))
    {
        TensorDesc d;
        d.name  = t.string(0);
        d.shape = t.vec<int32_t>(1);
        d.dtype = (DType)t.scalar<uint32_t>(2, 0);
        d.data  = t.vec<uint8_t>(3);
        block.tensors.push_back(std::move(d));
    }
    for (Table& o : blk.tables(1))
    {
        OperatorDesc d;
        d.op    = o.scalar<uint32_t>(0, 0);
        Table a = o.table(2);
        if (a.valid)
        {
            switch (d.op)
            {
                case Op_TRANSPOSE_CONV2D:    // out_pad, stride, local_bound, acc_type: the order of the
                                             // reference's TosaTransposeConv2dAttribute constructor
                                             // (tensor_ops_tests.cpp:293-296); no example graph confirms it
                    d.attr.pad         = a.vec<int32_t>(0);
                    d.attr.stride      = a.vec<int32_t>(1);
                    d.attr.local_bound = a.scalar<uint8_t>(2, 0) != 0;
                    d.attr.acc_type    = a.scalar<uint32_t>(3, 0);
                    break;
                case Op_AVG_POOL2D:    // kernel, stride, pad, acc_type / nan_mode: the order of the reference's
                case Op_MAX_POOL2D:    // TosaAvgPool2dAttribute constructor (tensor_ops_tests.cpp:539-540); no
                                       // example graph confirms it
                    d.attr.kernel = a.vec<int32_t>(0);
                    d.attr.stride = a.vec<int32_t>(1);
                    d.attr.pad    = a.vec<int32_t>(2);
                    if (d.op == Op_AVG_POOL2D)
                        d.attr.acc_type = a.scalar<uint32_t>(3, 0);
                    else
                        d.attr.nan_mode = a.scalar<uint32_t>(3, 0);
                    break;
                case Op_CONV2D:
                case Op_CONV3D:
                case Op_DEPTHWISE_CONV2D:
                    d.attr.pad         = a.vec<int32_t>(0);
                    d.attr.stride      = a.vec<int32_t>(1);
                    d.attr.dilation    = a.vec<int32_t>(2);
                    d.attr.local_bound = a.scalar<uint8_t>(3, 0) != 0;
                    d.attr.acc_type    = a.scalar<uint32_t>(4, 0);
                    break;
                case Op_RESCALE:
                    d.attr.scale32         = a.scalar<uint8_t>(0, 0) != 0;
                    d.attr.rounding_mode   = a.scalar<uint32_t>(1, 0);
                    d.attr.per_channel     = a.scalar<uint8_t>(2, 0) != 0;
                    d.attr.input_unsigned  = a.scalar<uint8_t>(3, 0) != 0;
                    d.attr.output_unsigned = a.scalar<uint8_t>(4, 0) != 0;
                    break;
                case Op_CLAMP:
                    d.attr.min_val  = a.vec<uint8_t>(0);
                    d.attr.max_val  = a.vec<uint8_t>(1);
                    d.attr.nan_mode = a.scalar<uint32_t>(2, 0);
                    break;
                default:
                    break;
            }
        }
        d.inputs  = o.strings(3);
        d.outputs = o.strings(4);
        block.operators.push_back(std::move(d));
    }
    block.inputs  = blk.strings(3);
    block.outputs = blk.strings(4);
    if (!b.ok)
    {
        err = path + ": truncated or malformed flatbuffer";
        return false;
    }
    return true;
}

// ---- .npy (format 1.0 / 2.0, C order only) -------------------------------------------------------------
const char* npy_descr_for(DType t)
{
    switch (t)
    {
        case DType_INT4:
        case DType_INT8:
            return "|i1";
        case DType_INT16:
            return "<i2";
        case DType_INT32:
            return "<i4";
        case DType_INT48:
            return "<i8";
        case DType_FP16:
            return "<f2";
        case DType_FP32:
            return "<f4";
        case DType_BF16:
            return "<u2";    // NumPy has no bfloat16: bit patterns
        default:
            return "";
    }
}

bool read_npy(const std::string& path, NpyArray& out, std::string& err)
{
    std::ifstream f(path, std::ios::binary);
    if (!f)
    {
        err = "cannot open " + path;
        return false;
    }
    std::vector<uint8_t> b((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    if (b.size() < 10 || memcmp(b.data(), "\x93NUMPY", 6) != 0)
    {
        err = path + ": not a .npy file";
        return false;
    }
    size_t hlen, hoff;
    if (b[6] == 1)
        hlen = b[8] | (b[9] << 8), hoff = 10;
    else
    {
        if (b.size() < 12)
        {
            err = path + ": truncated header";
            return false;
        }
        hlen = b[8] | (b[9] << 8) | (b[10] << 16) | ((size_t)b[11] << 24), hoff = 12;
    }
    if (hoff + hlen > b.size())
    {
        err = path + ": truncated header";
        return false;
    }
    const std::string h(reinterpret_cast<const char*>(b.data() + hoff), hlen);
    auto value_of = [&](const std::string& key) -> std::string {
        size_t k = h.find("'" + key + "'");
        if (k == std::string::npos)
            return "";
        k = h.find(':', k);
        return k == std::string::npos ? "" : h.substr(k + 1);
    };
    std::string d = value_of("descr");
    size_t q0 = d.find('\''), q1 = d.find('\'', q0 + 1);
    if (q0 == std::string::npos || q1 == std::string::npos)
    {
        err = path + ": unsupported descr";
        return false;
    }
    out.descr = d.substr(q0 + 1, q1 - q0 - 1);
    if (value_of("fortran_order").find("True") < 8)
    {
        err = path + ": fortran_order arrays are not supported";
        return false;
    }
    std::string s = value_of("shape");
    size_t p0 = s.find('('), p1 = s.find(')');
    out.shape.clear();
    if (p0 != std::string::npos && p1 != std::string::npos)
    {
        std::stringstream ss(s.substr(p0 + 1, p1 - p0 - 1));
        std::string tok;
        while (std::getline(ss, tok, ','))
        {
            bool digit = false;
            for (char c : tok)
                digit |= (c >= '0' && c <= '9');
            if (digit)
                out.shape.push_back(atoi(tok.c_str()));
        }
    }
    out.data.assign(b.begin() + hoff + hlen, b.end());
    return true;
}

bool write_npy(const std::string& path, const std::string& descr, const std::vector<int32_t>& shape,
               const void* data, size_t bytes, std::string& err)
{
    std::string sh = "(";
    for (size_t i = 0; i < shape.size(); i++)
        sh += std::to_string(shape[i]) + (shape.size() == 1 || i + 1 < shape.size() ? "," : "");
    sh += ")";
    std::string h = "{'descr': '" + descr + "', 'fortran_order': False, 'shape': " + sh + ", }";
    while ((10 + h.size() + 1) % 64 != 0)
        h += ' ';
    h += '\n';
    std::ofstream f(path, std::ios::binary);
    if (!f)
    {
        err = "cannot write " + path;
        return false;
    }
    const uint8_t pre[10] = { 0x93, 'N', 'U', 'M', 'P', 'Y', 1, 0, (uint8_t)(h.size() & 0xff), (uint8_t)(h.size() >> 8) };
    f.write(reinterpret_cast<const char*>(pre), 10);
    f.write(h.data(), (std::streamsize)h.size());
    f.write(reinterpret_cast<const char*>(data), (std::streamsize)bytes);
    return (bool)f;
}

}    // namespace tmi_host
