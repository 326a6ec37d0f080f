// Host side above the C ABI: a GraphNode-shaped adapter for the five operators of the hot path, the
// minimal graph runtime that drives it, and readers for the reference's on-disk formats.
//
// It mirrors the reference model's structure for this path (class and method names, operand order, status
// convention) so that a reference maintainer recognises every piece:
//   GraphNode::checkTensorAttributes / eval         reference_model/src/graph_node.h:176-179
//   SubgraphTraverser::initializeGraph ... evaluateAll  reference_model/src/subgraph_traverser.h:36-52
//   IModelRunner::initialize / setInput / run / getOutput  reference_model/include/model_runner.h:33-98
// but keeps tensors packed and device resident: an operator's eval() enqueues kernels through the C ABI
// (include/tosa_mi355.h) and hands a device pointer to its consumer; bytes come back to the host only for
// graph outputs.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "tosa_mi355.h"

namespace tmi_host
{

// reference_model/include/graph_status.h:18-23
enum class GraphStatus : int
{
    TOSA_VALID         = 0,
    TOSA_UNPREDICTABLE = 1,
    TOSA_ERROR         = 2,
};

// Operator and element-type numbers of the TOSA 1.0 serialization schema (CONV2D, RESCALE, CONST, INT8, INT32
// and FP32 are confirmed by the reference's example graphs).
enum Op : uint32_t
{
    Op_AVG_POOL2D       = 2,
    Op_CONV2D           = 3,
    Op_CONV3D           = 4,
    Op_DEPTHWISE_CONV2D = 5,
    Op_MATMUL           = 7,
    Op_MAX_POOL2D       = 8,
    Op_TRANSPOSE_CONV2D = 10,
    Op_CLAMP            = 11,
    Op_RESCALE          = 66,
    Op_CONST            = 67,
    Op_IDENTITY         = 68,
};

enum DType : uint32_t
{
    DType_UNKNOWN = 0,
    DType_BOOL    = 1,
    DType_INT4    = 2,
    DType_INT8    = 3,
    DType_INT16   = 4,
    DType_INT32   = 5,
    DType_INT48   = 6,
    DType_FP32    = 7,
    DType_FP16    = 8,
    DType_BF16    = 9,
};

size_t dtype_size(DType t);    // bytes per packed element, 0 if the type is not handled on this path
const char* op_name(uint32_t op);

// ---- serialized graph ------------------------------------------------------------------------------------
struct Attribute
{
    // Conv2dAttribute / DepthwiseConv2dAttribute / Conv3dAttribute; TransposeConv2dAttribute keeps out_pad in pad
    std::vector<int32_t> pad, stride, dilation;
    // AvgPool2dAttribute / MaxPool2dAttribute: kernel (+ stride, pad above; acc_type or nan_mode below)
    std::vector<int32_t> kernel;
    bool local_bound  = false;
    uint32_t acc_type = 0;
    // RescaleAttribute
    bool scale32 = false, per_channel = false, input_unsigned = false, output_unsigned = false;
    uint32_t rounding_mode = 0;
    // ClampAttribute (bytes of one value of the tensor's element type each)
    std::vector<uint8_t> min_val, max_val;
    uint32_t nan_mode = 0;
};

struct TensorDesc
{
    std::string name;
    std::vector<int32_t> shape;
    DType dtype = DType_UNKNOWN;
    std::vector<uint8_t> data;    // CONST payload (may carry alignment padding past the last element)
};

struct OperatorDesc
{
    uint32_t op = 0;
    Attribute attr;
    std::vector<std::string> inputs, outputs;
};

struct BasicBlock
{
    std::string name;
    std::vector<TensorDesc> tensors;
    std::vector<OperatorDesc> operators;
    std::vector<std::string> inputs, outputs;
};

// Reads region 0 / block 0 of a TOSA flatbuffer file (what TosaSerializationHandler::LoadFileTosaFlatbuffer
// provides to reference_model/src/main.cpp:286-337).  Returns false and sets `err` on malformed input.
bool load_tosa_file(const std::string& path, BasicBlock& block, std::string& err);

// ---- .npy ----------------------------------------------------------------------------------------------
struct NpyArray
{
    std::string descr;    // e.g. "|i1", "<i4", "<f2"
    std::vector<int32_t> shape;
    std::vector<uint8_t> data;
};
bool read_npy(const std::string& path, NpyArray& out, std::string& err);
bool write_npy(const std::string& path, const std::string& descr, const std::vector<int32_t>& shape,
               const void* data, size_t bytes, std::string& err);
const char* npy_descr_for(DType t);

// ---- runtime ---------------------------------------------------------------------------------------------
class GraphNode;
class SubgraphTraverser;

// A tensor of the graph: packed host bytes and/or a device buffer, with validity bits for each side
// (counterpart of TensorTemplate, reference_model/src/tensor.h:365-440).
class Tensor
{
public:
    Tensor(const TensorDesc& d);
    const std::string& getName() const { return name; }
    const std::vector<int32_t>& getShape() const { return shape; }
    int getRank() const { return (int)shape.size(); }
    DType getDtype() const { return dtype; }
    int64_t getElementCount() const;
    // a precise-mode result is held as fp64 whatever the serialized element type says
    size_t bytes() const { return (size_t)getElementCount() * (precise ? 8 : dtype_size(dtype)); }

    std::string name;
    std::vector<int32_t> shape;
    DType dtype;
    std::vector<uint8_t> host;
    void* dev          = nullptr;
    bool host_valid    = false;
    bool dev_valid     = false;
    bool is_const      = false;
    bool is_graph_io   = false;
    bool precise       = false;    // written by the fp64 precise / bounds pass of a floating-point operator
    GraphNode* producer = nullptr;
    std::vector<GraphNode*> consumers;

    // value of element 0 of a small CONST / input tensor as a sign-interpreted integer (zero points)
    bool scalar_value(int32_t& v) const;
};

class GraphNode
{
public:
    GraphNode(SubgraphTraverser* sgt, uint32_t op, uint64_t id);
    virtual ~GraphNode();
    virtual int checkTensorAttributes();
    virtual int eval();    // 0 = ok, 1 = stop evaluation (reference_model/src/subgraph_traverser.cpp:856-860)

    std::vector<std::string> inputNames, outputNames;
    std::vector<Tensor*> inputs, outputs;
    uint32_t nodeType;
    uint64_t nodeId;
    Attribute attribute;
    bool folded = false;    // evaluated as part of its producer's fused kernel; eval() only marks outputs valid

protected:
    int validateRequiredOperands();
    int validateRequiredRank(const Tensor* t, int rank_min, int rank_max);
    int error(const char* fmt, ...);    // printNodeValidationError + TOSA_ERROR; returns 1
    int call(int rc);                   // maps a C-ABI status onto the graph status; returns 0/1
    int requiredInputCount = -1, requiredOutputCount = -1;
    SubgraphTraverser* parent_sgt;
};

class SubgraphTraverser
{
public:
    explicit SubgraphTraverser(const BasicBlock& block, int device = 0);
    ~SubgraphTraverser();

    int initializeGraph();           // tensors + nodes from the serialized block, CONST data decoded
    int linkTensorsAndNodes();       // names -> pointers, producer/consumer lists, fusion peephole
    int validateGraph();             // checkTensorAttributes on every node
    int evaluateAll();               // topological evaluation, then one tmi_ctx_sync for the REQUIRE latch

    GraphStatus getGraphStatus() const { return status; }
    void setGraphStatus(GraphStatus s);
    Tensor* findTensorByName(const std::string& name) const;
    const std::vector<std::string>& inputNames() const { return block.inputs; }
    const std::vector<std::string>& outputNames() const { return block.outputs; }

    tmi_ctx_t* ctx = nullptr;
    void* device(Tensor* t);         // device pointer, uploading the host copy on first use
    void* device_out(Tensor* t);     // device pointer for a result (allocates, no upload)
    int download(Tensor* t);         // device -> host bytes
    std::string last_message;
    bool enable_fusion = true;
    // g_func_config.precise_mode / bounds_mode of the reference (include/func_config.h:60-61): floating-point
    // CONV2D / DEPTHWISE_CONV2D / MATMUL accumulate in fp64 (bounds mode: over absolute values) and write fp64
    bool precise_mode = false, bounds_mode = false;
    int kernels_launched = 0, nodes_folded = 0;

private:
    BasicBlock block;
    int device_id;
    GraphStatus status = GraphStatus::TOSA_VALID;
    std::vector<std::unique_ptr<Tensor>> tensors;
    std::vector<std::unique_ptr<GraphNode>> nodes;
    std::map<std::string, Tensor*> by_name;
};

// IModelRunner of the reference (reference_model/include/model_runner.h:33-98) on top of the traverser.
class ModelRunner
{
public:
    explicit ModelRunner(int device = 0) : device_id(device) {}
    GraphStatus initialize(const BasicBlock& block);
    int setInput(const std::string& name, const uint8_t* raw, size_t size);
    GraphStatus run();
    int getOutput(const std::string& name, uint8_t* raw, size_t size);
    SubgraphTraverser* traverser() { return sgt.get(); }
    void disableFusion() { fusion = false; }
    // compliance: a compliance test in precise mode (main.cpp:109-115); RESCALE's INEXACT_ROUND reads it
    void setPreciseMode(bool precise, bool bounds, bool compliance = false)
    {
        precise_mode = precise, bounds_mode = bounds, compliance_mode = compliance;
    }
    // g_func_config.tosa_level (func_config.h:63-66); all zero = NONE
    void setLevel(const tmi_level_t& l) { level = l; }

private:
    int device_id;
    bool fusion = true, precise_mode = false, bounds_mode = false, compliance_mode = false;
    tmi_level_t level = { 0, 0, 0, 0, 0 };
    std::unique_ptr<SubgraphTraverser> sgt;
};

}    // namespace tmi_host
