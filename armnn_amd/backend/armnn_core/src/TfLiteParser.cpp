// TfLite front end: reads a quantized .tflite model (FlatBuffers, schema tensorflow/lite/schema/schema.fbs version 3; the
// few accessors needed are written out, field numbers cited where used) and builds the INetwork the reference's parser
// would build for it (src/armnnTfLiteParser/TfLiteParser.cpp):
//   * one Input layer per subgraph input and one Output layer per subgraph output, binding id (tensor index << 8) +
//     subgraph index (GenerateLayerBindingId, :672-677), layer names "<Kind>:<subgraph>:<operator>";
//   * weights and biases as Constant layers feeding slots 1 and 2 (ParseConv2D :1275-1430, ParseDepthwiseConv2D
//     :1436-1560, ParseFullyConnected :3800-3960); per-channel int8 constants are QSymmS8 with their scales along
//     quantized_dimension, everything else int8 is QAsymmS8 (ToTensorInfo, :520-660);
//   * SAME padding front = total / 2 (CalcPadding, :406-427), pooling with PaddingMethod::Exclude and Floor rounding
//     (ParsePool, :2105-2200);
//   * a fused activation becomes an Activation layer behind the layer in the layer's own output quantization
//     (AddFusedActivationLayer, :5405-5464): ReLu, BoundedReLu(6, 0), BoundedReLu(1, -1);
//   * FULLY_CONNECTED flattens an input of more than two dimensions with a Reshape layer "Reshape_for:<name>" first and
//     keeps TfLite's [outputs, K] weights with m_TransposeWeightMatrix = true;
//   * PAD pads quantized tensors with their zero point (ParsePad, :2960-3010), MEAN becomes a Mean layer, RESHAPE and
//     SQUEEZE Reshape layers, RELU / RELU_N1_TO_1 / RELU6 Activation layers, SOFTMAX a Softmax layer with the file's beta.
// Only 8-bit quantized models of these operators are accepted; anything else is a ParseException that names it.
#include <armnnTfLiteParser/ITfLiteParser.hpp>

#include <armnn/Descriptors.hpp>
#include <armnn/Exceptions.hpp>

#include <algorithm>
#include <cstring>
#include <fstream>
#include <iterator>
#include <map>

namespace armnnTfLiteParser
{
using namespace armnn;

namespace
{
// ---- FlatBuffers ---------------------------------------------------------------------------------------------------------
class Buffer
{
public:
    explicit Buffer(const std::vector<uint8_t>& bytes) : m_Data(bytes.data()), m_Size(bytes.size()) {}
    template <typename T> T Get(size_t pos) const
    {
        if (pos > m_Size || m_Size - pos < sizeof(T)) throw ParseException("malformed flatbuffer: an offset leads outside the file");
        T v;
        std::memcpy(&v, m_Data + pos, sizeof(T));
        return v;
    }
    const uint8_t* Span(size_t pos, size_t bytes) const
    {
        if (pos > m_Size || m_Size - pos < bytes) throw ParseException("malformed flatbuffer: a vector is longer than the file");
        return m_Data + pos;
    }
    size_t Size() const { return m_Size; }
private:
    const uint8_t* m_Data;
    size_t m_Size;
};

// A FlatBuffers table: fields are looked up through the vtable the table points back to.
class Table
{
public:
    Table() = default;
    Table(const Buffer* buf, size_t pos) : m_Buf(buf), m_Pos(pos)
    {
        const int32_t back = buf->Get<int32_t>(pos);
        const long long vt = static_cast<long long>(pos) - back;
        if (vt < 0) throw ParseException("malformed flatbuffer: vtable outside the file");
        m_Vt = static_cast<size_t>(vt);
        m_VtSize = buf->Get<uint16_t>(m_Vt);
    }
    explicit operator bool() const { return m_Buf != nullptr; }
    template <typename T> T Scalar(unsigned int k, T fallback = T()) const
    {
        const size_t p = Field(k);
        return p ? m_Buf->Get<T>(p) : fallback;
    }
    Table Sub(unsigned int k) const
    {
        const size_t p = Field(k);
        return p ? Table(m_Buf, p + m_Buf->Get<uint32_t>(p)) : Table();
    }
    std::string String(unsigned int k) const
    {
        size_t start = 0, n = 0;
        Vector(k, start, n);
        return start ? std::string(reinterpret_cast<const char*>(m_Buf->Span(start, n)), n) : std::string();
    }
    template <typename T> std::vector<T> Numbers(unsigned int k) const
    {
        size_t start = 0, n = 0;
        Vector(k, start, n);
        std::vector<T> out(n);
        if (n) std::memcpy(out.data(), m_Buf->Span(start, n * sizeof(T)), n * sizeof(T));
        return out;
    }
    std::vector<Table> Tables(unsigned int k) const
    {
        size_t start = 0, n = 0;
        Vector(k, start, n);
        std::vector<Table> out;
        for (size_t i = 0; i < n; ++i)
        {
            const size_t p = start + 4 * i;
            out.emplace_back(m_Buf, p + m_Buf->Get<uint32_t>(p));
        }
        return out;
    }
private:
    size_t Field(unsigned int k) const
    {
        const size_t off = 4 + 2 * static_cast<size_t>(k);
        if (!m_Buf || off >= m_VtSize) return 0;
        const uint16_t rel = m_Buf->Get<uint16_t>(m_Vt + off);
        return rel ? m_Pos + rel : 0;
    }
    void Vector(unsigned int k, size_t& start, size_t& n) const
    {
        const size_t p = Field(k);
        if (!p) { start = 0; n = 0; return; }
        const size_t v = p + m_Buf->Get<uint32_t>(p);
        n = m_Buf->Get<uint32_t>(v);
        start = v + 4;
        if (n > m_Buf->Size()) throw ParseException("malformed flatbuffer: a vector is longer than the file");
    }
    const Buffer* m_Buf = nullptr;
    size_t m_Pos = 0, m_Vt = 0;
    uint16_t m_VtSize = 0;
};

// ---- schema constants ------------------------------------------------------------------------------------------------------
enum : int { kInt32 = 2, kUint8 = 3, kInt8 = 9 };                                                       // TensorType
enum : int { kAdd = 0, kAveragePool = 1, kConv = 3, kDepthwise = 4, kFullyConnected = 9, kMaxPool = 17, kRelu = 19,
             kReluN1To1 = 20, kRelu6 = 21, kReshape = 22, kSoftmax = 25, kPad = 34, kMean = 40, kSqueeze = 43 };   // BuiltinOperator
enum : int { kSame = 0, kValid = 1 };                                                                   // Padding

// CalcPadding, TfLiteParser.cpp:406-427
void CalcPadding(uint32_t inputSize, uint32_t filterSize, uint32_t stride, uint32_t dilation, uint32_t& front, uint32_t& back, int padding)
{
    front = back = 0;
    if (padding != kSame) return;
    const uint32_t outputSize = (inputSize + stride - 1) / stride;
    const uint32_t dilatedSize = filterSize + (dilation - 1) * (filterSize - 1);
    const uint32_t needed = (outputSize - 1) * stride + dilatedSize;
    if (needed > inputSize)
    {
        front = (needed - inputSize) / 2;
        back = (needed - inputSize) - front;
    }
}

std::vector<unsigned int> Dims(const TensorInfo& info)
{
    std::vector<unsigned int> d;
    for (unsigned int i = 0; i < info.GetNumDimensions(); ++i) d.push_back(info.GetShape()[i]);
    return d;
}

std::string Name(const char* kind, size_t subgraph, size_t op)
{
    return std::string(kind) + ":" + std::to_string(subgraph) + ":" + std::to_string(op);
}
} // namespace

class TfLiteParserImpl
{
public:
    INetworkPtr Create(const std::vector<uint8_t>& bytes)
    {
        m_Inputs.clear();
        m_Outputs.clear();
        if (bytes.size() < 8 || std::memcmp(bytes.data() + 4, "TFL3", 4) != 0)
            throw ParseException("not a TfLite flatbuffer (file identifier TFL3 missing)");
        const Buffer buf(bytes);
        const Table root(&buf, buf.Get<uint32_t>(0));
        m_OpCodes = root.Tables(1);                                 // Model.operator_codes
        const std::vector<Table> graphs = root.Tables(2);           // Model.subgraphs
        m_Buffers = root.Tables(4);                                 // Model.buffers
        if (graphs.size() != 1) throw ParseException(std::to_string(graphs.size()) + " subgraphs (one is supported)");
        m_SubgraphCount = graphs.size();
        const size_t sg = 0;
        const Table& graph = graphs[sg];
        m_Tensors = graph.Tables(0);                                // SubGraph.tensors
        m_Network = INetwork::Create();
        m_Slots.clear();

        for (int32_t t : graph.Numbers<int32_t>(1))                 // SubGraph.inputs
        {
            const TensorInfo info = Info(Index(t));
            const LayerBindingId id = static_cast<LayerBindingId>((static_cast<size_t>(t) << 8) + sg);
            const std::string name = m_Tensors[Index(t)].String(3);
            IConnectableLayer* layer = m_Network->AddInputLayer(id, name.c_str());
            layer->GetOutputSlot(0).SetTensorInfo(info);
            m_Slots[t] = &layer->GetOutputSlot(0);
            m_Inputs.emplace_back(name, BindingPointInfo(id, info));
        }
        const std::vector<Table> ops = graph.Tables(3);             // SubGraph.operators
        for (size_t k = 0; k < ops.size(); ++k) Operator(ops[k], sg, k);
        for (int32_t t : graph.Numbers<int32_t>(2))                 // SubGraph.outputs
        {
            const LayerBindingId id = static_cast<LayerBindingId>((static_cast<size_t>(t) << 8) + sg);
            const std::string name = m_Tensors[Index(t)].String(3);
            IConnectableLayer* layer = m_Network->AddOutputLayer(id, name.c_str());
            Slot(t, "a subgraph output")->Connect(layer->GetInputSlot(0));
            m_Outputs.emplace_back(name, BindingPointInfo(id, Info(Index(t))));
        }
        m_OpCodes.clear();
        m_Buffers.clear();
        m_Tensors.clear();
        m_Slots.clear();
        return std::move(m_Network);
    }

    std::vector<std::pair<std::string, BindingPointInfo>> m_Inputs, m_Outputs;
    size_t m_SubgraphCount = 0;

private:
    size_t Index(int32_t t) const
    {
        if (t < 0 || static_cast<size_t>(t) >= m_Tensors.size()) throw ParseException("tensor index " + std::to_string(t) + " is out of range");
        return static_cast<size_t>(t);
    }

    // ToTensorInfo (TfLiteParser.cpp:520-660) for the 8-bit quantized types and int32
    TensorInfo Info(size_t index, bool constant = false) const
    {
        const Table& t = m_Tensors[index];
        const std::vector<int32_t> dims = t.Numbers<int32_t>(0);    // Tensor.shape
        const int type = t.Scalar<int8_t>(1);                       // Tensor.type
        const Table q = t.Sub(4);                                   // Tensor.quantization
        const std::vector<float> scales = q ? q.Numbers<float>(2) : std::vector<float>();       // QuantizationParameters.scale
        const std::vector<int64_t> zeros = q ? q.Numbers<int64_t>(3) : std::vector<int64_t>();  // .zero_point
        const int32_t qdim = q ? q.Scalar<int32_t>(6) : 0;          // .quantized_dimension
        const std::string name = t.String(3);
        std::vector<unsigned int> shape;
        for (int32_t d : dims)
        {
            if (d < 0) throw ParseException("tensor '" + name + "' has a dynamic shape");
            shape.push_back(static_cast<unsigned int>(d));
        }
        if (shape.empty()) shape.push_back(1);
        DataType dtype;
        if (type == kInt32) dtype = DataType::Signed32;
        else if (type == kUint8) dtype = DataType::QAsymmU8;
        else if (type == kInt8) dtype = (constant && scales.size() > 1) ? DataType::QSymmS8 : DataType::QAsymmS8;
        else throw ParseException("tensor '" + name + "' has TensorType " + std::to_string(type) + "; only UINT8, INT8 and INT32 are read");
        const TensorShape ts(static_cast<unsigned int>(shape.size()), shape.data());
        TensorInfo info;
        if (scales.size() > 1)
        {
            for (int64_t z : zeros)
                if (z != 0) throw ParseException("tensor '" + name + "': per-channel quantization with non-zero zero points");
            if (qdim < 0 || static_cast<size_t>(qdim) >= shape.size()) throw ParseException("tensor '" + name + "': quantized_dimension out of range");
            info = TensorInfo(ts, dtype, scales, static_cast<unsigned int>(qdim));
        }
        else
        {
            if (scales.empty() && dtype != DataType::Signed32) throw ParseException("tensor '" + name + "' carries no quantization");
            info = TensorInfo(ts, dtype, scales.empty() ? 1.0f : scales[0], zeros.empty() ? 0 : static_cast<int32_t>(zeros[0]));
        }
        if (constant) info.SetConstant(true);
        return info;
    }

    IOutputSlot* Slot(int32_t t, const std::string& what) const
    {
        const auto it = m_Slots.find(t);
        if (it == m_Slots.end()) throw ParseException(what + " reads tensor " + std::to_string(t) + ", which nothing before it produces");
        return it->second;
    }

    // a Constant layer holding tensor t's buffer, or nullptr when the operator has no such input
    IConnectableLayer* Constant(int32_t t, const std::string& what, const std::string& name, TensorInfo& info)
    {
        if (t < 0) return nullptr;
        const Table& tensor = m_Tensors[Index(t)];
        const uint32_t b = tensor.Scalar<uint32_t>(2);              // Tensor.buffer
        if (b >= m_Buffers.size()) throw ParseException(what + ": buffer index out of range");
        const std::vector<uint8_t> data = m_Buffers[b].Numbers<uint8_t>(0);     // Buffer.data
        info = Info(Index(t), true);
        if (data.empty()) throw ParseException(what + " must be a constant tensor");
        if (data.size() != info.GetNumBytes()) throw ParseException(what + ": the buffer does not hold the tensor's shape");
        IConnectableLayer* layer = m_Network->AddConstantLayer(ConstTensor(info, data.data()), name.c_str());
        layer->GetOutputSlot(0).SetTensorInfo(info);
        return layer;
    }

    static void CheckBias(const TensorInfo& bias, const TensorInfo& weights, const std::string& what)
    {
        // ValidateBiasTensorQuantization, src/backends/backendsCommon/WorkloadData.cpp
        if (bias.GetDataType() != DataType::Signed32) throw ParseException(what + ": bias is not INT32");
        if (bias.GetQuantizationScales().size() != weights.GetQuantizationScales().size())
            throw ParseException(what + ": bias and weights differ in their number of quantization scales");
    }

    // AddFusedActivationLayer, TfLiteParser.cpp:5405-5464
    IOutputSlot* Fused(IOutputSlot* out, int code, const TensorInfo& info, const std::string& owner)
    {
        ActivationDescriptor d;
        std::string tag;
        switch (code)
        {
            case 0: return out;
            case 1: d.m_Function = ActivationFunction::ReLu; tag = "RELU"; break;
            case 2: d.m_Function = ActivationFunction::BoundedReLu; d.m_A = 1.0f; d.m_B = -1.0f; tag = "RELU_N1_TO_1"; break;
            case 3: d.m_Function = ActivationFunction::BoundedReLu; d.m_A = 6.0f; d.m_B = 0.0f; tag = "RELU6"; break;
            default: throw ParseException(owner + ": fused activation " + std::to_string(code) + " (NONE, RELU, RELU_N1_TO_1 and RELU6 are supported)");
        }
        IConnectableLayer* act = m_Network->AddActivationLayer(d, (owner + ":" + tag).c_str());
        out->Connect(act->GetInputSlot(0));
        act->GetOutputSlot(0).SetTensorInfo(info);
        return &act->GetOutputSlot(0);
    }

    void Expect(const TensorInfo& out, const std::vector<unsigned int>& shape, const std::string& what) const
    {
        // buffers are sized from the file's shapes and kernels from the operator's arithmetic: they have to agree
        bool same = out.GetNumDimensions() == shape.size();
        for (size_t i = 0; same && i < shape.size(); ++i) same = out.GetShape()[static_cast<unsigned int>(i)] == shape[i];
        if (!same) throw ParseException(what + ": the file's output shape is not what the operator produces");
    }

    void Operator(const Table& op, size_t sg, size_t k)
    {
        const uint32_t ci = op.Scalar<uint32_t>(0);                 // Operator.opcode_index
        if (ci >= m_OpCodes.size()) throw ParseException("operator " + std::to_string(k) + ": opcode index out of range");
        // OperatorCode.builtin_code (3) superseded deprecated_builtin_code (0, a byte) for codes above 127
        const int code = std::max<int>(m_OpCodes[ci].Scalar<int32_t>(3), m_OpCodes[ci].Scalar<int8_t>(0));
        const std::vector<int32_t> ins = op.Numbers<int32_t>(1);    // Operator.inputs
        const std::vector<int32_t> outs = op.Numbers<int32_t>(2);   // Operator.outputs
        const Table o = op.Sub(4);                                  // Operator.builtin_options
        if (ins.empty() || outs.size() != 1) throw ParseException("operator " + std::to_string(k) + " must have inputs and one output");
        const TensorInfo xi = Info(Index(ins[0]));
        const TensorInfo yi = Info(Index(outs[0]));
        IOutputSlot* x = nullptr;
        IOutputSlot* y = nullptr;
        auto input = [&](const std::string& what) { x = Slot(ins[0], what); };

        switch (code)
        {
        case kConv:
        case kDepthwise:
        {
            const bool dw = code == kDepthwise;
            const std::string name = Name(dw ? "DepthwiseConv2D" : "Conv2D", sg, k);
            input(name);
            if (ins.size() < 2 || !o) throw ParseException(name + ": weights and options are required");
            TensorInfo wi, bi;
            IConnectableLayer* w = Constant(ins[1], name + " weights", name + ":weights", wi);
            IConnectableLayer* b = ins.size() > 2 ? Constant(ins[2], name + " bias", name + ":bias", bi) : nullptr;
            if (b) CheckBias(bi, wi, name);
            const int padding = o.Scalar<int8_t>(0);                // Conv2DOptions / DepthwiseConv2DOptions.padding
            const int32_t sw = o.Scalar<int32_t>(1), sh = o.Scalar<int32_t>(2);
            const int act = o.Scalar<int8_t>(dw ? 4 : 3);
            const int32_t dwf = o.Scalar<int32_t>(dw ? 5 : 4, 1), dhf = o.Scalar<int32_t>(dw ? 6 : 5, 1);
            if (xi.GetNumDimensions() != 4 || wi.GetNumDimensions() != 4 || std::min(std::min(sw, sh), std::min(dwf, dhf)) < 1)
                throw ParseException(name + ": needs 4-D tensors and positive strides and dilations");
            const unsigned int h = xi.GetShape()[1], wd = xi.GetShape()[2], cin = xi.GetShape()[3];
            const unsigned int kh = wi.GetShape()[1], kw = wi.GetShape()[2];
            if (dw && (wi.GetShape()[0] != 1 || cin == 0 || wi.GetShape()[3] % cin != 0)) throw ParseException(name + ": weights must be [1, H, W, I * multiplier]");
            if (!dw && wi.GetShape()[3] != cin) throw ParseException(name + ": weights must be [O, H, W, I]");
            uint32_t pt, pb, pl, pr;
            CalcPadding(h, kh, static_cast<uint32_t>(sh), static_cast<uint32_t>(dhf), pt, pb, padding);
            CalcPadding(wd, kw, static_cast<uint32_t>(sw), static_cast<uint32_t>(dwf), pl, pr, padding);
            const unsigned int dkh = static_cast<unsigned int>(dhf) * (kh - 1) + 1, dkw = static_cast<unsigned int>(dwf) * (kw - 1) + 1;
            if (h + pt + pb < dkh || wd + pl + pr < dkw) throw ParseException(name + ": the filter is larger than the padded input");
            Expect(yi, {xi.GetShape()[0], (h + pt + pb - dkh) / static_cast<unsigned int>(sh) + 1, (wd + pl + pr - dkw) / static_cast<unsigned int>(sw) + 1,
                        dw ? wi.GetShape()[3] : wi.GetShape()[0]}, name);
            IConnectableLayer* layer;
            if (dw)
            {
                DepthwiseConvolution2dDescriptor d;
                d.m_PadTop = pt; d.m_PadBottom = pb; d.m_PadLeft = pl; d.m_PadRight = pr;
                d.m_StrideX = static_cast<uint32_t>(sw); d.m_StrideY = static_cast<uint32_t>(sh);
                d.m_DilationX = static_cast<uint32_t>(dwf); d.m_DilationY = static_cast<uint32_t>(dhf);
                d.m_BiasEnabled = b != nullptr;
                d.m_DataLayout = DataLayout::NHWC;
                layer = m_Network->AddDepthwiseConvolution2dLayer(d, name.c_str());
            }
            else
            {
                Convolution2dDescriptor d;
                d.m_PadTop = pt; d.m_PadBottom = pb; d.m_PadLeft = pl; d.m_PadRight = pr;
                d.m_StrideX = static_cast<uint32_t>(sw); d.m_StrideY = static_cast<uint32_t>(sh);
                d.m_DilationX = static_cast<uint32_t>(dwf); d.m_DilationY = static_cast<uint32_t>(dhf);
                d.m_BiasEnabled = b != nullptr;
                d.m_DataLayout = DataLayout::NHWC;
                layer = m_Network->AddConvolution2dLayer(d, name.c_str());
            }
            x->Connect(layer->GetInputSlot(0));
            w->GetOutputSlot(0).Connect(layer->GetInputSlot(1));
            if (b) b->GetOutputSlot(0).Connect(layer->GetInputSlot(2));
            layer->GetOutputSlot(0).SetTensorInfo(yi);
            y = Fused(&layer->GetOutputSlot(0), act, yi, name);
            break;
        }
        case kFullyConnected:
        {
            const std::string name = Name("FullyConnected", sg, k);
            input(name);
            if (ins.size() < 2) throw ParseException(name + ": weights are required");
            TensorInfo wi, bi;
            IConnectableLayer* w = Constant(ins[1], name + " weights", name + ":weights", wi);
            IConnectableLayer* b = ins.size() > 2 ? Constant(ins[2], name + " bias", name + ":bias", bi) : nullptr;
            if (b) CheckBias(bi, wi, name);
            if (wi.GetNumDimensions() != 2 || wi.GetShape()[1] == 0 || xi.GetNumElements() % wi.GetShape()[1] != 0)
                throw ParseException(name + ": weights must be [outputs, K] with K dividing the input");
            const unsigned int kdim = wi.GetShape()[1], rows = xi.GetNumElements() / kdim;
            FullyConnectedDescriptor d;
            d.m_BiasEnabled = b != nullptr;
            d.m_TransposeWeightMatrix = true;
            d.m_ConstantWeights = true;
            IConnectableLayer* layer = m_Network->AddFullyConnectedLayer(d, name.c_str());
            if (xi.GetNumDimensions() > 2 || xi.GetShape()[xi.GetNumDimensions() - 1] != kdim)
            {
                TensorInfo flat = xi;
                flat.SetShape(TensorShape({rows, kdim}));
                IConnectableLayer* reshape = m_Network->AddReshapeLayer(ReshapeDescriptor(flat.GetShape()), ("Reshape_for:" + name).c_str());
                x->Connect(reshape->GetInputSlot(0));
                reshape->GetOutputSlot(0).SetTensorInfo(flat);
                x = &reshape->GetOutputSlot(0);
            }
            if (yi.GetNumElements() != rows * wi.GetShape()[0]) throw ParseException(name + ": the file's output shape is not what the operator produces");
            TensorInfo out = yi;
            if (yi.GetNumDimensions() != 2) out.SetShape(TensorShape({rows, wi.GetShape()[0]}));
            x->Connect(layer->GetInputSlot(0));
            w->GetOutputSlot(0).Connect(layer->GetInputSlot(1));
            if (b) b->GetOutputSlot(0).Connect(layer->GetInputSlot(2));
            layer->GetOutputSlot(0).SetTensorInfo(out);
            y = Fused(&layer->GetOutputSlot(0), o ? o.Scalar<int8_t>(0) : 0, out, name);       // FullyConnectedOptions.fused_activation_function
            break;
        }
        case kAveragePool:
        case kMaxPool:
        {
            const std::string name = Name(code == kMaxPool ? "MaxPool2D" : "AveragePool2D", sg, k);
            input(name);
            if (!o) throw ParseException(name + ": options are required");
            const int padding = o.Scalar<int8_t>(0);                // Pool2DOptions
            const int32_t sw = o.Scalar<int32_t>(1), sh = o.Scalar<int32_t>(2), fw = o.Scalar<int32_t>(3), fh = o.Scalar<int32_t>(4);
            if (xi.GetNumDimensions() != 4 || std::min(std::min(sw, sh), std::min(fw, fh)) < 1) throw ParseException(name + ": needs a 4-D tensor and positive window and strides");
            const unsigned int h = xi.GetShape()[1], wd = xi.GetShape()[2];
            Pooling2dDescriptor d;
            d.m_PoolType = code == kMaxPool ? PoolingAlgorithm::Max : PoolingAlgorithm::Average;
            d.m_PoolWidth = static_cast<uint32_t>(fw); d.m_PoolHeight = static_cast<uint32_t>(fh);
            d.m_StrideX = static_cast<uint32_t>(sw); d.m_StrideY = static_cast<uint32_t>(sh);
            d.m_PaddingMethod = PaddingMethod::Exclude;
            d.m_OutputShapeRounding = OutputShapeRounding::Floor;
            d.m_DataLayout = DataLayout::NHWC;
            CalcPadding(h, d.m_PoolHeight, d.m_StrideY, 1u, d.m_PadTop, d.m_PadBottom, padding);
            CalcPadding(wd, d.m_PoolWidth, d.m_StrideX, 1u, d.m_PadLeft, d.m_PadRight, padding);
            if (h + d.m_PadTop + d.m_PadBottom < d.m_PoolHeight || wd + d.m_PadLeft + d.m_PadRight < d.m_PoolWidth) throw ParseException(name + ": the window is larger than the padded input");
            Expect(yi, {xi.GetShape()[0], (h + d.m_PadTop + d.m_PadBottom - d.m_PoolHeight) / d.m_StrideY + 1,
                        (wd + d.m_PadLeft + d.m_PadRight - d.m_PoolWidth) / d.m_StrideX + 1, xi.GetShape()[3]}, name);
            IConnectableLayer* layer = m_Network->AddPooling2dLayer(d, name.c_str());
            x->Connect(layer->GetInputSlot(0));
            layer->GetOutputSlot(0).SetTensorInfo(yi);
            y = Fused(&layer->GetOutputSlot(0), o.Scalar<int8_t>(5), yi, name);
            break;
        }
        case kAdd:
        {
            const std::string name = Name("Add", sg, k);
            input(name);
            if (ins.size() != 2) throw ParseException(name + ": two inputs are required");
            IOutputSlot* x1 = Slot(ins[1], name);
            if (Info(Index(ins[1])).GetShape() != xi.GetShape()) throw ParseException(name + ": broadcasting is not supported");
            Expect(yi, Dims(xi), name);
            IConnectableLayer* layer = m_Network->AddElementwiseBinaryLayer(ElementwiseBinaryDescriptor(BinaryOperation::Add), name.c_str());
            x->Connect(layer->GetInputSlot(0));
            x1->Connect(layer->GetInputSlot(1));
            layer->GetOutputSlot(0).SetTensorInfo(yi);
            y = Fused(&layer->GetOutputSlot(0), o ? o.Scalar<int8_t>(0) : 0, yi, name);        // AddOptions.fused_activation_function
            break;
        }
        case kPad:
        {
            const std::string name = Name("Pad", sg, k);
            input(name);
            if (ins.size() < 2) throw ParseException(name + ": paddings are required");
            const Table& pt = m_Tensors[Index(ins[1])];
            const uint32_t b = pt.Scalar<uint32_t>(2);
            if (b >= m_Buffers.size()) throw ParseException(name + ": buffer index out of range");
            const std::vector<uint8_t> raw = m_Buffers[b].Numbers<uint8_t>(0);
            if (pt.Scalar<int8_t>(1) != kInt32 || raw.size() != 8u * xi.GetNumDimensions() || xi.GetNumDimensions() > 4)
                throw ParseException(name + ": paddings must be a constant INT32 tensor with one (before, after) pair per dimension, at most 4 dimensions");
            std::vector<int32_t> p(raw.size() / 4);
            std::memcpy(p.data(), raw.data(), raw.size());
            PadDescriptor d;
            std::vector<unsigned int> shape;
            for (unsigned int i = 0; i < xi.GetNumDimensions(); ++i)
            {
                if (p[2 * i] < 0 || p[2 * i + 1] < 0) throw ParseException(name + ": negative padding");
                d.m_PadList.emplace_back(static_cast<unsigned int>(p[2 * i]), static_cast<unsigned int>(p[2 * i + 1]));
                shape.push_back(xi.GetShape()[i] + d.m_PadList.back().first + d.m_PadList.back().second);
            }
            Expect(yi, shape, name);
            // TfLite pads with the real number 0: the zero point in the tensor's own code (ParsePad, :2984-2989)
            d.m_PadValue = static_cast<float>(xi.GetQuantizationOffset());
            IConnectableLayer* layer = m_Network->AddPadLayer(d, name.c_str());
            x->Connect(layer->GetInputSlot(0));
            layer->GetOutputSlot(0).SetTensorInfo(yi);
            y = &layer->GetOutputSlot(0);
            break;
        }
        case kMean:
        {
            const std::string name = Name("Mean", sg, k);
            input(name);
            if (ins.size() < 2) throw ParseException(name + ": axes are required");
            const Table& at = m_Tensors[Index(ins[1])];
            const uint32_t b = at.Scalar<uint32_t>(2);
            if (b >= m_Buffers.size()) throw ParseException(name + ": buffer index out of range");
            const std::vector<uint8_t> raw = m_Buffers[b].Numbers<uint8_t>(0);
            if (at.Scalar<int8_t>(1) != kInt32 || raw.empty() || raw.size() % 4 != 0) throw ParseException(name + ": axes must be a constant INT32 tensor");
            std::vector<int32_t> axes(raw.size() / 4);
            std::memcpy(axes.data(), raw.data(), raw.size());
            const int rank = static_cast<int>(xi.GetNumDimensions());
            MeanDescriptor d;
            for (int32_t a : axes)
            {
                if (a < -rank || a >= rank) throw ParseException(name + ": axis out of range");
                d.m_Axis.push_back(static_cast<unsigned int>((a + rank) % rank));
            }
            std::sort(d.m_Axis.begin(), d.m_Axis.end());
            d.m_Axis.erase(std::unique(d.m_Axis.begin(), d.m_Axis.end()), d.m_Axis.end());
            d.m_KeepDims = o ? o.Scalar<int8_t>(0) != 0 : false;    // ReducerOptions.keep_dims
            std::vector<unsigned int> shape;
            for (unsigned int i = 0; i < xi.GetNumDimensions(); ++i)
            {
                const bool reduced = std::find(d.m_Axis.begin(), d.m_Axis.end(), i) != d.m_Axis.end();
                if (!reduced) shape.push_back(xi.GetShape()[i]);
                else if (d.m_KeepDims) shape.push_back(1);
            }
            if (shape.empty()) shape.push_back(1);
            Expect(yi, shape, name);
            IConnectableLayer* layer = m_Network->AddMeanLayer(d, name.c_str());
            x->Connect(layer->GetInputSlot(0));
            layer->GetOutputSlot(0).SetTensorInfo(yi);
            y = &layer->GetOutputSlot(0);
            break;
        }
        case kRelu:
        case kReluN1To1:
        case kRelu6:
        {
            // ParseRelu / ParseReluN1To1 / ParseRelu6 (ParseActivation, :3290-3380): a layer of its own, which re-quantizes
            // when the output tensor's quantization differs from the input's
            const char* tag = code == kRelu ? "RELU" : code == kRelu6 ? "RELU6" : "RELU_N1_TO_1";
            const std::string name = std::string("Activation:") + tag + ":" + std::to_string(sg) + ":" + std::to_string(k);
            input(name);
            Expect(yi, Dims(xi), name);
            ActivationDescriptor d;
            d.m_Function = code == kRelu ? ActivationFunction::ReLu : ActivationFunction::BoundedReLu;
            if (code == kRelu6) { d.m_A = 6.0f; d.m_B = 0.0f; }
            if (code == kReluN1To1) { d.m_A = 1.0f; d.m_B = -1.0f; }
            IConnectableLayer* layer = m_Network->AddActivationLayer(d, name.c_str());
            x->Connect(layer->GetInputSlot(0));
            layer->GetOutputSlot(0).SetTensorInfo(yi);
            y = &layer->GetOutputSlot(0);
            break;
        }
        case kReshape:
        case kSqueeze:
        {
            const std::string name = Name(code == kReshape ? "Reshape" : "Squeeze", sg, k);
            input(name);
            if (yi.GetNumElements() != xi.GetNumElements()) throw ParseException(name + ": input and output differ in their number of elements");
            if (code == kSqueeze)
            {
                // the output keeps the input's dimensions except some of extent 1
                unsigned int j = 0;
                bool ok = true;
                for (unsigned int i = 0; ok && i < xi.GetNumDimensions(); ++i)
                {
                    if (j < yi.GetNumDimensions() && xi.GetShape()[i] == yi.GetShape()[j]) ++j;
                    else ok = xi.GetShape()[i] == 1;
                }
                if (!ok || j != yi.GetNumDimensions()) throw ParseException(name + ": the output is not the input without some of its dimensions of extent 1");
            }
            IConnectableLayer* layer = m_Network->AddReshapeLayer(ReshapeDescriptor(yi.GetShape()), name.c_str());
            x->Connect(layer->GetInputSlot(0));
            layer->GetOutputSlot(0).SetTensorInfo(yi);
            y = &layer->GetOutputSlot(0);
            break;
        }
        case kSoftmax:
        {
            const std::string name = Name("Softmax", sg, k);
            input(name);
            Expect(yi, Dims(xi), name);
            SoftmaxDescriptor d;
            d.m_Beta = o ? o.Scalar<float>(0, 1.0f) : 1.0f;         // SoftmaxOptions.beta
            IConnectableLayer* layer = m_Network->AddSoftmaxLayer(d, name.c_str());
            x->Connect(layer->GetInputSlot(0));
            layer->GetOutputSlot(0).SetTensorInfo(yi);
            y = &layer->GetOutputSlot(0);
            break;
        }
        default:
            throw ParseException("operator " + std::to_string(k) + " has builtin code " + std::to_string(code) + ", which this parser does not read");
        }
        m_Slots[outs[0]] = y;
    }

    std::vector<Table> m_OpCodes, m_Buffers, m_Tensors;
    std::map<int32_t, IOutputSlot*> m_Slots;
    INetworkPtr m_Network{nullptr, [](INetwork*) {}};
};

// ---- ITfLiteParser ----------------------------------------------------------------------------------------------------------
ITfLiteParser::ITfLiteParser(const Optional<TfLiteParserOptions>& options) : pTfLiteParserImpl(new TfLiteParserImpl)
{
    if (options.has_value() && options.value().m_StandInLayerForUnsupported)
        throw InvalidArgumentException("ITfLiteParser: stand-in layers for unsupported operators are not offered");
}
ITfLiteParser::~ITfLiteParser() = default;
ITfLiteParser* ITfLiteParser::CreateRaw(const Optional<TfLiteParserOptions>& options) { return new ITfLiteParser(options); }
ITfLiteParserPtr ITfLiteParser::Create(const Optional<TfLiteParserOptions>& options) { return ITfLiteParserPtr(CreateRaw(options), &ITfLiteParser::Destroy); }
void ITfLiteParser::Destroy(ITfLiteParser* parser) { delete parser; }

INetworkPtr ITfLiteParser::CreateNetworkFromBinaryFile(const char* graphFile)
{
    if (!graphFile) throw InvalidArgumentException("Invalid (null) graph filename");
    std::ifstream in(graphFile, std::ios::binary);
    if (!in) throw FileNotFoundException(std::string("Cannot find the file (") + graphFile + ")");
    const std::vector<uint8_t> bytes((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    return pTfLiteParserImpl->Create(bytes);
}

INetworkPtr ITfLiteParser::CreateNetworkFromBinary(const std::vector<uint8_t>& binaryContent) { return pTfLiteParserImpl->Create(binaryContent); }

namespace
{
BindingPointInfo Find(const std::vector<std::pair<std::string, BindingPointInfo>>& all, size_t subgraphId, const std::string& name, const char* what)
{
    if (subgraphId != 0) throw ParseException("subgraph " + std::to_string(subgraphId) + " does not exist");
    for (const auto& e : all)
        if (e.first == name) return e.second;
    throw ParseException(std::string("No ") + what + " binding found for subgraph:0 and name:" + name);
}
std::vector<std::string> Names(const std::vector<std::pair<std::string, BindingPointInfo>>& all, size_t subgraphId)
{
    if (subgraphId != 0) throw ParseException("subgraph " + std::to_string(subgraphId) + " does not exist");
    std::vector<std::string> out;
    for (const auto& e : all) out.push_back(e.first);
    return out;
}
} // namespace

BindingPointInfo ITfLiteParser::GetNetworkInputBindingInfo(size_t subgraphId, const std::string& name) const { return Find(pTfLiteParserImpl->m_Inputs, subgraphId, name, "input"); }
BindingPointInfo ITfLiteParser::GetNetworkOutputBindingInfo(size_t subgraphId, const std::string& name) const { return Find(pTfLiteParserImpl->m_Outputs, subgraphId, name, "output"); }
size_t ITfLiteParser::GetSubgraphCount() const { return pTfLiteParserImpl->m_SubgraphCount; }
std::vector<std::string> ITfLiteParser::GetSubgraphInputTensorNames(size_t subgraphId) const { return Names(pTfLiteParserImpl->m_Inputs, subgraphId); }
std::vector<std::string> ITfLiteParser::GetSubgraphOutputTensorNames(size_t subgraphId) const { return Names(pTfLiteParserImpl->m_Outputs, subgraphId); }
} // namespace armnnTfLiteParser
