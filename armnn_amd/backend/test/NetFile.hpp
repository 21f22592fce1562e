// Reads a network file written by armnn_amd/netfile.py and builds the INetwork it describes: the benchmark networks
// with exactly the constants the device executor and the CPU checker use.  Fused activations of the file become
// Activation layers of their own, as a parser would add them; the backend folds them back in.
#pragma once
#include <armnn/ArmNN.hpp>

#include <cstdint>
#include <cstring>
#include <fstream>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

namespace netfile
{
using namespace armnn;

struct Const
{
    bool present = false;
    TensorInfo info;
    std::vector<uint8_t> bytes;
};

struct LayerRec
{
    std::string op, name, output;
    std::vector<std::string> inputs;
    int actFn = 0;
    float actA = 0.0f, actB = 0.0f;
    int32_t p[16] = {0};       // pad_top, pad_left, pad_bottom, pad_right, stride_x, stride_y, dilation_x, dilation_y, depthwise,
                               // pool_type, pool_w, pool_h, padding_method, transpose_weights, -, -
    float beta = 1.0f;
    Const weights, bias;
};

struct Net
{
    uint32_t batch = 0;
    std::string input, output;
    std::map<std::string, TensorInfo> tensors;
    std::vector<LayerRec> layers;
};

class Reader
{
public:
    explicit Reader(const std::string& path) : m_In(path, std::ios::binary)
    {
        if (!m_In) throw std::runtime_error("cannot open " + path);
    }
    template <typename T> T Get()
    {
        T v;
        m_In.read(reinterpret_cast<char*>(&v), sizeof(T));
        if (!m_In) throw std::runtime_error("network file ends early");
        return v;
    }
    std::string Str()
    {
        const uint32_t n = Get<uint32_t>();
        std::string s(n, '\0');
        m_In.read(s.data(), n);
        if (!m_In) throw std::runtime_error("network file ends early");
        return s;
    }
    void Bytes(void* dst, size_t n)
    {
        m_In.read(static_cast<char*>(dst), static_cast<std::streamsize>(n));
        if (!m_In) throw std::runtime_error("network file ends early");
    }
private:
    std::ifstream m_In;
};

inline DataType ToDataType(uint32_t code)
{
    switch (code)
    {
        case 0: return DataType::QAsymmS8;
        case 1: return DataType::QAsymmU8;
        case 2: return DataType::QSymmS8;
        case 3: return DataType::Signed32;
        case 4: return DataType::Float32;
        default: throw std::runtime_error("network file: unknown data type code");
    }
}

inline TensorShape ReadShape(Reader& r)
{
    const uint32_t rank = r.Get<uint32_t>();
    std::vector<unsigned int> dims(rank);
    for (auto& d : dims) d = r.Get<uint32_t>();
    return TensorShape(rank, dims.data());
}

inline Const ReadConst(Reader& r)
{
    Const c;
    c.present = r.Get<uint32_t>() != 0;
    if (!c.present) return c;
    const DataType t = ToDataType(r.Get<uint32_t>());
    const TensorShape shape = ReadShape(r);
    const uint32_t nScales = r.Get<uint32_t>();
    std::vector<float> scales(nScales);
    for (auto& s : scales) s = r.Get<float>();
    const int32_t offset = r.Get<int32_t>();
    const int32_t qdim = r.Get<int32_t>();
    if (qdim >= 0) c.info = TensorInfo(shape, t, scales, static_cast<unsigned int>(qdim), true);
    else c.info = TensorInfo(shape, t, scales.at(0), offset, true);
    c.bytes.resize(r.Get<uint64_t>());
    r.Bytes(c.bytes.data(), c.bytes.size());
    if (c.bytes.size() != c.info.GetNumBytes()) throw std::runtime_error("network file: constant size does not match its shape");
    return c;
}

inline Net Read(const std::string& path)
{
    Reader r(path);
    char magic[8];
    r.Bytes(magic, 8);
    if (std::memcmp(magic, "MI355XNT", 8) != 0 || r.Get<uint32_t>() != 1) throw std::runtime_error(path + ": not a network file of version 1");
    Net n;
    n.batch = r.Get<uint32_t>();
    const uint32_t nTensors = r.Get<uint32_t>(), nLayers = r.Get<uint32_t>();
    n.input = r.Str();
    n.output = r.Str();
    for (uint32_t i = 0; i < nTensors; ++i)
    {
        const std::string name = r.Str();
        const TensorShape shape = ReadShape(r);
        const DataType t = ToDataType(r.Get<uint32_t>());
        const float scale = r.Get<float>();
        const int32_t offset = r.Get<int32_t>();
        n.tensors[name] = TensorInfo(shape, t, scale, offset);
    }
    for (uint32_t i = 0; i < nLayers; ++i)
    {
        LayerRec l;
        l.op = r.Str();
        l.name = r.Str();
        const uint32_t nIn = r.Get<uint32_t>();
        for (uint32_t k = 0; k < nIn; ++k) l.inputs.push_back(r.Str());
        l.output = r.Str();
        l.actFn = r.Get<int32_t>();
        l.actA = r.Get<float>();
        l.actB = r.Get<float>();
        for (auto& v : l.p) v = r.Get<int32_t>();
        l.beta = r.Get<float>();
        l.weights = ReadConst(r);
        l.bias = ReadConst(r);
        n.layers.push_back(std::move(l));
    }
    return n;
}

/// The network as INetwork: input binding 0, output binding 0.  `net` must outlive the INetwork's optimization (constant
/// layers copy their data when they are added, as INetwork::AddConstantLayer does).
inline INetworkPtr Build(const Net& net)
{
    INetworkPtr g = INetwork::Create();
    std::map<std::string, IOutputSlot*> slot;
    IConnectableLayer* in = g->AddInputLayer(0, net.input.c_str());
    in->GetOutputSlot(0).SetTensorInfo(net.tensors.at(net.input));
    slot[net.input] = &in->GetOutputSlot(0);
    for (const LayerRec& l : net.layers)
    {
        const TensorInfo& outInfo = net.tensors.at(l.output);
        const TensorInfo& inInfo = net.tensors.at(l.inputs.at(0));
        IConnectableLayer* layer = nullptr;
        if (l.op == "conv" || l.op == "depthwise" || l.op == "fc")
        {
            IConnectableLayer* wl = g->AddConstantLayer(ConstTensor(l.weights.info, l.weights.bytes.data()), (l.name + "_w").c_str());
            IConnectableLayer* bl = l.bias.present ? g->AddConstantLayer(ConstTensor(l.bias.info, l.bias.bytes.data()), (l.name + "_b").c_str()) : nullptr;
            if (l.op == "fc")
            {
                FullyConnectedDescriptor d;
                d.m_BiasEnabled = l.bias.present;
                d.m_TransposeWeightMatrix = l.p[13] != 0;
                layer = g->AddFullyConnectedLayer(d, l.name.c_str());
            }
            else
            {
                // padding after the last row / column follows from the output extent (the file records the leading padding)
                const TensorShape& ws = l.weights.info.GetShape();
                const int kh = static_cast<int>(ws[1]), kw = static_cast<int>(ws[2]);
                const int needH = (static_cast<int>(outInfo.GetShape()[1]) - 1) * l.p[5] + (kh - 1) * l.p[7] + 1 - static_cast<int>(inInfo.GetShape()[1]);
                const int needW = (static_cast<int>(outInfo.GetShape()[2]) - 1) * l.p[4] + (kw - 1) * l.p[6] + 1 - static_cast<int>(inInfo.GetShape()[2]);
                const uint32_t padBottom = static_cast<uint32_t>(std::max(0, needH - l.p[0]));
                const uint32_t padRight = static_cast<uint32_t>(std::max(0, needW - l.p[1]));
                if (l.op == "conv")
                {
                    Convolution2dDescriptor d;
                    d.m_PadTop = l.p[0]; d.m_PadLeft = l.p[1]; d.m_PadBottom = padBottom; d.m_PadRight = padRight;
                    d.m_StrideX = l.p[4]; d.m_StrideY = l.p[5]; d.m_DilationX = l.p[6]; d.m_DilationY = l.p[7];
                    d.m_BiasEnabled = l.bias.present;
                    d.m_DataLayout = DataLayout::NHWC;
                    layer = g->AddConvolution2dLayer(d, l.name.c_str());
                }
                else
                {
                    DepthwiseConvolution2dDescriptor d;
                    d.m_PadTop = l.p[0]; d.m_PadLeft = l.p[1]; d.m_PadBottom = padBottom; d.m_PadRight = padRight;
                    d.m_StrideX = l.p[4]; d.m_StrideY = l.p[5]; d.m_DilationX = l.p[6]; d.m_DilationY = l.p[7];
                    d.m_BiasEnabled = l.bias.present;
                    d.m_DataLayout = DataLayout::NHWC;
                    layer = g->AddDepthwiseConvolution2dLayer(d, l.name.c_str());
                }
            }
            slot.at(l.inputs[0])->Connect(layer->GetInputSlot(0));
            wl->GetOutputSlot(0).SetTensorInfo(l.weights.info);
            wl->GetOutputSlot(0).Connect(layer->GetInputSlot(1));
            if (bl)
            {
                bl->GetOutputSlot(0).SetTensorInfo(l.bias.info);
                bl->GetOutputSlot(0).Connect(layer->GetInputSlot(2));
            }
        }
        else if (l.op == "pool")
        {
            Pooling2dDescriptor d;
            d.m_PoolType = l.p[9] == 0 ? PoolingAlgorithm::Max : PoolingAlgorithm::Average;
            d.m_PadTop = l.p[0]; d.m_PadLeft = l.p[1]; d.m_PadBottom = l.p[2]; d.m_PadRight = l.p[3];
            d.m_PoolWidth = l.p[10]; d.m_PoolHeight = l.p[11];
            d.m_StrideX = l.p[4]; d.m_StrideY = l.p[5];
            d.m_PaddingMethod = l.p[12] == 1 ? PaddingMethod::Exclude : PaddingMethod::IgnoreValue;
            d.m_DataLayout = DataLayout::NHWC;
            layer = g->AddPooling2dLayer(d, l.name.c_str());
            slot.at(l.inputs[0])->Connect(layer->GetInputSlot(0));
        }
        else if (l.op == "add")
        {
            layer = g->AddElementwiseBinaryLayer(ElementwiseBinaryDescriptor(BinaryOperation::Add), l.name.c_str());
            slot.at(l.inputs.at(0))->Connect(layer->GetInputSlot(0));
            slot.at(l.inputs.at(1))->Connect(layer->GetInputSlot(1));
        }
        else if (l.op == "reshape")
        {
            layer = g->AddReshapeLayer(ReshapeDescriptor(outInfo.GetShape()), l.name.c_str());
            slot.at(l.inputs[0])->Connect(layer->GetInputSlot(0));
        }
        else if (l.op == "softmax")
        {
            SoftmaxDescriptor d;
            d.m_Beta = l.beta;
            layer = g->AddSoftmaxLayer(d, l.name.c_str());
            slot.at(l.inputs[0])->Connect(layer->GetInputSlot(0));
        }
        else
        {
            throw std::runtime_error("network file: operation '" + l.op + "' is not supported by this reader");
        }
        layer->GetOutputSlot(0).SetTensorInfo(outInfo);
        IOutputSlot* out = &layer->GetOutputSlot(0);
        if (l.actFn != 0)
        {
            const ActivationDescriptor ad(l.actFn == 1 ? ActivationFunction::ReLu : ActivationFunction::BoundedReLu, l.actA, l.actB);
            IConnectableLayer* act = g->AddActivationLayer(ad, (l.name + "_act").c_str());
            out->Connect(act->GetInputSlot(0));
            act->GetOutputSlot(0).SetTensorInfo(outInfo);
            out = &act->GetOutputSlot(0);
        }
        slot[l.output] = out;
    }
    IConnectableLayer* o = g->AddOutputLayer(0, "output");
    slot.at(net.output)->Connect(o->GetInputSlot(0));
    return g;
}
} // namespace netfile
