// Helpers shared by the backend tests: seeded data, quantized layer builders on INetwork, and the same layers
// evaluated by the CPU oracle (test infrastructure; the product never links it).
#pragma once
#include <armnn/ArmNN.hpp>
#include <Layer.hpp>

#include <cpuref_oracle.h>

#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <string>
#include <vector>

namespace tu
{
using namespace armnn;

struct Rng
{
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed * 0x9E3779B97F4A7C15ull + 1) {}
    uint64_t Next() { s += 0x9E3779B97F4A7C15ull; uint64_t z = s; z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull; z = (z ^ (z >> 27)) * 0x94D049BB133111EBull; return z ^ (z >> 31); }
    int Range(int lo, int hi) { return lo + static_cast<int>(Next() % static_cast<uint64_t>(hi - lo + 1)); }
    float Uniform(float lo, float hi) { return lo + (hi - lo) * static_cast<float>(Next() >> 40) / 16777216.0f; }
};

inline TensorInfo ActInfo(std::initializer_list<unsigned int> shape, DataType t, float scale, int offset)
{
    return TensorInfo(TensorShape(shape), t, scale, offset);
}

inline std::vector<uint8_t> RandomActivations(const TensorInfo& info, uint64_t seed)
{
    Rng r(seed);
    std::vector<uint8_t> v(info.GetNumElements());
    for (auto& b : v) b = static_cast<uint8_t>(r.Range(0, 255));
    return v;
}

inline orc_tensor Orc(const TensorInfo& info, const void* data, const std::vector<float>& scales)
{
    orc_tensor t{};
    t.data = const_cast<void*>(data);
    switch (info.GetDataType())
    {
        case DataType::QAsymmS8: t.dtype = ORC_QASYMM_S8; break;
        case DataType::QAsymmU8: t.dtype = ORC_QASYMM_U8; break;
        case DataType::QSymmS8: t.dtype = ORC_QSYMM_S8; break;
        case DataType::Signed32: t.dtype = ORC_SIGNED32; break;
        default: t.dtype = ORC_FLOAT32; break;
    }
    t.ndim = info.GetNumDimensions();
    for (unsigned int i = 0; i < t.ndim; ++i) t.shape[i] = info.GetShape()[i];
    t.scales = scales.data();
    t.n_scales = static_cast<uint32_t>(scales.size());
    t.quant_dim = info.GetQuantizationDim().has_value() ? static_cast<int32_t>(info.GetQuantizationDim().value()) : -1;
    t.offset = info.GetQuantizationOffset();
    return t;
}

/// one quantized conv / depthwise / FC layer with its constants, enough to add it to a network and to the oracle
struct QLayer
{
    enum Kind { Conv, Depthwise, FullyConnected } kind = Conv;
    TensorInfo in, out, w, b;
    std::vector<int8_t> weights;
    std::vector<int32_t> bias;
    std::vector<float> wScales, bScales;
    unsigned int stride = 1, padTop = 0, padLeft = 0, padBottom = 0, padRight = 0;
    bool relu6 = false;
    float reluUpper = 6.0f;
};

inline unsigned int SameOut(unsigned int in, unsigned int stride) { return (in + stride - 1) / stride; }

/// SAME-padded conv (kind Conv / Depthwise) with per-axis QSymmS8 weights
inline QLayer MakeConv(QLayer::Kind kind, const TensorInfo& in, unsigned int co, unsigned int k, unsigned int stride,
                       float outScale, int outOffset, bool relu6, bool perAxis, uint64_t seed)
{
    QLayer l;
    l.kind = kind;
    l.in = in;
    l.stride = stride;
    l.relu6 = relu6;
    const unsigned int n = in.GetShape()[0], h = in.GetShape()[1], wd = in.GetShape()[2], ci = in.GetShape()[3];
    const unsigned int ho = SameOut(h, stride), wo = SameOut(wd, stride);
    const unsigned int totalH = std::max<int>(static_cast<int>((ho - 1) * stride + k) - static_cast<int>(h), 0);
    const unsigned int totalW = std::max<int>(static_cast<int>((wo - 1) * stride + k) - static_cast<int>(wd), 0);
    l.padTop = totalH / 2; l.padBottom = totalH - l.padTop;
    l.padLeft = totalW / 2; l.padRight = totalW - l.padLeft;
    l.out = TensorInfo(TensorShape({n, ho, wo, co}), in.GetDataType(), outScale, outOffset);
    Rng r(seed);
    const unsigned int taps = kind == QLayer::Depthwise ? k * k : k * k * ci;
    const unsigned int nScales = perAxis ? co : 1;
    for (unsigned int c = 0; c < nScales; ++c) l.wScales.push_back(r.Uniform(0.5f, 1.5f) * 0.02f / std::sqrt(static_cast<float>(taps)) * 3.0f);
    for (float s : l.wScales) l.bScales.push_back(in.GetQuantizationScale() * s);
    const TensorShape ws = kind == QLayer::Depthwise ? TensorShape({1, k, k, co}) : TensorShape({co, k, k, ci});
    const unsigned int qdim = kind == QLayer::Depthwise ? 3 : 0;
    l.w = perAxis ? TensorInfo(ws, DataType::QSymmS8, l.wScales, qdim, true) : TensorInfo(ws, DataType::QSymmS8, l.wScales[0], 0, true);
    l.b = perAxis ? TensorInfo(TensorShape({co}), DataType::Signed32, l.bScales, 0, true) : TensorInfo(TensorShape({co}), DataType::Signed32, l.bScales[0], 0, true);
    l.weights.resize(l.w.GetNumElements());
    for (auto& v : l.weights) v = static_cast<int8_t>(r.Range(-127, 127));
    l.bias.resize(co);
    for (auto& v : l.bias) v = r.Range(-2000, 2000);
    return l;
}

inline QLayer MakeFc(const TensorInfo& in, unsigned int o, float outScale, int outOffset, bool perAxis, uint64_t seed)
{
    QLayer l;
    l.kind = QLayer::FullyConnected;
    l.in = in;
    const unsigned int n = in.GetShape()[0];
    const unsigned int k = in.GetNumElements() / n;
    l.out = TensorInfo(TensorShape({n, o}), in.GetDataType(), outScale, outOffset);
    Rng r(seed);
    const unsigned int nScales = perAxis ? o : 1;
    for (unsigned int c = 0; c < nScales; ++c) l.wScales.push_back(r.Uniform(0.5f, 1.5f) * 0.06f / std::sqrt(static_cast<float>(k)));
    for (float s : l.wScales) l.bScales.push_back(in.GetQuantizationScale() * s);
    l.w = perAxis ? TensorInfo(TensorShape({o, k}), DataType::QSymmS8, l.wScales, 0, true) : TensorInfo(TensorShape({o, k}), DataType::QSymmS8, l.wScales[0], 0, true);
    l.b = perAxis ? TensorInfo(TensorShape({o}), DataType::Signed32, l.bScales, 0, true) : TensorInfo(TensorShape({o}), DataType::Signed32, l.bScales[0], 0, true);
    l.weights.resize(l.w.GetNumElements());
    for (auto& v : l.weights) v = static_cast<int8_t>(r.Range(-127, 127));
    l.bias.resize(o);
    for (auto& v : l.bias) v = r.Range(-2000, 2000);
    return l;
}

/// adds the layer (+ Constant layers, + a separate BoundedReLu Activation layer when relu6) and returns its output slot
inline IOutputSlot& AddToNetwork(INetwork& net, IOutputSlot& input, const QLayer& l, const std::string& name)
{
    IConnectableLayer* wl = net.AddConstantLayer(ConstTensor(l.w, l.weights.data()), (name + "_w").c_str());
    IConnectableLayer* bl = net.AddConstantLayer(ConstTensor(l.b, l.bias.data()), (name + "_b").c_str());
    IConnectableLayer* layer = nullptr;
    if (l.kind == QLayer::FullyConnected)
    {
        FullyConnectedDescriptor d;
        d.m_BiasEnabled = true;
        d.m_TransposeWeightMatrix = true;
        layer = net.AddFullyConnectedLayer(d, name.c_str());
    }
    else if (l.kind == QLayer::Conv)
    {
        Convolution2dDescriptor d;
        d.m_PadTop = l.padTop; d.m_PadBottom = l.padBottom; d.m_PadLeft = l.padLeft; d.m_PadRight = l.padRight;
        d.m_StrideX = d.m_StrideY = l.stride;
        d.m_BiasEnabled = true;
        d.m_DataLayout = DataLayout::NHWC;
        layer = net.AddConvolution2dLayer(d, name.c_str());
    }
    else
    {
        DepthwiseConvolution2dDescriptor d;
        d.m_PadTop = l.padTop; d.m_PadBottom = l.padBottom; d.m_PadLeft = l.padLeft; d.m_PadRight = l.padRight;
        d.m_StrideX = d.m_StrideY = l.stride;
        d.m_BiasEnabled = true;
        d.m_DataLayout = DataLayout::NHWC;
        layer = net.AddDepthwiseConvolution2dLayer(d, name.c_str());
    }
    input.Connect(layer->GetInputSlot(0));
    wl->GetOutputSlot(0).Connect(layer->GetInputSlot(1));
    bl->GetOutputSlot(0).Connect(layer->GetInputSlot(2));
    layer->GetOutputSlot(0).SetTensorInfo(l.out);
    if (!l.relu6) return layer->GetOutputSlot(0);
    IConnectableLayer* act = net.AddActivationLayer(ActivationDescriptor(ActivationFunction::BoundedReLu, l.reluUpper, 0.0f), (name + "_relu6").c_str());
    layer->GetOutputSlot(0).Connect(act->GetInputSlot(0));
    act->GetOutputSlot(0).SetTensorInfo(l.out);
    return act->GetOutputSlot(0);
}

/// what CpuRef would produce for the layer (and its Activation layer) on `input`
inline std::vector<uint8_t> OracleRun(const QLayer& l, const std::vector<uint8_t>& input)
{
    std::vector<uint8_t> out(l.out.GetNumElements());
    const std::vector<float> inS{l.in.GetQuantizationScale()}, outS{l.out.GetQuantizationScale()};
    orc_tensor ti = Orc(l.in, input.data(), inS);
    orc_tensor tw = Orc(l.w, l.weights.data(), l.wScales);
    orc_tensor tb = Orc(l.b, l.bias.data(), l.bScales);
    orc_tensor to = Orc(l.out, out.data(), outS);
    int rc = 0;
    if (l.kind == QLayer::FullyConnected) rc = orc_fully_connected(&ti, &tw, &tb, &to, 1, 1, 1);
    else
    {
        orc_conv_params p{};
        p.pad_top = l.padTop; p.pad_left = l.padLeft; p.stride_x = p.stride_y = l.stride; p.dilation_x = p.dilation_y = 1;
        p.bias_enabled = 1; p.data_layout = ORC_NHWC; p.depthwise = l.kind == QLayer::Depthwise;
        rc = orc_conv2d(&ti, &tw, &tb, &to, &p, 1);
    }
    if (rc != 0) throw std::runtime_error(std::string("oracle: ") + orc_last_error());
    if (l.relu6)
    {
        std::vector<uint8_t> act(out.size());
        orc_tensor ta = Orc(l.out, act.data(), outS);
        if (orc_activation(&to, &ta, ORC_ACT_BOUNDED_RELU, l.reluUpper, 0.0f) != 0) throw std::runtime_error(std::string("oracle: ") + orc_last_error());
        out.swap(act);
    }
    return out;
}

struct Diff { int maxAbs = 0; size_t mismatches = 0; size_t n = 0; };
inline Diff Compare(const std::vector<uint8_t>& a, const std::vector<uint8_t>& b, DataType t)
{
    Diff d;
    d.n = a.size();
    for (size_t i = 0; i < a.size() && i < b.size(); ++i)
    {
        const int x = t == DataType::QAsymmU8 ? a[i] : static_cast<int8_t>(a[i]);
        const int y = t == DataType::QAsymmU8 ? b[i] : static_cast<int8_t>(b[i]);
        const int e = std::abs(x - y);
        d.maxAbs = std::max(d.maxAbs, e);
        d.mismatches += e != 0;
    }
    if (a.size() != b.size()) d.maxAbs = 999;
    return d;
}

class FixedDeviceSpec : public IDeviceSpec
{
public:
    explicit FixedDeviceSpec(std::initializer_list<BackendId> ids) : m_Ids(ids) {}
    const BackendIdSet& GetSupportedBackends() const override { return m_Ids; }
private:
    BackendIdSet m_Ids;
};

inline const Layer* FindLayer(const Graph& g, const std::string& namePart)
{
    for (const auto& l : g.GetLayers())
        if (l->GetNameStr().find(namePart) != std::string::npos) return l.get();
    return nullptr;
}
inline size_t CountLayers(const Graph& g, LayerType t)
{
    size_t n = 0;
    for (const auto& l : g.GetLayers()) n += l->GetType() == t;
    return n;
}
} // namespace tu
