// Tests of the Mi355x backend through the Arm NN backend interfaces.
//   tag "cpu": host logic only -- registry, layer-support envelope, descriptor validation, sub-graph fusion, the arena
//              planner, behaviour when the process sees no device.  These never launch a kernel.
//   tag "gpu": INetwork -> Optimize -> LoadNetwork -> EnqueueWorkload on the device, checked against the CPU oracle
//              (every output byte within 1 LSB of CpuRef's) and against the C ABI called directly (identical bytes).
#include "MiniTest.hpp"
#include "HostTestBackend.hpp"
#include "TestUtils.hpp"

#include "../mi355x/Mi355xBackend.hpp"
#include "../mi355x/Mi355xBackendId.hpp"
#include "../mi355x/Mi355xDevice.hpp"
#include "../mi355x/Mi355xLayerSupport.hpp"
#include "../mi355x/Mi355xMemoryManager.hpp"
#include "../mi355x/Mi355xWorkloads.hpp"
#include "../mi355x/Mi355xTensorHandle.hpp"
#include "../mi355x/Mi355xWorkloadFactory.hpp"

#include "../mi355x/Mi355xTimer.hpp"
#include <Profiling.hpp>

#include <chrono>
#include <functional>
#include <sstream>
#include <thread>
#include <cstring>
#include <backendsCommon/TensorHandleFactoryRegistry.hpp>
#include <armnn/backends/WorkloadData.hpp>

using namespace armnn;
using namespace tu;

namespace
{
const BackendId kMi355x{Mi355xBackendId()};

// Input -> layer(s) -> Output
struct SingleLayerNet
{
    INetworkPtr net = INetwork::Create();
    SingleLayerNet(const QLayer& l)
    {
        IConnectableLayer* in = net->AddInputLayer(0, "input");
        in->GetOutputSlot(0).SetTensorInfo(l.in);
        IOutputSlot& out = AddToNetwork(*net, in->GetOutputSlot(0), l, "layer");
        IConnectableLayer* o = net->AddOutputLayer(0, "output");
        out.Connect(o->GetInputSlot(0));
    }
};

std::vector<uint8_t> RunOnRuntime(IRuntime& rt, const INetwork& net, const std::vector<BackendId>& prefs, const TensorInfo& inInfo,
                                  const std::vector<uint8_t>& input, const TensorInfo& outInfo, int repeats = 1,
                                  const INetworkProperties& properties = INetworkProperties(MemorySource::Undefined, MemorySource::Undefined),
                                  const std::function<void()>& whileLoaded = nullptr)
{
    IOptimizedNetworkPtr opt = Optimize(net, prefs, rt.GetDeviceSpec());
    NetworkId id = -1;
    std::string err;
    if (rt.LoadNetwork(id, std::move(opt), err, properties) != Status::Success) throw std::runtime_error("LoadNetwork failed: " + err);
    std::vector<uint8_t> out(outInfo.GetNumBytes());
    TensorInfo constIn = inInfo;
    constIn.SetConstant(true);
    for (int i = 0; i < repeats; ++i)
    {
        std::fill(out.begin(), out.end(), 0xA5);
        InputTensors ins{{0, ConstTensor(constIn, input.data())}};
        OutputTensors outs{{0, Tensor(outInfo, out.data())}};
        if (rt.EnqueueWorkload(id, ins, outs) != Status::Success) throw std::runtime_error("EnqueueWorkload failed");
    }
    if (whileLoaded) whileLoaded();
    rt.UnloadNetwork(id);
    return out;
}
} // namespace

// ---------------------------------------------------------------------------------------------------------------------
// cpu
// ---------------------------------------------------------------------------------------------------------------------
namespace
{
// The host-only cases test the rules of layer support and of the optimizer on machines without the device; layer support
// itself answers "no" there unless told to assume one (Mi355xDevice.hpp).
const bool g_AssumeDeviceForHostCases = (mi355x::AssumeDevice(true), true);
} // namespace

TEST_CASE("registry: Mi355x is registered by the static initializer", "cpu")
{
    CHECK(BackendRegistryInstance().IsBackendRegistered(kMi355x));
    CHECK(BackendRegistryInstance().GetBackendIdsAsString().find("Mi355x") != std::string::npos);
    auto backend = BackendRegistryInstance().GetFactory(kMi355x)();
    REQUIRE(backend != nullptr);
    CHECK(backend->GetId() == kMi355x);
    CHECK(backend->SupportsTensorAllocatorAPI());
    CHECK(backend->GetHandleFactoryPreferences().front() == std::string(Mi355xTensorHandleFactoryId()));
    CHECK_THROWS_AS(BackendRegistryInstance().Register(kMi355x, [] { return IBackendInternalUniquePtr(); }), InvalidArgumentException);
    CHECK(!HasCapability("Nonexistent", backend->GetCapabilities()));
    CHECK(HasCapability("ConstantTensorsAsInputs", backend->GetCapabilities()));
}

TEST_CASE("layer support: the accepted envelope and the reasons outside it", "cpu")
{
    Mi355xLayerSupport ls;
    std::string why;
    Optional<std::string&> reason(why);
    const TensorInfo in = ActInfo({1, 8, 8, 16}, DataType::QAsymmS8, 0.05f, -3);
    QLayer l = MakeConv(QLayer::Conv, in, 32, 3, 1, 0.1f, 5, false, true, 1);
    Convolution2dDescriptor d;
    d.m_DataLayout = DataLayout::NHWC;
    d.m_BiasEnabled = true;
    d.m_PadLeft = d.m_PadRight = d.m_PadTop = d.m_PadBottom = 1;
    CHECK(ls.IsLayerSupported(LayerType::Convolution2d, {l.in, l.out, l.w, l.b}, d, EmptyOptional(), EmptyOptional(), reason));

    Convolution2dDescriptor nchw = d;
    nchw.m_DataLayout = DataLayout::NCHW;
    CHECK(!ls.IsLayerSupported(LayerType::Convolution2d, {l.in, l.out, l.w, l.b}, nchw, EmptyOptional(), EmptyOptional(), reason));
    CHECK(why.find("NHWC") != std::string::npos);

    TensorInfo f32in = l.in;
    f32in.SetDataType(DataType::Float32);
    CHECK(!ls.IsLayerSupported(LayerType::Convolution2d, {f32in, l.out, l.w, l.b}, d, EmptyOptional(), EmptyOptional(), reason));
    CHECK(why.find("Float32") != std::string::npos);

    TensorInfo dynW = l.w;
    dynW.SetConstant(false);
    CHECK(!ls.IsLayerSupported(LayerType::Convolution2d, {l.in, l.out, dynW, l.b}, d, EmptyOptional(), EmptyOptional(), reason));
    CHECK(why.find("constant") != std::string::npos);

    TensorInfo badBias = l.b;
    badBias.SetQuantizationOffset(1);
    CHECK(!ls.IsLayerSupported(LayerType::Convolution2d, {l.in, l.out, l.w, badBias}, d, EmptyOptional(), EmptyOptional(), reason));

    TensorInfo u8out = l.out;
    u8out.SetDataType(DataType::QAsymmU8);
    CHECK(!ls.IsLayerSupported(LayerType::Convolution2d, {l.in, u8out, l.w, l.b}, d, EmptyOptional(), EmptyOptional(), reason));

    // more taps per output than a 32-bit accumulator is sure to hold (33 025): answered here, so that the optimizer falls
    // back instead of the plan being refused at the first inference.  Only shapes are looked at.
    {
        TensorInfo wideIn({1, 1, 1, 40000}, DataType::QAsymmS8, 0.05f, -3);
        TensorInfo wideW({8, 1, 1, 40000}, DataType::QSymmS8, 0.01f, 0);
        wideW.SetConstant(true);
        TensorInfo wideOut({1, 1, 1, 8}, DataType::QAsymmS8, 0.1f, 5);
        Convolution2dDescriptor plain;
        plain.m_DataLayout = DataLayout::NHWC;
        CHECK(!ls.IsLayerSupported(LayerType::Convolution2d, {wideIn, wideOut, wideW, TensorInfo()}, plain, EmptyOptional(), EmptyOptional(), reason));
        CHECK(why.find("33 025 taps") != std::string::npos);
        TensorInfo okIn({1, 1, 1, 33025}, DataType::QAsymmS8, 0.05f, -3), okW({8, 1, 1, 33025}, DataType::QSymmS8, 0.01f, 0);
        okW.SetConstant(true);
        CHECK(ls.IsLayerSupported(LayerType::Convolution2d, {okIn, wideOut, okW, TensorInfo()}, plain, EmptyOptional(), EmptyOptional(), reason));
        TensorInfo fcIn({2, 40000}, DataType::QAsymmS8, 0.05f, -3), fcW({40000, 8}, DataType::QSymmS8, 0.01f, 0), fcOut({2, 8}, DataType::QAsymmS8, 0.1f, 5);
        fcW.SetConstant(true);
        FullyConnectedDescriptor fd;
        fd.m_BiasEnabled = false;
        CHECK(!ls.IsLayerSupported(LayerType::FullyConnected, {fcIn, fcOut, fcW, TensorInfo()}, fd, EmptyOptional(), EmptyOptional(), reason));
        CHECK(why.find("33 025 taps") != std::string::npos);
    }

    // depthwise: [1,H,W,O] weights quantized along dimension 3
    QLayer dw = MakeConv(QLayer::Depthwise, in, 16, 3, 2, 0.1f, 5, false, true, 2);
    DepthwiseConvolution2dDescriptor dd;
    dd.m_DataLayout = DataLayout::NHWC;
    dd.m_BiasEnabled = true;
    dd.m_StrideX = dd.m_StrideY = 2;
    CHECK(ls.IsLayerSupported(LayerType::DepthwiseConvolution2d, {dw.in, dw.out, dw.w, dw.b}, dd, EmptyOptional(), EmptyOptional(), reason));
    TensorInfo wrongDim = dw.w;
    wrongDim.SetQuantizationDim(Optional<unsigned int>(0u));
    CHECK(!ls.IsLayerSupported(LayerType::DepthwiseConvolution2d, {dw.in, dw.out, wrongDim, dw.b}, dd, EmptyOptional(), EmptyOptional(), reason));

    // activations
    CHECK(ls.IsLayerSupported(LayerType::Activation, {in, in}, ActivationDescriptor(ActivationFunction::ReLu), EmptyOptional(), EmptyOptional(), reason));
    CHECK(ls.IsLayerSupported(LayerType::Activation, {in, in}, ActivationDescriptor(ActivationFunction::BoundedReLu, 6.f, 0.f), EmptyOptional(), EmptyOptional(), reason));
    CHECK(!ls.IsLayerSupported(LayerType::Activation, {in, in}, ActivationDescriptor(ActivationFunction::TanH), EmptyOptional(), EmptyOptional(), reason));
    CHECK(why.find("ReLu") != std::string::npos);

    // pooling / add / softmax / reshape
    Pooling2dDescriptor pd;
    pd.m_DataLayout = DataLayout::NHWC;
    pd.m_PoolType = PoolingAlgorithm::Average;
    pd.m_PoolWidth = pd.m_PoolHeight = 8;
    pd.m_StrideX = pd.m_StrideY = 1;
    const TensorInfo pooled = ActInfo({1, 1, 1, 16}, DataType::QAsymmS8, 0.05f, -3);
    CHECK(ls.IsLayerSupported(LayerType::Pooling2d, {in, pooled}, pd, EmptyOptional(), EmptyOptional(), reason));
    pd.m_PoolType = PoolingAlgorithm::L2;
    CHECK(!ls.IsLayerSupported(LayerType::Pooling2d, {in, pooled}, pd, EmptyOptional(), EmptyOptional(), reason));
    CHECK(ls.IsLayerSupported(LayerType::ElementwiseBinary, {in, in, in}, ElementwiseBinaryDescriptor(BinaryOperation::Add), EmptyOptional(), EmptyOptional(), reason));
    CHECK(!ls.IsLayerSupported(LayerType::ElementwiseBinary, {in, in, in}, ElementwiseBinaryDescriptor(BinaryOperation::Mul), EmptyOptional(), EmptyOptional(), reason));
    CHECK(!ls.IsLayerSupported(LayerType::ElementwiseBinary, {in, pooled, in}, ElementwiseBinaryDescriptor(BinaryOperation::Add), EmptyOptional(), EmptyOptional(), reason));
    SoftmaxDescriptor sd;
    const TensorInfo logits = ActInfo({4, 10}, DataType::QAsymmU8, 0.1f, 128);
    const TensorInfo probs = ActInfo({4, 10}, DataType::QAsymmU8, 1.0f / 256.0f, 0);
    CHECK(ls.IsLayerSupported(LayerType::Softmax, {logits, probs}, sd, EmptyOptional(), EmptyOptional(), reason));
    sd.m_Axis = 0;
    CHECK(!ls.IsLayerSupported(LayerType::Softmax, {logits, probs}, sd, EmptyOptional(), EmptyOptional(), reason));

    // Mean: over height and width only, kept dimensions or not
    const TensorInfo meanIn = ActInfo({2, 7, 7, 64}, DataType::QAsymmS8, 0.05f, -3);
    CHECK(ls.IsLayerSupported(LayerType::Mean, {meanIn, ActInfo({2, 1, 1, 64}, DataType::QAsymmS8, 0.05f, -3)}, MeanDescriptor({1, 2}, true), EmptyOptional(), EmptyOptional(), reason));
    CHECK(ls.IsLayerSupported(LayerType::Mean, {meanIn, ActInfo({2, 64}, DataType::QAsymmS8, 0.04f, 5)}, MeanDescriptor({2, 1}, false), EmptyOptional(), EmptyOptional(), reason));
    CHECK(!ls.IsLayerSupported(LayerType::Mean, {meanIn, ActInfo({2, 7, 7, 1}, DataType::QAsymmS8, 0.05f, -3)}, MeanDescriptor({3}, true), EmptyOptional(), EmptyOptional(), reason));
    CHECK_MSG(why.find("height and width") != std::string::npos, why);
    CHECK(!ls.IsLayerSupported(LayerType::Mean, {meanIn, ActInfo({2, 64, 1}, DataType::QAsymmS8, 0.05f, -3)}, MeanDescriptor({1, 2}, false), EmptyOptional(), EmptyOptional(), reason));

    // Pad: constant mode, ranks 1..4, the output shape must be the padded input shape
    PadDescriptor padDesc({{0, 0}, {1, 1}, {2, 0}, {0, 0}}, -3.0f);
    const TensorInfo padIn = ActInfo({1, 8, 8, 16}, DataType::QAsymmS8, 0.05f, -3), padOut = ActInfo({1, 10, 10, 16}, DataType::QAsymmS8, 0.05f, -3);
    CHECK(ls.IsLayerSupported(LayerType::Pad, {padIn, padOut}, padDesc, EmptyOptional(), EmptyOptional(), reason));
    CHECK(!ls.IsLayerSupported(LayerType::Pad, {padIn, ActInfo({1, 10, 9, 16}, DataType::QAsymmS8, 0.05f, -3)}, padDesc, EmptyOptional(), EmptyOptional(), reason));
    CHECK_MSG(why.find("output shape") != std::string::npos, why);
    padDesc.m_PaddingMode = PaddingMode::Reflect;
    CHECK(!ls.IsLayerSupported(LayerType::Pad, {padIn, padOut}, padDesc, EmptyOptional(), EmptyOptional(), reason));
    CHECK_MSG(why.find("constant") != std::string::npos, why);
    CHECK(ls.IsLayerSupported(LayerType::Reshape, {pooled, ActInfo({1, 16}, DataType::QAsymmS8, 0.05f, -3)}, ReshapeDescriptor(TensorShape({1, 16})), EmptyOptional(), EmptyOptional(), reason));
}

TEST_CASE("queue descriptors: Validate enforces the quantized conv rules", "cpu")
{
    const TensorInfo in = ActInfo({1, 8, 8, 16}, DataType::QAsymmS8, 0.05f, -3);
    QLayer l = MakeConv(QLayer::Conv, in, 32, 3, 1, 0.1f, 5, false, true, 3);
    Convolution2dQueueDescriptor q;
    q.m_Parameters.m_BiasEnabled = true;
    q.m_Parameters.m_DataLayout = DataLayout::NHWC;
    WorkloadInfo info;
    info.m_InputTensorInfos = {l.in, l.w, l.b};
    info.m_OutputTensorInfos = {l.out};
    CHECK_NOTHROW(q.Validate(info));

    WorkloadInfo bad = info;
    bad.m_InputTensorInfos[2].SetQuantizationOffset(7);                       // bias offset must be 0
    CHECK_THROWS_AS(q.Validate(bad), InvalidArgumentException);
    bad = info;
    bad.m_InputTensorInfos[2] = TensorInfo(TensorShape({32}), DataType::Signed32, 0.001f, 0, true);   // per-axis weights need per-axis bias
    CHECK_THROWS_AS(q.Validate(bad), InvalidArgumentException);
    bad = info;
    bad.m_InputTensorInfos[1].SetDataType(DataType::QAsymmU8);                // per-axis weights must be QSymmS8
    CHECK_THROWS_AS(q.Validate(bad), InvalidArgumentException);
    bad = info;
    bad.m_OutputTensorInfos[0].SetDataType(DataType::QAsymmU8);               // input and output types must match
    CHECK_THROWS_AS(q.Validate(bad), InvalidArgumentException);
    bad = info;
    bad.m_InputTensorInfos.pop_back();                                          // bias enabled means three inputs
    CHECK_THROWS_AS(q.Validate(bad), InvalidArgumentException);
    Convolution2dQueueDescriptor zeroStride = q;
    zeroStride.m_Parameters.m_StrideX = 0;
    CHECK_THROWS_AS(zeroStride.Validate(info), InvalidArgumentException);

    QLayer dw = MakeConv(QLayer::Depthwise, in, 16, 3, 1, 0.1f, 5, false, true, 4);
    DepthwiseConvolution2dQueueDescriptor dq;
    dq.m_Parameters.m_BiasEnabled = true;
    dq.m_Parameters.m_DataLayout = DataLayout::NHWC;
    WorkloadInfo dinfo;
    dinfo.m_InputTensorInfos = {dw.in, dw.w, dw.b};
    dinfo.m_OutputTensorInfos = {dw.out};
    CHECK_NOTHROW(dq.Validate(dinfo));
    WorkloadInfo dbad = dinfo;
    dbad.m_InputTensorInfos[1].SetShape(TensorShape({2, 3, 3, 8}));           // weights must be [1,H,W,O]
    CHECK_THROWS_AS(dq.Validate(dbad), InvalidArgumentException);
    DepthwiseConvolution2dQueueDescriptor dil = dq;
    dil.m_Parameters.m_DilationX = 0;
    CHECK_THROWS_AS(dil.Validate(dinfo), InvalidArgumentException);

    QLayer fc = MakeFc(ActInfo({2, 64}, DataType::QAsymmS8, 0.05f, 0), 10, 0.2f, 0, false, 5);
    FullyConnectedQueueDescriptor fq;
    fq.m_Parameters.m_BiasEnabled = true;
    fq.m_Parameters.m_TransposeWeightMatrix = true;
    WorkloadInfo finfo;
    finfo.m_InputTensorInfos = {fc.in, fc.w, fc.b};
    finfo.m_OutputTensorInfos = {fc.out};
    CHECK_NOTHROW(fq.Validate(finfo));
    WorkloadInfo fbad = finfo;
    fbad.m_InputTensorInfos[2].SetDataType(DataType::Float32);                // bias of a quantized layer is Signed32
    CHECK_THROWS_AS(fq.Validate(fbad), InvalidArgumentException);
}

TEST_CASE("arena planner: lifetimes that do not overlap share addresses, one retirement late", "cpu")
{
    Mi355xMemoryManager mm;
    const size_t a = mm.Reserve(1000);      // 1024
    const size_t b = mm.Reserve(5000);      // 5120
    CHECK(a == 0);
    CHECK(b == 1024);
    mm.Retire(a, 1000);                     // a's range is free once the next range has been retired
    const size_t c = mm.Reserve(512);
    CHECK(c == 6144);
    mm.Retire(c, 512);                      // now a's hole is free, c's is pending
    const size_t d = mm.Reserve(512);       // first half of a's hole
    CHECK(d == 0);
    const size_t e = mm.Reserve(512);       // second half
    CHECK(e == 512);
    mm.Retire(b, 5000);                     // frees c
    mm.Retire(d, 512);                      // frees b
    mm.Retire(e, 512);                      // frees d
    mm.Retire(0, 0);                        // (a lifetime of nothing) frees e: everything free again and coalesced
    const size_t f = mm.Reserve(6144 + 512);
    CHECK(f == 0);
    CHECK(mm.ArenaBytes() == 6144 + 512);
    const size_t g = mm.Reserve(100);       // grows past the end
    CHECK(g == 6144 + 512);
    mm.Retire(g, 100);
    mm.Retire(f, 6144 + 512);               // frees g's granule at the end
    const size_t h = mm.Reserve(300);       // the free tail is extended, not left behind
    CHECK(h == 6144 + 512);
    CHECK(mm.ArenaBytes() == 6144 + 512 + 512);
    CHECK(mm.ReservedTotal() > mm.ArenaBytes());
    CHECK_THROWS_AS(mm.Resolve(0), MemoryValidationException);   // nothing acquired yet
}

TEST_CASE("arena planner: the output of the layer behind a tensor's last consumer never lies over that tensor", "cpu")
{
    // the order in which a runtime walks a chain x -> depthwise -> t -> pointwise -> y -> next -> z: a layer's output begins
    // before the layer's inputs end
    Mi355xMemoryManager mm;
    const size_t x = mm.Reserve(4096);
    const size_t t = mm.Reserve(4096);      // depthwise: its output begins ...
    mm.Retire(x, 4096);                     // ... then its input ends
    const size_t y = mm.Reserve(4096);      // pointwise: reads t; a fused launch reads x and writes y
    CHECK(y != x);
    CHECK(y != t);
    mm.Retire(t, 4096);
    const size_t z = mm.Reserve(4096);      // the layer after: x's range is free by now
    CHECK(z == x);
}

TEST_CASE("tensor handle: lifecycle errors are reported, not ignored", "cpu")
{
    auto mm = std::make_shared<Mi355xMemoryManager>();
    const TensorInfo info = ActInfo({1, 4, 4, 8}, DataType::QAsymmS8, 0.1f, 0);
    Mi355xTensorHandle managed(info, mm, true);
    CHECK(managed.IsManaged());
    CHECK_THROWS_AS(managed.GetDevicePointer(), NullPointerException);
    managed.Manage();
    CHECK_THROWS_AS(managed.Manage(), InvalidArgumentException);
    CHECK_THROWS_AS(managed.GetDevicePointer(), MemoryValidationException);  // arena not acquired
    managed.Allocate();
    CHECK_THROWS_AS(managed.Allocate(), InvalidArgumentException);
    CHECK(managed.GetShape() == info.GetShape());
    CHECK(managed.GetStrides()[3] == 1);
    CHECK(managed.GetStrides()[0] == 4 * 4 * 8);
    Mi355xTensorHandle unmanaged(info, mm, false);
    CHECK(!unmanaged.IsManaged());
    CHECK_THROWS_AS(unmanaged.GetDevicePointer(), NullPointerException);     // Allocate() not called
}

namespace
{
INetworkPtr ConvReluNet(bool sameQuant, bool secondConsumer)
{
    INetworkPtr net = INetwork::Create();
    const TensorInfo in = ActInfo({1, 8, 8, 16}, DataType::QAsymmS8, 0.05f, -3);
    QLayer l = MakeConv(QLayer::Conv, in, 32, 3, 1, 0.1f, -128, false, true, 11);
    IConnectableLayer* input = net->AddInputLayer(0, "input");
    input->GetOutputSlot(0).SetTensorInfo(in);
    IOutputSlot& convOut = AddToNetwork(*net, input->GetOutputSlot(0), l, "conv");
    IConnectableLayer* act = net->AddActivationLayer(ActivationDescriptor(ActivationFunction::BoundedReLu, 6.0f, 0.0f), "relu6");
    convOut.Connect(act->GetInputSlot(0));
    TensorInfo actOut = l.out;
    if (!sameQuant) actOut.SetQuantizationScale(0.05f);
    act->GetOutputSlot(0).SetTensorInfo(actOut);
    IConnectableLayer* out = net->AddOutputLayer(0, "output");
    act->GetOutputSlot(0).Connect(out->GetInputSlot(0));
    if (secondConsumer)
    {
        IConnectableLayer* out2 = net->AddOutputLayer(1, "output2");
        convOut.Connect(out2->GetInputSlot(0));
    }
    return net;
}
} // namespace

TEST_CASE("optimize: BoundedReLu is folded into the convolution only when that changes no byte", "cpu")
{
    FixedDeviceSpec spec{kMi355x};
    {
        INetworkPtr net = ConvReluNet(true, false);
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec);
        const Graph& g = opt->GetGraph();
        CHECK(CountLayers(g, LayerType::Activation) == 0);
        CHECK(CountLayers(g, LayerType::Convolution2d) == 1);
        const Layer* fused = FindLayer(g, "fused-");
        REQUIRE(fused != nullptr);
        auto ad = fused->GetAdditionalInformation<ActivationDescriptor>();
        REQUIRE(ad != nullptr);
        CHECK(ad->m_Function == ActivationFunction::BoundedReLu);
        CHECK(ad->m_A == 6.0f);
        CHECK(fused->GetBackendId() == kMi355x);
        CHECK(fused->GetNumInputSlots() == 3);
        CHECK(fused->In(1).GetConnectedOutputSlot()->GetOwningLayer().GetType() == LayerType::Constant);
        CHECK(fused->Out(0).GetConnections()[0]->GetOwningLayer().GetType() == LayerType::Output);
        CHECK(CountLayers(g, LayerType::MemCopy) == 0);
    }
    {
        INetworkPtr net = ConvReluNet(false, false);       // the activation re-quantizes: it stays a layer
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec);
        CHECK(CountLayers(opt->GetGraph(), LayerType::Activation) == 1);
        CHECK(FindLayer(opt->GetGraph(), "fused-") == nullptr);
    }
    {
        INetworkPtr net = ConvReluNet(true, true);         // the pre-activation tensor is also a network output
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec);
        CHECK(CountLayers(opt->GetGraph(), LayerType::Activation) == 1);
    }
}

namespace
{
// input -> 3x3 conv + ReLU6 -> 1x1 conv (64 -> 256) --+
//   \-------------- 1x1 shortcut conv (64 -> 256) ----+-> Addition + ReLU -> output
struct ResidualBlock
{
    TensorInfo in, sum;
    QLayer first, last, shortcut;
    explicit ResidualBlock(unsigned int batch, unsigned int side = 16)
    {
        in = ActInfo({batch, side, side, 64}, DataType::QAsymmS8, 0.05f, -3);
        first = MakeConv(QLayer::Conv, in, 64, 3, 1, 0.04f, -128, true, true, 31);
        last = MakeConv(QLayer::Conv, first.out, 256, 1, 1, 0.09f, 5, false, true, 32);
        shortcut = MakeConv(QLayer::Conv, in, 256, 1, 1, 0.07f, -9, false, false, 33);
        sum = TensorInfo(last.out.GetShape(), DataType::QAsymmS8, 0.06f, -128);
    }
    INetworkPtr Build(bool lastAlsoAnOutput = false) const
    {
        INetworkPtr net = INetwork::Create();
        IConnectableLayer* input = net->AddInputLayer(0, "input");
        input->GetOutputSlot(0).SetTensorInfo(in);
        IOutputSlot& a = AddToNetwork(*net, input->GetOutputSlot(0), first, "first");
        IOutputSlot& b = AddToNetwork(*net, a, last, "last");
        IOutputSlot& c = AddToNetwork(*net, input->GetOutputSlot(0), shortcut, "shortcut");
        IConnectableLayer* add = net->AddElementwiseBinaryLayer(ElementwiseBinaryDescriptor(BinaryOperation::Add), "add");
        b.Connect(add->GetInputSlot(0));
        c.Connect(add->GetInputSlot(1));
        add->GetOutputSlot(0).SetTensorInfo(sum);
        IConnectableLayer* relu = net->AddActivationLayer(ActivationDescriptor(ActivationFunction::ReLu, 0.0f, 0.0f), "relu");
        add->GetOutputSlot(0).Connect(relu->GetInputSlot(0));
        relu->GetOutputSlot(0).SetTensorInfo(sum);
        IConnectableLayer* out = net->AddOutputLayer(0, "output");
        relu->GetOutputSlot(0).Connect(out->GetInputSlot(0));
        if (lastAlsoAnOutput)
        {
            IConnectableLayer* out2 = net->AddOutputLayer(1, "output2");
            b.Connect(out2->GetInputSlot(0));
        }
        return net;
    }
};

const Layer* ConvolutionNamed(const Graph& g, const std::string& name)
{
    for (const auto& l : g.GetLayers())
        if (l->GetType() == LayerType::Convolution2d && l->GetNameStr() == name) return l.get();
    return nullptr;
}

// input (64 channels) -> 3x3 conv to 256 channels + ReLU6 -> 1x1 conv back to 64 channels -+-> Addition + ReLU -> output
//   \------------------------------------------------------------------------------------+
// The 1x1 convolution's input is four times the sum and dies where the sum is born: an arena that shares addresses puts
// the sum there.
struct NarrowingResidualBlock
{
    TensorInfo in, sum;
    QLayer first, last;
    explicit NarrowingResidualBlock(unsigned int batch)
    {
        in = ActInfo({batch, 16, 16, 64}, DataType::QAsymmS8, 0.05f, -3);
        first = MakeConv(QLayer::Conv, in, 256, 3, 1, 0.04f, -128, true, true, 41);
        last = MakeConv(QLayer::Conv, first.out, 64, 1, 1, 0.09f, 5, false, true, 42);
        sum = TensorInfo(last.out.GetShape(), DataType::QAsymmS8, 0.06f, -128);
    }
    INetworkPtr Build() const
    {
        INetworkPtr net = INetwork::Create();
        IConnectableLayer* input = net->AddInputLayer(0, "input");
        input->GetOutputSlot(0).SetTensorInfo(in);
        IOutputSlot& a = AddToNetwork(*net, input->GetOutputSlot(0), first, "first");
        IOutputSlot& b = AddToNetwork(*net, a, last, "last");
        IConnectableLayer* add = net->AddElementwiseBinaryLayer(ElementwiseBinaryDescriptor(BinaryOperation::Add), "add");
        input->GetOutputSlot(0).Connect(add->GetInputSlot(0));
        b.Connect(add->GetInputSlot(1));
        add->GetOutputSlot(0).SetTensorInfo(sum);
        IConnectableLayer* relu = net->AddActivationLayer(ActivationDescriptor(ActivationFunction::ReLu, 0.0f, 0.0f), "relu");
        add->GetOutputSlot(0).Connect(relu->GetInputSlot(0));
        relu->GetOutputSlot(0).SetTensorInfo(sum);
        IConnectableLayer* out = net->AddOutputLayer(0, "output");
        relu->GetOutputSlot(0).Connect(out->GetInputSlot(0));
        return net;
    }
};

bool MarkedForAnAddition(const Layer* l)
{
    auto ad = l ? l->GetAdditionalInformation<ActivationDescriptor>() : nullptr;
    return ad && ad->m_Function == ActivationFunction::Linear && ad->m_A == 1.0f && ad->m_B == 0.0f;
}
} // namespace

TEST_CASE("optimize: a convolution that feeds one Addition and nothing else is marked for it, unless the network says no", "cpu")
{
    FixedDeviceSpec spec{kMi355x};
    ResidualBlock block(1);
    {
        INetworkPtr net = block.Build();
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec);
        const Graph& g = opt->GetGraph();
        CHECK(CountLayers(g, LayerType::Convolution2d) == 3);
        CHECK(CountLayers(g, LayerType::ElementwiseBinary) == 1);
        CHECK(CountLayers(g, LayerType::Activation) == 0);
        CHECK(MarkedForAnAddition(ConvolutionNamed(g, "last")));
        CHECK(MarkedForAnAddition(ConvolutionNamed(g, "shortcut")));
        const Layer* first = FindLayer(g, "fused-first_relu6-into-first");
        REQUIRE(first != nullptr);
        CHECK(!MarkedForAnAddition(first));
        const Layer* add = FindLayer(g, "fused-relu-into-add");
        REQUIRE(add != nullptr);
        CHECK(&add->In(0).GetConnectedOutputSlot()->GetOwningLayer() == ConvolutionNamed(g, "last"));
        CHECK(&add->In(1).GetConnectedOutputSlot()->GetOwningLayer() == ConvolutionNamed(g, "shortcut"));
    }
    {
        INetworkPtr net = block.Build(true);               // the convolution's own output is wanted as well
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec);
        CHECK(!MarkedForAnAddition(ConvolutionNamed(opt->GetGraph(), "last")));
        CHECK(MarkedForAnAddition(ConvolutionNamed(opt->GetGraph(), "shortcut")));
    }
    {
        INetworkPtr net = block.Build();
        OptimizerOptionsOpaque options;
        options.AddModelOption(BackendOptions("Mi355x", {{"FuseAdditions", false}}));
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec, options);
        CHECK(!MarkedForAnAddition(ConvolutionNamed(opt->GetGraph(), "last")));
        CHECK(!MarkedForAnAddition(ConvolutionNamed(opt->GetGraph(), "shortcut")));
        // model options that name the backend: it still hands out layer support and factories (the interface's defaults
        // answer with nothing then, IBackendInternal.cpp:24-58, 88-102)
        Mi355xBackend backend;
        CHECK(backend.GetLayerSupport(options.GetModelOptions()) != nullptr);
        CHECK(backend.CreateWorkloadFactory(IBackendInternal::IMemoryManagerSharedPtr(), options.GetModelOptions()) != nullptr);
        TensorHandleFactoryRegistry registry;
        backend.RegisterTensorHandleFactories(registry);
        CHECK(backend.CreateWorkloadFactory(registry, options.GetModelOptions()) != nullptr);
    }
}

namespace
{
// input [n, 2, 2, 16] -> Reshape -> FullyConnected (64 -> 10) + ReLU6 -> output
INetworkPtr ReshapeFcNet(const TensorShape& reshaped, bool reshapedAlsoAnOutput)
{
    INetworkPtr net = INetwork::Create();
    const TensorInfo in = ActInfo({2, 2, 2, 16}, DataType::QAsymmS8, 0.05f, -3);
    TensorInfo flat = in;
    flat.SetShape(reshaped);
    QLayer fc = MakeFc(flat, 10, 0.1f, -128, true, 17);
    fc.relu6 = true;
    IConnectableLayer* input = net->AddInputLayer(0, "input");
    input->GetOutputSlot(0).SetTensorInfo(in);
    IConnectableLayer* reshape = net->AddReshapeLayer(ReshapeDescriptor(reshaped), "reshape");
    input->GetOutputSlot(0).Connect(reshape->GetInputSlot(0));
    reshape->GetOutputSlot(0).SetTensorInfo(flat);
    IOutputSlot& out = AddToNetwork(*net, reshape->GetOutputSlot(0), fc, "fc");
    IConnectableLayer* output = net->AddOutputLayer(0, "output");
    out.Connect(output->GetInputSlot(0));
    if (reshapedAlsoAnOutput)
    {
        IConnectableLayer* out2 = net->AddOutputLayer(1, "output2");
        reshape->GetOutputSlot(0).Connect(out2->GetInputSlot(0));
    }
    return net;
}
} // namespace

TEST_CASE("optimize: a Reshape that only flattens what follows the batch goes into the FullyConnected behind it", "cpu")
{
    FixedDeviceSpec spec{kMi355x};
    {
        INetworkPtr net = ReshapeFcNet(TensorShape({2, 64}), false);
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec);
        const Graph& g = opt->GetGraph();
        CHECK(CountLayers(g, LayerType::Reshape) == 0);
        CHECK(CountLayers(g, LayerType::Activation) == 0);
        CHECK(CountLayers(g, LayerType::FullyConnected) == 1);
        const Layer* fc = FindLayer(g, "folded-reshape-into-fc");
        REQUIRE(fc != nullptr);
        CHECK(fc->GetType() == LayerType::FullyConnected);
        CHECK(fc->In(0).GetConnectedOutputSlot()->GetOwningLayer().GetType() == LayerType::Input);
        CHECK(fc->In(0).GetConnectedOutputSlot()->GetTensorInfo().GetNumDimensions() == 4);
        CHECK(fc->In(1).GetConnectedOutputSlot()->GetOwningLayer().GetType() == LayerType::Constant);
        CHECK(fc->Out(0).GetTensorInfo().GetShape() == TensorShape({2, 10}));
        auto ad = fc->GetAdditionalInformation<ActivationDescriptor>();
        REQUIRE(ad != nullptr);
        CHECK(ad->m_Function == ActivationFunction::BoundedReLu);
    }
    {
        INetworkPtr net = ReshapeFcNet(TensorShape({1, 128}), false);      // the batch dimension changes: rows would differ
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec);
        CHECK(CountLayers(opt->GetGraph(), LayerType::Reshape) == 1);
    }
    {
        INetworkPtr net = ReshapeFcNet(TensorShape({2, 64}), true);        // the flattened tensor is wanted as well
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec);
        CHECK(CountLayers(opt->GetGraph(), LayerType::Reshape) == 1);
    }
}

namespace
{
using PadList = std::vector<std::pair<unsigned int, unsigned int>>;

TensorInfo Padded(const TensorInfo& in, const PadList& pads)
{
    std::vector<unsigned int> dims;
    for (unsigned int k = 0; k < in.GetNumDimensions(); ++k) dims.push_back(in.GetShape()[k] + pads[k].first + pads[k].second);
    TensorInfo out = in;
    out.SetShape(TensorShape(static_cast<unsigned int>(dims.size()), dims.data()));
    return out;
}

// Input -> Pad -> conv / depthwise (+ BoundedReLu); `extraConsumer` makes the padded tensor a network output as well
INetworkPtr PadConvNet(const TensorInfo& in, const PadList& pads, float padValue, const QLayer& conv, bool extraConsumer = false)
{
    INetworkPtr net = INetwork::Create();
    IConnectableLayer* input = net->AddInputLayer(0, "input");
    input->GetOutputSlot(0).SetTensorInfo(in);
    IConnectableLayer* pad = net->AddPadLayer(PadDescriptor(pads, padValue), "pad");
    input->GetOutputSlot(0).Connect(pad->GetInputSlot(0));
    pad->GetOutputSlot(0).SetTensorInfo(Padded(in, pads));
    IOutputSlot& out = AddToNetwork(*net, pad->GetOutputSlot(0), conv, "conv");
    IConnectableLayer* o = net->AddOutputLayer(0, "output");
    out.Connect(o->GetInputSlot(0));
    if (extraConsumer)
    {
        IConnectableLayer* o2 = net->AddOutputLayer(1, "padded");
        pad->GetOutputSlot(0).Connect(o2->GetInputSlot(0));
    }
    return net;
}

// Input -> Pad -> Pooling2d
INetworkPtr PadPoolNet(const TensorInfo& in, const PadList& pads, float padValue, const Pooling2dDescriptor& pool, const TensorInfo& out)
{
    INetworkPtr net = INetwork::Create();
    IConnectableLayer* input = net->AddInputLayer(0, "input");
    input->GetOutputSlot(0).SetTensorInfo(in);
    IConnectableLayer* pad = net->AddPadLayer(PadDescriptor(pads, padValue), "pad");
    input->GetOutputSlot(0).Connect(pad->GetInputSlot(0));
    pad->GetOutputSlot(0).SetTensorInfo(Padded(in, pads));
    IConnectableLayer* p = net->AddPooling2dLayer(pool, "pool");
    pad->GetOutputSlot(0).Connect(p->GetInputSlot(0));
    p->GetOutputSlot(0).SetTensorInfo(out);
    IConnectableLayer* o = net->AddOutputLayer(0, "output");
    p->GetOutputSlot(0).Connect(o->GetInputSlot(0));
    return net;
}

Pooling2dDescriptor Pool3x3s2(PoolingAlgorithm algo)
{
    Pooling2dDescriptor d;
    d.m_PoolType = algo;
    d.m_PoolWidth = d.m_PoolHeight = 3;
    d.m_StrideX = d.m_StrideY = 2;
    d.m_DataLayout = DataLayout::NHWC;
    return d;
}
} // namespace

TEST_CASE("optimize: a Pad of height and width moves into the layer behind it when the padded value is neutral there", "cpu")
{
    FixedDeviceSpec spec{kMi355x};
    const TensorInfo in = ActInfo({2, 10, 12, 16}, DataType::QAsymmS8, 0.05f, -3);
    const PadList hw{{0, 0}, {1, 2}, {3, 0}, {0, 0}};
    const QLayer conv = MakeConv(QLayer::Conv, Padded(in, hw), 32, 3, 1, 0.1f, -128, true, true, 41);     // SAME: own padding 1
    {
        INetworkPtr net = PadConvNet(in, hw, -3.0f, conv);                  // the zero point: what a skipped tap contributes
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec);
        const Graph& g = opt->GetGraph();
        CHECK(CountLayers(g, LayerType::Pad) == 0);
        CHECK(CountLayers(g, LayerType::Activation) == 0);
        CHECK(CountLayers(g, LayerType::Convolution2d) == 1);
        const Layer* folded = FindLayer(g, "folded-pad-into-conv");
        REQUIRE(folded != nullptr);
        CHECK(folded->GetNameStr().find("fused-") == 0);
        const auto& d = static_cast<const Convolution2dDescriptor&>(folded->GetParameters());
        CHECK(d.m_PadTop == 2); CHECK(d.m_PadBottom == 3); CHECK(d.m_PadLeft == 4); CHECK(d.m_PadRight == 1);
        CHECK(folded->GetAdditionalInformation<ActivationDescriptor>() != nullptr);
        CHECK(folded->In(0).GetConnectedOutputSlot()->GetOwningLayer().GetType() == LayerType::Input);
        CHECK(folded->In(1).GetConnectedOutputSlot()->GetOwningLayer().GetType() == LayerType::Constant);
        CHECK(folded->In(2).GetConnectedOutputSlot()->GetOwningLayer().GetType() == LayerType::Constant);
        CHECK(folded->Out(0).GetTensorInfo().GetShape() == conv.out.GetShape());
    }
    {
        INetworkPtr net = PadConvNet(in, hw, 0.0f, conv);                   // code 0 is the real number 0.15 here: not neutral
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec);
        CHECK(CountLayers(opt->GetGraph(), LayerType::Pad) == 1);
        CHECK(FindLayer(opt->GetGraph(), "folded-") == nullptr);
        CHECK(FindLayer(opt->GetGraph(), "fused-") != nullptr);             // the activation is still fused
    }
    {
        const PadList withChannels{{0, 0}, {1, 1}, {1, 1}, {0, 16}};
        QLayer c2 = MakeConv(QLayer::Conv, Padded(in, withChannels), 8, 1, 1, 0.1f, -128, false, true, 42);
        IOptimizedNetworkPtr opt = Optimize(*PadConvNet(in, withChannels, -3.0f, c2), {kMi355x}, spec);
        CHECK(CountLayers(opt->GetGraph(), LayerType::Pad) == 1);
    }
    {
        IOptimizedNetworkPtr opt = Optimize(*PadConvNet(in, hw, -3.0f, conv, true), {kMi355x}, spec);      // the padded tensor is read elsewhere
        CHECK(CountLayers(opt->GetGraph(), LayerType::Pad) == 1);
    }
    {
        const QLayer dw = MakeConv(QLayer::Depthwise, Padded(in, hw), 16, 3, 2, 0.1f, -128, false, true, 43);
        IOptimizedNetworkPtr opt = Optimize(*PadConvNet(in, hw, -3.0f, dw), {kMi355x}, spec);
        CHECK(CountLayers(opt->GetGraph(), LayerType::Pad) == 0);
        REQUIRE(FindLayer(opt->GetGraph(), "folded-pad-into-conv") != nullptr);
        CHECK(FindLayer(opt->GetGraph(), "folded-pad-into-conv")->GetType() == LayerType::DepthwiseConvolution2d);
    }
    // pooling: Max needs a value no element can undercut, Average needs zeros that count in the divisor
    const TensorInfo padded = Padded(in, hw);
    const TensorInfo pooled = ActInfo({2, (padded.GetShape()[1] - 3) / 2 + 1, (padded.GetShape()[2] - 3) / 2 + 1, 16}, DataType::QAsymmS8, 0.05f, -3);
    {
        IOptimizedNetworkPtr opt = Optimize(*PadPoolNet(in, hw, -128.0f, Pool3x3s2(PoolingAlgorithm::Max), pooled), {kMi355x}, spec);
        CHECK(CountLayers(opt->GetGraph(), LayerType::Pad) == 0);
        const Layer* p = FindLayer(opt->GetGraph(), "folded-pad-into-pool");
        REQUIRE(p != nullptr);
        const auto& d = static_cast<const Pooling2dDescriptor&>(p->GetParameters());
        CHECK(d.m_PaddingMethod == PaddingMethod::IgnoreValue);
        CHECK(d.m_PadTop == 1); CHECK(d.m_PadBottom == 2); CHECK(d.m_PadLeft == 3); CHECK(d.m_PadRight == 0);
    }
    {
        IOptimizedNetworkPtr opt = Optimize(*PadPoolNet(in, hw, -3.0f, Pool3x3s2(PoolingAlgorithm::Max), pooled), {kMi355x}, spec);
        CHECK(CountLayers(opt->GetGraph(), LayerType::Pad) == 1);           // an element below the zero point would lose to the padding
    }
    {
        IOptimizedNetworkPtr opt = Optimize(*PadPoolNet(in, hw, -3.0f, Pool3x3s2(PoolingAlgorithm::Average), pooled), {kMi355x}, spec);
        CHECK(CountLayers(opt->GetGraph(), LayerType::Pad) == 0);
    }
    {
        Pooling2dDescriptor own = Pool3x3s2(PoolingAlgorithm::Average);     // padding of its own, left out of the divisor
        own.m_PadLeft = own.m_PadRight = 1;
        own.m_PaddingMethod = PaddingMethod::Exclude;
        const TensorInfo o2 = ActInfo({2, pooled.GetShape()[1], (padded.GetShape()[2] + 2 - 3) / 2 + 1, 16}, DataType::QAsymmS8, 0.05f, -3);
        IOptimizedNetworkPtr opt = Optimize(*PadPoolNet(in, hw, -3.0f, own, o2), {kMi355x}, spec);
        CHECK(CountLayers(opt->GetGraph(), LayerType::Pad) == 1);
    }
}

TEST_CASE("profiling: events nest as their scopes do, exist only while the profiler is on, and print as JSON", "cpu")
{
    IProfiler profiler;
    ProfilerManager::GetInstance().RegisterProfiler(&profiler);
    {
        // off: nothing is recorded, and the device timer handed to the macro is never started (no device is needed)
        ARMNN_SCOPED_PROFILING_EVENT_WITH_INSTRUMENTS(kMi355x, EmptyOptional(), std::string("ignored"), Mi355xTimer(), WallClockTimer())
    }
    CHECK(profiler.GetEvents().empty());
    profiler.EnableProfiling(true);
    CHECK(profiler.IsProfilingEnabled());
    {
        ARMNN_SCOPED_PROFILING_EVENT(BackendId(), "outer");
        {
            ARMNN_SCOPED_PROFILING_EVENT_GUID(kMi355x, "inner \"quoted\"", arm::pipe::ProfilingGuid(42));
            std::this_thread::sleep_for(std::chrono::milliseconds(2));
        }
        ARMNN_SCOPED_PROFILING_EVENT(kMi355x, "second inner");
    }
    WorkloadInfo info;
    info.m_Name = "conv";
    info.m_InputTensorInfos = {ActInfo({1, 8, 8, 16}, DataType::QAsymmS8, 0.05f, -3)};
    info.m_ConvolutionMethod = Optional<std::string>("igemm 64x64");
    Convolution2dDescriptor cd;
    cd.m_PadLeft = 3;
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Conv_Construct", cd, info, arm::pipe::ProfilingGuid(7))
    ProfilerManager::GetInstance().RegisterProfiler(nullptr);

    const auto& events = profiler.GetEvents();
    REQUIRE(events.size() == 3);
    CHECK(events[0]->GetName() == "outer");
    CHECK(events[0]->GetParentEvent() == nullptr);
    CHECK(events[1]->GetParentEvent() == events[0].get());
    CHECK(events[2]->GetParentEvent() == events[0].get());
    const std::vector<Measurement> inner = events[1]->GetMeasurements();
    REQUIRE(inner.size() == 1);
    CHECK(inner[0].m_Unit == Measurement::TIME_US);
    CHECK(inner[0].m_Value >= 2000.0);
    CHECK(events[0]->GetMeasurements()[0].m_Value >= inner[0].m_Value);

    std::ostringstream table, json;
    profiler.AnalyzeEventsAndWriteResults(table);
    CHECK(table.str().find("  second inner") != std::string::npos);
    profiler.Print(json);
    const std::string j = json.str();
    CHECK(j.find("\"ArmNN\"") != std::string::npos);
    CHECK(j.find("\"inner \\\"quoted\\\"_#1\"") != std::string::npos);
    CHECK(j.find("\"GUID\": 42") != std::string::npos);
    CHECK(j.find("\"ConvolutionMethod\": \"igemm 64x64\"") != std::string::npos);
    CHECK(j.find("pad (l,r,t,b) 3,0,0,0") != std::string::npos);
    CHECK(j.find("\"outer_#0\"") < j.find("\"second inner_#2\""));
    size_t open = 0, close = 0;
    for (char c : j) { open += c == '{'; close += c == '}'; }
    CHECK(open == close);
    CHECK(profiler.GetEvents().empty());       // printing starts a new recording
}

TEST_CASE("optimize: unsupported layers fall back along the preference list, with copies between backends", "cpu")
{
    testhost::Register();
    INetworkPtr net = INetwork::Create();
    const TensorInfo in = ActInfo({1, 8, 8, 16}, DataType::QAsymmS8, 0.05f, -3);
    QLayer c1 = MakeConv(QLayer::Conv, in, 16, 1, 1, 0.05f, -3, false, true, 21);
    QLayer c2 = MakeConv(QLayer::Conv, c1.out, 8, 1, 1, 0.05f, -3, false, true, 22);
    IConnectableLayer* input = net->AddInputLayer(0, "input");
    input->GetOutputSlot(0).SetTensorInfo(in);
    IOutputSlot& s1 = AddToNetwork(*net, input->GetOutputSlot(0), c1, "conv1");
    IConnectableLayer* lin = net->AddActivationLayer(ActivationDescriptor(ActivationFunction::Linear, 1.0f, 0.0f), "identity");
    s1.Connect(lin->GetInputSlot(0));
    lin->GetOutputSlot(0).SetTensorInfo(c1.out);
    IOutputSlot& s2 = AddToNetwork(*net, lin->GetOutputSlot(0), c2, "conv2");
    IConnectableLayer* out = net->AddOutputLayer(0, "output");
    s2.Connect(out->GetInputSlot(0));

    FixedDeviceSpec both{kMi355x, testhost::Id()};
    std::vector<std::string> messages;
    IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x, testhost::Id()}, both, OptimizerOptionsOpaque(), Optional<std::vector<std::string>&>(messages));
    const Graph& g = opt->GetGraph();
    CHECK(FindLayer(g, "identity")->GetBackendId() == testhost::Id());
    CHECK(FindLayer(g, "conv1")->GetBackendId() == kMi355x);
    CHECK(CountLayers(g, LayerType::MemCopy) == 2);
    bool warned = false;
    for (const auto& m : messages) warned |= m.find("Activation") != std::string::npos && m.find("falling back") != std::string::npos;
    CHECK(warned);

    // no backend takes the convolution: Optimize refuses
    FixedDeviceSpec hostOnly{testhost::Id()};
    CHECK_THROWS_AS(Optimize(*net, {kMi355x, testhost::Id()}, hostOnly), InvalidArgumentException);
    // no preferred backend is present at all
    FixedDeviceSpec none{};
    CHECK_THROWS_AS(Optimize(*net, {kMi355x}, none), InvalidArgumentException);
    CHECK_THROWS_AS(Optimize(*net, {}, both), InvalidArgumentException);
}

namespace
{
// Input -> identity x n -> Output on one backend
INetworkPtr IdentityChain(const TensorInfo& info, int n)
{
    INetworkPtr net = INetwork::Create();
    IConnectableLayer* input = net->AddInputLayer(0, "input");
    input->GetOutputSlot(0).SetTensorInfo(info);
    IOutputSlot* last = &input->GetOutputSlot(0);
    for (int i = 0; i < n; ++i)
    {
        IConnectableLayer* l = net->AddActivationLayer(ActivationDescriptor(ActivationFunction::Linear, 1.0f, 0.0f), ("identity" + std::to_string(i)).c_str());
        last->Connect(l->GetInputSlot(0));
        l->GetOutputSlot(0).SetTensorInfo(info);
        last = &l->GetOutputSlot(0);
    }
    IConnectableLayer* out = net->AddOutputLayer(0, "output");
    last->Connect(out->GetInputSlot(0));
    return net;
}
} // namespace

TEST_CASE("memory plan: the runtime places the tensors of a backend that lets it, in buffers from that backend's allocator", "cpu")
{
    testhost::RegisterPlanned();
    const BackendId planned = testhost::PlannedId();
    const TensorInfo info = ActInfo({1, 5, 5, 10}, DataType::QAsymmS8, 0.05f, -3);     // 250 bytes -> blocks of 252
    const std::vector<uint8_t> input = RandomActivations(info, 77);
    const INetworkProperties external(MemorySource::Undefined, MemorySource::Undefined, false, ProfilingDetailsMethod::Undefined, true);
    testhost::AllocatorLog& log = testhost::AllocatorLog::Default();

    // not asked for: the backend's own tensors, no allocator call
    {
        log = testhost::AllocatorLog();
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        INetworkPtr net = IdentityChain(info, 3);
        CHECK(RunOnRuntime(*rt, *net, {planned}, info, input, info, 2) == input);
        CHECK(log.allocations == 0);
    }
    // asked for, no strategy named: every tensor (the input and the three layers' outputs) a buffer of its own, taken
    // with the first inference and given back when the network goes
    {
        log = testhost::AllocatorLog();
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        INetworkPtr net = IdentityChain(info, 3);
        IOptimizedNetworkPtr opt = Optimize(*net, {planned}, rt->GetDeviceSpec());
        NetworkId id = -1;
        std::string err;
        REQUIRE(rt->LoadNetwork(id, std::move(opt), err, external) == Status::Success);
        CHECK(log.allocations == 0);
        std::vector<uint8_t> out(info.GetNumBytes());
        TensorInfo constIn = info;
        constIn.SetConstant(true);
        for (int i = 0; i < 2; ++i)
            CHECK(rt->EnqueueWorkload(id, {{0, ConstTensor(constIn, input.data())}}, {{0, Tensor(info, out.data())}}) == Status::Success);
        CHECK(out == input);
        CHECK(log.allocations == 4);
        CHECK(log.bytes == 4 * 252u);
        CHECK(log.frees == 0);
        rt->UnloadNetwork(id);
        CHECK(log.frees == 4);
    }
    // a strategy and an allocator of the caller's: one buffer; tensors whose lifetimes do not meet share addresses
    {
        log = testhost::AllocatorLog();
        testhost::AllocatorLog mine;
        IRuntime::CreationOptions options;
        options.m_CustomAllocatorMap[planned] = std::make_shared<testhost::CountingAllocator>(mine);
        options.m_MemoryOptimizerStrategyMap[planned] = std::make_shared<testhost::PackingStrategy>();
        {
            IRuntimePtr rt = IRuntime::Create(options);
            INetworkPtr net = IdentityChain(info, 5);
            CHECK(RunOnRuntime(*rt, *net, {planned}, info, input, info, 2, external) == input);
            CHECK(log.allocations == 0);
            CHECK(mine.allocations == 1);
            CHECK(mine.frees == 1);
            // input, then five outputs in a chain: two slots of 256 bytes alternate, and the network's output, alive to the
            // end, needs no third one because it is the last tensor
            CHECK(mine.bytes == 256u + 252u);
        }
        // the runtime took its registrations with it
        CHECK(BackendRegistryInstance().GetAllocators().count(planned) == 0);
        CHECK(BackendRegistryInstance().GetMemoryOptimizerStrategies().count(planned) == 0);
    }
    // an allocator the backend cannot work with: the backend is left out
    {
        testhost::AllocatorLog mine;
        IRuntime::CreationOptions options;
        options.m_CustomAllocatorMap[planned] = std::make_shared<testhost::CountingAllocator>(mine, MemorySource::DmaBuf);
        IRuntimePtr rt = IRuntime::Create(options);
        CHECK(rt->GetDeviceSpec().GetSupportedBackends().count(planned) == 0);
        CHECK(BackendRegistryInstance().GetAllocators().count(planned) == 0);
    }
}

TEST_CASE("memory plan: the backend lists the capability, hands out an allocator and refuses allocators it cannot check", "cpu")
{
    Mi355xBackend backend;
    bool listed = false;
    const BackendCapabilities caps = backend.GetCapabilities();
    for (size_t i = 0; i < caps.GetOptionCount(); ++i)
        if (caps.GetOption(i).GetName() == "ExternallyManagedMemory") listed = caps.GetOption(i).GetValue().AsBool();
    CHECK(listed);
    std::unique_ptr<ICustomAllocator> allocator = backend.GetDefaultAllocator();
    REQUIRE(allocator != nullptr);
    CHECK(allocator->GetMemorySourceType() == MemorySource::Malloc);
    char buffer[8];
    CHECK(allocator->GetMemoryRegionAtOffset(buffer, 5) == buffer + 5);
    testhost::AllocatorLog log;
    std::string why;
    CHECK(!backend.UseCustomMemoryAllocator(nullptr, why));
    CHECK(!backend.UseCustomMemoryAllocator(std::make_shared<testhost::CountingAllocator>(log, MemorySource::DmaBuf), why));
    CHECK(why.find("Malloc") != std::string::npos);
    if (mi355x::DeviceCount() == 0)
    {
        CHECK(!backend.UseCustomMemoryAllocator(std::make_shared<testhost::CountingAllocator>(log), why));
        CHECK(why.find("no device") != std::string::npos);
        CHECK(log.allocations == 0);
    }
    // adopted device ranges: an overlap turns the lanes off until the overlapping range goes
    const unsigned int lanesBefore = mi355x::Lanes();
    mi355x::SetLanes(2);
    char* base = reinterpret_cast<char*>(uintptr_t(0x10000));
    CHECK(mi355x::LanesFor(32) == 2);
    const bool a = mi355x::NoteAdoptedRange(base, 1000);
    const bool b = mi355x::NoteAdoptedRange(base + 1000, 1000);      // touching is not overlapping
    CHECK(!a);
    CHECK(!b);
    CHECK(mi355x::LanesFor(32) == 2);
    const bool c = mi355x::NoteAdoptedRange(base + 500, 100);
    CHECK(c);
    CHECK(mi355x::LanesFor(32) == 1);
    mi355x::ForgetAdoptedRange(base + 500, 100, c);
    CHECK(mi355x::LanesFor(32) == 2);
    mi355x::ForgetAdoptedRange(base, 1000, a);
    mi355x::ForgetAdoptedRange(base + 1000, 1000, b);
    const bool d = mi355x::NoteAdoptedRange(base + 500, 100);        // nothing left to overlap with
    CHECK(!d);
    mi355x::ForgetAdoptedRange(base + 500, 100, d);
    mi355x::SetLanes(lanesBefore);
}

TEST_CASE("runtime: importing is refused politely where a backend cannot adopt memory, and loudly when misused", "cpu")
{
    testhost::Register();
    // Input -> identity -> Output on the host test backend, whose tensor handles cannot adopt caller memory
    INetworkPtr net = INetwork::Create();
    const TensorInfo info = ActInfo({1, 4, 4, 8}, DataType::QAsymmS8, 0.05f, -3);
    IConnectableLayer* input = net->AddInputLayer(0, "input");
    input->GetOutputSlot(0).SetTensorInfo(info);
    IConnectableLayer* lin = net->AddActivationLayer(ActivationDescriptor(ActivationFunction::Linear, 1.0f, 0.0f), "identity");
    input->GetOutputSlot(0).Connect(lin->GetInputSlot(0));
    lin->GetOutputSlot(0).SetTensorInfo(info);
    IConnectableLayer* out = net->AddOutputLayer(0, "output");
    lin->GetOutputSlot(0).Connect(out->GetInputSlot(0));
    FixedDeviceSpec hostOnly{testhost::Id()};
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    NetworkId id = -1;
    std::string err;
    REQUIRE(rt->LoadNetwork(id, Optimize(*net, {testhost::Id()}, hostOnly), err) == Status::Success);

    std::vector<uint8_t> x = RandomActivations(info, 5), y(info.GetNumBytes(), 0);
    TensorInfo constInfo = info;
    constInfo.SetConstant(true);
    InputTensors ins{{0, ConstTensor(constInfo, x.data())}};
    OutputTensors outs{{0, Tensor(info, y.data())}};
    CHECK_THROWS_AS(rt->ImportInputs(id, ins), MemoryImportException);                      // no memory source named
    CHECK_THROWS_AS(rt->ImportOutputs(id, outs, MemorySource::Undefined), MemoryImportException);
    InputTensors twice{{0, ConstTensor(constInfo, x.data())}, {0, ConstTensor(constInfo, x.data())}};
    CHECK_THROWS_AS(rt->ImportInputs(id, twice, MemorySource::Malloc), MemoryImportException);   // more tensors than inputs
    CHECK(rt->ImportInputs(id, ins, MemorySource::Malloc).empty());                         // cannot adopt: left out, no error
    CHECK(rt->ImportOutputs(id, outs, MemorySource::Malloc).empty());
    CHECK_THROWS_AS(rt->EnqueueWorkload(id, {}, outs, {0}), InvalidArgumentException);       // id 0 was never imported
    CHECK_THROWS_AS(rt->EnqueueWorkload(id, ins, outs, {0}), InvalidArgumentException);      // list + ids exceed the inputs
    CHECK_THROWS_AS(rt->ClearImportedInputs(id, {0}), InvalidArgumentException);
    CHECK(rt->EnqueueWorkload(id, ins, outs) == Status::Success);                            // the copying path is untouched
    CHECK(x == y);
}

TEST_CASE("runtime: without a device the backend is left out and nothing runs on a substitute", "cpu")
{
    if (mi355x::DeviceCount() > 0)
    {
        std::printf("    (a device is present: the no-device path is covered where there is none)\n");
        return;
    }
    Mi355xBackend backend;
    CHECK_THROWS_AS(backend.CreateBackendContext(IRuntime::CreationOptions()), BackendUnavailableException);
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    CHECK(rt->GetDeviceSpec().GetSupportedBackends().count(kMi355x) == 0);
    QLayer l = MakeConv(QLayer::Conv, ActInfo({1, 8, 8, 16}, DataType::QAsymmS8, 0.05f, -3), 32, 3, 1, 0.1f, 5, true, true, 31);
    SingleLayerNet n(l);
    CHECK_THROWS_AS(Optimize(*n.net, {kMi355x}, rt->GetDeviceSpec()), InvalidArgumentException);
    // A runtime that lists the backend all the same (Arm NN's own does so for every dynamically loaded backend) gets "no"
    // with the reason for every layer, and the next backend of the preference list takes the layers.
    FixedDeviceSpec both{kMi355x, testhost::Id()};
    testhost::Register();
    {
        struct Restore { ~Restore() { mi355x::AssumeDevice(true); } } restore;
        mi355x::AssumeDevice(false);
        std::string why;
        const TensorInfo info = ActInfo({1, 4, 4, 8}, DataType::QAsymmS8, 0.05f, -3);
        const ActivationDescriptor relu(ActivationFunction::ReLu, 0.0f, 0.0f);
        CHECK(!backend.GetLayerSupport()->IsLayerSupported(LayerType::Activation, {info, info}, relu, EmptyOptional(), EmptyOptional(),
                                                           Optional<std::string&>(why)));
        CHECK_MSG(why.find("no MI355X device") != std::string::npos, why);
        INetworkPtr net = INetwork::Create();
        IConnectableLayer* input = net->AddInputLayer(0, "input");
        input->GetOutputSlot(0).SetTensorInfo(info);
        IConnectableLayer* lin = net->AddActivationLayer(ActivationDescriptor(ActivationFunction::Linear, 1.0f, 0.0f), "identity");
        input->GetOutputSlot(0).Connect(lin->GetInputSlot(0));
        lin->GetOutputSlot(0).SetTensorInfo(info);
        IConnectableLayer* out = net->AddOutputLayer(0, "output");
        lin->GetOutputSlot(0).Connect(out->GetInputSlot(0));
        IOptimizedNetworkPtr fallen = Optimize(*net, {kMi355x, testhost::Id()}, both);
        for (const auto& layer : fallen->GetGraph().GetLayers()) CHECK(layer->GetBackendId() == testhost::Id());
        CHECK_THROWS_AS(Optimize(*n.net, {kMi355x}, both), InvalidArgumentException);
    }
    // workloads exist without a device, but executing one fails loudly
    FixedDeviceSpec pretend{kMi355x};
    IOptimizedNetworkPtr opt = Optimize(*n.net, {kMi355x}, pretend);
    NetworkId id = -1;
    std::string err;
    CHECK(rt->LoadNetwork(id, std::move(opt), err) == Status::Failure);
    CHECK_MSG(err.find("unavailable") != std::string::npos || err.find("failed") != std::string::npos, err);
}

// ---------------------------------------------------------------------------------------------------------------------
// gpu
// ---------------------------------------------------------------------------------------------------------------------
namespace
{
// what CpuRef's Addition followed by its ReLU Activation (in the sum's quantization) gives
std::vector<uint8_t> OracleAddRelu(const TensorInfo& i0, const std::vector<uint8_t>& x0, const TensorInfo& i1, const std::vector<uint8_t>& x1,
                                   const TensorInfo& sum)
{
    std::vector<uint8_t> added(sum.GetNumBytes()), out(sum.GetNumBytes());
    const std::vector<float> s0{i0.GetQuantizationScale()}, s1{i1.GetQuantizationScale()}, so{sum.GetQuantizationScale()};
    orc_tensor t0 = Orc(i0, x0.data(), s0), t1 = Orc(i1, x1.data(), s1), ta = Orc(sum, added.data(), so), to = Orc(sum, out.data(), so);
    if (orc_add(&t0, &t1, &ta) != 0) throw std::runtime_error(std::string("oracle: ") + orc_last_error());
    if (orc_activation(&ta, &to, ORC_ACT_RELU, 0.0f, 0.0f) != 0) throw std::runtime_error(std::string("oracle: ") + orc_last_error());
    return out;
}

void CheckSingleLayer(const QLayer& l, uint64_t seed, const char* what)
{
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    REQUIRE(rt->GetDeviceSpec().GetSupportedBackends().count(kMi355x) == 1);
    SingleLayerNet n(l);
    const std::vector<uint8_t> input = RandomActivations(l.in, seed);
    const std::vector<uint8_t> got = RunOnRuntime(*rt, *n.net, {kMi355x}, l.in, input, l.out, 2);
    const std::vector<uint8_t> want = OracleRun(l, input);
    const Diff d = Compare(got, want, l.out.GetDataType());
    std::printf("    %s: %zu outputs, max |diff| %d LSB, exact %.5f\n", what, d.n, d.maxAbs, 1.0 - static_cast<double>(d.mismatches) / static_cast<double>(d.n));
    CHECK(d.maxAbs <= 1);
    CHECK(static_cast<double>(d.mismatches) <= 0.002 * static_cast<double>(d.n));
    // not a constant answer
    size_t distinct = 0;
    bool seen[256] = {false};
    for (uint8_t v : got) if (!seen[v]) { seen[v] = true; ++distinct; }
    CHECK(distinct > 8);
}
} // namespace

TEST_CASE("runtime: Convolution2d 3x3 s2, per-axis QSymmS8 weights, QAsymmS8, fused BoundedReLu", "gpu")
{
    CheckSingleLayer(MakeConv(QLayer::Conv, ActInfo({2, 23, 19, 16}, DataType::QAsymmS8, 0.0235f, -7), 48, 3, 2, 0.0235f, -128, true, true, 101), 1, "conv3x3");
}

TEST_CASE("runtime: pointwise Convolution2d, per-tensor weights, QAsymmU8", "gpu")
{
    CheckSingleLayer(MakeConv(QLayer::Conv, ActInfo({3, 14, 14, 64}, DataType::QAsymmU8, 0.0235f, 120), 128, 1, 1, 0.03f, 110, false, false, 102), 2, "conv1x1-u8");
}

namespace
{
// the same layer with per-tensor QAsymmU8 weights: every code moved up by the zero point
QLayer WithUint8Weights(QLayer l, int zeroPoint)
{
    l.w = TensorInfo(l.w.GetShape(), DataType::QAsymmU8, l.wScales[0], zeroPoint, true);
    for (auto& v : l.weights) v = static_cast<int8_t>(static_cast<uint8_t>(std::min(255, std::max(0, static_cast<int>(v) + zeroPoint))));
    return l;
}
} // namespace

TEST_CASE("runtime: per-tensor QAsymmU8 weights with a zero point: Convolution2d, DepthwiseConvolution2d, stem, FullyConnected", "gpu")
{
    const TensorInfo in = ActInfo({2, 21, 17, 32}, DataType::QAsymmU8, 0.0235f, 119);
    CheckSingleLayer(WithUint8Weights(MakeConv(QLayer::Conv, in, 64, 3, 1, 0.03f, 7, true, false, 141), 93), 11, "conv3x3 zw=93");
    CheckSingleLayer(WithUint8Weights(MakeConv(QLayer::Conv, in, 48, 1, 1, 0.03f, 7, false, false, 142), 160), 12, "conv1x1 zw=160");
    CheckSingleLayer(WithUint8Weights(MakeConv(QLayer::Depthwise, in, 32, 3, 2, 0.03f, 7, true, false, 143), 93), 13, "depthwise zw=93");
    CheckSingleLayer(WithUint8Weights(MakeConv(QLayer::Conv, ActInfo({2, 30, 30, 3}, DataType::QAsymmU8, 0.0078f, 128), 32, 3, 2, 0.0235f, 0, true, false, 144), 151), 14, "stem zw=151");
    CheckSingleLayer(WithUint8Weights(MakeFc(ActInfo({5, 256}, DataType::QAsymmU8, 0.02f, 63), 100, 0.25f, 30, false, 145), 93), 15, "fc zw=93");
}

TEST_CASE("runtime: stem Convolution2d with 3 input channels", "gpu")
{
    CheckSingleLayer(MakeConv(QLayer::Conv, ActInfo({2, 32, 32, 3}, DataType::QAsymmS8, 0.0078f, 0), 32, 3, 2, 0.0235f, -128, true, true, 103), 3, "stem");
}

TEST_CASE("runtime: DepthwiseConvolution2d 3x3, per-axis weights, fused BoundedReLu", "gpu")
{
    CheckSingleLayer(MakeConv(QLayer::Depthwise, ActInfo({2, 28, 28, 64}, DataType::QAsymmS8, 0.0235f, -128), 64, 3, 1, 0.0235f, -128, true, true, 104), 4, "dw3x3");
    CheckSingleLayer(MakeConv(QLayer::Depthwise, ActInfo({1, 15, 15, 24}, DataType::QAsymmU8, 0.0235f, 3), 24, 3, 2, 0.0235f, 0, true, true, 105), 5, "dw3x3-s2-u8");
}

namespace
{
std::vector<uint8_t> OraclePad(const TensorInfo& in, const std::vector<uint8_t>& input, const PadList& pads, float value)
{
    const TensorInfo outInfo = Padded(in, pads);
    std::vector<uint8_t> out(outInfo.GetNumElements());
    const std::vector<float> s{in.GetQuantizationScale()};
    orc_tensor ti = Orc(in, input.data(), s), to = Orc(outInfo, out.data(), s);
    std::vector<uint32_t> before;
    for (const auto& p : pads) before.push_back(p.first);
    if (orc_pad(&ti, &to, before.data(), value) != 0) throw std::runtime_error(std::string("oracle: ") + orc_last_error());
    return out;
}

std::vector<uint8_t> OraclePool(const TensorInfo& in, const std::vector<uint8_t>& input, const Pooling2dDescriptor& d, const TensorInfo& outInfo)
{
    std::vector<uint8_t> out(outInfo.GetNumElements());
    const std::vector<float> si{in.GetQuantizationScale()}, so{outInfo.GetQuantizationScale()};
    orc_tensor ti = Orc(in, input.data(), si), to = Orc(outInfo, out.data(), so);
    orc_pool_params p{};
    p.pool_type = d.m_PoolType == PoolingAlgorithm::Max ? ORC_POOL_MAX : ORC_POOL_AVERAGE;
    p.padding_method = d.m_PaddingMethod == PaddingMethod::Exclude ? ORC_PAD_EXCLUDE : ORC_PAD_IGNORE_VALUE;
    p.pad_left = d.m_PadLeft; p.pad_right = d.m_PadRight; p.pad_top = d.m_PadTop; p.pad_bottom = d.m_PadBottom;
    p.pool_w = d.m_PoolWidth; p.pool_h = d.m_PoolHeight; p.stride_x = d.m_StrideX; p.stride_y = d.m_StrideY;
    if (orc_pooling2d(&ti, &to, &p, ORC_NHWC) != 0) throw std::runtime_error(std::string("oracle: ") + orc_last_error());
    return out;
}
} // namespace

TEST_CASE("runtime: Pad runs on the device; folded into the layer behind it, it gives the bytes of the two layers run apart", "gpu")
{
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    REQUIRE(rt->GetDeviceSpec().GetSupportedBackends().count(kMi355x) == 1);
    const TensorInfo in = ActInfo({2, 21, 19, 16}, DataType::QAsymmS8, 0.0235f, -7);
    const PadList hw{{0, 0}, {1, 2}, {3, 0}, {0, 0}};
    const TensorInfo padded = Padded(in, hw);
    const std::vector<uint8_t> input = RandomActivations(in, 77);

    // the layer on its own, with a value that is nobody's neutral element
    auto padOnly = [&](float value) {
        INetworkPtr net = INetwork::Create();
        IConnectableLayer* i = net->AddInputLayer(0, "input");
        i->GetOutputSlot(0).SetTensorInfo(in);
        IConnectableLayer* p = net->AddPadLayer(PadDescriptor(hw, value), "pad");
        i->GetOutputSlot(0).Connect(p->GetInputSlot(0));
        p->GetOutputSlot(0).SetTensorInfo(padded);
        IConnectableLayer* o = net->AddOutputLayer(0, "output");
        p->GetOutputSlot(0).Connect(o->GetInputSlot(0));
        return net;
    };
    CHECK(Compare(RunOnRuntime(*rt, *padOnly(11.0f), {kMi355x}, in, input, padded), OraclePad(in, input, hw, 11.0f), DataType::QAsymmS8).mismatches == 0);
    const std::vector<uint8_t> paddedBytes = RunOnRuntime(*rt, *padOnly(-7.0f), {kMi355x}, in, input, padded);
    CHECK(Compare(paddedBytes, OraclePad(in, input, hw, -7.0f), DataType::QAsymmS8).mismatches == 0);

    for (QLayer::Kind kind : {QLayer::Conv, QLayer::Depthwise})
    {
        const QLayer conv = MakeConv(kind, padded, kind == QLayer::Conv ? 48 : 16, 3, kind == QLayer::Conv ? 1 : 2, 0.0235f, -128, true, true, 78);
        INetworkPtr folded = PadConvNet(in, hw, -7.0f, conv);
        {
            IOptimizedNetworkPtr opt = Optimize(*folded, {kMi355x}, rt->GetDeviceSpec());
            CHECK(CountLayers(opt->GetGraph(), LayerType::Pad) == 0);
        }
        const std::vector<uint8_t> got = RunOnRuntime(*rt, *folded, {kMi355x}, in, input, conv.out);
        SingleLayerNet apart(conv);
        const std::vector<uint8_t> twoSteps = RunOnRuntime(*rt, *apart.net, {kMi355x}, padded, paddedBytes, conv.out);
        CHECK(Compare(got, twoSteps, DataType::QAsymmS8).mismatches == 0);
        const Diff d = Compare(got, OracleRun(conv, paddedBytes), DataType::QAsymmS8);
        std::printf("    pad folded into %s: max |diff| %d LSB vs oracle, exact %.5f\n", kind == QLayer::Conv ? "conv" : "depthwise", d.maxAbs,
                    1.0 - static_cast<double>(d.mismatches) / static_cast<double>(d.n));
        CHECK(d.maxAbs <= 1);
    }

    for (PoolingAlgorithm algo : {PoolingAlgorithm::Max, PoolingAlgorithm::Average})
    {
        const Pooling2dDescriptor pool = Pool3x3s2(algo);
        const TensorInfo pooled = ActInfo({2, (padded.GetShape()[1] - 3) / 2 + 1, (padded.GetShape()[2] - 3) / 2 + 1, 16}, DataType::QAsymmS8, 0.03f, -20);
        const float value = algo == PoolingAlgorithm::Max ? -128.0f : -7.0f;
        INetworkPtr folded = PadPoolNet(in, hw, value, pool, pooled);
        {
            IOptimizedNetworkPtr opt = Optimize(*folded, {kMi355x}, rt->GetDeviceSpec());
            CHECK(CountLayers(opt->GetGraph(), LayerType::Pad) == 0);
        }
        const std::vector<uint8_t> got = RunOnRuntime(*rt, *folded, {kMi355x}, in, input, pooled);
        // CpuRef folds the same way (RefBackend.cpp:95-117) and then runs Pooling2d with the summed padding ignored
        Pooling2dDescriptor summed = pool;
        summed.m_PadTop = hw[1].first; summed.m_PadBottom = hw[1].second; summed.m_PadLeft = hw[2].first; summed.m_PadRight = hw[2].second;
        summed.m_PaddingMethod = PaddingMethod::IgnoreValue;
        CHECK(Compare(got, OraclePool(in, input, summed, pooled), DataType::QAsymmS8).mismatches == 0);
        // The first window of every row lies wholly on the three padded columns.  Averaging gives the zero point either
        // way; Max gives the reference's "nothing to pool" value 0.0 (Pooling2d.cpp:212-219) once folded, where the two
        // layers run apart would give the lowest code -- so for Max only the other windows can be compared with that.
        const std::vector<uint8_t> apart = OraclePool(padded, OraclePad(in, input, hw, value), pool, pooled);
        size_t differing = 0;
        const unsigned int wo = pooled.GetShape()[2], c = pooled.GetShape()[3];
        for (size_t i = 0; i < got.size(); ++i)
            if (got[i] != apart[i] && !(algo == PoolingAlgorithm::Max && (i / c) % wo == 0)) ++differing;
        CHECK(differing == 0);
    }
}

TEST_CASE("runtime: Mean over height and width gives the bytes of the global average pooling it runs as", "gpu")
{
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    REQUIRE(rt->GetDeviceSpec().GetSupportedBackends().count(kMi355x) == 1);
    for (bool keep : {true, false})
    {
        const TensorInfo in = ActInfo({16, 7, 5, 96}, DataType::QAsymmU8, 0.0235f, 3);
        const TensorInfo out = keep ? ActInfo({16, 1, 1, 96}, DataType::QAsymmU8, 0.02f, 1) : ActInfo({16, 96}, DataType::QAsymmU8, 0.02f, 1);
        INetworkPtr net = INetwork::Create();
        IConnectableLayer* i = net->AddInputLayer(0, "input");
        i->GetOutputSlot(0).SetTensorInfo(in);
        IConnectableLayer* mean = net->AddMeanLayer(MeanDescriptor({1, 2}, keep), "mean");
        i->GetOutputSlot(0).Connect(mean->GetInputSlot(0));
        mean->GetOutputSlot(0).SetTensorInfo(out);
        IConnectableLayer* o = net->AddOutputLayer(0, "output");
        mean->GetOutputSlot(0).Connect(o->GetInputSlot(0));
        const std::vector<uint8_t> x = RandomActivations(in, 321);
        const std::vector<uint8_t> got = RunOnRuntime(*rt, *net, {kMi355x}, in, x, out, 2);
        Pooling2dDescriptor whole;
        whole.m_PoolType = PoolingAlgorithm::Average;
        whole.m_PoolWidth = 5; whole.m_PoolHeight = 7; whole.m_StrideX = whole.m_StrideY = 1;
        whole.m_DataLayout = DataLayout::NHWC;
        CHECK(got == OraclePool(in, x, whole, ActInfo({16, 1, 1, 96}, DataType::QAsymmU8, 0.02f, 1)));
    }
}

TEST_CASE("runtime: FullyConnected, per-axis weights", "gpu")
{
    CheckSingleLayer(MakeFc(ActInfo({5, 1, 1, 256}, DataType::QAsymmS8, 0.02f, -128), 100, 0.09f, -20, true, 106), 6, "fc");
}

namespace
{
// stem conv -> (dw -> pw)* -> global average pool -> FC -> softmax, relu6 everywhere it belongs.
// The default is two depthwise-separable blocks on a 32x32 image; `full` is MobileNetV1-1.0 (13 blocks, 1001 classes).
struct MiniMobileNet
{
    std::vector<QLayer> layers;        // convolutions, then the FullyConnected layer last
    TensorInfo in, pooled, logits, probs;
    unsigned int classes = 10;
    MiniMobileNet(unsigned int batch, DataType t, unsigned int resolution = 32, bool full = false)
    {
        const int zp = t == DataType::QAsymmU8 ? 0 : -128;
        in = ActInfo({batch, resolution, resolution, 3}, t, 0.0078f, t == DataType::QAsymmU8 ? 128 : 0);
        layers.push_back(MakeConv(QLayer::Conv, in, 32, 3, 2, 0.0235f, zp, true, true, 201));
        std::vector<std::pair<unsigned int, unsigned int>> blocks = {{1, 64}, {2, 128}};     // (depthwise stride, pointwise channels)
        if (full) blocks = {{1, 64}, {2, 128}, {1, 128}, {2, 256}, {1, 256}, {2, 512}, {1, 512}, {1, 512}, {1, 512}, {1, 512}, {1, 512}, {2, 1024}, {1, 1024}};
        uint64_t seed = 202;
        for (const auto& blk : blocks)
        {
            const unsigned int c = layers.back().out.GetShape()[3];
            layers.push_back(MakeConv(QLayer::Depthwise, layers.back().out, c, 3, blk.first, 0.0235f, zp, true, true, seed++));
            layers.push_back(MakeConv(QLayer::Conv, layers.back().out, blk.second, 1, 1, 0.0235f, zp, true, true, seed++));
        }
        const unsigned int channels = layers.back().out.GetShape()[3];
        classes = full ? 1001 : 10;
        pooled = TensorInfo(TensorShape({batch, 1, 1, channels}), t, 0.0235f, zp);
        layers.push_back(MakeFc(pooled, classes, 0.1f, t == DataType::QAsymmU8 ? 128 : 0, true, seed++));
        logits = layers.back().out;
        probs = TensorInfo(TensorShape({batch, classes}), t, 1.0f / 256.0f, zp);
    }

    INetworkPtr Build() const
    {
        INetworkPtr net = INetwork::Create();
        IConnectableLayer* input = net->AddInputLayer(0, "input");
        input->GetOutputSlot(0).SetTensorInfo(in);
        IOutputSlot* slot = &input->GetOutputSlot(0);
        const size_t nConv = layers.size() - 1;
        for (size_t i = 0; i < nConv; ++i) slot = &AddToNetwork(*net, *slot, layers[i], "l" + std::to_string(i));
        Pooling2dDescriptor pd;
        pd.m_DataLayout = DataLayout::NHWC;
        pd.m_PoolType = PoolingAlgorithm::Average;
        pd.m_PoolWidth = layers[nConv - 1].out.GetShape()[2];
        pd.m_PoolHeight = layers[nConv - 1].out.GetShape()[1];
        pd.m_StrideX = pd.m_StrideY = 1;
        IConnectableLayer* pool = net->AddPooling2dLayer(pd, "avgpool");
        slot->Connect(pool->GetInputSlot(0));
        pool->GetOutputSlot(0).SetTensorInfo(pooled);
        slot = &AddToNetwork(*net, pool->GetOutputSlot(0), layers[nConv], "logits");
        IConnectableLayer* sm = net->AddSoftmaxLayer(SoftmaxDescriptor(), "softmax");
        slot->Connect(sm->GetInputSlot(0));
        sm->GetOutputSlot(0).SetTensorInfo(probs);
        IConnectableLayer* out = net->AddOutputLayer(0, "output");
        sm->GetOutputSlot(0).Connect(out->GetInputSlot(0));
        return net;
    }

    // the same layers through the C ABI, one call after the other, every tensor in a buffer of its own
    std::vector<uint8_t> RunDirect(const std::vector<uint8_t>& input) const
    {
        auto check = [](int rc, const char* what) { if (rc) throw std::runtime_error(std::string(what) + ": " + mi355x_last_error()); };
        const unsigned int batch = in.GetShape()[0];
        std::vector<void*> bufs;
        auto alloc = [&](size_t n) { void* p = nullptr; check(mi355x_malloc(&p, n), "malloc"); bufs.push_back(p); return p; };
        void* cur = alloc(input.size());
        check(mi355x_memcpy_h2d(cur, input.data(), input.size(), nullptr), "h2d");
        for (size_t i = 0; i < layers.size(); ++i)
        {
            const QLayer& l = layers[i];
            mi355x_const_quant wq{MI355X_QSYMM_S8, 0, static_cast<uint32_t>(l.wScales.size()), l.wScales.data()};
            mi355x_const_quant bq{MI355X_SIGNED32, 0, static_cast<uint32_t>(l.bScales.size()), l.bScales.data()};
            if (i + 1 == layers.size())
            {
                const TensorInfo& last = layers[i - 1].out;
                mi355x_pool2d_desc pd{};
                pd.in_h = last.GetShape()[1]; pd.in_w = last.GetShape()[2]; pd.channels = last.GetShape()[3]; pd.out_h = pd.out_w = 1;
                pd.pool_w = pd.in_w; pd.pool_h = pd.in_h; pd.stride_x = pd.stride_y = 1;
                pd.pool_type = 1; pd.padding_method = 1;
                pd.input = mi355x::ToQuant(last); pd.output = mi355x::ToQuant(pooled);
                void* next = alloc(pooled.GetNumBytes());
                check(mi355x_pool2d_run(&pd, batch, cur, next, nullptr), "pool");
                cur = next;
                mi355x_fc_desc fd{};
                fd.k = last.GetShape()[3]; fd.out_features = classes; fd.transpose_weights = 1; fd.bias_enabled = 1;
                fd.input = mi355x::ToQuant(l.in); fd.output = mi355x::ToQuant(l.out);
                mi355x_fc_t plan = nullptr;
                check(mi355x_fc_create(&fd, l.weights.data(), &wq, l.bias.data(), &bq, &plan), "fc_create");
                next = alloc(l.out.GetNumBytes());
                check(mi355x_fc_run(plan, batch, cur, next, nullptr), "fc_run");
                check(mi355x_device_synchronize(), "sync");
                mi355x_fc_destroy(plan);
                cur = next;
                continue;
            }
            mi355x_conv2d_desc d{};
            d.in_h = l.in.GetShape()[1]; d.in_w = l.in.GetShape()[2]; d.in_c = l.in.GetShape()[3];
            d.out_h = l.out.GetShape()[1]; d.out_w = l.out.GetShape()[2]; d.out_c = l.out.GetShape()[3];
            d.kernel_h = l.w.GetShape()[1]; d.kernel_w = l.w.GetShape()[2];
            d.pad_top = l.padTop; d.pad_left = l.padLeft; d.stride_x = d.stride_y = l.stride; d.dilation_x = d.dilation_y = 1;
            d.depthwise = l.kind == QLayer::Depthwise; d.bias_enabled = 1;
            d.input = mi355x::ToQuant(l.in); d.output = mi355x::ToQuant(l.out);
            d.activation = MI355X_ACT_BOUNDED_RELU; d.activation_a = 6.0f; d.activation_b = 0.0f;
            mi355x_conv2d_t plan = nullptr;
            check(mi355x_conv2d_create(&d, l.weights.data(), &wq, l.bias.data(), &bq, &plan), "conv_create");
            void* next = alloc(l.out.GetNumBytes());
            check(mi355x_conv2d_run(plan, batch, cur, next, nullptr), "conv_run");
            check(mi355x_device_synchronize(), "sync");
            mi355x_conv2d_destroy(plan);
            cur = next;
        }
        const mi355x_quant qi = mi355x::ToQuant(logits), qo = mi355x::ToQuant(probs);
        void* sm = alloc(probs.GetNumBytes());
        check(mi355x_softmax_run(batch, classes, 1.0f, &qi, &qo, cur, sm, nullptr), "softmax");
        std::vector<uint8_t> out(probs.GetNumBytes());
        check(mi355x_memcpy_d2h(out.data(), sm, out.size(), nullptr), "d2h");
        check(mi355x_device_synchronize(), "sync");
        for (void* p : bufs) mi355x_free(p);
        return out;
    }
};
} // namespace

TEST_CASE("runtime: a small MobileNet gives the bytes of the same C-ABI calls made one by one", "gpu")
{
    for (DataType t : {DataType::QAsymmS8, DataType::QAsymmU8})
    {
        MiniMobileNet m(4, t);
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        INetworkPtr net = m.Build();
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec());
        CHECK(CountLayers(opt->GetGraph(), LayerType::Activation) == 0);       // all five relu6 folded
        CHECK(CountLayers(opt->GetGraph(), LayerType::MemCopy) == 0);
        opt.reset();
        const std::vector<uint8_t> input = RandomActivations(m.in, 77);
        const std::vector<uint8_t> got = RunOnRuntime(*rt, *net, {kMi355x}, m.in, input, m.probs, 3);
        const std::vector<uint8_t> want = m.RunDirect(input);
        const Diff d = Compare(got, want, t);
        std::printf("    %s: %zu outputs, %zu differ\n", GetDataTypeName(t), d.n, d.mismatches);
        CHECK(d.mismatches == 0);
        // probabilities of a row sum to about 1 (256 codes)
        for (unsigned int r = 0; r < 4; ++r)
        {
            int sum = 0;
            for (unsigned int c = 0; c < 10; ++c) sum += t == DataType::QAsymmU8 ? got[r * 10 + c] : static_cast<int8_t>(got[r * 10 + c]) + 128;
            CHECK(std::abs(sum - 256) <= 10);
        }
    }
}

TEST_CASE("profiling: every workload of a profiled network reports its device time, and its kernel in the details", "gpu")
{
    MiniMobileNet m(4, DataType::QAsymmS8);
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    INetworkPtr net = m.Build();
    IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec());
    NetworkId id = -1;
    std::string err;
    REQUIRE(rt->LoadNetwork(id, std::move(opt), err, INetworkProperties(MemorySource::Undefined, MemorySource::Undefined, true)) == Status::Success);
    const std::shared_ptr<IProfiler> profiler = rt->GetProfiler(id);
    REQUIRE(profiler != nullptr);
    CHECK(profiler->IsProfilingEnabled());
    const std::vector<uint8_t> input = RandomActivations(m.in, 5);
    std::vector<uint8_t> out(m.probs.GetNumBytes());
    TensorInfo constIn = m.in;
    constIn.SetConstant(true);
    auto run = [&] {
        InputTensors ins{{0, ConstTensor(constIn, input.data())}};
        OutputTensors outs{{0, Tensor(m.probs, out.data())}};
        REQUIRE(rt->EnqueueWorkload(id, ins, outs) == Status::Success);
    };
    run();                                     // builds the plans
    { std::ostringstream drop; profiler->Print(drop); }
    run();
    const std::vector<uint8_t> profiled = out;

    size_t workloads = 0;
    double deviceUs = 0.0, executeWallUs = 0.0;
    for (const auto& e : profiler->GetEvents())
    {
        if (e->GetName() == "Execute") executeWallUs = e->GetMeasurements().at(0).m_Value;
        if (e->GetBackendId() != kMi355x) continue;
        ++workloads;
        CHECK(e->GetParentEvent() != nullptr && e->GetParentEvent()->GetName() == "Execute");
        bool hasDevice = false;
        for (const Measurement& meas : e->GetMeasurements())
            if (meas.m_Name == "Device time") { hasDevice = true; deviceUs += meas.m_Value; CHECK(meas.m_Value > 0.0); CHECK(meas.m_Value < 5000.0); }
        CHECK(hasDevice);
    }
    CHECK(workloads == 5);                     // stem, depthwise + pointwise (the depthwise workload leaves its execution to the
                                               // convolution behind it, whose event covers both), pool (the second depthwise +
                                               // pointwise pair leaves its execution to the pooling over the whole image behind
                                               // it), fc, softmax; the activations are fused
    std::ostringstream json;
    profiler->Print(json);
    const std::string j = json.str();
    std::printf("    %zu device workloads, %.1f us on the device, Execute %.1f us on the host\n", workloads, deviceUs, executeWallUs);
    CHECK(j.find("Mi355xConvolution2dWorkload_Execute") != std::string::npos);
    CHECK(j.find("Mi355xDepthwiseConvolution2dWorkload_Plan") != std::string::npos);
    CHECK(j.find("\"ConvolutionMethod\": \"") != std::string::npos);
    CHECK(j.find("Device time_#0") != std::string::npos);

    // the same bytes with the profiler off, and then no events
    profiler->EnableProfiling(false);
    run();
    CHECK(out == profiled);
    CHECK(profiler->GetEvents().empty());
    rt->UnloadNetwork(id);
}

TEST_CASE("runtime: MobileNetV1-224 batch 64 through EnqueueWorkload equals the C-ABI calls; host-to-host images/s printed", "gpu")
{
    MiniMobileNet m(64, DataType::QAsymmS8, 224, true);
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    INetworkPtr net = m.Build();
    IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec());
    CHECK(CountLayers(opt->GetGraph(), LayerType::Activation) == 0);
    CHECK(CountLayers(opt->GetGraph(), LayerType::MemCopy) == 0);
    NetworkId id = -1;
    std::string err;
    REQUIRE(rt->LoadNetwork(id, std::move(opt), err) == Status::Success);
    const std::vector<uint8_t> input = RandomActivations(m.in, 78);
    std::vector<uint8_t> got(m.probs.GetNumBytes());
    TensorInfo constIn = m.in;
    constIn.SetConstant(true);
    InputTensors ins{{0, ConstTensor(constIn, input.data())}};
    OutputTensors outs{{0, Tensor(m.probs, got.data())}};
    for (int i = 0; i < 3; ++i) REQUIRE(rt->EnqueueWorkload(id, ins, outs) == Status::Success);      // plans are built on the first call
    const int steps = 20;
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; ++i) REQUIRE(rt->EnqueueWorkload(id, ins, outs) == Status::Success);
    const double sec = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    std::printf("    EnqueueWorkload, pageable host buffers in and out (9.6 MB + 64 KB per call): %.3f ms per batch of 64 = %.0f images/s\n",
                1e3 * sec / steps, 64.0 * steps / sec);
    rt->UnloadNetwork(id);
    const std::vector<uint8_t> want = m.RunDirect(input);
    const Diff d = Compare(got, want, DataType::QAsymmS8);
    std::printf("    %zu outputs, %zu differ from the one-by-one C-ABI calls\n", d.n, d.mismatches);
    CHECK(d.mismatches == 0);
}

namespace
{
struct PinnedBuffer
{
    void* p = nullptr;
    size_t n = 0;
    explicit PinnedBuffer(size_t bytes) : n(bytes) { if (mi355x_host_alloc(&p, bytes ? bytes : 1) != 0) throw std::runtime_error(mi355x_last_error()); }
    ~PinnedBuffer() { mi355x_host_free(p); }
    uint8_t* bytes() const { return static_cast<uint8_t*>(p); }
};
} // namespace

TEST_CASE("runtime: pinned caller buffers are adopted as network input and output, pageable ones are not", "gpu")
{
    MiniMobileNet m(4, DataType::QAsymmS8);
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    INetworkPtr net = m.Build();
    NetworkId id = -1;
    std::string err;
    REQUIRE(rt->LoadNetwork(id, Optimize(*net, {kMi355x}, rt->GetDeviceSpec()), err) == Status::Success);
    TensorInfo constIn = m.in;
    constIn.SetConstant(true);

    // reference: the copying path
    const std::vector<uint8_t> x1 = RandomActivations(m.in, 81), x2 = RandomActivations(m.in, 82);
    std::vector<uint8_t> want1(m.probs.GetNumBytes()), want2(m.probs.GetNumBytes());
    REQUIRE(rt->EnqueueWorkload(id, {{0, ConstTensor(constIn, x1.data())}}, {{0, Tensor(m.probs, want1.data())}}) == Status::Success);
    REQUIRE(rt->EnqueueWorkload(id, {{0, ConstTensor(constIn, x2.data())}}, {{0, Tensor(m.probs, want2.data())}}) == Status::Success);
    CHECK(want1 != want2);

    // pageable memory cannot be adopted: no id comes back, nothing throws
    std::vector<uint8_t> pageable(m.in.GetNumBytes() + 64);
    uint8_t* aligned = pageable.data() + (16 - reinterpret_cast<uintptr_t>(pageable.data()) % 16) % 16;
    CHECK(rt->ImportInputs(id, {{0, ConstTensor(constIn, aligned)}}, MemorySource::Malloc).empty());

    PinnedBuffer in(m.in.GetNumBytes()), out(m.probs.GetNumBytes());
    // a misaligned address inside pinned memory is refused as well
    CHECK(rt->ImportInputs(id, {{0, ConstTensor(constIn, in.bytes() + 4)}}, MemorySource::Malloc).empty() || m.in.GetNumBytes() < 8);
    const std::vector<ImportedInputId> inIds = rt->ImportInputs(id, {{0, ConstTensor(constIn, in.p)}}, MemorySource::Malloc);
    const std::vector<ImportedOutputId> outIds = rt->ImportOutputs(id, {{0, Tensor(m.probs, out.p)}}, MemorySource::Malloc);
    REQUIRE(inIds.size() == 1);
    REQUIRE(outIds.size() == 1);
    CHECK(inIds[0] == 0);
    CHECK(outIds[0] == 0);

    // both adopted: the caller fills its buffer, enqueues with the ids only, and finds the result in its buffer
    std::memcpy(in.p, x1.data(), x1.size());
    std::memset(out.p, 0xA5, out.n);
    REQUIRE(rt->EnqueueWorkload(id, {}, {}, inIds, outIds) == Status::Success);
    CHECK(std::memcmp(out.p, want1.data(), want1.size()) == 0);
    std::memcpy(in.p, x2.data(), x2.size());
    REQUIRE(rt->EnqueueWorkload(id, {}, {}, inIds, outIds) == Status::Success);
    CHECK(std::memcmp(out.p, want2.data(), want2.size()) == 0);

    // mixed: adopted input, copied output -- and back to plain copies, which must not see the adopted memory any more
    std::vector<uint8_t> got(m.probs.GetNumBytes(), 0);
    std::memcpy(in.p, x1.data(), x1.size());
    REQUIRE(rt->EnqueueWorkload(id, {}, {{0, Tensor(m.probs, got.data())}}, inIds) == Status::Success);
    CHECK(got == want1);
    std::memset(out.p, 0x5A, out.n);
    REQUIRE(rt->EnqueueWorkload(id, {{0, ConstTensor(constIn, x2.data())}}, {{0, Tensor(m.probs, got.data())}}) == Status::Success);
    CHECK(got == want2);
    CHECK(out.bytes()[0] == 0x5A);

    rt->ClearImportedInputs(id, inIds);
    rt->ClearImportedOutputs(id, outIds);
    CHECK_THROWS_AS(rt->EnqueueWorkload(id, {}, {}, inIds, outIds), InvalidArgumentException);

    // device memory is adopted too, and then used in place
    void* devIn = nullptr;
    REQUIRE(mi355x_malloc(&devIn, m.in.GetNumBytes()) == 0);
    REQUIRE(mi355x_memcpy_h2d(devIn, x2.data(), x2.size(), nullptr) == 0);
    REQUIRE(mi355x_device_synchronize() == 0);
    const std::vector<ImportedInputId> devIds = rt->ImportInputs(id, {{0, ConstTensor(constIn, devIn)}}, MemorySource::Malloc);
    REQUIRE(devIds.size() == 1);
    REQUIRE(rt->EnqueueWorkload(id, {}, {{0, Tensor(m.probs, got.data())}}, devIds) == Status::Success);
    CHECK(got == want2);
    rt->ClearImportedInputs(id, devIds);
    mi355x_free(devIn);
    REQUIRE(rt->EnqueueWorkload(id, {{0, ConstTensor(constIn, x1.data())}}, {{0, Tensor(m.probs, got.data())}}) == Status::Success);
    CHECK(got == want1);
    rt->UnloadNetwork(id);
}

TEST_CASE("runtime: MobileNetV1-224 batch 64 with adopted pinned input and output; host-to-host images/s printed", "gpu")
{
    MiniMobileNet m(64, DataType::QAsymmS8, 224, true);
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    INetworkPtr net = m.Build();
    NetworkId id = -1;
    std::string err;
    REQUIRE(rt->LoadNetwork(id, Optimize(*net, {kMi355x}, rt->GetDeviceSpec()), err) == Status::Success);
    TensorInfo constIn = m.in;
    constIn.SetConstant(true);
    const std::vector<uint8_t> input = RandomActivations(m.in, 78);
    std::vector<uint8_t> want(m.probs.GetNumBytes());
    REQUIRE(rt->EnqueueWorkload(id, {{0, ConstTensor(constIn, input.data())}}, {{0, Tensor(m.probs, want.data())}}) == Status::Success);

    PinnedBuffer in(m.in.GetNumBytes()), out(m.probs.GetNumBytes());
    const auto inIds = rt->ImportInputs(id, {{0, ConstTensor(constIn, in.p)}}, MemorySource::Malloc);
    const auto outIds = rt->ImportOutputs(id, {{0, Tensor(m.probs, out.p)}}, MemorySource::Malloc);
    REQUIRE(inIds.size() == 1);
    REQUIRE(outIds.size() == 1);
    std::memcpy(in.p, input.data(), input.size());
    for (int i = 0; i < 3; ++i) REQUIRE(rt->EnqueueWorkload(id, {}, {}, inIds, outIds) == Status::Success);
    CHECK(std::memcmp(out.p, want.data(), want.size()) == 0);
    const int steps = 20;
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; ++i) REQUIRE(rt->EnqueueWorkload(id, {}, {}, inIds, outIds) == Status::Success);
    const double sec = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    std::printf("    EnqueueWorkload, adopted pinned buffers (one transfer of 9.6 MB in, one of 64 KB out, no host copies): "
                "%.3f ms per batch of 64 = %.0f images/s\n", 1e3 * sec / steps, 64.0 * steps / sec);
    CHECK(std::memcmp(out.p, want.data(), want.size()) == 0);
    rt->UnloadNetwork(id);
}

TEST_CASE("runtime: intermediate tensors share an arena smaller than their sum", "gpu")
{
    MiniMobileNet m(4, DataType::QAsymmS8);
    INetworkPtr net = m.Build();
    FixedDeviceSpec spec{kMi355x};
    IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, spec);
    // replay the runtime's handle protocol by hand against one backend instance; addresses are shared only where
    // everything runs on one stream
    const unsigned int lanesBefore = mi355x::Lanes();
    mi355x::SetLanes(1);
    {
        Mi355xBackend backend;
        TensorHandleFactoryRegistry registry;
        backend.RegisterTensorHandleFactories(registry);
        auto factory = backend.CreateWorkloadFactory(registry);
        auto* hf = dynamic_cast<Mi355xTensorHandleFactory*>(registry.GetFactory(Mi355xTensorHandleFactory::GetIdStatic()));
        REQUIRE(hf != nullptr);
        std::vector<std::unique_ptr<ITensorHandle>> handles;
        size_t total = 0;
        const std::vector<Layer*> order = opt->GetGraph().TopologicalSort();
        ITensorHandle* previous = nullptr;
        for (Layer* l : order)
        {
            if (l->GetType() == LayerType::Constant || l->GetType() == LayerType::Input || l->GetNumOutputSlots() == 0) continue;
            handles.push_back(hf->CreateTensorHandle(l->Out(0).GetTensorInfo(), true));
            handles.back()->Manage();
            total += l->Out(0).GetTensorInfo().GetNumBytes();
            if (previous) previous->Allocate();      // a chain: the producer's input dies once the layer is placed
            previous = handles.back().get();
        }
        if (previous) previous->Allocate();
        const size_t arena = hf->GetMemoryManager()->ArenaBytes();
        std::printf("    sum of intermediates %zu bytes, arena %zu bytes\n", total, arena);
        CHECK(arena < total);
        CHECK(arena >= 2 * 4 * 16 * 16 * 32u);      // the two largest neighbours must both fit
        CHECK_NOTHROW(registry.AquireMemory());
        CHECK(dynamic_cast<Mi355xTensorHandle*>(handles[0].get())->GetDevicePointer() != nullptr);
        registry.ReleaseMemory();
        (void)factory;
    }
    mi355x::SetLanes(lanesBefore);
}

namespace
{
// pinned host memory: the device reaches it, so the backend accepts the allocator
class PinnedAllocator : public ICustomAllocator
{
public:
    void* allocate(size_t size, size_t) override
    {
        void* p = nullptr;
        mi355x::Check(mi355x_host_alloc(&p, size ? size : 1), "mi355x_host_alloc");
        ++allocations;
        return p;
    }
    void free(void* p) override { mi355x::Synchronize(); mi355x_host_free(p); ++frees; }
    MemorySource GetMemorySourceType() override { return MemorySource::Malloc; }
    void* GetMemoryRegionAtOffset(void* buffer, size_t offset, size_t = 0) override { return static_cast<char*>(buffer) + offset; }
    int allocations = 0, frees = 0;
};
} // namespace

TEST_CASE("memory plan: tensors placed by the runtime give the same bytes; lanes run only while no two of them share addresses", "gpu")
{
    const unsigned int lanesBefore = mi355x::Lanes();
    mi355x::SetLanes(2);
    MiniMobileNet m(32, DataType::QAsymmS8);
    const std::vector<uint8_t> input = RandomActivations(m.in, 321);
    const std::vector<uint8_t> want = m.RunDirect(input);
    const INetworkProperties external(MemorySource::Undefined, MemorySource::Undefined, false, ProfilingDetailsMethod::Undefined, true);

    // the backend's allocator, every tensor a buffer of its own
    {
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        INetworkPtr net = m.Build();
        unsigned int lanesWhile = 0;
        CHECK(RunOnRuntime(*rt, *net, {kMi355x}, m.in, input, m.probs, 3, external, [&] { lanesWhile = mi355x::LanesFor(32); }) == want);
        CHECK(lanesWhile == 2);
    }
    // a strategy that lets tensors share addresses: the same bytes, on one stream
    {
        IRuntime::CreationOptions options;
        options.m_MemoryOptimizerStrategyMap[kMi355x] = std::make_shared<testhost::PackingStrategy>();
        IRuntimePtr rt = IRuntime::Create(options);
        INetworkPtr net = m.Build();
        unsigned int lanesWhile = 0;
        CHECK(RunOnRuntime(*rt, *net, {kMi355x}, m.in, input, m.probs, 3, external, [&] { lanesWhile = mi355x::LanesFor(32); }) == want);
        CHECK(lanesWhile == 1);
        CHECK(mi355x::LanesFor(32) == 2);          // the network is gone, and its ranges with it
    }
    // the caller's allocator, pinned memory: accepted; tensors keep a device copy of their own
    {
        auto pinned = std::make_shared<PinnedAllocator>();
        IRuntime::CreationOptions options;
        options.m_CustomAllocatorMap[kMi355x] = pinned;
        options.m_MemoryOptimizerStrategyMap[kMi355x] = std::make_shared<testhost::PackingStrategy>();
        {
            IRuntimePtr rt = IRuntime::Create(options);
            REQUIRE(rt->GetDeviceSpec().GetSupportedBackends().count(kMi355x) == 1);
            const int probes = pinned->allocations;
            CHECK(probes == 1);
            CHECK(pinned->frees == 1);
            INetworkPtr net = m.Build();
            unsigned int lanesWhile = 0;
            CHECK(RunOnRuntime(*rt, *net, {kMi355x}, m.in, input, m.probs, 3, external, [&] { lanesWhile = mi355x::LanesFor(32); }) == want);
            CHECK(lanesWhile == 2);
            CHECK(pinned->allocations == probes + 1);
            CHECK(pinned->frees == pinned->allocations);
        }
    }
    // pageable memory: refused, and the backend is not offered
    {
        testhost::AllocatorLog log;
        IRuntime::CreationOptions options;
        options.m_CustomAllocatorMap[kMi355x] = std::make_shared<testhost::CountingAllocator>(log);
        IRuntimePtr rt = IRuntime::Create(options);
        CHECK(rt->GetDeviceSpec().GetSupportedBackends().count(kMi355x) == 0);
        CHECK(log.allocations == 1);
        CHECK(log.frees == 1);
    }
    // Allocate() without a lifetime, as the runtime does for the output of a Constant layer: memory of the tensor's own
    {
        auto mm = std::make_shared<Mi355xMemoryManager>(false);
        Mi355xTensorHandle constant(ActInfo({1, 4, 4, 8}, DataType::QAsymmS8, 0.1f, 0), mm, true);
        constant.Allocate();
        CHECK(constant.GetDevicePointer() != nullptr);
        CHECK_THROWS_AS(constant.Allocate(), InvalidArgumentException);
    }
    mi355x::SetLanes(lanesBefore);
}

TEST_CASE("runtime: two host threads, each with a runtime and a network of its own, share the backend's streams", "gpu")
{
    // the forked / joined state of the lanes belongs to the calling thread; the streams are the process's
    MiniMobileNet a(32, DataType::QAsymmS8), b(16, DataType::QAsymmU8);
    const std::vector<uint8_t> inA = RandomActivations(a.in, 31), inB = RandomActivations(b.in, 32);
    const std::vector<uint8_t> wantA = a.RunDirect(inA), wantB = b.RunDirect(inB);
    std::vector<std::string> problems(2);
    auto work = [&](int which) {
        try
        {
            const MiniMobileNet& m = which == 0 ? a : b;
            const std::vector<uint8_t>& in = which == 0 ? inA : inB;
            const std::vector<uint8_t>& want = which == 0 ? wantA : wantB;
            IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
            INetworkPtr net = m.Build();
            for (int i = 0; i < 4; ++i)
                if (RunOnRuntime(*rt, *net, {kMi355x}, m.in, in, m.probs, 3) != want) problems[which] = "bytes differ in pass " + std::to_string(i);
        }
        catch (const std::exception& e) { problems[which] = e.what(); }
    };
    std::thread t0(work, 0), t1(work, 1);
    t0.join();
    t1.join();
    CHECK_MSG(problems[0].empty(), problems[0]);
    CHECK_MSG(problems[1].empty(), problems[1]);
}

TEST_CASE("runtime: a batch run as two or four slices on streams of their own gives the bytes of the unsplit run", "gpu")
{
    const unsigned int lanesBefore = mi355x::Lanes();
    MiniMobileNet m(32, DataType::QAsymmS8);
    const std::vector<uint8_t> input = RandomActivations(m.in, 123);
    std::vector<std::vector<uint8_t>> results;
    for (unsigned int lanes : {1u, 2u, 4u})
    {
        mi355x::SetLanes(lanes);
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        INetworkPtr net = m.Build();
        results.push_back(RunOnRuntime(*rt, *net, {kMi355x}, m.in, input, m.probs, 3));
    }
    CHECK(results[0] == m.RunDirect(input));
    CHECK(results[1] == results[0]);
    CHECK(results[2] == results[0]);

    // a padded batch, a batch too small to split and a layer on another backend in the middle all fall back to joined
    // execution without the caller noticing
    mi355x::SetLanes(2);
    {
        MiniMobileNet small(4, DataType::QAsymmS8);
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        INetworkPtr net = small.Build();
        const std::vector<uint8_t> in4 = RandomActivations(small.in, 124);
        CHECK(RunOnRuntime(*rt, *net, {kMi355x}, small.in, in4, small.probs, 2) == small.RunDirect(in4));
    }
    {
        // Input -> Pad (batch 16 -> 18: not splittable) -> Pooling2d (batch 18: splits into 9 + 9) -> Output
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        const TensorInfo in = ActInfo({16, 12, 12, 16}, DataType::QAsymmS8, 0.05f, -3);
        const PadList pads{{1, 1}, {0, 0}, {0, 0}, {0, 0}};
        const TensorInfo padded = Padded(in, pads);
        const TensorInfo pooled = ActInfo({18, 5, 5, 16}, DataType::QAsymmS8, 0.05f, -3);
        INetworkPtr net = PadPoolNet(in, pads, 9.0f, Pool3x3s2(PoolingAlgorithm::Max), pooled);
        const std::vector<uint8_t> x = RandomActivations(in, 125);
        const std::vector<uint8_t> got = RunOnRuntime(*rt, *net, {kMi355x}, in, x, pooled, 2);
        CHECK(got == OraclePool(padded, OraclePad(in, x, pads, 9.0f), Pool3x3s2(PoolingAlgorithm::Max), pooled));
    }
    mi355x::SetLanes(lanesBefore);
}

TEST_CASE("runtime: an Addition runs the convolution that feeds it in one launch and gives the bytes of the two layers run apart", "gpu")
{
    const unsigned int lanesBefore = mi355x::Lanes();
    for (unsigned int lanes : {1u, 2u})
    {
        mi355x::SetLanes(lanes);
        ResidualBlock block(16);
        const std::vector<uint8_t> input = RandomActivations(block.in, 91);
        TensorInfo constIn = block.in;
        constIn.SetConstant(true);
        std::vector<uint8_t> results[2];
        size_t convolutionsExecuted[2] = {0, 0};
        for (int fused = 0; fused < 2; ++fused)
        {
            IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
            INetworkPtr net = block.Build();
            OptimizerOptionsOpaque options;
            options.AddModelOption(BackendOptions("Mi355x", {{"FuseAdditions", fused == 1}}));
            IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec(), options);
            NetworkId id = -1;
            std::string err;
            REQUIRE(rt->LoadNetwork(id, std::move(opt), err, INetworkProperties(MemorySource::Undefined, MemorySource::Undefined, true)) == Status::Success);
            std::vector<uint8_t>& out = results[fused];
            out.assign(block.sum.GetNumBytes(), 0);
            for (int pass = 0; pass < 2; ++pass)
            {
                { std::ostringstream drop; rt->GetProfiler(id)->Print(drop); }
                InputTensors ins{{0, ConstTensor(constIn, input.data())}};
                OutputTensors outs{{0, Tensor(block.sum, out.data())}};
                REQUIRE(rt->EnqueueWorkload(id, ins, outs) == Status::Success);
            }
            for (const auto& e : rt->GetProfiler(id)->GetEvents())
                if (e->GetName().find("Mi355xConvolution2dWorkload_Execute") != std::string::npos) ++convolutionsExecuted[fused];
            rt->UnloadNetwork(id);
        }
        std::printf("    lanes %u: convolution workloads that executed on their own: %zu apart, %zu with the Addition taking one over\n", lanes,
                    convolutionsExecuted[0], convolutionsExecuted[1]);
        CHECK(convolutionsExecuted[0] == 3);
        CHECK(convolutionsExecuted[1] == 2);
        CHECK(results[0] == results[1]);

        // and both follow CpuRef's arithmetic.  Its float accumulation may round a convolution output the other way once
        // in thousands of values; such a code passes through the 1x1 convolution and counts 0.09 / 0.06 = 1.5 codes in the sum
        const std::vector<uint8_t> a = OracleRun(block.first, input);
        const std::vector<uint8_t> b = OracleRun(block.last, a);
        const std::vector<uint8_t> c = OracleRun(block.shortcut, input);
        const Diff d = Compare(results[1], OracleAddRelu(block.last.out, b, block.shortcut.out, c, block.sum), DataType::QAsymmS8);
        std::printf("    residual block vs oracle: max |diff| %d, exact %.5f\n", d.maxAbs, 1.0 - static_cast<double>(d.mismatches) / static_cast<double>(d.n));
        CHECK(d.maxAbs <= 2);
        CHECK(d.mismatches * 1000 <= d.n);
    }
    mi355x::SetLanes(lanesBefore);
}

// input -> 3x3 depthwise + ReLU6 -> 1x1 conv + ReLU6 -> 3x3 depthwise (stride 2) + ReLU6 -> 1x1 conv + ReLU6 -> output
struct SeparableBlocks
{
    TensorInfo in;
    QLayer dw1, pw1, dw2, pw2;
    SeparableBlocks(unsigned int batch, unsigned int side, DataType type)
    {
        in = ActInfo({batch, side, side, 32}, type, 0.0235f, type == DataType::QAsymmU8 ? 128 : 0);
        const int zero = type == DataType::QAsymmU8 ? 0 : -128;
        dw1 = MakeConv(QLayer::Depthwise, in, 32, 3, 1, 0.0235f, zero, true, true, 51);
        pw1 = MakeConv(QLayer::Conv, dw1.out, 64, 1, 1, 0.0235f, zero, true, true, 52);
        dw2 = MakeConv(QLayer::Depthwise, pw1.out, 64, 3, 2, 0.0235f, zero, true, true, 53);
        pw2 = MakeConv(QLayer::Conv, dw2.out, 128, 1, 1, 0.0235f, zero, true, true, 54);
    }
    INetworkPtr Build(bool firstDepthwiseAlsoAnOutput = false) const
    {
        INetworkPtr net = INetwork::Create();
        IConnectableLayer* input = net->AddInputLayer(0, "input");
        input->GetOutputSlot(0).SetTensorInfo(in);
        IOutputSlot& a = AddToNetwork(*net, input->GetOutputSlot(0), dw1, "dw1");
        IOutputSlot& b = AddToNetwork(*net, a, pw1, "pw1");
        IOutputSlot& c = AddToNetwork(*net, b, dw2, "dw2");
        IOutputSlot& d = AddToNetwork(*net, c, pw2, "pw2");
        IConnectableLayer* out = net->AddOutputLayer(0, "output");
        d.Connect(out->GetInputSlot(0));
        if (firstDepthwiseAlsoAnOutput)
        {
            IConnectableLayer* out2 = net->AddOutputLayer(1, "output2");
            a.Connect(out2->GetInputSlot(0));
        }
        return net;
    }
};

TEST_CASE("runtime: a 1x1 convolution runs the depthwise layer in front of it in one launch and gives the bytes of the two layers run apart", "gpu")
{
    const unsigned int lanesBefore = mi355x::Lanes();
    for (DataType type : {DataType::QAsymmU8, DataType::QAsymmS8})
        for (unsigned int lanes : {2u, 1u})
        {
            mi355x::SetLanes(lanes);
            // 64 images of 48 x 48: the first pair has 2304 tiles of 8 x 8 per launch in one lane and 1152 in each of two (the
            // library recommends one launch from 1024 on), the second pair 576 / 288: formed, and run as two launches
            SeparableBlocks blocks(64, 48, type);
            const std::vector<uint8_t> input = RandomActivations(blocks.in, 93);
            TensorInfo constIn = blocks.in;
            constIn.SetConstant(true);
            std::vector<uint8_t> results[2];
            unsigned long long formed[2], fused[2], apart[2];
            for (int on = 0; on < 2; ++on)
            {
                const unsigned long long f0 = Mi355xConvolution2dWorkload::DepthwisePairsFormed(), r0 = Mi355xConvolution2dWorkload::DepthwisePairsRunFused(),
                                         a0 = Mi355xConvolution2dWorkload::DepthwisePairsRunApart();
                IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
                INetworkPtr net = blocks.Build();
                OptimizerOptionsOpaque options;
                options.AddModelOption(BackendOptions("Mi355x", {{"FuseDepthwisePointwise", on == 1}}));
                IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec(), options);
                NetworkId id = -1;
                std::string err;
                REQUIRE(rt->LoadNetwork(id, std::move(opt), err) == Status::Success);
                results[on].assign(blocks.pw2.out.GetNumBytes(), 0);
                for (int pass = 0; pass < 2; ++pass)
                {
                    InputTensors ins{{0, ConstTensor(constIn, input.data())}};
                    OutputTensors outs{{0, Tensor(blocks.pw2.out, results[on].data())}};
                    REQUIRE(rt->EnqueueWorkload(id, ins, outs) == Status::Success);
                }
                rt->UnloadNetwork(id);
                formed[on] = Mi355xConvolution2dWorkload::DepthwisePairsFormed() - f0;
                fused[on] = Mi355xConvolution2dWorkload::DepthwisePairsRunFused() - r0;
                apart[on] = Mi355xConvolution2dWorkload::DepthwisePairsRunApart() - a0;
            }
            std::printf("    %s, lanes %u: pairs formed %llu, executions as one launch %llu, as two %llu\n", type == DataType::QAsymmU8 ? "uint8" : "int8", lanes,
                        formed[1], fused[1], apart[1]);
            CHECK(formed[0] == 0);
            CHECK(formed[1] == 2);
            CHECK(fused[1] + apart[1] == 4);               // two pairs, two inferences
            // in lanes every tensor has memory of its own; on one stream the arena frees a range one retirement late, so that a
            // pair's output never lies over its input: either way the first pair runs as one launch
            CHECK(fused[1] == 2);
            CHECK(results[0] == results[1]);
            const std::vector<uint8_t> a = OracleRun(blocks.dw1, input);
            const std::vector<uint8_t> b = OracleRun(blocks.pw1, a);
            const std::vector<uint8_t> c = OracleRun(blocks.dw2, b);
            const std::vector<uint8_t> d = OracleRun(blocks.pw2, c);
            const Diff diff = Compare(results[1], d, type);
            std::printf("    separable blocks vs oracle: max |diff| %d, exact %.5f\n", diff.maxAbs, 1.0 - static_cast<double>(diff.mismatches) / static_cast<double>(diff.n));
            // (four layers deep: a code that CpuRef's float accumulation rounds the other way in an early layer is multiplied by
            // the weights behind it; per layer the bar is 1 LSB, which the library's own tests hold on every kernel)
            CHECK(diff.maxAbs <= 8);
            CHECK(diff.mismatches * 1000 <= diff.n);
        }
    mi355x::SetLanes(lanesBefore);
}

TEST_CASE("runtime: a depthwise layer whose output is read by a second consumer stays a launch of its own", "gpu")
{
    SeparableBlocks blocks(4, 24, DataType::QAsymmU8);
    const std::vector<uint8_t> input = RandomActivations(blocks.in, 94);
    TensorInfo constIn = blocks.in;
    constIn.SetConstant(true);
    const unsigned long long f0 = Mi355xConvolution2dWorkload::DepthwisePairsFormed();
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    INetworkPtr net = blocks.Build(true);
    IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec(), OptimizerOptionsOpaque());
    NetworkId id = -1;
    std::string err;
    REQUIRE(rt->LoadNetwork(id, std::move(opt), err) == Status::Success);
    std::vector<uint8_t> out(blocks.pw2.out.GetNumBytes(), 0), out2(blocks.dw1.out.GetNumBytes(), 0);
    InputTensors ins{{0, ConstTensor(constIn, input.data())}};
    OutputTensors outs{{0, Tensor(blocks.pw2.out, out.data())}, {1, Tensor(blocks.dw1.out, out2.data())}};
    REQUIRE(rt->EnqueueWorkload(id, ins, outs) == Status::Success);
    rt->UnloadNetwork(id);
    CHECK(Mi355xConvolution2dWorkload::DepthwisePairsFormed() - f0 == 1);       // dw2 + pw2 only
    const std::vector<uint8_t> a = OracleRun(blocks.dw1, input);
    const Diff d1 = Compare(out2, a, DataType::QAsymmU8);
    CHECK(d1.maxAbs <= 1);
    CHECK(d1.mismatches * 100 <= d1.n);
}

// Input -> 1x1 convolution (ReLu6 fused by the backend's own rewrite) -> pooling over the whole image [-> second output]
struct PointwiseThenGlobalPooling
{
    TensorInfo in, pooled;
    QLayer pw;
    Pooling2dDescriptor pd;
    PointwiseThenGlobalPooling(unsigned int batch, unsigned int side, unsigned int ci, unsigned int co, DataType type, PoolingAlgorithm algo)
    {
        in = ActInfo({batch, side, side, ci}, type, 0.0235f, type == DataType::QAsymmU8 ? 128 : 0);
        pw = MakeConv(QLayer::Conv, in, co, 1, 1, 0.04f, type == DataType::QAsymmU8 ? 0 : -128, true, true, 61);
        pooled = ActInfo({batch, 1, 1, co}, type, 0.03f, type == DataType::QAsymmU8 ? 2 : -126);
        pd.m_DataLayout = DataLayout::NHWC;
        pd.m_PoolType = algo;
        pd.m_PoolWidth = pd.m_PoolHeight = side;
        pd.m_StrideX = pd.m_StrideY = 1;
    }
    INetworkPtr Build(bool convolutionAlsoAnOutput = false) const
    {
        INetworkPtr net = INetwork::Create();
        IConnectableLayer* input = net->AddInputLayer(0, "input");
        input->GetOutputSlot(0).SetTensorInfo(in);
        IOutputSlot& a = AddToNetwork(*net, input->GetOutputSlot(0), pw, "pw");
        IConnectableLayer* pool = net->AddPooling2dLayer(pd, "pool");
        a.Connect(pool->GetInputSlot(0));
        pool->GetOutputSlot(0).SetTensorInfo(pooled);
        IConnectableLayer* out = net->AddOutputLayer(0, "output");
        pool->GetOutputSlot(0).Connect(out->GetInputSlot(0));
        if (convolutionAlsoAnOutput)
        {
            IConnectableLayer* out2 = net->AddOutputLayer(1, "output2");
            a.Connect(out2->GetInputSlot(0));
        }
        return net;
    }
};

TEST_CASE("runtime: a pooling over the whole image runs the 1x1 convolution in front of it in one launch and gives the bytes of the two layers run apart", "gpu")
{
    const unsigned int lanesBefore = mi355x::Lanes();
    for (DataType type : {DataType::QAsymmU8, DataType::QAsymmS8})
        for (PoolingAlgorithm algo : {PoolingAlgorithm::Average, PoolingAlgorithm::Max})
            for (unsigned int lanes : {2u, 1u})
            {
                mi355x::SetLanes(lanes);
                // 16 images of 7 x 7, 128 -> 1024 channels: four images x 64 channels per block, 64 blocks per launch in one lane
                // and 32 in each of two (the library recommends one launch from 32 on)
                PointwiseThenGlobalPooling pair(16, 7, 128, 1024, type, algo);
                const std::vector<uint8_t> input = RandomActivations(pair.in, 95);
                TensorInfo constIn = pair.in;
                constIn.SetConstant(true);
                std::vector<uint8_t> results[2];
                unsigned long long formed[2], fused[2], apart[2];
                for (int on = 0; on < 2; ++on)
                {
                    const unsigned long long f0 = Mi355xPooling2dWorkload::PairsFormed(), r0 = Mi355xPooling2dWorkload::PairsRunFused(),
                                             a0 = Mi355xPooling2dWorkload::PairsRunApart();
                    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
                    INetworkPtr net = pair.Build();
                    OptimizerOptionsOpaque options;
                    options.AddModelOption(BackendOptions("Mi355x", {{"FuseConvolutionPooling", on == 1}}));
                    IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec(), options);
                    NetworkId id = -1;
                    std::string err;
                    REQUIRE(rt->LoadNetwork(id, std::move(opt), err) == Status::Success);
                    results[on].assign(pair.pooled.GetNumBytes(), 0);
                    for (int pass = 0; pass < 2; ++pass)
                    {
                        InputTensors ins{{0, ConstTensor(constIn, input.data())}};
                        OutputTensors outs{{0, Tensor(pair.pooled, results[on].data())}};
                        REQUIRE(rt->EnqueueWorkload(id, ins, outs) == Status::Success);
                    }
                    rt->UnloadNetwork(id);
                    formed[on] = Mi355xPooling2dWorkload::PairsFormed() - f0;
                    fused[on] = Mi355xPooling2dWorkload::PairsRunFused() - r0;
                    apart[on] = Mi355xPooling2dWorkload::PairsRunApart() - a0;
                }
                CHECK(formed[0] == 0);
                CHECK(formed[1] == 1);
                CHECK(fused[1] == 2);                        // one pair, two inferences
                CHECK(apart[1] == 0);
                CHECK(results[0] == results[1]);
                const std::vector<uint8_t> a = OracleRun(pair.pw, input);
                const std::vector<uint8_t> b = OraclePool(pair.pw.out, a, pair.pd, pair.pooled);
                const Diff diff = Compare(results[1], b, type);
                std::printf("    %s, %s, lanes %u: convolution + pooling vs oracle: max |diff| %d, exact %.5f\n", type == DataType::QAsymmU8 ? "uint8" : "int8",
                            algo == PoolingAlgorithm::Max ? "max" : "average", lanes, diff.maxAbs,
                            1.0 - static_cast<double>(diff.mismatches) / static_cast<double>(diff.n));
                CHECK(diff.maxAbs <= 1);
                CHECK(diff.mismatches * 50 <= diff.n);
            }
    mi355x::SetLanes(lanesBefore);
}

TEST_CASE("runtime: a 1x1 convolution whose output is read by a second consumer, or pooled in small windows, stays a launch of its own", "gpu")
{
    {
        PointwiseThenGlobalPooling pair(16, 7, 128, 1024, DataType::QAsymmU8, PoolingAlgorithm::Average);
        const std::vector<uint8_t> input = RandomActivations(pair.in, 96);
        TensorInfo constIn = pair.in;
        constIn.SetConstant(true);
        const unsigned long long f0 = Mi355xPooling2dWorkload::PairsFormed();
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        INetworkPtr net = pair.Build(true);
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec(), OptimizerOptionsOpaque());
        NetworkId id = -1;
        std::string err;
        REQUIRE(rt->LoadNetwork(id, std::move(opt), err) == Status::Success);
        std::vector<uint8_t> out(pair.pooled.GetNumBytes(), 0), out2(pair.pw.out.GetNumBytes(), 0);
        InputTensors ins{{0, ConstTensor(constIn, input.data())}};
        OutputTensors outs{{0, Tensor(pair.pooled, out.data())}, {1, Tensor(pair.pw.out, out2.data())}};
        REQUIRE(rt->EnqueueWorkload(id, ins, outs) == Status::Success);
        rt->UnloadNetwork(id);
        CHECK(Mi355xPooling2dWorkload::PairsFormed() - f0 == 0);
        // the convolution's tensor exists and the pooling read it
        CHECK(out == OraclePool(pair.pw.out, out2, pair.pd, pair.pooled));
        const Diff d1 = Compare(out2, OracleRun(pair.pw, input), DataType::QAsymmU8);
        CHECK(d1.maxAbs <= 1);
    }
    {
        // 3 x 3 windows at stride 2 over an 8 x 8 image: not the whole image
        PointwiseThenGlobalPooling pair(4, 8, 128, 64, DataType::QAsymmS8, PoolingAlgorithm::Max);
        pair.pd.m_PoolWidth = pair.pd.m_PoolHeight = 3;
        pair.pd.m_StrideX = pair.pd.m_StrideY = 2;
        pair.pooled = ActInfo({4, 3, 3, 64}, DataType::QAsymmS8, 0.04f, -128);
        const std::vector<uint8_t> input = RandomActivations(pair.in, 97);
        TensorInfo constIn = pair.in;
        constIn.SetConstant(true);
        const unsigned long long f0 = Mi355xPooling2dWorkload::PairsFormed();
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        INetworkPtr net = pair.Build();
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec(), OptimizerOptionsOpaque());
        NetworkId id = -1;
        std::string err;
        REQUIRE(rt->LoadNetwork(id, std::move(opt), err) == Status::Success);
        std::vector<uint8_t> out(pair.pooled.GetNumBytes(), 0);
        InputTensors ins{{0, ConstTensor(constIn, input.data())}};
        OutputTensors outs{{0, Tensor(pair.pooled, out.data())}};
        REQUIRE(rt->EnqueueWorkload(id, ins, outs) == Status::Success);
        rt->UnloadNetwork(id);
        CHECK(Mi355xPooling2dWorkload::PairsFormed() - f0 == 0);
        const Diff d = Compare(out, OraclePool(pair.pw.out, OracleRun(pair.pw, input), pair.pd, pair.pooled), DataType::QAsymmS8);
        CHECK(d.maxAbs <= 1);
    }
    {
        // two images: one block row of 16 blocks per launch, fewer than the library recommends as one launch -- the pair is
        // formed and runs as two launches
        PointwiseThenGlobalPooling pair(2, 7, 128, 1024, DataType::QAsymmU8, PoolingAlgorithm::Average);
        const std::vector<uint8_t> input = RandomActivations(pair.in, 98);
        TensorInfo constIn = pair.in;
        constIn.SetConstant(true);
        const unsigned long long f0 = Mi355xPooling2dWorkload::PairsFormed(), r0 = Mi355xPooling2dWorkload::PairsRunFused(),
                                 a0 = Mi355xPooling2dWorkload::PairsRunApart();
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        INetworkPtr net = pair.Build();
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec(), OptimizerOptionsOpaque());
        NetworkId id = -1;
        std::string err;
        REQUIRE(rt->LoadNetwork(id, std::move(opt), err) == Status::Success);
        std::vector<uint8_t> out(pair.pooled.GetNumBytes(), 0);
        InputTensors ins{{0, ConstTensor(constIn, input.data())}};
        OutputTensors outs{{0, Tensor(pair.pooled, out.data())}};
        REQUIRE(rt->EnqueueWorkload(id, ins, outs) == Status::Success);
        rt->UnloadNetwork(id);
        CHECK(Mi355xPooling2dWorkload::PairsFormed() - f0 == 1);
        CHECK(Mi355xPooling2dWorkload::PairsRunFused() - r0 == 0);
        CHECK(Mi355xPooling2dWorkload::PairsRunApart() - a0 == 1);
        const Diff d = Compare(out, OraclePool(pair.pw.out, OracleRun(pair.pw, input), pair.pd, pair.pooled), DataType::QAsymmU8);
        CHECK(d.maxAbs <= 1);
    }
}

TEST_CASE("runtime: an Addition whose sum was placed over the convolution's input runs the pair as two launches, same bytes", "gpu")
{
    const unsigned int lanesBefore = mi355x::Lanes();
    mi355x::SetLanes(1);
    // The backend's own arena frees a range one retirement late, which keeps a pair's output off the pair's input; a runtime
    // that plans the memory itself makes no such promise: with a packing strategy the sum lands on the dead 256-channel
    // tensor the last convolution reads.
    const INetworkProperties external(MemorySource::Undefined, MemorySource::Undefined, false, ProfilingDetailsMethod::Undefined, true);
    {
        NarrowingResidualBlock block(4);
        const std::vector<uint8_t> input = RandomActivations(block.in, 92);
        TensorInfo constIn = block.in;
        constIn.SetConstant(true);
        std::vector<uint8_t> results[2];
        unsigned long long pairs[2] = {0, 0}, apart[2] = {0, 0};
        for (int fused = 0; fused < 2; ++fused)
        {
            const unsigned long long pairsBefore = Mi355xAdditionWorkload::PairsFormed(), apartBefore = Mi355xAdditionWorkload::PairsRunApart();
            IRuntime::CreationOptions creation;
            creation.m_MemoryOptimizerStrategyMap[kMi355x] = std::make_shared<testhost::PackingStrategy>();
            IRuntimePtr rt = IRuntime::Create(creation);
            INetworkPtr net = block.Build();
            OptimizerOptionsOpaque options;
            options.AddModelOption(BackendOptions("Mi355x", {{"FuseAdditions", fused == 1}}));
            IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec(), options);
            NetworkId id = -1;
            std::string err;
            REQUIRE(rt->LoadNetwork(id, std::move(opt), err, external) == Status::Success);
            results[fused].assign(block.sum.GetNumBytes(), 0);
            InputTensors ins{{0, ConstTensor(constIn, input.data())}};
            OutputTensors outs{{0, Tensor(block.sum, results[fused].data())}};
            REQUIRE(rt->EnqueueWorkload(id, ins, outs) == Status::Success);
            rt->UnloadNetwork(id);
            pairs[fused] = Mi355xAdditionWorkload::PairsFormed() - pairsBefore;
            apart[fused] = Mi355xAdditionWorkload::PairsRunApart() - apartBefore;
        }
        std::printf("    pairs formed %llu, executions that ran as two launches %llu\n", pairs[1], apart[1]);
        CHECK(pairs[0] == 0);
        CHECK(pairs[1] == 1);
        CHECK(apart[0] == 0);
        CHECK(apart[1] == 1);                              // the strategy puts the sum at the start of the dead 256-channel tensor
        CHECK(results[0] == results[1]);
        const std::vector<uint8_t> a = OracleRun(block.first, input);
        const std::vector<uint8_t> b = OracleRun(block.last, a);
        const Diff d = Compare(results[1], OracleAddRelu(block.in, input, block.last.out, b, block.sum), DataType::QAsymmS8);
        std::printf("    narrowing residual block vs oracle: max |diff| %d, exact %.5f\n", d.maxAbs, 1.0 - static_cast<double>(d.mismatches) / static_cast<double>(d.n));
        CHECK(d.maxAbs <= 2);
        CHECK(d.mismatches * 1000 <= d.n);
    }
    // the same network in the backend's own arena, one stream: the pair runs as one launch
    {
        NarrowingResidualBlock block(4);
        const std::vector<uint8_t> input = RandomActivations(block.in, 92);
        const unsigned long long pairsBefore = Mi355xAdditionWorkload::PairsFormed(), apartBefore = Mi355xAdditionWorkload::PairsRunApart();
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        INetworkPtr net = block.Build();
        const std::vector<uint8_t> got = RunOnRuntime(*rt, *net, {kMi355x}, block.in, input, block.sum);
        CHECK(Mi355xAdditionWorkload::PairsFormed() - pairsBefore == 1);
        CHECK(Mi355xAdditionWorkload::PairsRunApart() - apartBefore == 0);
        const std::vector<uint8_t> a = OracleRun(block.first, input);
        const std::vector<uint8_t> b = OracleRun(block.last, a);
        const Diff d = Compare(got, OracleAddRelu(block.in, input, block.last.out, b, block.sum), DataType::QAsymmS8);
        CHECK(d.maxAbs <= 2);
        CHECK(d.mismatches * 1000 <= d.n);
    }
    mi355x::SetLanes(lanesBefore);
}

TEST_CASE("runtime: two networks loaded side by side pair their own convolutions and Additions, and survive each other's unloading", "gpu")
{
    // every loaded network has a workload factory of its own, and a pairing never leaves its factory: load A, load B, run
    // both interleaved, unload A, run B again
    ResidualBlock blockA(4);
    NarrowingResidualBlock blockB(2);
    const std::vector<uint8_t> inA = RandomActivations(blockA.in, 191), inB = RandomActivations(blockB.in, 192);
    TensorInfo constA = blockA.in, constB = blockB.in;
    constA.SetConstant(true);
    constB.SetConstant(true);
    auto runAlone = [&](INetworkPtr net, const TensorInfo& cin, const std::vector<uint8_t>& in, const TensorInfo& out) {
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        OptimizerOptionsOpaque options;
        options.AddModelOption(BackendOptions("Mi355x", {{"FuseAdditions", false}}));
        IOptimizedNetworkPtr opt = Optimize(*net, {kMi355x}, rt->GetDeviceSpec(), options);
        NetworkId id = -1;
        std::string err;
        REQUIRE(rt->LoadNetwork(id, std::move(opt), err) == Status::Success);
        std::vector<uint8_t> result(out.GetNumBytes(), 0);
        REQUIRE(rt->EnqueueWorkload(id, InputTensors{{0, ConstTensor(cin, in.data())}}, OutputTensors{{0, Tensor(out, result.data())}}) == Status::Success);
        return result;
    };
    const std::vector<uint8_t> wantA = runAlone(blockA.Build(), constA, inA, blockA.sum);
    const std::vector<uint8_t> wantB = runAlone(blockB.Build(), constB, inB, blockB.sum);

    const unsigned long long pairsBefore = Mi355xAdditionWorkload::PairsFormed();
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    NetworkId idA = -1, idB = -1;
    std::string err;
    {
        INetworkPtr netA = blockA.Build(), netB = blockB.Build();
        IOptimizedNetworkPtr optA = Optimize(*netA, {kMi355x}, rt->GetDeviceSpec(), OptimizerOptionsOpaque());
        IOptimizedNetworkPtr optB = Optimize(*netB, {kMi355x}, rt->GetDeviceSpec(), OptimizerOptionsOpaque());
        REQUIRE(rt->LoadNetwork(idA, std::move(optA), err) == Status::Success);
        REQUIRE(rt->LoadNetwork(idB, std::move(optB), err) == Status::Success);
    }
    CHECK(Mi355xAdditionWorkload::PairsFormed() - pairsBefore == 2);
    std::vector<uint8_t> gotA(blockA.sum.GetNumBytes(), 0), gotB(blockB.sum.GetNumBytes(), 0);
    for (int pass = 0; pass < 2; ++pass)
    {
        REQUIRE(rt->EnqueueWorkload(idA, InputTensors{{0, ConstTensor(constA, inA.data())}}, OutputTensors{{0, Tensor(blockA.sum, gotA.data())}}) == Status::Success);
        REQUIRE(rt->EnqueueWorkload(idB, InputTensors{{0, ConstTensor(constB, inB.data())}}, OutputTensors{{0, Tensor(blockB.sum, gotB.data())}}) == Status::Success);
        CHECK(gotA == wantA);
        CHECK(gotB == wantB);
    }
    REQUIRE(rt->UnloadNetwork(idA) == Status::Success);
    std::fill(gotB.begin(), gotB.end(), 0);
    REQUIRE(rt->EnqueueWorkload(idB, InputTensors{{0, ConstTensor(constB, inB.data())}}, OutputTensors{{0, Tensor(blockB.sum, gotB.data())}}) == Status::Success);
    CHECK(gotB == wantB);
}

TEST_CASE("runtime: a layer the device lacks runs on the next backend and the copies preserve the data", "gpu")
{
    testhost::Register();
    const TensorInfo in = ActInfo({2, 12, 12, 32}, DataType::QAsymmS8, 0.0235f, -128);
    QLayer c1 = MakeConv(QLayer::Conv, in, 32, 1, 1, 0.0235f, -128, true, true, 301);
    QLayer c2 = MakeConv(QLayer::Conv, c1.out, 64, 3, 1, 0.0235f, -128, true, true, 302);
    auto build = [&](bool withIdentity) {
        INetworkPtr net = INetwork::Create();
        IConnectableLayer* input = net->AddInputLayer(0, "input");
        input->GetOutputSlot(0).SetTensorInfo(in);
        IOutputSlot* s = &AddToNetwork(*net, input->GetOutputSlot(0), c1, "conv1");
        if (withIdentity)
        {
            IConnectableLayer* lin = net->AddActivationLayer(ActivationDescriptor(ActivationFunction::Linear, 1.0f, 0.0f), "identity");
            s->Connect(lin->GetInputSlot(0));
            lin->GetOutputSlot(0).SetTensorInfo(c1.out);
            s = &lin->GetOutputSlot(0);
        }
        s = &AddToNetwork(*net, *s, c2, "conv2");
        IConnectableLayer* out = net->AddOutputLayer(0, "output");
        s->Connect(out->GetInputSlot(0));
        return net;
    };
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    REQUIRE(rt->GetDeviceSpec().GetSupportedBackends().count(testhost::Id()) == 1);
    const std::vector<uint8_t> input = RandomActivations(in, 9);
    const int before = testhost::CopyActivationWorkload::Executions();
    INetworkPtr split = build(true), whole = build(false);
    const std::vector<uint8_t> a = RunOnRuntime(*rt, *split, {kMi355x, testhost::Id()}, in, input, c2.out);
    CHECK(testhost::CopyActivationWorkload::Executions() == before + 1);
    const std::vector<uint8_t> b = RunOnRuntime(*rt, *whole, {kMi355x}, in, input, c2.out);
    CHECK(Compare(a, b, DataType::QAsymmS8).mismatches == 0);
    const std::vector<uint8_t> want = OracleRun(c2, OracleRun(c1, input));
    // two layers deep, a 1-LSB difference after the first layer may move a few second-layer outputs by more; the
    // bound that holds per layer is checked by the single-layer cases above
    const Diff d = Compare(a, want, DataType::QAsymmS8);
    std::printf("    two layers vs oracle: max |diff| %d, exact %.5f\n", d.maxAbs, 1.0 - static_cast<double>(d.mismatches) / static_cast<double>(d.n));
    CHECK(d.maxAbs <= 2);
    CHECK(static_cast<double>(d.mismatches) <= 0.01 * static_cast<double>(d.n));
}

TEST_CASE("runtime: new inputs give new outputs, bad bindings are refused, a failing plan fails the load or the inference", "gpu")
{
    IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
    QLayer l = MakeConv(QLayer::Conv, ActInfo({1, 16, 16, 16}, DataType::QAsymmS8, 0.0235f, -5), 32, 3, 1, 0.0235f, -128, true, true, 401);
    SingleLayerNet n(l);
    IOptimizedNetworkPtr opt = Optimize(*n.net, {kMi355x}, rt->GetDeviceSpec());
    NetworkId id = -1;
    std::string err;
    REQUIRE(rt->LoadNetwork(id, std::move(opt), err) == Status::Success);
    CHECK(rt->GetInputTensorInfo(id, 0) == l.in);
    CHECK(rt->GetOutputTensorInfo(id, 0) == l.out);
    CHECK_THROWS_AS(rt->GetInputTensorInfo(id, 5), InvalidArgumentException);
    TensorInfo cin = l.in;
    cin.SetConstant(true);
    for (uint64_t seed : {1u, 2u, 3u})
    {
        const std::vector<uint8_t> input = RandomActivations(l.in, seed);
        std::vector<uint8_t> out(l.out.GetNumBytes());
        CHECK(rt->EnqueueWorkload(id, {{0, ConstTensor(cin, input.data())}}, {{0, Tensor(l.out, out.data())}}) == Status::Success);
        CHECK(Compare(out, OracleRun(l, input), DataType::QAsymmS8).maxAbs <= 1);
    }
    std::vector<uint8_t> small(8), out(l.out.GetNumBytes());
    TensorInfo wrong = ActInfo({1, 1, 1, 8}, DataType::QAsymmS8, 0.0235f, -5);
    wrong.SetConstant(true);
    CHECK_THROWS_AS(rt->EnqueueWorkload(id, {{0, ConstTensor(wrong, small.data())}}, {{0, Tensor(l.out, out.data())}}), InvalidArgumentException);
    CHECK_THROWS_AS(rt->EnqueueWorkload(id, {}, {{0, Tensor(l.out, out.data())}}), InvalidArgumentException);
    CHECK(rt->UnloadNetwork(id) == Status::Success);
    CHECK(rt->UnloadNetwork(id) == Status::Failure);
    CHECK_THROWS_AS(rt->EnqueueWorkload(id, {}, {}), InvalidArgumentException);
}
