// The backend inside the REAL Arm NN runtime (libarmnn.so built from an Arm NN source tree; this file and the backend
// sources are compiled against that tree's own headers).  Host logic only, no device needed:
//   * IRuntime::Create with CreationOptions::m_DynamicBackendsPath finds Amd_Mi355x_backend.so by its file name, accepts
//     its backend API version and registers the id it reports (DynamicBackendUtils.cpp, Runtime.cpp LoadDynamicBackends);
//   * the factory the registry now holds creates the backend, whose id, capabilities and layer support answer through
//     the public handles (BackendHelper.hpp);
//   * without a device CreateBackendContext throws BackendUnavailableException, which the runtime swallows, layer support
//     answers "unsupported" with a reason, and Optimize({Mi355x, CpuRef}) places every layer on CpuRef, whose result the
//     runtime then computes;
//   * destroying the runtime deregisters the dynamic backend again.
// Usage: real_runtime_tests <directory that holds Amd_Mi355x_backend.so>
#include <armnn/ArmNN.hpp>
#include <armnn/BackendHelper.hpp>
#include <armnn/BackendRegistry.hpp>
#include <armnn/backends/IBackendInternal.hpp>

#include <cstdio>
#include <algorithm>
#include <cstdlib>
#include <memory>
#include <sstream>
#include <string>
#include <vector>

using namespace armnn;

namespace
{
int g_failed = 0, g_checked = 0;
#define CHECK(cond) do { ++g_checked; if (!(cond)) { ++g_failed; std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); } } while (0)
}

int main(int argc, char** argv)
{
    if (argc < 2) { std::fprintf(stderr, "usage: %s <dynamic backend directory>\n", argv[0]); return 2; }
    std::setvbuf(stdout, nullptr, _IOLBF, 0);
    if (argv[1][0] != '/') { std::fprintf(stderr, "the runtime only searches absolute paths (DynamicBackendUtils.cpp IsPathValid)\n"); return 2; }
    const BackendId mi("Mi355x");
    CHECK(!BackendRegistryInstance().IsBackendRegistered(mi));
    {
        IRuntime::CreationOptions options;
        options.m_DynamicBackendsPath = argv[1];
        IRuntimePtr runtime = IRuntime::Create(options);

        // ---- found, version accepted, registered under its own id
        CHECK(BackendRegistryInstance().IsBackendRegistered(mi));
        if (!BackendRegistryInstance().IsBackendRegistered(mi)) { std::printf("the backend was not loaded from %s\n", argv[1]); return 1; }
        std::printf("registered backends: %s\n", BackendRegistryInstance().GetBackendIdsAsString().c_str());
        const BackendIdSet& supported = runtime->GetDeviceSpec().GetSupportedBackends();
        const bool listed = supported.count(mi) != 0;
        std::printf("device spec lists Mi355x: %s (the runtime adds every registered dynamic backend, Runtime.cpp:684-687)\n", listed ? "yes" : "no");

        // ---- the object behind the factory
        auto factory = BackendRegistryInstance().GetFactory(mi);
        CHECK(static_cast<bool>(factory));
        IBackendInternalUniquePtr backend = factory();
        CHECK(backend != nullptr);
        CHECK(backend->GetId() == mi);
        CHECK(IBackendInternal::GetApiVersion() >= BackendVersion({1, 0}));
        const BackendCapabilities caps = backend->GetCapabilities();
        CHECK(caps.GetBackendId() == mi);
        CHECK(HasCapability("ConstantTensorsAsInputs", caps) || HasCapability("NonConstWeights", caps));
        bool unavailable = false;
        try
        {
            (void)backend->CreateBackendContext(options);
        }
        catch (const BackendUnavailableException& e)
        {
            unavailable = true;
            std::printf("no device here: CreateBackendContext throws BackendUnavailableException (%s)\n", e.what());
        }
        std::printf("backend context %s\n", unavailable ? "unavailable (ignored by the runtime)" : "created: a device is present");

        // ---- layer support through the public handle
        LayerSupportHandle handle = GetILayerSupportByBackendId(mi);
        CHECK(handle.IsBackendRegistered());
        const TensorInfo in({1, 8, 8, 16}, DataType::QAsymmS8, 0.05f, -3);
        const TensorInfo out({1, 8, 8, 32}, DataType::QAsymmS8, 0.1f, -128);
        TensorInfo weights({32, 3, 3, 16}, DataType::QSymmS8, 0.01f, 0);
        weights.SetConstant(true);
        TensorInfo bias({32}, DataType::Signed32, 0.05f * 0.01f, 0);
        bias.SetConstant(true);
        Convolution2dDescriptor cd;
        cd.m_PadLeft = cd.m_PadRight = cd.m_PadTop = cd.m_PadBottom = 1;
        cd.m_StrideX = cd.m_StrideY = 1;
        cd.m_BiasEnabled = true;
        cd.m_DataLayout = DataLayout::NHWC;
        std::string reason;
        const bool convOk = handle.IsConvolution2dSupported(in, out, cd, weights, Optional<TensorInfo>(bias), Optional<std::string&>(reason));
        std::printf("IsConvolution2dSupported(QAsymmS8 NHWC 3x3): %s%s%s\n", convOk ? "yes" : "no", reason.empty() ? "" : " - ", reason.c_str());
        CHECK(convOk == !unavailable);                       // supported exactly when there is a device to run it on
        if (unavailable) CHECK(!reason.empty());
        std::string reasonF;
        const TensorInfo fin({1, 8, 8, 16}, DataType::Float32), fout({1, 8, 8, 32}, DataType::Float32);
        TensorInfo fw({32, 3, 3, 16}, DataType::Float32);
        fw.SetConstant(true);
        cd.m_BiasEnabled = false;
        CHECK(!handle.IsConvolution2dSupported(fin, fout, cd, fw, EmptyOptional(), Optional<std::string&>(reasonF)));
        CHECK(!reasonF.empty());                             // float convolutions are never ours, and we say why

        // ---- Optimize with a fallback, then run.  Known answer first: constant data, one output checked by hand.
        auto convNet = [&](const std::vector<int8_t>& wdata, const std::vector<int32_t>& bdata, const TensorInfo& out) {
            INetworkPtr net = INetwork::Create();
            IConnectableLayer* input = net->AddInputLayer(0);
            Convolution2dDescriptor d = cd;
            d.m_BiasEnabled = true;
            IConnectableLayer* wl = net->AddConstantLayer(ConstTensor(weights, wdata.data()));
            IConnectableLayer* bl = net->AddConstantLayer(ConstTensor(bias, bdata.data()));
            IConnectableLayer* conv = net->AddConvolution2dLayer(d, "conv");
            IConnectableLayer* output = net->AddOutputLayer(0);
            input->GetOutputSlot(0).SetTensorInfo(in);
            wl->GetOutputSlot(0).SetTensorInfo(weights);
            bl->GetOutputSlot(0).SetTensorInfo(bias);
            conv->GetOutputSlot(0).SetTensorInfo(out);
            input->GetOutputSlot(0).Connect(conv->GetInputSlot(0));
            wl->GetOutputSlot(0).Connect(conv->GetInputSlot(1));
            bl->GetOutputSlot(0).Connect(conv->GetInputSlot(2));
            conv->GetOutputSlot(0).Connect(output->GetInputSlot(0));
            return net;
        };
        std::string lastProfile;
        OptimizerOptionsOpaque optimizerOptions;
        auto run = [&](INetwork& net, const std::vector<BackendId>& prefs, const TensorInfo& inInfo, const std::vector<int8_t>& x,
                       const TensorInfo& outInfo, std::string& placement) {
            std::vector<std::string> messages;
            std::vector<int8_t> y(outInfo.GetNumElements(), 0);
            IOptimizedNetworkPtr opt(nullptr, [](IOptimizedNetwork*) {});
            try
            {
                opt = Optimize(net, prefs, runtime->GetDeviceSpec(), optimizerOptions, Optional<std::vector<std::string>&>(messages));
            }
            catch (const Exception& e)
            {
                std::printf("Optimize: %s\n", e.what());
            }
            for (const std::string& m : messages) std::printf("optimizer: %s\n", m.c_str());
            CHECK(opt != nullptr);
            if (!opt) return y;
            NetworkId id = 0;
            std::string err;
            const Status loaded = runtime->LoadNetwork(id, std::move(opt), err);
            if (loaded != Status::Success) std::printf("LoadNetwork: %s\n", err.c_str());
            CHECK(loaded == Status::Success);
            if (loaded != Status::Success) return y;
            TensorInfo cin = inInfo;
            cin.SetConstant(true);
            runtime->GetProfiler(id)->EnableProfiling(true);
            CHECK(runtime->EnqueueWorkload(id, {{0, ConstTensor(cin, x.data())}}, {{0, Tensor(outInfo, y.data())}}) == Status::Success);
            std::ostringstream prof;
            runtime->GetProfiler(id)->Print(prof);
            lastProfile = prof.str();
            placement = lastProfile.find("Mi355x") != std::string::npos ? "Mi355x" : "CpuRef";
            runtime->UnloadNetwork(id);
            return y;
        };
        {
            std::string where;
            INetworkPtr net = convNet(std::vector<int8_t>(weights.GetNumElements(), 3), std::vector<int32_t>(32, 100), out);
            const std::vector<int8_t> y = run(*net, {mi, BackendId("CpuRef")}, in, std::vector<int8_t>(in.GetNumElements(), 7), out, where);
            // centre pixel: 9 taps x 16 channels of (7 - (-3)) * 0.05 * 3 * 0.01 = 2.16, + 100 * 0.0005 = 2.21 -> 22 codes above -128
            CHECK(y[(4 * 8 + 4) * 32] == -128 + 22);
            std::printf("constant convolution ran on %s: centre output code %d\n", where.c_str(), static_cast<int>(y[(4 * 8 + 4) * 32]));
            CHECK((where == "Mi355x") == !unavailable);
        }
        // ---- random data: {Mi355x, CpuRef} against {CpuRef} alone.  On a machine with the device that is this backend's
        //      integer-accumulating convolution against the reference implementation's float accumulation: within one
        //      code everywhere (the tolerance of the reference's own quantized layer tests, TensorHelpers.hpp:24-31),
        //      equal nearly everywhere.
        auto compare = [&](const std::vector<int8_t>& got, const std::vector<int8_t>& want, const char* what, const std::string& where) {
            size_t differing = 0;
            int worst = 0, lo = 127, hi = -128;
            for (size_t i = 0; i < got.size(); ++i)
            {
                differing += got[i] != want[i];
                worst = std::max(worst, std::abs(static_cast<int>(got[i]) - static_cast<int>(want[i])));
                lo = std::min<int>(lo, want[i]);
                hi = std::max<int>(hi, want[i]);
            }
            std::printf("%s on %s against CpuRef: %zu of %zu bytes differ, max |difference| %d, codes span [%d, %d]\n", what, where.c_str(),
                        differing, got.size(), worst, lo, hi);
            CHECK(worst <= 1);
            CHECK(differing * 100 <= got.size());
            CHECK(hi - lo > 100);
            if (unavailable) CHECK(differing == 0);
        };
        {
            uint64_t state = 0x9E3779B97F4A7C15ull;
            auto next = [&]() { state ^= state << 13; state ^= state >> 7; state ^= state << 17; return state; };
            std::vector<int8_t> w(weights.GetNumElements()), x(in.GetNumElements());
            std::vector<int32_t> b(32);
            for (auto& v : w) v = static_cast<int8_t>(static_cast<int>(next() % 81) - 40);
            for (auto& v : x) v = static_cast<int8_t>(static_cast<int>(next() % 256) - 128);
            for (auto& v : b) v = static_cast<int32_t>(next() % 4001) - 2000;
            const TensorInfo spread({1, 8, 8, 32}, DataType::QAsymmS8, 0.25f, 4);
            std::string where, whereRef;
            INetworkPtr net = convNet(w, b, spread);
            const std::vector<int8_t> got = run(*net, {mi, BackendId("CpuRef")}, in, x, spread, where);
            INetworkPtr net2 = convNet(w, b, spread);
            const std::vector<int8_t> want = run(*net2, {BackendId("CpuRef")}, in, x, spread, whereRef);
            compare(got, want, "random convolution", where);
            CHECK(whereRef == "CpuRef");
        }
        // ---- a small MobileNet-shaped network with per-channel weight scales, fused activations to fold, a strided
        //      depthwise layer, a pointwise layer, global average pooling and a fully connected layer
        {
            uint64_t state = 0xD1B54A32D192ED03ull;
            auto next = [&]() { state ^= state << 13; state ^= state >> 7; state ^= state << 17; return state; };
            auto scales = [&](unsigned int n, float base) {
                std::vector<float> v(n);
                for (auto& f : v) f = base * (0.5f + static_cast<float>(next() % 1000) / 1000.0f);
                return v;
            };
            struct Held { std::vector<int8_t> w; std::vector<int32_t> b; };
            std::vector<std::unique_ptr<Held>> held;
            auto build = [&](int depth) {
                state = 0xD1B54A32D192ED03ull;
                held.clear();
                INetworkPtr net = INetwork::Create();
                const TensorInfo t0({2, 16, 16, 16}, DataType::QAsymmS8, 0.04f, -5);
                IConnectableLayer* input = net->AddInputLayer(0);
                input->GetOutputSlot(0).SetTensorInfo(t0);
                IOutputSlot* cur = &input->GetOutputSlot(0);
                TensorInfo curInfo = t0;
                auto constants = [&](IConnectableLayer* layer, const TensorShape& wshape, unsigned int channels, unsigned int qdim, float wbase) {
                    // CpuRef's FullyConnected wants weights of the input's type (RefLayerSupport.cpp IsFullyConnectedSupported):
                    // one scale, QAsymmS8, there; per-channel QSymmS8 for the convolutions
                    const bool perTensor = layer->GetType() == LayerType::FullyConnected;
                    const std::vector<float> ws = perTensor ? std::vector<float>(channels, wbase) : scales(channels, wbase);
                    TensorInfo wi = perTensor ? TensorInfo(wshape, DataType::QAsymmS8, wbase, 0) : TensorInfo(wshape, DataType::QSymmS8, ws, qdim);
                    wi.SetConstant(true);
                    std::vector<float> bs(channels);
                    for (unsigned int c = 0; c < channels; ++c) bs[c] = ws[c] * curInfo.GetQuantizationScale();
                    TensorInfo bi = perTensor ? TensorInfo({channels}, DataType::Signed32, bs[0], 0) : TensorInfo({channels}, DataType::Signed32, bs, 0);
                    bi.SetConstant(true);
                    held.emplace_back(new Held);
                    Held& h = *held.back();
                    h.w.resize(wi.GetNumElements());
                    h.b.resize(channels);
                    for (auto& v : h.w) v = static_cast<int8_t>(static_cast<int>(next() % 255) - 127);
                    for (auto& v : h.b) v = static_cast<int32_t>(next() % 2001) - 1000;
                    IConnectableLayer* wl = net->AddConstantLayer(ConstTensor(wi, h.w.data()));
                    IConnectableLayer* bl = net->AddConstantLayer(ConstTensor(bi, h.b.data()));
                    wl->GetOutputSlot(0).SetTensorInfo(wi);
                    bl->GetOutputSlot(0).SetTensorInfo(bi);
                    cur->Connect(layer->GetInputSlot(0));
                    wl->GetOutputSlot(0).Connect(layer->GetInputSlot(1));
                    bl->GetOutputSlot(0).Connect(layer->GetInputSlot(2));
                };
                auto finish = [&](IConnectableLayer* layer, const TensorInfo& info, int act) {
                    layer->GetOutputSlot(0).SetTensorInfo(info);
                    cur = &layer->GetOutputSlot(0);
                    curInfo = info;
                    if (act != 0)
                    {
                        const ActivationDescriptor ad(act == 1 ? ActivationFunction::ReLu : ActivationFunction::BoundedReLu, 6.0f, 0.0f);
                        IConnectableLayer* a = net->AddActivationLayer(ad);
                        cur->Connect(a->GetInputSlot(0));
                        a->GetOutputSlot(0).SetTensorInfo(info);
                        cur = &a->GetOutputSlot(0);
                    }
                };
                Convolution2dDescriptor c1;
                c1.m_PadLeft = c1.m_PadRight = c1.m_PadTop = c1.m_PadBottom = 1;
                c1.m_StrideX = c1.m_StrideY = 1;
                c1.m_BiasEnabled = true;
                c1.m_DataLayout = DataLayout::NHWC;
                IConnectableLayer* l1 = net->AddConvolution2dLayer(c1, "conv3x3");
                constants(l1, {32, 3, 3, 16}, 32, 0, 0.004f);
                finish(l1, TensorInfo({2, 16, 16, 32}, DataType::QAsymmS8, 6.0f / 255.0f, -128), 2);
                DepthwiseConvolution2dDescriptor d2;
                d2.m_PadLeft = d2.m_PadTop = 0;
                d2.m_PadRight = d2.m_PadBottom = 1;
                d2.m_StrideX = d2.m_StrideY = 2;
                d2.m_BiasEnabled = true;
                d2.m_DataLayout = DataLayout::NHWC;
                IConnectableLayer* l2 = net->AddDepthwiseConvolution2dLayer(d2, "depthwise3x3s2");
                constants(l2, {1, 3, 3, 32}, 32, 3, 0.01f);
                finish(l2, TensorInfo({2, 8, 8, 32}, DataType::QAsymmS8, 0.03f, -128), 1);
                Convolution2dDescriptor c3;
                c3.m_StrideX = c3.m_StrideY = 1;
                c3.m_BiasEnabled = true;
                c3.m_DataLayout = DataLayout::NHWC;
                IConnectableLayer* l3 = net->AddConvolution2dLayer(c3, "pointwise");
                constants(l3, {64, 1, 1, 32}, 64, 0, 0.006f);
                finish(l3, TensorInfo({2, 8, 8, 64}, DataType::QAsymmS8, 6.0f / 255.0f, -128), 2);
                if (depth == 3)
                {
                    IConnectableLayer* output = net->AddOutputLayer(0);
                    cur->Connect(output->GetInputSlot(0));
                    return net;
                }
                if (depth == 4)
                {
                    // a residual connection: a 1x1 convolution of the trunk, added to the trunk, then ReLU
                    IOutputSlot* trunk = cur;
                    IConnectableLayer* l4 = net->AddConvolution2dLayer(c3, "branch");
                    constants(l4, {64, 1, 1, 64}, 64, 0, 0.005f);
                    finish(l4, TensorInfo({2, 8, 8, 64}, DataType::QAsymmS8, 0.05f, 3), 0);
                    IConnectableLayer* add = net->AddElementwiseBinaryLayer(ElementwiseBinaryDescriptor(BinaryOperation::Add), "add");
                    cur->Connect(add->GetInputSlot(0));
                    trunk->Connect(add->GetInputSlot(1));
                    finish(add, TensorInfo({2, 8, 8, 64}, DataType::QAsymmS8, 0.04f, -128), 1);
                    IConnectableLayer* output = net->AddOutputLayer(0);
                    cur->Connect(output->GetInputSlot(0));
                    return net;
                }
                Pooling2dDescriptor p4;
                p4.m_PoolType = PoolingAlgorithm::Average;
                p4.m_PoolWidth = p4.m_PoolHeight = 8;
                p4.m_StrideX = p4.m_StrideY = 8;
                p4.m_DataLayout = DataLayout::NHWC;
                IConnectableLayer* l4 = net->AddPooling2dLayer(p4, "pool");
                cur->Connect(l4->GetInputSlot(0));
                finish(l4, TensorInfo({2, 1, 1, 64}, DataType::QAsymmS8, 6.0f / 255.0f, -128), 0);
                IConnectableLayer* l5 = net->AddReshapeLayer(ReshapeDescriptor(TensorShape({2, 64})), "reshape");
                cur->Connect(l5->GetInputSlot(0));
                finish(l5, TensorInfo({2, 64}, DataType::QAsymmS8, 6.0f / 255.0f, -128), 0);
                FullyConnectedDescriptor f6;
                f6.m_BiasEnabled = true;
                f6.m_TransposeWeightMatrix = true;
                IConnectableLayer* l6 = net->AddFullyConnectedLayer(f6, "fc");
                constants(l6, {10, 64}, 10, 0, 0.008f);
                finish(l6, TensorInfo({2, 10}, DataType::QAsymmS8, 0.3f, 3), 0);
                IConnectableLayer* output = net->AddOutputLayer(0);
                cur->Connect(output->GetInputSlot(0));
                return net;
            };
            const TensorInfo t0({2, 16, 16, 16}, DataType::QAsymmS8, 0.04f, -5);
            std::vector<int8_t> x(t0.GetNumElements());
            uint64_t xs = 88172645463325252ull;
            for (auto& v : x) { xs ^= xs << 13; xs ^= xs >> 7; xs ^= xs << 17; v = static_cast<int8_t>(static_cast<int>(xs % 256) - 128); }
            for (int depth : {3, 6})
            {
                const TensorInfo tout = depth == 3 ? TensorInfo({2, 8, 8, 64}, DataType::QAsymmS8, 6.0f / 255.0f, -128)
                                                   : TensorInfo({2, 10}, DataType::QAsymmS8, 0.3f, 3);
                std::string where, whereRef;
                INetworkPtr a = build(depth);
                const std::vector<int8_t> got = run(*a, {mi, BackendId("CpuRef")}, t0, x, tout, where);
                INetworkPtr b = build(depth);
                const std::vector<int8_t> want = run(*b, {BackendId("CpuRef")}, t0, x, tout, whereRef);
                compare(got, want, depth == 3 ? "convolution + ReLU6, strided depthwise + ReLU, pointwise + ReLU6" : "the same, then pooling, reshape, fully connected",
                        where);
            }
            // ---- a residual connection.  The backend's Addition workload runs the convolution that feeds it inside its
            //      own launch; with BackendOptions("Mi355x", {{"FuseAdditions", false}}) among the model options the two stay
            //      apart.  Same bytes either way, and one convolution workload fewer executes on its own.
            {
                auto executed = [&] {
                    size_t n = 0;
                    for (size_t at = lastProfile.find("Mi355xConvolution2dWorkload_Execute"); at != std::string::npos;
                         at = lastProfile.find("Mi355xConvolution2dWorkload_Execute", at + 1))
                        ++n;
                    return n;
                };
                const TensorInfo tout({2, 8, 8, 64}, DataType::QAsymmS8, 0.04f, -128);
                std::string where, whereApart, whereRef;
                INetworkPtr a = build(4);
                const std::vector<int8_t> got = run(*a, {mi, BackendId("CpuRef")}, t0, x, tout, where);
                const size_t together = executed();
                optimizerOptions.AddModelOption(BackendOptions("Mi355x", {{"FuseAdditions", false}}));
                INetworkPtr b = build(4);
                const std::vector<int8_t> apart = run(*b, {mi, BackendId("CpuRef")}, t0, x, tout, whereApart);
                const size_t alone = executed();
                optimizerOptions = OptimizerOptionsOpaque();
                INetworkPtr c = build(4);
                const std::vector<int8_t> want = run(*c, {BackendId("CpuRef")}, t0, x, tout, whereRef);
                compare(got, want, "convolution, depthwise, pointwise, then a 1x1 convolution added to its own input + ReLU", where);
                CHECK(got == apart);
                if (!unavailable)
                {
                    std::printf("convolution workloads executing on their own: %zu with the Addition taking one over, %zu apart\n", together, alone);
                    CHECK(alone > 0);
                    CHECK(together + (alone / 3) == alone);      // each workload appears the same number of times in the printed profile
                }
            }
        }
    }
    // ---- the runtime's destructor takes the dynamic backend out of the registry again
    CHECK(!BackendRegistryInstance().IsBackendRegistered(mi));
    std::printf("%d checks, %d failed\n", g_checked, g_failed);
    return g_failed == 0 ? 0 : 1;
}
