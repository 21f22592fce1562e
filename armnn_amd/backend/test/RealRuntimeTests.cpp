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
#include <cstdlib>
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
    const BackendId mi("Mi355x");
    CHECK(!BackendRegistryInstance().IsBackendRegistered(mi));
    {
        IRuntime::CreationOptions options;
        options.m_DynamicBackendsPath = argv[1];
        IRuntimePtr runtime = IRuntime::Create(options);

        // ---- found, version accepted, registered under its own id
        CHECK(BackendRegistryInstance().IsBackendRegistered(mi));
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

        // ---- Optimize with a fallback, then run: the bytes are CpuRef's either way of placing the layers
        INetworkPtr net = INetwork::Create();
        IConnectableLayer* input = net->AddInputLayer(0);
        std::vector<int8_t> wdata(weights.GetNumElements(), 3);
        std::vector<int32_t> bdata(32, 100);
        cd.m_BiasEnabled = true;
        IConnectableLayer* wl = net->AddConstantLayer(ConstTensor(weights, wdata.data()));
        IConnectableLayer* bl = net->AddConstantLayer(ConstTensor(bias, bdata.data()));
        IConnectableLayer* conv = net->AddConvolution2dLayer(cd, "conv");
        IConnectableLayer* output = net->AddOutputLayer(0);
        input->GetOutputSlot(0).SetTensorInfo(in);
        wl->GetOutputSlot(0).SetTensorInfo(weights);
        bl->GetOutputSlot(0).SetTensorInfo(bias);
        conv->GetOutputSlot(0).SetTensorInfo(out);
        input->GetOutputSlot(0).Connect(conv->GetInputSlot(0));
        wl->GetOutputSlot(0).Connect(conv->GetInputSlot(1));
        bl->GetOutputSlot(0).Connect(conv->GetInputSlot(2));
        conv->GetOutputSlot(0).Connect(output->GetInputSlot(0));
        std::vector<std::string> messages;
        IOptimizedNetworkPtr opt = Optimize(*net, {mi, BackendId("CpuRef")}, runtime->GetDeviceSpec(), OptimizerOptionsOpaque(),
                                            Optional<std::vector<std::string>&>(messages));
        CHECK(opt != nullptr);
        for (const std::string& m : messages) std::printf("optimizer: %s\n", m.c_str());
        NetworkId id = 0;
        std::string err;
        const Status loaded = runtime->LoadNetwork(id, std::move(opt), err);
        if (loaded != Status::Success) std::printf("LoadNetwork: %s\n", err.c_str());
        CHECK(loaded == Status::Success);
        if (loaded == Status::Success)
        {
            std::vector<int8_t> x(in.GetNumElements(), 7), y(out.GetNumElements(), 0);
            TensorInfo cin = in;
            cin.SetConstant(true);
            CHECK(runtime->EnqueueWorkload(id, {{0, ConstTensor(cin, x.data())}}, {{0, Tensor(out, y.data())}}) == Status::Success);
            // centre pixel: 9 taps x 16 channels of (7 - (-3)) * 0.05 * 3 * 0.01 = 2.16, + 100 * 0.0005 = 2.21 -> 22 codes above -128
            CHECK(y[(4 * 8 + 4) * 32] == -128 + 22);
            std::printf("EnqueueWorkload through the fallback placement: centre output code %d\n", static_cast<int>(y[(4 * 8 + 4) * 32]));
            runtime->UnloadNetwork(id);
        }
    }
    // ---- the runtime's destructor takes the dynamic backend out of the registry again
    CHECK(!BackendRegistryInstance().IsBackendRegistered(mi));
    std::printf("%d checks, %d failed\n", g_checked, g_failed);
    return g_failed == 0 ? 0 : 1;
}
