// The backend as a dynamically loaded object: this executable links the host core only; "Mi355x" becomes known to it
// when the runtime scans IRuntime::CreationOptions::m_DynamicBackendsPath and finds Amd_Mi355x_backend.so.
#include "MiniTest.hpp"
#include "TestUtils.hpp"

#include <armnn/backends/DynamicBackend.hpp>

#include <cstdio>
#include <fstream>
#include <unistd.h>
#include <sys/stat.h>

using namespace armnn;
using namespace tu;

namespace
{
std::string LibDir()
{
    if (const char* env = std::getenv("MI355X_BACKEND_DIR")) return env;
    char buf[4096];
    const ssize_t n = readlink("/proc/self/exe", buf, sizeof(buf) - 1);
    std::string exe(buf, n > 0 ? static_cast<size_t>(n) : 0);
    return exe.substr(0, exe.rfind('/')) + "/../../../lib";
}
} // namespace

TEST_CASE("dynamic: only <vendor>_<name>_backend.so[.N...] files are candidates", "cpu")
{
    char tmpl[] = "/tmp/mi355x_dyn_XXXXXX";
    REQUIRE(mkdtemp(tmpl) != nullptr);
    const std::string dir = tmpl;
    const char* names[] = {"Amd_Mi355x_backend.so", "Arm_GpuAcc_backend.so.1", "Arm_GpuAcc_backend.so.1.2.3", "libarmnn.so",
                           "Amd_Mi355x_backend.so.", "Amd__backend.so", "Amd_Mi355x_backend_so", "Amd_Mi-355x_backend.so", "_Mi355x_backend.so"};
    for (const char* n : names) std::ofstream(dir + "/" + n) << "x";
    const std::vector<std::string> found = DynamicBackendUtils::GetSharedObjects(dir);
    // the pattern's dot before "so" is unescaped, as in DynamicBackendUtils.cpp:228-231, so "backend_so" passes too
    CHECK(found.size() == 4);
    for (const std::string& f : found)
        CHECK(f.find("Amd_Mi355x_backend.so") != std::string::npos || f.find("Arm_GpuAcc_backend.so.1") != std::string::npos ||
              f.find("Amd_Mi355x_backend_so") != std::string::npos);
    // files that are not loadable objects are skipped, not fatal
    CHECK(DynamicBackendUtils::RegisterDynamicBackends(found).empty());
    for (const char* n : names) std::remove((dir + "/" + n).c_str());
    rmdir(dir.c_str());
    CHECK(DynamicBackendUtils::GetSharedObjects("/nonexistent/dir").empty());
    CHECK(DynamicBackendUtils::GetSharedObjects("").empty());
    CHECK(DynamicBackendUtils::IsBackendCompatible(BackendVersion(1, 0)));
    CHECK(!DynamicBackendUtils::IsBackendCompatible(BackendVersion(2, 0)));
    CHECK(!DynamicBackendUtils::IsBackendCompatible(BackendVersion(1, 7)));
}

TEST_CASE("dynamic: the runtime loads Amd_Mi355x_backend.so and registers Mi355x", "cpu")
{
    CHECK(!BackendRegistryInstance().IsBackendRegistered("Mi355x"));
    {
        IRuntime::CreationOptions options;
        options.m_DynamicBackendsPath = LibDir();
        IRuntimePtr rt = IRuntime::Create(options);
        CHECK_MSG(BackendRegistryInstance().IsBackendRegistered("Mi355x"), "looked in " + LibDir());
        auto backend = BackendRegistryInstance().GetFactory("Mi355x")();
        REQUIRE(backend != nullptr);
        CHECK(backend->GetId() == BackendId("Mi355x"));
        CHECK(backend->GetLayerSupport() != nullptr);
    }
    // dynamic backends leave the registry with the runtime that loaded them
    CHECK(!BackendRegistryInstance().IsBackendRegistered("Mi355x"));
}

TEST_CASE("dynamic: a convolution runs through the loaded backend", "gpu")
{
    IRuntime::CreationOptions options;
    options.m_DynamicBackendsPath = LibDir();
    IRuntimePtr rt = IRuntime::Create(options);
    REQUIRE(rt->GetDeviceSpec().GetSupportedBackends().count("Mi355x") == 1);
    QLayer l = MakeConv(QLayer::Conv, ActInfo({2, 14, 14, 32}, DataType::QAsymmS8, 0.0235f, -128), 64, 3, 1, 0.0235f, -128, true, true, 501);
    INetworkPtr net = INetwork::Create();
    IConnectableLayer* in = net->AddInputLayer(0, "input");
    in->GetOutputSlot(0).SetTensorInfo(l.in);
    IOutputSlot& o = AddToNetwork(*net, in->GetOutputSlot(0), l, "conv");
    IConnectableLayer* out = net->AddOutputLayer(0, "output");
    o.Connect(out->GetInputSlot(0));
    IOptimizedNetworkPtr opt = Optimize(*net, {"Mi355x"}, rt->GetDeviceSpec());
    NetworkId id = -1;
    std::string err;
    REQUIRE(rt->LoadNetwork(id, std::move(opt), err) == Status::Success);
    const std::vector<uint8_t> input = RandomActivations(l.in, 5);
    std::vector<uint8_t> got(l.out.GetNumBytes());
    TensorInfo cin = l.in;
    cin.SetConstant(true);
    REQUIRE(rt->EnqueueWorkload(id, {{0, ConstTensor(cin, input.data())}}, {{0, Tensor(l.out, got.data())}}) == Status::Success);
    const Diff d = Compare(got, OracleRun(l, input), DataType::QAsymmS8);
    std::printf("    max |diff| %d LSB, exact %.5f\n", d.maxAbs, 1.0 - static_cast<double>(d.mismatches) / static_cast<double>(d.n));
    CHECK(d.maxAbs <= 1);
    rt->UnloadNetwork(id);
}
