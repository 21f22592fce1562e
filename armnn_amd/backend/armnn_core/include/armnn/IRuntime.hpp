// Minimal host core: IRuntime with the names of include/armnn/IRuntime.hpp:41-183.
#pragma once
#include "BackendOptions.hpp"
#include "INetwork.hpp"
#include "Tensor.hpp"
#include "Types.hpp"
#include <memory>
#include <string>

namespace armnn
{
struct INetworkProperties
{
    INetworkProperties(bool asyncEnabled = false, MemorySource inputSource = MemorySource::Undefined,
                       MemorySource outputSource = MemorySource::Undefined, bool profilingEnabled = false)
        : m_AsyncEnabled(asyncEnabled), m_InputSource(inputSource), m_OutputSource(outputSource), m_ProfilingEnabled(profilingEnabled) {}
    const bool m_AsyncEnabled;
    const MemorySource m_InputSource;
    const MemorySource m_OutputSource;
    const bool m_ProfilingEnabled;
};

class IRuntime;
using IRuntimePtr = std::unique_ptr<IRuntime, void (*)(IRuntime* runtime)>;
class RuntimeImpl;

class IRuntime
{
public:
    struct CreationOptions
    {
        CreationOptions() = default;
        /// directory scanned for <vendor>_<name>_backend.so files; empty = none
        std::string m_DynamicBackendsPath;
        bool m_EnableGpuProfiling = false;
        std::vector<BackendOptions> m_BackendOptions;
    };

    static IRuntime* CreateRaw(const CreationOptions& options);
    static IRuntimePtr Create(const CreationOptions& options);
    static void Destroy(IRuntime* runtime);

    Status LoadNetwork(NetworkId& networkIdOut, IOptimizedNetworkPtr network);
    Status LoadNetwork(NetworkId& networkIdOut, IOptimizedNetworkPtr network, std::string& errorMessage);
    Status LoadNetwork(NetworkId& networkIdOut, IOptimizedNetworkPtr network, std::string& errorMessage,
                       const INetworkProperties& networkProperties);
    TensorInfo GetInputTensorInfo(NetworkId networkId, LayerBindingId layerId) const;
    TensorInfo GetOutputTensorInfo(NetworkId networkId, LayerBindingId layerId) const;
    Status EnqueueWorkload(NetworkId networkId, const InputTensors& inputTensors, const OutputTensors& outputTensors);
    Status UnloadNetwork(NetworkId networkId);
    const IDeviceSpec& GetDeviceSpec() const;
    ~IRuntime();
protected:
    IRuntime(const CreationOptions& options);
private:
    std::unique_ptr<RuntimeImpl> pRuntimeImpl;
};
} // namespace armnn
