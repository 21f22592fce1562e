// Minimal host core: IRuntime with the names of include/armnn/IRuntime.hpp:41-183.
#pragma once
#include "BackendOptions.hpp"
#include "INetwork.hpp"
#include "IProfiler.hpp"
#include "Tensor.hpp"
#include "Types.hpp"
#include "BackendId.hpp"
#include "backends/ICustomAllocator.hpp"
#include "backends/IMemoryOptimizerStrategy.hpp"
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace armnn
{
struct INetworkProperties
{
    INetworkProperties(MemorySource inputSource, MemorySource outputSource, bool profilingEnabled = false,
                       ProfilingDetailsMethod detailsMethod = ProfilingDetailsMethod::Undefined,
                       bool externalMemoryManagementEnabled = false)
        : m_ProfilingEnabled(profilingEnabled), m_OutputNetworkDetailsMethod(detailsMethod), m_InputSource(inputSource),
          m_OutputSource(outputSource), m_ExternalMemoryManagementEnabled(externalMemoryManagementEnabled) {}
    const bool m_ProfilingEnabled;
    const ProfilingDetailsMethod m_OutputNetworkDetailsMethod;
    const MemorySource m_InputSource;
    const MemorySource m_OutputSource;
    /// the runtime plans the memory of intermediate tensors itself (a strategy places them in buffers taken from the
    /// backend's allocator) for every backend that lists the capability ExternallyManagedMemory
    const bool m_ExternalMemoryManagementEnabled;
    virtual ~INetworkProperties() {}
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
        /// per backend: the allocator the buffers of a caller-side memory plan come from (the backend must accept it)
        std::map<BackendId, std::shared_ptr<ICustomAllocator>> m_CustomAllocatorMap;
        /// per backend: the strategy that places tensors into those buffers (default: every tensor a buffer of its own)
        std::map<BackendId, std::shared_ptr<IMemoryOptimizerStrategy>> m_MemoryOptimizerStrategyMap;
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
    /// Lets the tensor handles bound to the given inputs / outputs adopt the caller's memory once, for use in any number
    /// of EnqueueWorkload calls.  Returns the indices (in the order of the network's input / output layers) that were
    /// adopted; a tensor the backend cannot adopt is left out, not reported as an error.  MemorySource::Undefined throws
    /// MemoryImportException.
    std::vector<ImportedInputId> ImportInputs(NetworkId networkId, const InputTensors& inputTensors,
                                              MemorySource forceImportMemorySource = MemorySource::Undefined);
    std::vector<ImportedOutputId> ImportOutputs(NetworkId networkId, const OutputTensors& outputTensors,
                                                MemorySource forceImportMemorySource = MemorySource::Undefined);
    void ClearImportedInputs(NetworkId networkId, const std::vector<ImportedInputId> inputIds);
    void ClearImportedOutputs(NetworkId networkId, const std::vector<ImportedOutputId> outputIds);
    /// inputs / outputs named in the pre-imported id lists are not passed again in the tensor lists
    Status EnqueueWorkload(NetworkId networkId, const InputTensors& inputTensors, const OutputTensors& outputTensors,
                           std::vector<ImportedInputId> preImportedInputIds = {},
                           std::vector<ImportedOutputId> preImportedOutputIds = {});
    Status UnloadNetwork(NetworkId networkId);
    /// the profiler of a loaded network; events are recorded while it is enabled (INetworkProperties::m_ProfilingEnabled
    /// turns it on at load time)
    const std::shared_ptr<IProfiler> GetProfiler(NetworkId networkId) const;
    const IDeviceSpec& GetDeviceSpec() const;
    ~IRuntime();
protected:
    IRuntime(const CreationOptions& options);
private:
    std::unique_ptr<RuntimeImpl> pRuntimeImpl;
};
} // namespace armnn
