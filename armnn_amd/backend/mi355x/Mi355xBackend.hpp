// IBackendInternal of the Mi355x backend (RefBackend, src/backends/reference/RefBackend.hpp:11-75 and RefBackend.cpp,
// is the CpuRef counterpart).  The id is "Mi355x" -- not GpuAcc, which names the OpenCL backend.
#pragma once
#include <armnn/backends/IBackendInternal.hpp>

namespace armnn
{
class Mi355xBackend : public IBackendInternal
{
public:
    Mi355xBackend() = default;
    ~Mi355xBackend() override = default;

    static const BackendId& GetIdStatic();
    const BackendId& GetId() const override { return GetIdStatic(); }

    IBackendInternal::IMemoryManagerUniquePtr CreateMemoryManager() const override;
    IBackendInternal::IWorkloadFactoryPtr CreateWorkloadFactory(const IBackendInternal::IMemoryManagerSharedPtr& memoryManager = nullptr) const override;
    IBackendInternal::IWorkloadFactoryPtr CreateWorkloadFactory(TensorHandleFactoryRegistry& tensorHandleFactoryRegistry) const override;
    /// The backend reads its model options ("FuseAdditions") when it optimizes a network; factories and layer support do
    /// not depend on them.  The overloads exist because the defaults answer with nothing once the options name the backend
    /// (IBackendInternal.cpp:24-58, 88-102).
    IBackendInternal::IWorkloadFactoryPtr CreateWorkloadFactory(const IBackendInternal::IMemoryManagerSharedPtr& memoryManager,
                                                                const ModelOptions& modelOptions) const override;
    IBackendInternal::IWorkloadFactoryPtr CreateWorkloadFactory(TensorHandleFactoryRegistry& tensorHandleFactoryRegistry,
                                                                const ModelOptions& modelOptions) const override;
    IBackendInternal::ILayerSupportSharedPtr GetLayerSupport(const ModelOptions& modelOptions) const override;
    /// throws BackendUnavailableException when the process sees no MI355X; the runtime then leaves the backend out
    IBackendInternal::IBackendContextPtr CreateBackendContext(const IRuntime::CreationOptions&) const override;
    IBackendInternal::ILayerSupportSharedPtr GetLayerSupport() const override;
    /// folds ReLu / BoundedReLu Activation layers into the Convolution2d / DepthwiseConvolution2d / FullyConnected /
    /// Add layer that feeds them, when that is byte-for-byte what the two separate layers would produce
    OptimizationViews OptimizeSubgraphView(const SubgraphView& subgraph, const ModelOptions& modelOptions) const override;
    std::vector<ITensorHandleFactory::FactoryId> GetHandleFactoryPreferences() const override;
    void RegisterTensorHandleFactories(TensorHandleFactoryRegistry& registry) override;
    BackendCapabilities GetCapabilities() const override;
    /// device memory for a memory plan made outside the backend (INetworkProperties::m_ExternalMemoryManagementEnabled)
    std::unique_ptr<ICustomAllocator> GetDefaultAllocator() const override;
    /// Accepts an allocator of MemorySource::Malloc whose memory the device reaches (device memory, or pinned host memory);
    /// one probe allocation decides.  The runtime then takes the buffers of caller-side memory plans from it.  Weights and
    /// other constants stay in memory the backend allocates itself.
    bool UseCustomMemoryAllocator(std::shared_ptr<ICustomAllocator> allocator, armnn::Optional<std::string&> errMsg) override;
};
} // namespace armnn
