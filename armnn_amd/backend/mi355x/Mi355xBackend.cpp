#include "Mi355xBackend.hpp"
#include "Mi355xBackendId.hpp"
#include "Mi355xDevice.hpp"
#include "Mi355xLayerSupport.hpp"
#include "Mi355xTensorHandle.hpp"
#include "Mi355xWorkloadFactory.hpp"

#include <Layer.hpp>
#include <armnn/BackendRegistry.hpp>
#include <armnn/backends/IBackendContext.hpp>
#include <backendsCommon/TensorHandleFactoryRegistry.hpp>

#include <set>

namespace armnn
{
namespace
{
// selects and warms up the device when the runtime is created; waits for outstanding work before a network goes away
class Mi355xBackendContext : public IBackendContext
{
public:
    explicit Mi355xBackendContext(const IRuntime::CreationOptions& options) : IBackendContext(options) { mi355x::EnsureDevice(); }
    bool BeforeLoadNetwork(NetworkId) override { return true; }
    bool AfterLoadNetwork(NetworkId) override { return true; }
    bool BeforeUnloadNetwork(NetworkId) override { mi355x::Synchronize(); return true; }
    bool AfterUnloadNetwork(NetworkId) override { return true; }
    bool AfterEnqueueWorkload(NetworkId) override { return true; }
};

bool SameQuantization(const TensorInfo& a, const TensorInfo& b)
{
    return a.GetDataType() == b.GetDataType() && a.GetQuantizationScales() == b.GetQuantizationScales() &&
           a.GetQuantizationOffset() == b.GetQuantizationOffset();
}

bool Fusable(const Layer& base)
{
    switch (base.GetType())
    {
        case LayerType::Convolution2d: case LayerType::DepthwiseConvolution2d: case LayerType::FullyConnected: return true;
        case LayerType::ElementwiseBinary:
            return static_cast<const ElementwiseBinaryDescriptor&>(base.GetParameters()).m_Operation == BinaryOperation::Add;
        default: return false;
    }
}
} // namespace

const BackendId& Mi355xBackend::GetIdStatic()
{
    static const BackendId s_Id{Mi355xBackendId()};
    return s_Id;
}

IBackendInternal::IMemoryManagerUniquePtr Mi355xBackend::CreateMemoryManager() const
{
    return std::make_unique<Mi355xMemoryManager>();
}

IBackendInternal::IWorkloadFactoryPtr Mi355xBackend::CreateWorkloadFactory(const IBackendInternal::IMemoryManagerSharedPtr& memoryManager) const
{
    return std::make_unique<Mi355xWorkloadFactory>(std::dynamic_pointer_cast<Mi355xMemoryManager>(memoryManager));
}

IBackendInternal::IWorkloadFactoryPtr Mi355xBackend::CreateWorkloadFactory(TensorHandleFactoryRegistry& registry) const
{
    // handles made by the registered tensor handle factory and by the workload factory share one arena
    if (auto* existing = dynamic_cast<Mi355xTensorHandleFactory*>(registry.GetFactory(Mi355xTensorHandleFactory::GetIdStatic())))
        return std::make_unique<Mi355xWorkloadFactory>(existing->GetMemoryManager());
    auto memoryManager = std::make_shared<Mi355xMemoryManager>();
    registry.RegisterMemoryManager(memoryManager);
    registry.RegisterFactory(std::make_unique<Mi355xTensorHandleFactory>(memoryManager));
    return std::make_unique<Mi355xWorkloadFactory>(memoryManager);
}

IBackendInternal::IBackendContextPtr Mi355xBackend::CreateBackendContext(const IRuntime::CreationOptions& options) const
{
    return std::make_unique<Mi355xBackendContext>(options);
}

IBackendInternal::ILayerSupportSharedPtr Mi355xBackend::GetLayerSupport() const
{
    static ILayerSupportSharedPtr layerSupport{new Mi355xLayerSupport};
    return layerSupport;
}

std::vector<ITensorHandleFactory::FactoryId> Mi355xBackend::GetHandleFactoryPreferences() const
{
    return {Mi355xTensorHandleFactory::GetIdStatic()};
}

void Mi355xBackend::RegisterTensorHandleFactories(TensorHandleFactoryRegistry& registry)
{
    if (registry.GetFactory(Mi355xTensorHandleFactory::GetIdStatic()) != nullptr) return;
    auto memoryManager = std::make_shared<Mi355xMemoryManager>();
    registry.RegisterMemoryManager(memoryManager);
    registry.RegisterFactory(std::make_unique<Mi355xTensorHandleFactory>(memoryManager));
}

BackendCapabilities Mi355xBackend::GetCapabilities() const
{
    return BackendCapabilities(Mi355xBackendId(), {{"NonConstWeights", false},
                                                   {"AsyncExecution", false},
                                                   {"ProtectedContentAllocation", false},
                                                   {"ConstantTensorsAsInputs", true},
                                                   {"PreImportIOTensors", true},
                                                   {"ExternallyManagedMemory", false},
                                                   {"MultiAxisPacking", false},
                                                   {"SingleAxisPacking", false}});
}

// A quantized ReLu / BoundedReLu whose input and output share one quantization is an integer clamp
// (workloads/Activation.cpp:33-42 between a decoder and an encoder of the same scale and offset), which the device
// kernels apply in their epilogue.  With different quantizations the Activation layer re-quantizes and stays a layer
// of its own.  The replacement layer carries the ActivationDescriptor as its additional-info object, as the Neon and
// CL backends do (src/backends/aclCommon/ArmComputeSubgraphUtils.hpp:60-109).
OptimizationViews Mi355xBackend::OptimizeSubgraphView(const SubgraphView& subgraph, const ModelOptions& modelOptions) const
{
    OptimizationViews views(modelOptions);
    const SubgraphView::IConnectableLayers& layers = subgraph.GetIConnectableLayers();
    std::set<const IConnectableLayer*> members(layers.begin(), layers.end());
    std::set<const IConnectableLayer*> consumed;

    for (IConnectableLayer* il : layers)
    {
        if (consumed.count(il)) continue;
        Layer* base = PolymorphicDowncast<Layer*>(il);
        if (!Fusable(*base) || base->GetAdditionalInformation<ActivationDescriptor>() != nullptr) continue;
        OutputSlot& out = base->GetOutputSlot(0);
        if (out.GetNumConnections() != 1) continue;
        Layer* act = &out.GetConnections()[0]->GetOwningLayer();
        if (act->GetType() != LayerType::Activation || !members.count(act) || consumed.count(act)) continue;
        const auto& ad = static_cast<const ActivationDescriptor&>(act->GetParameters());
        if (ad.m_Function != ActivationFunction::ReLu && ad.m_Function != ActivationFunction::BoundedReLu) continue;
        if (!SameQuantization(out.GetTensorInfo(), act->GetOutputSlot(0).GetTensorInfo())) continue;

        const std::string name = std::string("fused-") + act->GetName() + "-into-" + base->GetName();
        INetwork& net = views.GetINetworkRef();
        IConnectableLayer* replacement = nullptr;
        switch (base->GetType())
        {
            case LayerType::Convolution2d:
                replacement = net.AddConvolution2dLayer(static_cast<const Convolution2dDescriptor&>(base->GetParameters()), name.c_str());
                break;
            case LayerType::DepthwiseConvolution2d:
                replacement = net.AddDepthwiseConvolution2dLayer(static_cast<const DepthwiseConvolution2dDescriptor&>(base->GetParameters()), name.c_str());
                break;
            case LayerType::FullyConnected:
                replacement = net.AddFullyConnectedLayer(static_cast<const FullyConnectedDescriptor&>(base->GetParameters()), name.c_str());
                break;
            default:
                replacement = net.AddElementwiseBinaryLayer(static_cast<const ElementwiseBinaryDescriptor&>(base->GetParameters()), name.c_str());
                break;
        }
        replacement->GetOutputSlot(0).SetTensorInfo(act->GetOutputSlot(0).GetTensorInfo());
        PolymorphicDowncast<Layer*>(replacement)->SetAdditionalInfoForObject(std::make_shared<ActivationDescriptor>(ad));

        SubgraphView::IInputSlots ins;
        for (unsigned int i = 0; i < base->GetNumInputSlots(); ++i) ins.push_back(&base->GetInputSlot(i));
        SubgraphView::IOutputSlots outs{&act->GetOutputSlot(0)};
        SubgraphView substitutable({base, act}, std::move(ins), std::move(outs));
        views.AddSubstitution({std::move(substitutable), SubgraphView(replacement)});
        consumed.insert(base);
        consumed.insert(act);
    }

    for (IConnectableLayer* il : layers)
        if (!consumed.count(il)) views.AddUntouchedSubgraph(SubgraphView(il));
    return views;
}
} // namespace armnn
