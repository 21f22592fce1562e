#include "Mi355xBackend.hpp"
#include "Mi355xDefaultAllocator.hpp"
#include "Mi355xBackendId.hpp"
#include "Mi355xDevice.hpp"
#include "Mi355xLayerSupport.hpp"
#include "Mi355xTensorHandle.hpp"
#include "Mi355xWorkloadFactory.hpp"
#include "Mi355xWorkloads.hpp"

#include <Layer.hpp>
#include <armnn/BackendOptions.hpp>
#include <armnn/BackendRegistry.hpp>
#include <armnn/backends/IBackendContext.hpp>
#include <backendsCommon/TensorHandleFactoryRegistry.hpp>

#include <limits>
#include <set>
#include <string>
#include <utility>

namespace armnn
{
namespace
{
// selects and warms up the device when the runtime is created; waits for outstanding work before a network goes away
class Mi355xBackendContext : public IBackendContext
{
public:
    explicit Mi355xBackendContext(const IRuntime::CreationOptions& options) : IBackendContext(options)
    {
        mi355x::EnsureDevice();
        // BackendOptions("Mi355x", {{"Lanes", n}}): into how many slices a batch is split (1 = one stream, addresses shared)
        ParseOptions(options.m_BackendOptions, Mi355xBackendId(), [](const std::string& name, const BackendOptions::Var& value) {
            if (name == "Lanes" && value.IsInt() && value.AsInt() >= 1 && value.AsInt() <= static_cast<int>(mi355x::kMaxLanes))
                mi355x::SetLanes(static_cast<unsigned int>(value.AsInt()));
        });
    }
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
// ---- Pad folding (src/armnn/optimizations/FoldPadIntoLayer2d.hpp:21-145) ---------------------------------------------
// the stored value that stands for the real number 0 (:21-24)
float ZeroElement(const TensorInfo& info) { return static_cast<float>(info.IsQuantized() ? info.GetQuantizationOffset() : 0); }

// the smallest value the tensor's type can hold (:26-56: -infinity quantized, i.e. saturated)
float LowestElement(const TensorInfo& info)
{
    switch (info.GetDataType())
    {
        case DataType::QAsymmU8: return 0.0f;
        case DataType::QAsymmS8: case DataType::QSymmS8: return -128.0f;
        default: return -std::numeric_limits<float>::infinity();
    }
}

// height and width padding of `pad` added to the layer's own; batch and channels must be unpadded (:93-120)
template <typename Descriptor>
bool AddPadding(const PadDescriptor& pad, Descriptor& d)
{
    if (pad.m_PaddingMode != PaddingMode::Constant || pad.m_PadList.size() != 4) return false;
    const bool nhwc = d.m_DataLayout == DataLayout::NHWC;
    const unsigned int channels = nhwc ? 3 : 1, height = nhwc ? 1 : 2, width = nhwc ? 2 : 3;
    const std::pair<unsigned int, unsigned int> none{0u, 0u};
    if (pad.m_PadList[0] != none || pad.m_PadList[channels] != none) return false;
    d.m_PadLeft += pad.m_PadList[width].first;
    d.m_PadRight += pad.m_PadList[width].second;
    d.m_PadTop += pad.m_PadList[height].first;
    d.m_PadBottom += pad.m_PadList[height].second;
    return true;
}

// convolutions skip padded taps, which equals multiplying by the zero element (:58-69)
template <typename Descriptor>
bool FoldPad(const PadDescriptor& pad, Descriptor& d, const TensorInfo& padded)
{
    return pad.m_PadValue == ZeroElement(padded) && AddPadding(pad, d);
}

// (:71-77, :122-145) max pooling ignores anything not above the lowest value; average pooling needs zeros that count in
// the divisor, so it cannot keep padding of its own that is excluded from it
bool FoldPadIntoPooling(const PadDescriptor& pad, Pooling2dDescriptor& d, const TensorInfo& padded)
{
    const bool isMax = d.m_PoolType == PoolingAlgorithm::Max;
    const bool ownPadding = d.m_PadLeft || d.m_PadRight || d.m_PadTop || d.m_PadBottom;
    if (!isMax && ownPadding && d.m_PaddingMethod == PaddingMethod::Exclude) return false;
    if (isMax ? !(pad.m_PadValue <= LowestElement(padded)) : pad.m_PadValue != ZeroElement(padded)) return false;
    if (!AddPadding(pad, d)) return false;
    d.m_PaddingMethod = PaddingMethod::IgnoreValue;
    return true;
}
} // namespace

const BackendId& Mi355xBackend::GetIdStatic()
{
    static const BackendId s_Id{Mi355xBackendId()};
    return s_Id;
}

IBackendInternal::IMemoryManagerUniquePtr Mi355xBackend::CreateMemoryManager() const
{
    return std::make_unique<Mi355xMemoryManager>(mi355x::Lanes() == 1);
}

IBackendInternal::IWorkloadFactoryPtr Mi355xBackend::CreateWorkloadFactory(const IBackendInternal::IMemoryManagerSharedPtr& memoryManager) const
{
    return std::make_unique<Mi355xWorkloadFactory>(std::dynamic_pointer_cast<Mi355xMemoryManager>(memoryManager));
}

namespace
{
// The registry as this backend leaves it: one memory manager, one tensor handle factory, paired with itself for imports --
// the same factory makes the handles that adopt caller memory (RefBackend.cpp:34-48 and :190-203 pair likewise); without
// the pairing LoadedNetwork finds no import factory (LoadedNetwork.cpp:433-447) and ImportInputs / ImportOutputs adopt
// nothing.
Mi355xTensorHandleFactory& EnsureFactories(TensorHandleFactoryRegistry& registry)
{
    if (auto* existing = dynamic_cast<Mi355xTensorHandleFactory*>(registry.GetFactory(Mi355xTensorHandleFactory::GetIdStatic()))) return *existing;
    auto memoryManager = std::make_shared<Mi355xMemoryManager>(mi355x::Lanes() == 1);
    registry.RegisterMemoryManager(memoryManager);
    auto factory = std::make_unique<Mi355xTensorHandleFactory>(memoryManager);
    Mi355xTensorHandleFactory& made = *factory;
    registry.RegisterCopyAndImportFactoryPair(Mi355xTensorHandleFactory::GetIdStatic(), Mi355xTensorHandleFactory::GetIdStatic());
    registry.RegisterFactory(std::move(factory));
    return made;
}
} // namespace

// LoadedNetwork calls this without RegisterTensorHandleFactories (LoadedNetwork.cpp:265-272), the optimizer calls that
// without this (Network.cpp CreateSupportedBackends): either leaves the registry complete.  Handles made by the registered
// tensor handle factory and by the workload factory share one arena.
IBackendInternal::IWorkloadFactoryPtr Mi355xBackend::CreateWorkloadFactory(TensorHandleFactoryRegistry& registry) const
{
    return std::make_unique<Mi355xWorkloadFactory>(EnsureFactories(registry).GetMemoryManager());
}

IBackendInternal::IWorkloadFactoryPtr Mi355xBackend::CreateWorkloadFactory(const IBackendInternal::IMemoryManagerSharedPtr& memoryManager,
                                                                           const ModelOptions&) const
{
    return CreateWorkloadFactory(memoryManager);
}
IBackendInternal::IWorkloadFactoryPtr Mi355xBackend::CreateWorkloadFactory(TensorHandleFactoryRegistry& registry, const ModelOptions&) const
{
    return CreateWorkloadFactory(registry);
}
IBackendInternal::ILayerSupportSharedPtr Mi355xBackend::GetLayerSupport(const ModelOptions&) const { return GetLayerSupport(); }

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
    EnsureFactories(registry);
}

std::unique_ptr<ICustomAllocator> Mi355xBackend::GetDefaultAllocator() const
{
    return std::make_unique<Mi355xDefaultAllocator>();
}

bool Mi355xBackend::UseCustomMemoryAllocator(std::shared_ptr<ICustomAllocator> allocator, armnn::Optional<std::string&> errMsg)
{
    auto refuse = [&](const std::string& why)
    {
        if (errMsg) errMsg.value() = "Mi355x: " + why;
        return false;
    };
    if (!allocator) return refuse("null allocator");
    if (allocator->GetMemorySourceType() != MemorySource::Malloc) return refuse("only allocators of MemorySource::Malloc are supported");
    if (mi355x::DeviceCount() == 0) return refuse("no device to check the allocator's memory against");
    void* probe = nullptr;
    try
    {
        mi355x::EnsureDevice();
        probe = allocator->allocate(256, 16);
    }
    catch (const std::exception& e)
    {
        return refuse(std::string("the allocator's probe allocation failed: ") + e.what());
    }
    void* device = nullptr;
    int isDevice = 0;
    const bool reachable = probe && mi355x_host_device_pointer(probe, &device, &isDevice) == 0 && device != nullptr;
    if (probe) allocator->free(probe);
    if (!reachable) return refuse("the allocator returns memory the device cannot reach (pageable host memory); use device or pinned memory");
    return true;
}

BackendCapabilities Mi355xBackend::GetCapabilities() const
{
    return BackendCapabilities(Mi355xBackendId(), {{"NonConstWeights", false},
                                                   {"AsyncExecution", false},
                                                   {"ProtectedContentAllocation", false},
                                                   {"ConstantTensorsAsInputs", true},
                                                   {"PreImportIOTensors", true},
                                                   {"ExternallyManagedMemory", true},
                                                   {"MultiAxisPacking", false},
                                                   {"SingleAxisPacking", false}});
}

// Two rewrites, alone or together on one layer:
//
// * A quantized ReLu / BoundedReLu whose input and output share one quantization is an integer clamp
//   (workloads/Activation.cpp:33-42 between a decoder and an encoder of the same scale and offset), which the device
//   kernels apply in their epilogue.  With different quantizations the Activation layer re-quantizes and stays a layer
//   of its own.  The replacement layer carries the ActivationDescriptor as its additional-info object, as the Neon and
//   CL backends do (src/backends/aclCommon/ArmComputeSubgraphUtils.hpp:60-109).
// * A Convolution2d without an activation whose output goes to one Addition of this backend and nowhere else is marked
//   (Mi355xFeedsOnlyAnAddition): the two workloads may then run as one launch (Mi355xAdditionWorkload).
// * A DepthwiseConvolution2d whose output goes to one unpadded 1x1 stride-1 Convolution2d of this backend and nowhere else
//   is marked (Mi355xLayerNote, which also carries the fused activation): the two workloads may then run as one launch
//   (Mi355xConvolution2dWorkload::TakeOver).
// * An unpadded 1x1 stride-1 Convolution2d whose output goes to one Pooling2d of this backend over the whole unpadded image
//   and nowhere else is marked the same way: the two workloads may then run as one launch (Mi355xPooling2dWorkload::TakeOver).
// * A Reshape that only flattens the dimensions behind the batch, in front of a FullyConnected, is dropped: the
//   FullyConnected reads the unflattened tensor (same bytes in the same order).
// * A constant Pad of height and width in front of a Convolution2d, DepthwiseConvolution2d or Pooling2d moves into that
//   layer's own padding when the padded value is the layer's neutral element, as CpuRef does
//   (src/backends/reference/RefBackend.cpp:72-184 with the rules of src/armnn/optimizations/FoldPadIntoLayer2d.hpp:21-145).
OptimizationViews Mi355xBackend::OptimizeSubgraphView(const SubgraphView& subgraph, const ModelOptions& modelOptions) const
{
    OptimizationViews views(modelOptions);
    const SubgraphView::IConnectableLayers& layers = subgraph.GetIConnectableLayers();
    std::set<const IConnectableLayer*> members(layers.begin(), layers.end());
    std::set<const IConnectableLayer*> consumed;
    // BackendOptions("Mi355x", {{"FuseAdditions", false}}) among the network's model options keeps every Addition a launch of its own
    bool fuseAdditions = true;
    // ... {{"FuseDepthwisePointwise", false}} keeps every depthwise layer and the 1x1 convolution behind it two launches
    bool fuseDepthwisePointwise = true;
    // ... {{"FuseConvolutionPooling", false}} keeps every 1x1 convolution and the pooling over its whole image two launches
    bool fuseConvolutionPooling = true;
    ParseOptions(modelOptions, Mi355xBackendId(), [&](const std::string& name, const BackendOptions::Var& value) {
        if (name == "FuseAdditions" && value.IsBool()) fuseAdditions = value.AsBool();
        if (name == "FuseDepthwisePointwise" && value.IsBool()) fuseDepthwisePointwise = value.AsBool();
        if (name == "FuseConvolutionPooling" && value.IsBool()) fuseConvolutionPooling = value.AsBool();
    });

    for (IConnectableLayer* il : layers)
    {
        if (consumed.count(il)) continue;
        Layer* base = PolymorphicDowncast<Layer*>(il);
        const LayerType type = base->GetType();

        // the descriptor the replacement would get; the Pad in front of the layer, if its padding fits into it
        Convolution2dDescriptor conv;
        DepthwiseConvolution2dDescriptor depthwise;
        Pooling2dDescriptor pooling;
        Layer* pad = nullptr;
        if (type == LayerType::Convolution2d || type == LayerType::DepthwiseConvolution2d || type == LayerType::Pooling2d)
        {
            if (type == LayerType::Convolution2d) conv = static_cast<const Convolution2dDescriptor&>(base->GetParameters());
            if (type == LayerType::DepthwiseConvolution2d) depthwise = static_cast<const DepthwiseConvolution2dDescriptor&>(base->GetParameters());
            if (type == LayerType::Pooling2d) pooling = static_cast<const Pooling2dDescriptor&>(base->GetParameters());
            OutputSlot* source = base->GetInputSlot(0).GetConnectedOutputSlot();
            Layer* producer = source ? &source->GetOwningLayer() : nullptr;
            if (producer && producer->GetType() == LayerType::Pad && members.count(producer) && !consumed.count(producer) &&
                source->GetNumConnections() == 1 && producer->GetInputSlot(0).GetConnectedOutputSlot() != nullptr)
            {
                const auto& pd = static_cast<const PadDescriptor&>(producer->GetParameters());
                const TensorInfo& padded = source->GetTensorInfo();
                const bool folded = type == LayerType::Convolution2d ? FoldPad(pd, conv, padded)
                                  : type == LayerType::DepthwiseConvolution2d ? FoldPad(pd, depthwise, padded)
                                  : FoldPadIntoPooling(pd, pooling, padded);
                if (folded) pad = producer;
            }
        }

        // the Reshape in front of a FullyConnected, if it only flattens what follows the batch: FullyConnected takes the
        // unflattened tensor as it is (FullyConnectedLayer.cpp:64-80 infers {shape[0], outputs} from any input;
        // WorkloadData.cpp:1036-1098 admits 2 or 4 dimensions), and the copy the Reshape workload would make goes away
        Layer* flat = nullptr;
        if (type == LayerType::FullyConnected)
        {
            OutputSlot* source = base->GetInputSlot(0).GetConnectedOutputSlot();
            Layer* producer = source ? &source->GetOwningLayer() : nullptr;
            if (producer && producer->GetType() == LayerType::Reshape && members.count(producer) && !consumed.count(producer) &&
                source->GetNumConnections() == 1 && producer->GetInputSlot(0).GetConnectedOutputSlot() != nullptr)
            {
                const TensorInfo& before = producer->GetInputSlot(0).GetConnectedOutputSlot()->GetTensorInfo();
                const TensorInfo& after = source->GetTensorInfo();
                if ((before.GetNumDimensions() == 2 || before.GetNumDimensions() == 4) && after.GetNumDimensions() == 2 &&
                    before.GetShape()[0] == after.GetShape()[0] && before.GetNumElements() == after.GetNumElements() &&
                    SameQuantization(before, after))
                    flat = producer;
            }
        }

        // the Activation behind the layer, if it is a clamp in the layer's own output quantization
        Layer* act = nullptr;
        if (Fusable(*base) && base->GetAdditionalInformation<ActivationDescriptor>() == nullptr && base->GetOutputSlot(0).GetNumConnections() == 1)
        {
            Layer* next = &base->GetOutputSlot(0).GetConnections()[0]->GetOwningLayer();
            if (next->GetType() == LayerType::Activation && members.count(next) && !consumed.count(next))
            {
                const auto& ad = static_cast<const ActivationDescriptor&>(next->GetParameters());
                if ((ad.m_Function == ActivationFunction::ReLu || ad.m_Function == ActivationFunction::BoundedReLu) &&
                    SameQuantization(base->GetOutputSlot(0).GetTensorInfo(), next->GetOutputSlot(0).GetTensorInfo()))
                    act = next;
            }
        }
        // a Convolution2d whose only consumer is an Addition of this backend: its workload may run inside that Addition's
        bool residual = false;
        if (fuseAdditions && type == LayerType::Convolution2d && !act && base->GetAdditionalInformation<ActivationDescriptor>() == nullptr &&
            base->GetOutputSlot(0).GetNumConnections() == 1)
        {
            Layer* next = &base->GetOutputSlot(0).GetConnections()[0]->GetOwningLayer();
            if (next->GetType() == LayerType::ElementwiseBinary && members.count(next) &&
                static_cast<const ElementwiseBinaryDescriptor&>(next->GetParameters()).m_Operation == BinaryOperation::Add &&
                next->GetInputSlot(0).GetConnectedOutputSlot() != next->GetInputSlot(1).GetConnectedOutputSlot())
                residual = true;
        }
        // a DepthwiseConvolution2d (with the Activation fused into it, if any) whose only consumer is an unpadded 1x1 stride-1
        // Convolution2d of this backend: the two workloads may run as one launch (Mi355xConvolution2dWorkload::TakeOver)
        bool pointwiseNext = false;
        if (fuseDepthwisePointwise && type == LayerType::DepthwiseConvolution2d)
        {
            Layer* lastOfThis = act ? act : base;
            if (lastOfThis->GetOutputSlot(0).GetNumConnections() == 1)
            {
                InputSlot* to = lastOfThis->GetOutputSlot(0).GetConnections()[0];
                Layer* next = &to->GetOwningLayer();
                if (next->GetType() == LayerType::Convolution2d && members.count(next) && to->GetSlotIndex() == 0)
                {
                    const auto& nd = static_cast<const Convolution2dDescriptor&>(next->GetParameters());
                    const OutputSlot* weights = next->GetInputSlot(1).GetConnectedOutputSlot();
                    pointwiseNext = weights != nullptr && weights->GetTensorInfo().GetNumDimensions() == 4 &&
                                    weights->GetTensorInfo().GetShape()[1] == 1 && weights->GetTensorInfo().GetShape()[2] == 1 &&
                                    nd.m_StrideX == 1 && nd.m_StrideY == 1 && nd.m_PadLeft == 0 && nd.m_PadRight == 0 && nd.m_PadTop == 0 &&
                                    nd.m_PadBottom == 0 && nd.m_DataLayout == DataLayout::NHWC;
                }
            }
            // (a layer that already carries the mark needs no second replacement)
            if (pointwiseNext && !pad && !act)
                if (const Mi355xLayerNote* note = Mi355xLayerNote::From(base->GetAdditionalInformation<ActivationDescriptor>().get()))
                    if (note->onlyConsumerIsAPointwiseConvolution) pointwiseNext = false;
        }
        // an unpadded 1x1 stride-1 Convolution2d (with the Activation fused into it, if any) whose only consumer is a Pooling2d
        // of this backend over the whole unpadded image: the two workloads may run as one launch
        // (Mi355xPooling2dWorkload::TakeOver)
        bool poolingNext = false;
        if (fuseConvolutionPooling && type == LayerType::Convolution2d && !residual && !pad)
        {
            Layer* lastOfThis = act ? act : base;
            const OutputSlot* weights = base->GetInputSlot(1).GetConnectedOutputSlot();
            const bool pointwise = weights != nullptr && weights->GetTensorInfo().GetNumDimensions() == 4 &&
                                   weights->GetTensorInfo().GetShape()[1] == 1 && weights->GetTensorInfo().GetShape()[2] == 1 &&
                                   conv.m_StrideX == 1 && conv.m_StrideY == 1 && conv.m_PadLeft == 0 && conv.m_PadRight == 0 &&
                                   conv.m_PadTop == 0 && conv.m_PadBottom == 0 && conv.m_DataLayout == DataLayout::NHWC;
            if (pointwise && lastOfThis->GetOutputSlot(0).GetNumConnections() == 1)
            {
                Layer* next = &lastOfThis->GetOutputSlot(0).GetConnections()[0]->GetOwningLayer();
                if (next->GetType() == LayerType::Pooling2d && members.count(next))
                {
                    const auto& pd = static_cast<const Pooling2dDescriptor&>(next->GetParameters());
                    const TensorInfo& image = lastOfThis->GetOutputSlot(0).GetTensorInfo();
                    const TensorInfo& pooled = next->GetOutputSlot(0).GetTensorInfo();
                    poolingNext = pd.m_DataLayout == DataLayout::NHWC && image.GetNumDimensions() == 4 && pooled.GetNumDimensions() == 4 &&
                                  pd.m_PoolHeight == image.GetShape()[1] && pd.m_PoolWidth == image.GetShape()[2] &&
                                  pooled.GetShape()[1] == 1 && pooled.GetShape()[2] == 1 && pd.m_PadLeft == 0 && pd.m_PadRight == 0 &&
                                  pd.m_PadTop == 0 && pd.m_PadBottom == 0 &&
                                  (pd.m_PoolType == PoolingAlgorithm::Max || pd.m_PoolType == PoolingAlgorithm::Average);
                }
            }
            if (poolingNext && !act)
                if (const Mi355xLayerNote* note = Mi355xLayerNote::From(base->GetAdditionalInformation<ActivationDescriptor>().get()))
                    if (note->onlyConsumerIsAGlobalPooling) poolingNext = false;
        }
        if (!pad && !act && !residual && !flat && !pointwiseNext && !poolingNext) continue;

        std::string name = base->GetName();
        if (pad) name = std::string("folded-") + pad->GetName() + "-into-" + name;
        if (flat) name = std::string("folded-") + flat->GetName() + "-into-" + name;
        if (act) name = std::string("fused-") + act->GetName() + "-into-" + name;
        INetwork& net = views.GetINetworkRef();
        IConnectableLayer* replacement = nullptr;
        switch (type)
        {
            case LayerType::Convolution2d: replacement = net.AddConvolution2dLayer(conv, name.c_str()); break;
            case LayerType::DepthwiseConvolution2d: replacement = net.AddDepthwiseConvolution2dLayer(depthwise, name.c_str()); break;
            case LayerType::Pooling2d: replacement = net.AddPooling2dLayer(pooling, name.c_str()); break;
            case LayerType::FullyConnected:
                replacement = net.AddFullyConnectedLayer(static_cast<const FullyConnectedDescriptor&>(base->GetParameters()), name.c_str());
                break;
            default:
                replacement = net.AddElementwiseBinaryLayer(static_cast<const ElementwiseBinaryDescriptor&>(base->GetParameters()), name.c_str());
                break;
        }
        Layer* last = act ? act : base;
        replacement->GetOutputSlot(0).SetTensorInfo(last->GetOutputSlot(0).GetTensorInfo());
        if (pointwiseNext || poolingNext)
        {
            auto carried = base->GetAdditionalInformation<ActivationDescriptor>();
            PolymorphicDowncast<Layer*>(replacement)->SetAdditionalInfoForObject(
                Mi355xLayerNote::Make(act ? &static_cast<const ActivationDescriptor&>(act->GetParameters()) : carried.get(), pointwiseNext,
                                      poolingNext));
        }
        else if (act)
            PolymorphicDowncast<Layer*>(replacement)->SetAdditionalInfoForObject(
                std::make_shared<ActivationDescriptor>(static_cast<const ActivationDescriptor&>(act->GetParameters())));
        else if (auto carried = base->GetAdditionalInformation<ActivationDescriptor>())
            PolymorphicDowncast<Layer*>(replacement)->SetAdditionalInfoForObject(carried);
        else if (residual)
            PolymorphicDowncast<Layer*>(replacement)->SetAdditionalInfoForObject(std::make_shared<ActivationDescriptor>(Mi355xFeedsOnlyAnAddition()));

        SubgraphView::IConnectableLayers replaced;
        SubgraphView::IInputSlots ins;
        Layer* front = pad ? pad : flat;
        if (front) replaced.push_back(front);
        replaced.push_back(base);
        if (act) replaced.push_back(act);
        ins.push_back(front ? &front->GetInputSlot(0) : &base->GetInputSlot(0));
        for (unsigned int i = 1; i < base->GetNumInputSlots(); ++i) ins.push_back(&base->GetInputSlot(i));
        SubgraphView::IOutputSlots outs{&last->GetOutputSlot(0)};
        SubgraphView substitutable(std::move(replaced), std::move(ins), std::move(outs));
        views.AddSubstitution({std::move(substitutable), SubgraphView(replacement)});
        for (Layer* l : {pad, flat, base, act})
            if (l) consumed.insert(l);
    }

    for (IConnectableLayer* il : layers)
        if (!consumed.count(il)) views.AddUntouchedSubgraph(SubgraphView(il));
    return views;
}
} // namespace armnn
