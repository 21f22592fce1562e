// Minimal host core: what src/backends/backendsCommon provides to every backend -- registry, tensor-handle-factory
// registry, descriptor validation, the generic copy workload, dynamic backend loading, layer-support dispatch.
#include <Layer.hpp>
#include <armnn/BackendRegistry.hpp>
#include <armnn/backends/DynamicBackend.hpp>
#include <armnn/backends/IBackendInternal.hpp>
#include <armnn/backends/MemCopyWorkload.hpp>
#include <backendsCommon/TensorHandleFactoryRegistry.hpp>
#include <armnn/backends/WorkloadData.hpp>
#include <armnn/backends/WorkloadFactory.hpp>

#include <dirent.h>
#include <dlfcn.h>

#include <algorithm>
#include <atomic>
#include <cstring>
#include <regex>
#include <set>
#include <sstream>

namespace arm { namespace pipe {
ProfilingGuid IProfilingService::GetNextGuid()
{
    static std::atomic<uint64_t> next{1};
    return ProfilingGuid(next.fetch_add(1));
}
}} // namespace arm::pipe

namespace armnn
{
const ITensorHandleFactory::FactoryId ITensorHandleFactory::LegacyFactoryId = "armnn_legacy_factory";
const ITensorHandleFactory::FactoryId ITensorHandleFactory::DeferredFactoryId = "armnn_deferred_factory";

// ---- BackendRegistry (src/armnn/BackendRegistry.cpp:14-60) ---------------------------------------------------
BackendRegistry& BackendRegistryInstance()
{
    static BackendRegistry instance;
    return instance;
}

void BackendRegistry::Register(const BackendId& id, FactoryFunction factory)
{
    if (m_Factories.find(id) != m_Factories.end())
        throw InvalidArgumentException(std::string(id) + " already registered as IBackend factory", CHECK_LOCATION());
    m_Factories[id] = factory;
}
bool BackendRegistry::IsBackendRegistered(const BackendId& id) const { return m_Factories.find(id) != m_Factories.end(); }
BackendRegistry::FactoryFunction BackendRegistry::GetFactory(const BackendId& id) const
{
    auto it = m_Factories.find(id);
    if (it == m_Factories.end()) throw InvalidArgumentException(std::string(id) + " has no IBackend factory registered", CHECK_LOCATION());
    return it->second;
}
size_t BackendRegistry::Size() const { return m_Factories.size(); }
BackendIdSet BackendRegistry::GetBackendIds() const
{
    BackendIdSet s;
    for (const auto& f : m_Factories) s.insert(f.first);
    return s;
}
std::string BackendRegistry::GetBackendIdsAsString() const
{
    std::vector<std::string> ids;
    for (const auto& f : m_Factories) ids.push_back(f.first.Get());
    std::sort(ids.begin(), ids.end());
    std::string out = "[";
    for (size_t i = 0; i < ids.size(); ++i) out += (i ? " " : "") + ids[i];
    return out + "]";
}
void BackendRegistry::Deregister(const BackendId& id) { m_Factories.erase(id); }
void BackendRegistry::RegisterAllocator(const BackendId& id, std::shared_ptr<ICustomAllocator> alloc)
{
    if (m_CustomMemoryAllocatorMap.count(id)) throw InvalidArgumentException("Allocator for backend " + id.Get() + " already registered");
    m_CustomMemoryAllocatorMap[id] = std::move(alloc);
}
std::unordered_map<BackendId, std::shared_ptr<ICustomAllocator>> BackendRegistry::GetAllocators() { return m_CustomMemoryAllocatorMap; }
void BackendRegistry::DeregisterAllocator(const BackendId& id) { m_CustomMemoryAllocatorMap.erase(id); }
void BackendRegistry::RegisterMemoryOptimizerStrategy(const BackendId& id, std::shared_ptr<IMemoryOptimizerStrategy> strategy)
{
    if (m_MemoryOptimizerStrategyMap.count(id)) throw InvalidArgumentException("Memory optimizer strategy for backend " + id.Get() + " already registered");
    m_MemoryOptimizerStrategyMap[id] = std::move(strategy);
}
std::unordered_map<BackendId, std::shared_ptr<IMemoryOptimizerStrategy>> BackendRegistry::GetMemoryOptimizerStrategies() { return m_MemoryOptimizerStrategyMap; }
void BackendRegistry::DeregisterMemoryOptimizerStrategy(const BackendId& id) { m_MemoryOptimizerStrategyMap.erase(id); }

// ---- TensorHandleFactoryRegistry -----------------------------------------------------------------------------
void TensorHandleFactoryRegistry::RegisterFactory(std::unique_ptr<ITensorHandleFactory> f)
{
    if (!f) throw InvalidArgumentException("RegisterFactory: null factory");
    for (const auto& e : m_Factories)
        if (e->GetId() == f->GetId()) return;
    m_Factories.push_back(std::move(f));
}
void TensorHandleFactoryRegistry::RegisterMemoryManager(std::shared_ptr<IMemoryManager> m) { m_MemoryManagers.push_back(std::move(m)); }
ITensorHandleFactory* TensorHandleFactoryRegistry::GetFactory(ITensorHandleFactory::FactoryId id) const
{
    for (const auto& f : m_Factories)
        if (f->GetId() == id) return f.get();
    return nullptr;
}
void TensorHandleFactoryRegistry::RegisterCopyAndImportFactoryPair(ITensorHandleFactory::FactoryId c, ITensorHandleFactory::FactoryId i)
{
    m_FactoryMappings[c] = i;
}
ITensorHandleFactory::FactoryId TensorHandleFactoryRegistry::GetMatchingImportFactoryId(ITensorHandleFactory::FactoryId c)
{
    auto it = m_FactoryMappings.find(c);
    return it == m_FactoryMappings.end() ? ITensorHandleFactory::FactoryId() : it->second;
}
void TensorHandleFactoryRegistry::AquireMemory() { for (auto& m : m_MemoryManagers) m->Acquire(); }
void TensorHandleFactoryRegistry::ReleaseMemory() { for (auto& m : m_MemoryManagers) m->Release(); }

// ---- descriptor validation (src/backends/backendsCommon/WorkloadData.cpp) -----------------------------------
namespace
{
void Require(bool cond, const std::string& msg)
{
    if (!cond) throw InvalidArgumentException(msg);
}

void ValidateNumInputsOutputs(const WorkloadInfo& info, const std::string& name, size_t nin, size_t nout)
{
    Require(info.m_InputTensorInfos.size() == nin, name + ": Requires exactly " + std::to_string(nin) + " input(s). " +
                                                        std::to_string(info.m_InputTensorInfos.size()) + " have been provided.");
    Require(info.m_OutputTensorInfos.size() == nout, name + ": Requires exactly " + std::to_string(nout) + " output(s). " +
                                                          std::to_string(info.m_OutputTensorInfos.size()) + " have been provided.");
}

void ValidateDims(const TensorInfo& t, const std::string& name, unsigned int dims, const char* what)
{
    Require(t.GetNumDimensions() == dims, name + ": Expected " + std::to_string(dims) + " dimensions but got " +
                                              std::to_string(t.GetNumDimensions()) + " dimensions for " + what + " tensor.");
}

// WorkloadData.cpp:28-45
Optional<DataType> GetBiasDataType(DataType inputDataType)
{
    switch (inputDataType)
    {
        case DataType::Float16: return DataType::Float16;
        case DataType::BFloat16: case DataType::Float32: return DataType::Float32;
        case DataType::QAsymmS8: case DataType::QAsymmU8: case DataType::QSymmS8: case DataType::QSymmS16: return DataType::Signed32;
        default: throw InvalidArgumentException("GetBiasDataType: invalid input data type");
    }
}

// WorkloadData.cpp:180-205: bias offset must be 0; a per-axis bias must carry as many scales as the weights
void ValidateBiasTensorQuantization(const TensorInfo& bias, const TensorInfo& weights, const std::string& name)
{
    Require(bias.GetQuantizationOffset() == 0, name + ": Quantization offset for bias value expected to be 0, but got " +
                                                   std::to_string(bias.GetQuantizationOffset()));
    if (bias.HasMultipleQuantizationScales())
    {
        Require(weights.HasMultipleQuantizationScales(), name + ": Per-axis quantization parameters not set on weights, despite being set on bias.");
        Require(bias.GetQuantizationScales().size() == weights.GetQuantizationScales().size(),
                name + ": Expected matching number of per-axis quantization scales for weights and bias.");
    }
}

// WorkloadData.cpp:353-393
void ValidatePerAxisQuantization(const TensorInfo& input, const TensorInfo& output, const TensorInfo& weights,
                                 const Optional<TensorInfo>& bias, const std::string& name)
{
    if (!weights.HasPerAxisQuantization()) return;
    const DataType inputType = input.GetDataType();
    Require(inputType == DataType::QAsymmS8 || inputType == DataType::QAsymmU8 || inputType == DataType::QSymmS8,
            name + ": Per-axis quantization is only supported for 8-bit quantized inputs.");
    Require(output.GetDataType() == inputType, name + ": input and output data types must match for per-axis quantization.");
    Require(weights.GetDataType() == DataType::QSymmS8, name + ": weights must be QSymmS8 for per-axis quantization.");
    Require(weights.GetQuantizationDim().has_value(), name + ": Quantization dimension for per-axis quantization not set on tensor weights.");
    Require(weights.GetQuantizationOffset() == 0, name + ": Quantization offset for per-axis quantization expected to be 0 on tensor weights.");
    if (bias.has_value())
    {
        Require(bias.value().GetDataType() == DataType::Signed32, name + ": bias must be Signed32 for per-axis quantization.");
        Require(bias.value().HasPerAxisQuantization(), name + ": Per-axis quantization parameters not set on bias tensor, despite being set on weight tensor.");
    }
}

void ValidateTypesMatch(const TensorInfo& a, const TensorInfo& b, const std::string& name, const char* an, const char* bn)
{
    Require(a.GetDataType() == b.GetDataType(), name + ": " + an + " & " + bn + " must have identical data types.");
}
} // namespace

void QueueDescriptor::ValidateInputsOutputs(const std::string& descName, unsigned int numExpectedIn, unsigned int numExpectedOut) const
{
    Require(m_Inputs.size() == numExpectedIn, descName + ": Number of inputs (" + std::to_string(m_Inputs.size()) + ") does not match expected (" + std::to_string(numExpectedIn) + ")");
    Require(m_Outputs.size() == numExpectedOut, descName + ": Number of outputs (" + std::to_string(m_Outputs.size()) + ") does not match expected (" + std::to_string(numExpectedOut) + ")");
    for (auto* h : m_Inputs) Require(h != nullptr, descName + ": Invalid NULL input");
    for (auto* h : m_Outputs) Require(h != nullptr, descName + ": Invalid NULL output");
}

void MemCopyQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    ValidateNumInputsOutputs(info, "MemCopyQueueDescriptor", 1, 1);
    Require(info.m_InputTensorInfos[0].GetNumElements() == info.m_OutputTensorInfos[0].GetNumElements(),
            "MemCopyQueueDescriptor: input and output must have the same number of elements");
    Require(m_Inputs.size() == m_Outputs.size(), "MemCopyQueueDescriptor: Number of inputs and outputs do not match");
}

void ConstantQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    ValidateNumInputsOutputs(info, "ConstantQueueDescriptor", 0, 1);
    Require(m_LayerOutput != nullptr, "ConstantQueueDescriptor: No const input specified.");
}

void ActivationQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    ValidateNumInputsOutputs(info, "ActivationQueueDescriptor", 1, 1);
    ValidateTypesMatch(info.m_InputTensorInfos[0], info.m_OutputTensorInfos[0], "ActivationQueueDescriptor", "input", "output");
    Require(info.m_InputTensorInfos[0].GetShape() == info.m_OutputTensorInfos[0].GetShape(), "ActivationQueueDescriptor: input and output shapes differ");
}

// WorkloadData.cpp:1253-1328
void Convolution2dQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    const std::string name = "Convolution2dQueueDescriptor";
    ValidateNumInputsOutputs(info, name, m_Parameters.GetNumInputs(), 1);
    const TensorInfo& in = info.m_InputTensorInfos[0];
    const TensorInfo& out = info.m_OutputTensorInfos[0];
    const TensorInfo& w = info.m_InputTensorInfos[1];
    ValidateDims(in, name, 4, "input");
    ValidateDims(out, name, 4, "output");
    ValidateDims(w, name, 4, "weight");
    Optional<TensorInfo> bias;
    if (m_Parameters.m_BiasEnabled)
    {
        bias = MakeOptional<TensorInfo>(info.m_InputTensorInfos[2]);
        Require(bias.value().GetDataType() == GetBiasDataType(in.GetDataType()).value(), name + ": bias has an unexpected data type.");
        ValidateBiasTensorQuantization(bias.value(), w, name);
    }
    Require(m_Parameters.m_StrideX > 0 && m_Parameters.m_StrideY > 0,
            name + ": strideX (provided " + std::to_string(m_Parameters.m_StrideX) + ") and strideY (provided " +
                std::to_string(m_Parameters.m_StrideY) + ") cannot be either negative or 0.");
    ValidatePerAxisQuantization(in, out, w, bias, name);
    ValidateTypesMatch(in, out, name, "input", "output");
}

// WorkloadData.cpp:1392-1494
void DepthwiseConvolution2dQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    const std::string name = "DepthwiseConvolution2dQueueDescriptor";
    ValidateNumInputsOutputs(info, name, m_Parameters.GetNumInputs(), 1);
    const TensorInfo& in = info.m_InputTensorInfos[0];
    const TensorInfo& out = info.m_OutputTensorInfos[0];
    const TensorInfo& w = info.m_InputTensorInfos[1];
    ValidateDims(in, name, 4, "input");
    ValidateDims(out, name, 4, "output");
    ValidateDims(w, name, 4, "weight");
    Require(m_Parameters.m_DilationX >= 1 && m_Parameters.m_DilationY >= 1,
            name + ": dilationX (provided " + std::to_string(m_Parameters.m_DilationX) + ") and dilationY (provided " +
                std::to_string(m_Parameters.m_DilationY) + ") cannot be smaller than 1.");
    Require(m_Parameters.m_StrideX > 0 && m_Parameters.m_StrideY > 0, name + ": strideX and strideY cannot be either negative or 0.");
    Require(w.GetShape()[0] == 1, name + ": The weight format in armnn is expected to be [1, H, W, Cout]. But first dimension is not equal to 1.");
    const unsigned int channelIndex = m_Parameters.m_DataLayout == DataLayout::NCHW ? 1 : 3;
    const unsigned int cout = out.GetShape()[channelIndex];
    Require(w.GetShape()[3] == cout || w.GetShape()[1] == cout,
            name + ": The weight format in armnn is expected to be [1, H, W, Cout]. But 4th dimension is not equal to Cout.");
    Optional<TensorInfo> bias;
    if (m_Parameters.m_BiasEnabled)
    {
        bias = MakeOptional<TensorInfo>(info.m_InputTensorInfos[2]);
        ValidateBiasTensorQuantization(bias.value(), w, name);
        Require(bias.value().GetDataType() == GetBiasDataType(in.GetDataType()).value(), name + ": bias has an unexpected data type.");
    }
    ValidatePerAxisQuantization(in, out, w, bias, name);
    ValidateTypesMatch(in, out, name, "input", "output");
}

// WorkloadData.cpp:1036-1098
void FullyConnectedQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    const std::string name = "FullyConnectedQueueDescriptor";
    ValidateNumInputsOutputs(info, name, m_Parameters.GetNumInputs(), 1);
    const TensorInfo& in = info.m_InputTensorInfos[0];
    const TensorInfo& out = info.m_OutputTensorInfos[0];
    const TensorInfo& w = info.m_InputTensorInfos[1];
    ValidateDims(out, name, 2, "output");
    Require(in.GetNumDimensions() == 2 || in.GetNumDimensions() == 4, name + ": Input tensor must have 2 or 4 dimensions.");
    ValidateDims(w, name, 2, "weight");
    if (m_Parameters.m_BiasEnabled)
    {
        const TensorInfo& b = info.m_InputTensorInfos[2];
        ValidateBiasTensorQuantization(b, w, name);
        Require(b.GetDataType() == GetBiasDataType(in.GetDataType()).value(), name + ": bias has an unexpected data type.");
        ValidateDims(b, name, 1, "bias");
    }
    ValidateTypesMatch(in, out, name, "input", "output");
}

void Pooling2dQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    const std::string name = "Pooling2dQueueDescriptor";
    ValidateNumInputsOutputs(info, name, 1, 1);
    ValidateDims(info.m_InputTensorInfos[0], name, 4, "input");
    ValidateDims(info.m_OutputTensorInfos[0], name, 4, "output");
    ValidateTypesMatch(info.m_InputTensorInfos[0], info.m_OutputTensorInfos[0], name, "input", "output");
}

// WorkloadData.cpp:2439-2482
void MeanQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    const std::string name = "MeanQueueDescriptor";
    ValidateNumInputsOutputs(info, name, 1, 1);
    const TensorInfo& in = info.m_InputTensorInfos[0];
    const TensorInfo& out = info.m_OutputTensorInfos[0];
    ValidateTypesMatch(in, out, name, "input", "output");
    const unsigned int rank = in.GetNumDimensions();
    const unsigned int axes = static_cast<unsigned int>(m_Parameters.m_Axis.size());
    const unsigned int expected = m_Parameters.m_KeepDims ? rank : m_Parameters.m_Axis.empty() ? 1u : (rank > axes ? rank - axes : 1u);
    ValidateDims(out, name, expected, "output");
}

// WorkloadData.cpp:2484-2504
void PadQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    const std::string name = "PadQueueDescriptor";
    ValidateNumInputsOutputs(info, name, 1, 1);
    const TensorInfo& in = info.m_InputTensorInfos[0];
    ValidateDims(info.m_OutputTensorInfos[0], name, in.GetNumDimensions(), "output");
    Require(m_Parameters.m_PadList.size() == in.GetNumDimensions(),
            name + ": the pad list needs one entry per input dimension (" + std::to_string(in.GetNumDimensions()) +
            "), not " + std::to_string(m_Parameters.m_PadList.size()));
}

void SoftmaxQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    const std::string name = "SoftmaxQueueDescriptor";
    ValidateNumInputsOutputs(info, name, 1, 1);
    ValidateTypesMatch(info.m_InputTensorInfos[0], info.m_OutputTensorInfos[0], name, "input", "output");
    Require(info.m_InputTensorInfos[0].GetShape() == info.m_OutputTensorInfos[0].GetShape(), name + ": input and output shapes differ");
}

void ElementwiseBinaryQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    const std::string name = "ElementwiseBinaryQueueDescriptor";
    ValidateNumInputsOutputs(info, name, 2, 1);
    ValidateTypesMatch(info.m_InputTensorInfos[0], info.m_InputTensorInfos[1], name, "input_0", "input_1");
    ValidateTypesMatch(info.m_InputTensorInfos[0], info.m_OutputTensorInfos[0], name, "input", "output");
}

void ReshapeQueueDescriptor::Validate(const WorkloadInfo& info) const
{
    const std::string name = "ReshapeQueueDescriptor";
    ValidateNumInputsOutputs(info, name, 1, 1);
    Require(info.m_InputTensorInfos[0].GetNumElements() == info.m_OutputTensorInfos[0].GetNumElements(),
            name + ": input and output must have the same number of elements");
}

// ---- generic copy (MemCopyWorkload.cpp:44-64; WorkloadUtils.hpp:46-211 for dense tensors) ---------------------
CopyMemGenericWorkload::CopyMemGenericWorkload(const MemCopyQueueDescriptor& descriptor, const WorkloadInfo& info)
    : BaseWorkload<MemCopyQueueDescriptor>(descriptor, info) {}

void CopyMemGenericWorkload::Execute() const
{
    for (size_t i = 0; i < m_Data.m_Inputs.size(); ++i)
    {
        const ITensorHandle* src = m_Data.m_Inputs[i];
        ITensorHandle* dst = m_Data.m_Outputs[i];
        const TensorShape shape = src->GetShape();
        const TensorShape strides = src->GetStrides();
        const size_t bytes = shape.GetNumDimensions() ? static_cast<size_t>(shape[0]) * strides[0] : 0;
        const void* s = src->Map();
        void* d = dst->Map();
        if (s && d && bytes) std::memcpy(d, s, bytes);
        src->Unmap();
        dst->Unmap();
    }
}

// ---- layer-support dispatch (WorkloadFactory.cpp:70-94, info lists :258-291; BackendHelper.cpp:371-423) -----
bool IWorkloadFactory::IsLayerSupported(const BackendId& backendId, const IConnectableLayer& connectableLayer, Optional<DataType>,
                                        std::string& outReasonIfUnsupported, const ModelOptions& modelOptions)
{
    Optional<std::string&> reason = outReasonIfUnsupported;
    if (!BackendRegistryInstance().IsBackendRegistered(backendId))
    {
        outReasonIfUnsupported = std::string("backend ") + backendId.Get() + " is not registered";
        return false;
    }
    auto backend = BackendRegistryInstance().GetFactory(backendId)();
    auto support = backend->GetLayerSupport(modelOptions);
    const Layer& layer = *PolymorphicDowncast<const Layer*>(&connectableLayer);
    std::vector<TensorInfo> infos;
    auto in = [&](unsigned int i) { return layer.In(i).GetConnectedOutputSlot()->GetTensorInfo(); };
    auto out = [&](unsigned int i) { return layer.Out(i).GetTensorInfo(); };
    switch (layer.GetType())
    {
        case LayerType::Convolution2d:
        case LayerType::DepthwiseConvolution2d:
        case LayerType::FullyConnected:
        {
            // {input, output, weights, biases}; an empty TensorInfo stands in for a disabled bias
            infos = {in(0), out(0), in(1)};
            infos.push_back(layer.GetNumInputSlots() > 2 ? in(2) : TensorInfo());
            // constant weights only unless the backend advertises NonConstWeights (BackendHelper.cpp:381-406)
            bool nonConstWeights = false;
            const BackendCapabilities caps = backend->GetCapabilities();
            for (size_t i = 0; i < caps.GetOptionCount(); ++i)
                if (caps.GetOption(i).GetName() == "NonConstWeights" && caps.GetOption(i).GetValue().IsBool())
                    nonConstWeights = caps.GetOption(i).GetValue().AsBool();
            if (!nonConstWeights && (!infos[2].IsConstant() || (layer.GetNumInputSlots() > 2 && !infos[3].IsConstant())))
            {
                outReasonIfUnsupported = "Backend is not capable of supporting dynamic weights (NonConstWeights) and weights/bias are set as dynamic (non constant).";
                return false;
            }
            break;
        }
        case LayerType::ElementwiseBinary: infos = {in(0), in(1), out(0)}; break;
        case LayerType::Input: infos = {out(0)}; break;
        case LayerType::Output: infos = {in(0)}; break;
        case LayerType::Constant: infos = {out(0)}; break;
        default: infos = {in(0), out(0)}; break;
    }
    return support->IsLayerSupported(layer.GetType(), infos, layer.GetParameters(), EmptyOptional(), EmptyOptional(), reason);
}

// ---- OptimizationViews (backendsCommon/OptimizationViews.cpp:11-75) ---------------------------------------------
OptimizationViews::OptimizationViews(const NetworkOptions& networkOptions) : m_INetwork(INetwork::Create(networkOptions)) {}
void OptimizationViews::AddSubstitution(SubstitutionPair&& substitution) { m_SuccesfulOptimizations.emplace_back(std::move(substitution)); }
void OptimizationViews::AddFailedSubgraph(SubgraphView&& subgraph) { m_FailedOptimizations.emplace_back(std::move(subgraph)); }
void OptimizationViews::AddUntouchedSubgraph(SubgraphView&& subgraph) { m_UntouchedSubgraphs.emplace_back(std::move(subgraph)); }
void OptimizationViews::AddDeletedSubgraph(SubgraphView&& subgraph) { m_DeletedSubgraphs.emplace_back(std::move(subgraph)); }
OptimizationViews::Substitutions& OptimizationViews::GetSubstitutions() { return m_SuccesfulOptimizations; }
const OptimizationViews::Substitutions& OptimizationViews::GetSubstitutions() const { return m_SuccesfulOptimizations; }
const OptimizationViews::Subgraphs& OptimizationViews::GetFailedSubgraphs() const { return m_FailedOptimizations; }
const OptimizationViews::Subgraphs& OptimizationViews::GetUntouchedSubgraphs() const { return m_UntouchedSubgraphs; }
const OptimizationViews::Subgraphs& OptimizationViews::GetDeletedSubgraphs() const { return m_DeletedSubgraphs; }
INetwork* OptimizationViews::GetINetwork() { return m_INetwork.get(); }
INetwork& OptimizationViews::GetINetworkRef() { return *m_INetwork; }

bool OptimizationViews::Validate(const SubgraphView& original) const
{
    std::multiset<const IConnectableLayer*> seen;
    auto add = [&](const SubgraphView& v) { for (auto* l : v.GetIConnectableLayers()) seen.insert(l); };
    for (const auto& s : m_SuccesfulOptimizations)
    {
        if (s.m_SubstitutableSubgraph.GetNumInputSlots() != s.m_ReplacementSubgraph.GetNumInputSlots() ||
            s.m_SubstitutableSubgraph.GetNumOutputSlots() != s.m_ReplacementSubgraph.GetNumOutputSlots())
            return false;
        add(s.m_SubstitutableSubgraph);
    }
    for (const auto& v : m_FailedOptimizations) add(v);
    for (const auto& v : m_UntouchedSubgraphs) add(v);
    for (const auto& v : m_DeletedSubgraphs) add(v);
    if (seen.size() != original.GetIConnectableLayers().size()) return false;
    for (auto* l : original.GetIConnectableLayers())
        if (seen.count(l) != 1) return false;
    return true;
}

// default: nothing to optimise, the whole view is untouched (backendsCommon/IBackendInternal.cpp:106-118)
OptimizationViews IBackendInternal::OptimizeSubgraphView(const SubgraphView& subgraph) const
{
    OptimizationViews result;
    result.AddUntouchedSubgraph(SubgraphView(subgraph));
    return result;
}

// ---- dynamic backends (backendsCommon/DynamicBackendUtils.cpp, DynamicBackend.cpp) ------------------------------
std::vector<std::string> DynamicBackendUtils::GetSharedObjects(const std::string& path)
{
    std::vector<std::string> out;
    if (path.empty()) return out;
    DIR* dir = opendir(path.c_str());
    if (!dir) return out;
    const std::regex pattern("^[a-zA-Z0-9]+_[a-zA-Z0-9]+_backend.so(\\.[0-9]+)*$");
    while (dirent* e = readdir(dir))
        if (std::regex_match(std::string(e->d_name), pattern)) out.push_back(path + "/" + e->d_name);
    closedir(dir);
    std::sort(out.begin(), out.end());
    return out;
}

bool DynamicBackendUtils::IsBackendCompatible(const BackendVersion& v)
{
    const BackendVersion api = IBackendInternal::GetApiVersion();
    return v.m_Major == api.m_Major && v.m_Minor <= api.m_Minor;
}

BackendIdSet DynamicBackendUtils::RegisterDynamicBackends(const std::vector<std::string>& sharedObjects)
{
    BackendIdSet registered;
    for (const std::string& so : sharedObjects)
    {
        void* handle = dlopen(so.c_str(), RTLD_LAZY | RTLD_GLOBAL);
        if (!handle) continue;
        using IdFn = const char* (*)();
        using VersionFn = void (*)(uint32_t*, uint32_t*);
        using FactoryFn = void* (*)();
        auto idFn = reinterpret_cast<IdFn>(dlsym(handle, "GetBackendId"));
        auto versionFn = reinterpret_cast<VersionFn>(dlsym(handle, "GetVersion"));
        auto factoryFn = reinterpret_cast<FactoryFn>(dlsym(handle, "BackendFactory"));
        if (!idFn || !versionFn || !factoryFn) { dlclose(handle); continue; }
        BackendVersion v;
        versionFn(&v.m_Major, &v.m_Minor);
        if (!IsBackendCompatible(v)) { dlclose(handle); continue; }
        const BackendId id(idFn());
        if (BackendRegistryInstance().IsBackendRegistered(id)) continue;   // first one wins; keep the object loaded
        BackendRegistryInstance().Register(id, [factoryFn]() {
            return IBackendInternalUniquePtr(static_cast<IBackendInternal*>(factoryFn()));
        });
        registered.insert(id);
    }
    return registered;
}
} // namespace armnn
