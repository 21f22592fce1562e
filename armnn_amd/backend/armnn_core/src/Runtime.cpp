// Minimal host core: IRuntime -- backend discovery, LoadNetwork (tensor handles, workloads, constants), and
// EnqueueWorkload (src/armnn/Runtime.cpp:301-574, src/armnn/LoadedNetwork.cpp:82-360 and :845-1100).
#include <algorithm>
#include <atomic>
#include <Layer.hpp>
#include <Profiling.hpp>
#include <armnn/BackendRegistry.hpp>
#include <armnn/IRuntime.hpp>
#include <armnn/Utils.hpp>
#include <armnn/backends/DynamicBackend.hpp>
#include <armnn/backends/IBackendInternal.hpp>
#include <backendsCommon/TensorHandleFactoryRegistry.hpp>
#include <armnn/backends/WorkloadFactory.hpp>

#include <cstring>
#include <iostream>
#include <map>
#include <mutex>

namespace armnn
{
namespace
{
std::atomic<int> g_LogThreshold{static_cast<int>(LogSeverity::Warning)};
std::atomic<bool> g_LogToStdout{false};
} // namespace

void ConfigureLogging(bool printToStandardOutput, bool, LogSeverity severity)
{
    g_LogToStdout.store(printToStandardOutput);
    g_LogThreshold.store(static_cast<int>(severity));
}
bool LogsAt(LogSeverity severity) { return static_cast<int>(severity) >= g_LogThreshold.load(); }
bool LogsToStandardOutput() { return g_LogToStdout.load(); }

namespace
{
std::ostream& LogStream() { return LogsToStandardOutput() ? std::cout : std::cerr; }

class DeviceSpec final : public IDeviceSpec
{
public:
    const BackendIdSet& GetSupportedBackends() const override { return m_Supported; }
    BackendIdSet m_Supported;
    BackendIdSet m_Dynamic;
};

struct BackendSlot
{
    IBackendInternalUniquePtr backend;
    IBackendInternal::IWorkloadFactoryPtr factory;
    ITensorHandleFactory* handleFactory = nullptr;   // preferred tensor handle factory, null: use the workload factory
    bool external = false;                           // the runtime, not the backend, places this backend's tensors in memory
};

bool HasMatchingCapability(const BackendOptions::BackendOption& wanted, const BackendCapabilities& capabilities)
{
    for (size_t i = 0; i < capabilities.GetOptionCount(); ++i)
    {
        const auto& have = capabilities.GetOption(i);
        if (have.GetName() != wanted.GetName()) continue;
        if (wanted.GetValue().IsBool() && have.GetValue().IsBool()) return wanted.GetValue().AsBool() == have.GetValue().AsBool();
        return false;
    }
    return false;
}

// every block a bin of its own, at offset 0 (ConstantMemoryStrategy,
// src/backends/backendsCommon/memoryOptimizerStrategyLibrary/strategies/ConstantMemoryStrategy.cpp:22-38)
class ConstantMemoryStrategy final : public IMemoryOptimizerStrategy
{
public:
    std::string GetName() const override { return "ConstantMemoryStrategy"; }
    MemBlockStrategyType GetMemBlockStrategyType() const override { return MemBlockStrategyType::SingleAxisPacking; }
    std::vector<MemBin> Optimize(std::vector<MemBlock>& blocks) override
    {
        std::vector<MemBin> bins;
        for (MemBlock& b : blocks)
        {
            b.m_Offset = 0;
            MemBin bin;
            bin.m_MemSize = b.m_MemSize;
            bin.m_MemBlocks.push_back(b);
            bins.push_back(std::move(bin));
        }
        return bins;
    }
};

// the buffers of a memory plan and the tensors placed in them (src/backends/backendsCommon/MemoryManager.hpp:13-70)
struct PlannedTensor
{
    ITensorHandle* handle = nullptr;
    size_t offset = 0;
};
struct PlannedBuffer
{
    std::shared_ptr<ICustomAllocator> allocator;
    size_t bytes = 0;
    void* memory = nullptr;
    std::vector<PlannedTensor> tensors;
};

// makes a profiler the calling thread's current one for a scope
class CurrentProfiler
{
public:
    explicit CurrentProfiler(IProfiler* profiler) : m_Previous(ProfilerManager::GetInstance().GetProfiler()) { ProfilerManager::GetInstance().RegisterProfiler(profiler); }
    ~CurrentProfiler() { ProfilerManager::GetInstance().RegisterProfiler(m_Previous); }
private:
    IProfiler* m_Previous;
};

class LoadedNetwork
{
public:
    LoadedNetwork(IOptimizedNetworkPtr net, const INetworkProperties& properties) : m_Net(std::move(net)), m_Profiler(std::make_shared<IProfiler>())
    {
        const bool profilingEnabled = properties.m_ProfilingEnabled;
        // the network's profiler is the thread's current one while its workloads are built and run
        // (LoadedNetwork.cpp:131-136, :845-852)
        m_Profiler->EnableProfiling(profilingEnabled);
        CurrentProfiler current(m_Profiler.get());
        Graph& graph = m_Net->GetGraph();
        m_Order = graph.TopologicalSort();

        // one backend object, handle factory and workload factory per backend in use (LoadedNetwork.cpp:169-260)
        for (Layer* l : m_Order)
        {
            const BackendId& id = l->GetBackendId();
            if (m_Backends.count(id)) continue;
            BackendSlot slot;
            slot.backend = BackendRegistryInstance().GetFactory(id)();
            if (slot.backend->SupportsTensorAllocatorAPI())
            {
                // the backend registers its tensor handle factories from CreateWorkloadFactory (LoadedNetwork.cpp:265-272
                // calls nothing else)
                slot.factory = slot.backend->CreateWorkloadFactory(m_Registry, m_Net->GetModelOptions());
                slot.handleFactory = m_Registry.GetFactory(slot.backend->GetHandleFactoryPreferences().front());
            }
            else
            {
                IBackendInternal::IMemoryManagerSharedPtr mm = slot.backend->CreateMemoryManager();
                if (mm) m_Registry.RegisterMemoryManager(mm);
                slot.factory = slot.backend->CreateWorkloadFactory(mm, m_Net->GetModelOptions());
            }
            if (!slot.factory) throw RuntimeException("backend " + id.Get() + " returned no workload factory");
            // LoadedNetwork.cpp:252-262
            slot.external = properties.m_ExternalMemoryManagementEnabled &&
                            HasMatchingCapability(BackendOptions::BackendOption{"ExternallyManagedMemory", true}, slot.backend->GetCapabilities());
            m_Backends.emplace(id, std::move(slot));
        }

        // Tensor handles in execution order.  Manage() opens a tensor's lifetime when its producer is reached and
        // Allocate() closes it after its last consumer, so a pooling memory manager can overlap tensors whose
        // lifetimes do not (LoadedNetwork.cpp:262-330, Layer::CreateTensorHandles, Graph::AllocateDynamicBuffers).  The
        // output of a Constant layer is created like the others but gets memory that lasts by an Allocate() without a
        // lifetime (Graph.cpp:237-252).  Where the runtime plans the memory itself, the backend's tensors are created
        // unmanaged, their lifetimes go into a memory profile (LoadedNetwork.cpp:1596-1718) and each is handed its place
        // before the first inference.
        std::map<const OutputSlot*, unsigned int> remaining;
        std::map<const OutputSlot*, size_t> blockOf;              // external tensors: index into `profile`
        struct Lifetime { BackendId backend; ITensorHandle* handle; unsigned int start, end; size_t bytes; };
        std::vector<Lifetime> profile;
        unsigned int timestep = 0;
        for (Layer* l : m_Order)
        {
            BackendSlot& slot = m_Backends.at(l->GetBackendId());
            const bool constant = l->GetType() == LayerType::Constant;
            const bool external = slot.external && !constant;
            const bool managed = !external;
            for (unsigned int o = 0; o < l->GetNumOutputSlots(); ++o)
            {
                OutputSlot& out = l->Out(o);
                std::unique_ptr<ITensorHandle> h = slot.handleFactory ? slot.handleFactory->CreateTensorHandle(out.GetTensorInfo(), managed)
                                                                      : slot.factory->CreateTensorHandle(out.GetTensorInfo(), managed);
                if (!h) throw RuntimeException(std::string("no tensor handle for layer ") + l->GetName());
                if (constant)
                {
                    h->Allocate();
                    out.SetTensorHandle(std::move(h));
                    remaining[&out] = ~0u;
                    continue;
                }
                if (external)
                {
                    const size_t bytes = (out.GetTensorInfo().GetNumBytes() + 3) / 4 * 4;
                    blockOf[&out] = profile.size();
                    profile.push_back(Lifetime{l->GetBackendId(), h.get(), timestep, timestep, bytes});
                    out.SetTensorHandle(std::move(h));
                    remaining[&out] = ~0u;
                    continue;
                }
                // a tensor read by a network output must survive until the caller has copied it out
                bool pinned = !managed;
                for (InputSlot* c : out.GetConnections()) pinned |= c->GetOwningLayer().GetType() == LayerType::Output;
                if (managed) h->Manage();
                out.SetTensorHandle(std::move(h));
                remaining[&out] = pinned ? ~0u : out.GetNumConnections();
                if (!managed || out.GetNumConnections() == 0 || pinned) m_AllocateLast.push_back(out.GetTensorHandle());
            }
            CreateWorkloadFor(*l, slot);
            for (unsigned int i = 0; i < l->GetNumInputSlots(); ++i)
            {
                const OutputSlot* src = l->In(i).GetConnectedOutputSlot();
                auto ext = blockOf.find(src);
                // alive until its last consumer; what a network output reads, until the caller has copied it out
                if (ext != blockOf.end())
                    profile[ext->second].end = l->GetType() == LayerType::Output ? static_cast<unsigned int>(m_Order.size()) : std::max(profile[ext->second].end, timestep);
                unsigned int& r = remaining[src];
                if (r != ~0u && --r == 0) src->GetTensorHandle()->Allocate();
            }
            ++timestep;
        }
        for (ITensorHandle* h : m_AllocateLast) h->Allocate();
        m_AllocateLast.clear();

        // the memory plan: per backend, a strategy packs the blocks into bins; every bin becomes one buffer of the
        // backend's allocator (LoadedNetwork.cpp:517-541 and :1722-1764)
        {
            std::map<BackendId, std::vector<MemBlock>> blocks;
            for (size_t i = 0; i < profile.size(); ++i)
                blocks[profile[i].backend].emplace_back(profile[i].start, profile[i].end, profile[i].bytes, 0, static_cast<unsigned int>(i));
            auto strategies = BackendRegistryInstance().GetMemoryOptimizerStrategies();
            auto allocators = BackendRegistryInstance().GetAllocators();
            for (auto& perBackend : blocks)
            {
                const BackendId& id = perBackend.first;
                ConstantMemoryStrategy constantStrategy;
                IMemoryOptimizerStrategy* strategy = strategies.count(id) ? strategies[id].get() : &constantStrategy;
                std::shared_ptr<ICustomAllocator> allocator = allocators.count(id) ? allocators[id]
                                                                                   : std::shared_ptr<ICustomAllocator>(m_Backends.at(id).backend->GetDefaultAllocator());
                for (const MemBin& bin : strategy->Optimize(perBackend.second))
                {
                    PlannedBuffer buffer;
                    buffer.allocator = allocator;
                    buffer.bytes = bin.m_MemSize;
                    for (const MemBlock& b : bin.m_MemBlocks) buffer.tensors.push_back(PlannedTensor{profile.at(b.m_Index).handle, b.m_Offset});
                    m_Plan.push_back(std::move(buffer));
                }
            }
        }

        m_Registry.AquireMemory();
        for (auto& w : m_Constants) w->PostAllocationConfigure();
        for (auto& w : m_Workloads) w->PostAllocationConfigure();
        for (auto& b : m_Backends) b.second.factory->AfterWorkloadsCreated();
        // constant layers produce their output once (LoadedNetwork.cpp:342-357)
        for (auto& w : m_Constants) w->Execute();
        for (Layer* l : m_Order)
        {
            Binding b;
            b.layer = l;
            if (l->GetType() == LayerType::Input) { b.slot = &l->Out(0); m_Inputs.push_back(std::move(b)); }
            else if (l->GetType() == LayerType::Output) { b.slot = const_cast<OutputSlot*>(l->In(0).GetConnectedOutputSlot()); m_Outputs.push_back(std::move(b)); }
        }
    }

    ~LoadedNetwork()
    {
        m_Constants.clear();
        m_Workloads.clear();
        m_Registry.ReleaseMemory();
        // LoadedNetwork::FreeWorkingMemory, LoadedNetwork.cpp:1199-1225
        for (PlannedBuffer& b : m_Plan)
        {
            for (PlannedTensor& t : b.tensors) t.handle->Unimport();
            if (b.memory) b.allocator->free(b.memory);
        }
    }

    size_t GetNumPlannedBuffers() const { return m_Plan.size(); }

    const std::shared_ptr<IProfiler>& GetProfiler() const { return m_Profiler; }

    const Layer* FindBinding(LayerType type, LayerBindingId id) const
    {
        for (const Layer* l : m_Order)
            if (l->GetType() == type && l->GetBindingId() == id) return l;
        return nullptr;
    }

    TensorInfo GetInputTensorInfo(LayerBindingId id) const
    {
        const Layer* l = FindBinding(LayerType::Input, id);
        if (!l) throw InvalidArgumentException("No input layer is associated with id " + std::to_string(id));
        return l->Out(0).GetTensorInfo();
    }
    TensorInfo GetOutputTensorInfo(LayerBindingId id) const
    {
        const Layer* l = FindBinding(LayerType::Output, id);
        if (!l) throw InvalidArgumentException("No output layer is associated with id " + std::to_string(id));
        return l->In(0).GetConnectedOutputSlot()->GetTensorInfo();
    }

    Status Enqueue(const InputTensors& inputs, const OutputTensors& outputs, const std::vector<ImportedInputId>& preIn = {},
                   const std::vector<ImportedOutputId>& preOut = {})
    {
        // a tensor comes either in the list or pre-imported; together they must cover the network (LoadedNetwork.cpp:800-806)
        if (inputs.size() + preIn.size() != m_Net->GetNumInputs()) throw InvalidArgumentException("Number of inputs provided does not match network.");
        if (outputs.size() + preOut.size() != m_Net->GetNumOutputs()) throw InvalidArgumentException("Number of outputs provided does not match network.");
        std::lock_guard<std::mutex> lock(m_Mutex);
        CurrentProfiler current(m_Profiler.get());
        ARMNN_SCOPED_PROFILING_EVENT(BackendId(), "EnqueueWorkload");
        AllocateWorkingMemory();
        for (ImportedInputId id : preIn)
            if (id >= m_Inputs.size() || !m_Inputs[id].adopted) throw InvalidArgumentException("EnqueueWorkload: input " + std::to_string(id) + " was not imported");
        for (ImportedOutputId id : preOut)
            if (id >= m_Outputs.size() || !m_Outputs[id].adopted) throw InvalidArgumentException("EnqueueWorkload: output " + std::to_string(id) + " was not imported");
        // workloads read adopted memory for the ids named in this call and the network's own tensors for the rest
        for (unsigned int i = 0; i < m_Inputs.size(); ++i) Point(m_Inputs[i], std::find(preIn.begin(), preIn.end(), i) != preIn.end());
        for (unsigned int i = 0; i < m_Outputs.size(); ++i) Point(m_Outputs[i], std::find(preOut.begin(), preOut.end(), i) != preOut.end());
        for (const auto& in : inputs)
        {
            const Layer* l = FindBinding(LayerType::Input, in.first);
            if (!l) throw InvalidArgumentException("No input layer is associated with id " + std::to_string(in.first));
            const TensorInfo& info = l->Out(0).GetTensorInfo();
            if (in.second.GetNumBytes() != info.GetNumBytes()) throw InvalidArgumentException("Input tensor size does not match the network's");
            ITensorHandle* h = l->Out(0).GetTensorHandle();
            void* dst = h->Map();
            std::memcpy(dst, in.second.GetMemoryArea(), info.GetNumBytes());
            h->Unmap();
        }
        {
            ARMNN_SCOPED_PROFILING_EVENT(BackendId(), "Execute");
            // constant workloads are part of the queue that runs for every inference (LoadedNetwork.cpp:366-394): a backend
            // that wants its constants uploaded once has to see to that itself
            for (auto& w : m_Constants) w->Execute();
            for (auto& w : m_Workloads) w->Execute();
        }
        for (const auto& out : outputs)
        {
            const Layer* l = FindBinding(LayerType::Output, out.first);
            if (!l) throw InvalidArgumentException("No output layer is associated with id " + std::to_string(out.first));
            const OutputSlot* src = l->In(0).GetConnectedOutputSlot();
            if (out.second.GetNumBytes() != src->GetTensorInfo().GetNumBytes()) throw InvalidArgumentException("Output tensor size does not match the network's");
            const ITensorHandle* h = src->GetTensorHandle();
            const void* p = h->Map();
            std::memcpy(out.second.GetMemoryArea(), p, src->GetTensorInfo().GetNumBytes());
            h->Unmap();
        }
        // an adopted output is complete once its handle has been mapped: that is where a device backend waits for its
        // queue (the SyncMemGeneric workload of LoadedNetwork.cpp:905-918)
        for (ImportedOutputId id : preOut)
        {
            m_Outputs[id].imported->Map(true);
            m_Outputs[id].imported->Unmap();
        }
        return Status::Success;
    }

private:
    // the planned buffers come into being with the first inference; every tensor then adopts its place
    // (LoadedNetwork::AllocateWorkingMemory, LoadedNetwork.cpp:1162-1197)
    void AllocateWorkingMemory()
    {
        if (m_WorkingMemoryAllocated) return;
        for (PlannedBuffer& b : m_Plan)
        {
            b.memory = b.allocator->allocate(b.bytes, 0);
            for (PlannedTensor& t : b.tensors)
                t.handle->Import(b.allocator->GetMemoryRegionAtOffset(b.memory, t.offset), b.allocator->GetMemorySourceType());
        }
        m_WorkingMemoryAllocated = true;
    }

    template <typename Desc>
    void Fill(Desc& d, WorkloadInfo& info, Layer& l)
    {
        for (unsigned int i = 0; i < l.GetNumInputSlots(); ++i)
        {
            const OutputSlot* src = l.In(i).GetConnectedOutputSlot();
            d.m_Inputs.push_back(src->GetTensorHandle());
            info.m_InputTensorInfos.push_back(src->GetTensorInfo());
        }
        for (unsigned int o = 0; o < l.GetNumOutputSlots(); ++o)
        {
            d.m_Outputs.push_back(l.Out(o).GetTensorHandle());
            info.m_OutputTensorInfos.push_back(l.Out(o).GetTensorInfo());
        }
        d.m_AdditionalInfoObject = l.GetAdditionalInformation<void>().get();
        info.m_Name = l.GetNameStr();
    }

    template <typename Desc, typename Params>
    std::unique_ptr<IWorkload> Make(Layer& l, BackendSlot& slot)
    {
        Desc d;
        WorkloadInfo info;
        Fill(d, info, l);
        d.m_Parameters = static_cast<const Params&>(l.GetParameters());
        return slot.factory->CreateWorkload(l.GetType(), d, info);
    }

    void CreateWorkloadFor(Layer& l, BackendSlot& slot)
    {
        std::unique_ptr<IWorkload> w;
        switch (l.GetType())
        {
            case LayerType::Input:
            case LayerType::Output:
                return;   // the runtime itself moves data between caller memory and the bound tensor handles
            case LayerType::Constant:
            {
                ConstantQueueDescriptor d;
                WorkloadInfo info;
                Fill(d, info, l);
                d.m_LayerOutput = l.m_LayerOutput.get();
                w = slot.factory->CreateWorkload(LayerType::Constant, d, info);
                if (!w) throw RuntimeException(std::string("No workload created for layer (name: '") + l.GetName() + "' type: 'Constant')");
                m_Constants.push_back(std::move(w));
                return;
            }
            case LayerType::MemCopy:
            {
                MemCopyQueueDescriptor d;
                WorkloadInfo info;
                Fill(d, info, l);
                w = slot.factory->CreateWorkload(LayerType::MemCopy, d, info);
                break;
            }
            case LayerType::Convolution2d: w = Make<Convolution2dQueueDescriptor, Convolution2dDescriptor>(l, slot); break;
            case LayerType::DepthwiseConvolution2d: w = Make<DepthwiseConvolution2dQueueDescriptor, DepthwiseConvolution2dDescriptor>(l, slot); break;
            case LayerType::FullyConnected: w = Make<FullyConnectedQueueDescriptor, FullyConnectedDescriptor>(l, slot); break;
            case LayerType::Activation: w = Make<ActivationQueueDescriptor, ActivationDescriptor>(l, slot); break;
            case LayerType::Pooling2d: w = Make<Pooling2dQueueDescriptor, Pooling2dDescriptor>(l, slot); break;
            case LayerType::Mean: w = Make<MeanQueueDescriptor, MeanDescriptor>(l, slot); break;
            case LayerType::Pad: w = Make<PadQueueDescriptor, PadDescriptor>(l, slot); break;
            case LayerType::Softmax: w = Make<SoftmaxQueueDescriptor, SoftmaxDescriptor>(l, slot); break;
            case LayerType::ElementwiseBinary: w = Make<ElementwiseBinaryQueueDescriptor, ElementwiseBinaryDescriptor>(l, slot); break;
            case LayerType::Reshape: w = Make<ReshapeQueueDescriptor, ReshapeDescriptor>(l, slot); break;
        }
        if (!w)
            throw RuntimeException(std::string("No workload created for layer (name: '") + l.GetName() + "' type: '" +
                                   GetLayerTypeAsCString(l.GetType()) + "' backend: '" + l.GetBackendId().Get() + "')");
        m_WorkloadOf[&l] = m_Workloads.size();
        m_Workloads.push_back(std::move(w));
    }

    // ---- pre-imported inputs and outputs (LoadedNetwork.cpp:1402-1560 and :796-960) ---------------------------------
    struct Binding
    {
        Layer* layer = nullptr;                               // the Input / Output layer
        OutputSlot* slot = nullptr;                           // the tensor it binds
        std::unique_ptr<ITensorHandle> imported;              // handle that adopts caller memory (created on first use)
        bool adopted = false;                                 // Import() succeeded and has not been cleared
        bool inUse = false;                                   // the workloads currently point at `imported`
    };

    // workloads (with the slot index) that read / write `slot`
    std::vector<std::pair<IWorkload*, unsigned int>> Readers(const OutputSlot& slot) const
    {
        std::vector<std::pair<IWorkload*, unsigned int>> r;
        for (InputSlot* c : slot.GetConnections())
        {
            auto it = m_WorkloadOf.find(&c->GetOwningLayer());
            if (it != m_WorkloadOf.end()) r.emplace_back(m_Workloads[it->second].get(), c->GetSlotIndex());
        }
        return r;
    }
    std::pair<IWorkload*, unsigned int> Writer(const OutputSlot& slot) const
    {
        auto it = m_WorkloadOf.find(&slot.GetOwningLayer());
        if (it == m_WorkloadOf.end()) return {nullptr, 0u};
        return {m_Workloads[it->second].get(), slot.CalculateIndexOnOwner()};
    }

    void Point(Binding& b, bool toImported)
    {
        if (b.inUse == toImported) return;
        ITensorHandle* h = toImported ? b.imported.get() : b.slot->GetTensorHandle();
        if (b.layer->GetType() == LayerType::Output)
        {
            const auto w = Writer(*b.slot);
            if (w.first) w.first->ReplaceOutputTensorHandle(h, w.second);
        }
        for (const auto& r : Readers(*b.slot)) r.first->ReplaceInputTensorHandle(h, r.second);
        b.inUse = toImported;
    }

    bool TryImport(Binding& b, void* memory, MemorySource source)
    {
        // the tensor must be produced and consumed by workloads that accept another handle
        const bool isOutput = b.layer->GetType() == LayerType::Output;
        if (isOutput)
        {
            const auto w = Writer(*b.slot);
            if (!w.first || !w.first->SupportsTensorHandleReplacement()) return false;
        }
        for (const auto& r : Readers(*b.slot))
            if (!r.first->SupportsTensorHandleReplacement()) return false;
        if (!b.imported)
        {
            const Layer& owner = isOutput ? b.slot->GetOwningLayer() : b.slot->GetConnections().empty() ? *b.layer : b.slot->GetConnections().front()->GetOwningLayer();
            BackendSlot& bs = m_Backends.at(owner.GetBackendId());
            if (!bs.handleFactory) return false;
            // the factory the backend paired with its copying factory for imports (LoadedNetwork.cpp:433-447)
            ITensorHandleFactory* importFactory = m_Registry.GetFactory(m_Registry.GetMatchingImportFactoryId(bs.handleFactory->GetId()));
            if (!importFactory || (importFactory->GetImportFlags() & static_cast<MemorySourceFlags>(source)) == 0) return false;
            b.imported = importFactory->CreateTensorHandle(b.slot->GetTensorInfo(), false);
            if (!b.imported) return false;
        }
        try
        {
            if (b.adopted) { Point(b, false); b.imported->Unimport(); b.adopted = false; }
            if (b.imported->CanBeImported(memory, source) && b.imported->Import(memory, source)) b.adopted = true;
        }
        catch (const MemoryImportException& e)
        {
            if (LogsAt(LogSeverity::Error)) LogStream() << "armnn: an error occurred attempting to import a tensor: " << e.what() << "\n";
        }
        return b.adopted;
    }

public:
    std::vector<ImportedInputId> ImportInputs(const InputTensors& inputs, MemorySource source)
    {
        if (source == MemorySource::Undefined) throw MemoryImportException("ImportInputs: Memory Import failed, no memory source given");
        if (inputs.size() > m_Inputs.size()) throw MemoryImportException("ImportInputs: The number of tensors provided exceeds the number of inputs.");
        std::lock_guard<std::mutex> lock(m_Mutex);
        std::vector<ImportedInputId> ids;
        for (unsigned int i = 0; i < m_Inputs.size(); ++i)
            for (const auto& t : inputs)
                if (t.first == m_Inputs[i].layer->GetBindingId() && t.second.GetNumBytes() == m_Inputs[i].slot->GetTensorInfo().GetNumBytes() &&
                    TryImport(m_Inputs[i], const_cast<void*>(t.second.GetMemoryArea()), source))
                    ids.push_back(i);
        return ids;
    }

    std::vector<ImportedOutputId> ImportOutputs(const OutputTensors& outputs, MemorySource source)
    {
        if (source == MemorySource::Undefined) throw MemoryImportException("ImportOutputs: Memory Import failed, no memory source given");
        if (outputs.size() > m_Outputs.size()) throw MemoryImportException("ImportOutputs: The number of tensors provided exceeds the number of outputs.");
        std::lock_guard<std::mutex> lock(m_Mutex);
        std::vector<ImportedOutputId> ids;
        for (unsigned int i = 0; i < m_Outputs.size(); ++i)
            for (const auto& t : outputs)
                if (t.first == m_Outputs[i].layer->GetBindingId() && t.second.GetNumBytes() == m_Outputs[i].slot->GetTensorInfo().GetNumBytes() &&
                    TryImport(m_Outputs[i], t.second.GetMemoryArea(), source))
                    ids.push_back(i);
        return ids;
    }

    void ClearImported(bool inputs, const std::vector<unsigned int>& ids)
    {
        std::lock_guard<std::mutex> lock(m_Mutex);
        std::vector<Binding>& all = inputs ? m_Inputs : m_Outputs;
        for (unsigned int id : ids)
        {
            if (id >= all.size() || !all[id].adopted) throw InvalidArgumentException("ClearImported: id " + std::to_string(id) + " is not an imported tensor");
            Point(all[id], false);
            all[id].imported->Unimport();
            all[id].adopted = false;
        }
    }

private:
    std::vector<Binding> m_Inputs, m_Outputs;                 // in the order of the network's Input / Output layers
    std::map<const Layer*, size_t> m_WorkloadOf;

    IOptimizedNetworkPtr m_Net;
    std::shared_ptr<IProfiler> m_Profiler;
    std::vector<Layer*> m_Order;
    TensorHandleFactoryRegistry m_Registry;
    std::map<BackendId, BackendSlot> m_Backends;
    std::vector<std::unique_ptr<IWorkload>> m_Constants;
    std::vector<std::unique_ptr<IWorkload>> m_Workloads;
    std::vector<ITensorHandle*> m_AllocateLast;
    std::vector<PlannedBuffer> m_Plan;
    bool m_WorkingMemoryAllocated = false;
    std::mutex m_Mutex;
};
} // namespace

class RuntimeImpl
{
public:
    explicit RuntimeImpl(const IRuntime::CreationOptions& options)
    {
        // dynamic backends first, so they are part of the registry scan (Runtime.cpp:655-676)
        if (!options.m_DynamicBackendsPath.empty())
            m_DeviceSpec.m_Dynamic = DynamicBackendUtils::RegisterDynamicBackends(DynamicBackendUtils::GetSharedObjects(options.m_DynamicBackendsPath));
        // a backend whose context cannot be created is not offered to Optimize (Runtime.cpp:377-470)
        for (const BackendId& id : BackendRegistryInstance().GetBackendIds())
        {
            try
            {
                auto backend = BackendRegistryInstance().GetFactory(id)();
                auto context = backend->CreateBackendContext(options);
                // a backend that cannot work with the allocator the caller chose for it is not used (Runtime.cpp:395-413)
                auto allocator = options.m_CustomAllocatorMap.find(id);
                if (allocator != options.m_CustomAllocatorMap.end())
                {
                    if (!allocator->second) throw Exception("Allocator associated with id " + id.Get() + " is null");
                    std::string err;
                    if (!backend->UseCustomMemoryAllocator(allocator->second, err))
                    {
                        if (LogsAt(LogSeverity::Warning)) LogStream() << "armnn: the backend " << id << " reported an error when trying to use the provided custom allocator."
                                  << " Backend won't be used. ErrorMsg: " << err << "\n";
                        continue;
                    }
                    BackendRegistryInstance().RegisterAllocator(id, allocator->second);
                    m_AllocatorsAdded.insert(id);
                }
                auto strategy = options.m_MemoryOptimizerStrategyMap.find(id);
                if (strategy != options.m_MemoryOptimizerStrategyMap.end() && strategy->second)
                {
                    BackendRegistryInstance().RegisterMemoryOptimizerStrategy(id, strategy->second);
                    m_StrategiesAdded.insert(id);
                }
                if (context) m_Contexts.emplace(id, std::move(context));
                m_DeviceSpec.m_Supported.insert(id);
            }
            catch (const BackendUnavailableException& e)
            {
                if (LogsAt(LogSeverity::Warning)) LogStream() << "armnn: backend " << id << " is unavailable and ignored: " << e.what() << "\n";
            }
        }
    }

    ~RuntimeImpl()
    {
        m_Networks.clear();
        m_Contexts.clear();
        for (const BackendId& id : m_AllocatorsAdded) BackendRegistryInstance().DeregisterAllocator(id);
        for (const BackendId& id : m_StrategiesAdded) BackendRegistryInstance().DeregisterMemoryOptimizerStrategy(id);
        for (const BackendId& id : m_DeviceSpec.m_Dynamic) BackendRegistryInstance().Deregister(id);
    }

    Status LoadNetwork(NetworkId& idOut, IOptimizedNetworkPtr network, std::string& error,
                       const INetworkProperties& properties = INetworkProperties(MemorySource::Undefined, MemorySource::Undefined))
    {
        NetworkId id;
        {
            std::lock_guard<std::mutex> lock(m_NetworksMutex);
            id = m_NextId++;
        }
        idOut = id;
        for (auto& c : m_Contexts) c.second->BeforeLoadNetwork(id);
        std::unique_ptr<LoadedNetwork> loaded;
        try
        {
            // built outside the lock (plans are created and constants uploaded here); only the map is guarded, as
            // RuntimeImpl::LoadNetwork does with m_Mutex (src/armnn/Runtime.cpp:153-200)
            loaded = std::make_unique<LoadedNetwork>(std::move(network), properties);
        }
        catch (const Exception& e)
        {
            error = e.what();
            return Status::Failure;
        }
        {
            std::lock_guard<std::mutex> lock(m_NetworksMutex);
            m_Networks[id] = std::move(loaded);
        }
        for (auto& c : m_Contexts) c.second->AfterLoadNetwork(id);
        return Status::Success;
    }

    LoadedNetwork& Get(NetworkId id) const
    {
        std::lock_guard<std::mutex> lock(m_NetworksMutex);
        auto it = m_Networks.find(id);
        if (it == m_Networks.end()) throw InvalidArgumentException("Unknown network id " + std::to_string(id));
        return *it->second;
    }

    Status Enqueue(NetworkId id, const InputTensors& in, const OutputTensors& out, const std::vector<ImportedInputId>& preIn = {},
                   const std::vector<ImportedOutputId>& preOut = {})
    {
        LoadedNetwork& net = Get(id);
        Status s = Status::Failure;
        try
        {
            s = net.Enqueue(in, out, preIn, preOut);
        }
        catch (const RuntimeException& e)
        {
            // a failing workload ends the inference, not the process (LoadedNetwork.cpp:1088-1100)
            if (LogsAt(LogSeverity::Error)) LogStream() << "armnn: an error occurred attempting to execute a workload: " << e.what() << "\n";
            return Status::Failure;
        }
        for (auto& c : m_Contexts) c.second->AfterEnqueueWorkload(id);
        return s;
    }

    Status Unload(NetworkId id)
    {
        for (auto& c : m_Contexts) c.second->BeforeUnloadNetwork(id);
        std::unique_ptr<LoadedNetwork> gone;
        {
            std::lock_guard<std::mutex> lock(m_NetworksMutex);
            auto it = m_Networks.find(id);
            if (it != m_Networks.end())
            {
                gone = std::move(it->second);
                m_Networks.erase(it);
            }
        }
        const bool erased = gone != nullptr;
        gone.reset();                           // the network's memory is released outside the lock
        for (auto& c : m_Contexts) c.second->AfterUnloadNetwork(id);
        return erased ? Status::Success : Status::Failure;
    }

    DeviceSpec m_DeviceSpec;
private:
    std::map<BackendId, IBackendInternal::IBackendContextPtr> m_Contexts;
    std::map<NetworkId, std::unique_ptr<LoadedNetwork>> m_Networks;
    mutable std::mutex m_NetworksMutex;         // guards m_Networks and m_NextId: networks may be loaded, run and unloaded from several threads
    BackendIdSet m_AllocatorsAdded, m_StrategiesAdded;
    NetworkId m_NextId = 0;
};

IRuntime::IRuntime(const CreationOptions& options) : pRuntimeImpl(new RuntimeImpl(options)) {}
IRuntime::~IRuntime() = default;
IRuntime* IRuntime::CreateRaw(const CreationOptions& options) { return new IRuntime(options); }
IRuntimePtr IRuntime::Create(const CreationOptions& options) { return IRuntimePtr(CreateRaw(options), &IRuntime::Destroy); }
void IRuntime::Destroy(IRuntime* runtime) { delete runtime; }
Status IRuntime::LoadNetwork(NetworkId& id, IOptimizedNetworkPtr network)
{
    std::string ignored;
    return pRuntimeImpl->LoadNetwork(id, std::move(network), ignored);
}
Status IRuntime::LoadNetwork(NetworkId& id, IOptimizedNetworkPtr network, std::string& error) { return pRuntimeImpl->LoadNetwork(id, std::move(network), error); }
Status IRuntime::LoadNetwork(NetworkId& id, IOptimizedNetworkPtr network, std::string& error, const INetworkProperties& properties)
{
    return pRuntimeImpl->LoadNetwork(id, std::move(network), error, properties);
}
const std::shared_ptr<IProfiler> IRuntime::GetProfiler(NetworkId id) const { return pRuntimeImpl->Get(id).GetProfiler(); }
TensorInfo IRuntime::GetInputTensorInfo(NetworkId id, LayerBindingId layerId) const { return pRuntimeImpl->Get(id).GetInputTensorInfo(layerId); }
TensorInfo IRuntime::GetOutputTensorInfo(NetworkId id, LayerBindingId layerId) const { return pRuntimeImpl->Get(id).GetOutputTensorInfo(layerId); }
Status IRuntime::EnqueueWorkload(NetworkId id, const InputTensors& in, const OutputTensors& out, std::vector<ImportedInputId> preIn,
                                 std::vector<ImportedOutputId> preOut)
{
    return pRuntimeImpl->Enqueue(id, in, out, preIn, preOut);
}
std::vector<ImportedInputId> IRuntime::ImportInputs(NetworkId id, const InputTensors& in, MemorySource source) { return pRuntimeImpl->Get(id).ImportInputs(in, source); }
std::vector<ImportedOutputId> IRuntime::ImportOutputs(NetworkId id, const OutputTensors& out, MemorySource source) { return pRuntimeImpl->Get(id).ImportOutputs(out, source); }
void IRuntime::ClearImportedInputs(NetworkId id, const std::vector<ImportedInputId> ids) { pRuntimeImpl->Get(id).ClearImported(true, ids); }
void IRuntime::ClearImportedOutputs(NetworkId id, const std::vector<ImportedOutputId> ids) { pRuntimeImpl->Get(id).ClearImported(false, ids); }
Status IRuntime::UnloadNetwork(NetworkId id) { return pRuntimeImpl->Unload(id); }
const IDeviceSpec& IRuntime::GetDeviceSpec() const { return pRuntimeImpl->m_DeviceSpec; }
} // namespace armnn
