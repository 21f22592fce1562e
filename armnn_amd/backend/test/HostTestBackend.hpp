// "TestHost": a second backend for tests of fallback and of copies between backends.  It keeps tensors in host
// memory and implements only what those tests need -- Input, Output, MemCopy, Constant, and Activation(Linear) with
// a = 1, b = 0 on equally quantized tensors, which is a byte copy.  Test infrastructure; it ships in no library.
#pragma once
#include <armnn/BackendRegistry.hpp>
#include <armnn/backends/IBackendInternal.hpp>
#include <armnn/backends/MemCopyWorkload.hpp>
#include <armnn/backends/TensorHandle.hpp>
#include <armnn/backends/Workload.hpp>
#include <armnn/utility/PolymorphicDowncast.hpp>

#include <cstring>
#include <vector>

namespace testhost
{
using namespace armnn;

inline const BackendId& Id() { static const BackendId id("TestHost"); return id; }

class HostHandle : public ITensorHandle
{
public:
    explicit HostHandle(const TensorInfo& info) : m_Info(info) {}
    void Manage() override {}
    void Allocate() override { m_Data.resize(m_Info.GetNumBytes()); }
    ITensorHandle* GetParent() const override { return nullptr; }
    const void* Map(bool) const override
    {
        if (m_Adopted) return m_Adopted;
        if (m_Data.empty()) m_Data.resize(m_Info.GetNumBytes());
        return m_Data.data();
    }
    unsigned int GetImportFlags() const override { return static_cast<unsigned int>(MemorySource::Malloc); }
    bool CanBeImported(void* memory, MemorySource source) override { return memory && source == MemorySource::Malloc; }
    bool Import(void* memory, MemorySource source) override { if (!CanBeImported(memory, source)) return false; m_Adopted = memory; return true; }
    void Unimport() override { m_Adopted = nullptr; }
    void* Adopted() const { return m_Adopted; }
    void Unmap() const override {}
    TensorShape GetStrides() const override { return GetUnpaddedTensorStrides(m_Info); }
    TensorShape GetShape() const override { return m_Info.GetShape(); }
    void CopyOutTo(void* memory) const override { std::memcpy(memory, Map(true), m_Info.GetNumBytes()); }
    void CopyInFrom(const void* memory) override { std::memcpy(const_cast<void*>(Map(true)), memory, m_Info.GetNumBytes()); }
private:
    TensorInfo m_Info;
    mutable std::vector<unsigned char> m_Data;
    void* m_Adopted = nullptr;
};

class CopyActivationWorkload : public BaseWorkload<ActivationQueueDescriptor>
{
public:
    CopyActivationWorkload(const ActivationQueueDescriptor& d, const WorkloadInfo& info) : BaseWorkload<ActivationQueueDescriptor>(d, info), m_Bytes(info.m_InputTensorInfos[0].GetNumBytes()) {}
    void Execute() const override
    {
        const void* s = m_Data.m_Inputs[0]->Map(true);
        void* d = m_Data.m_Outputs[0]->Map(true);
        std::memcpy(d, s, m_Bytes);
        m_Data.m_Inputs[0]->Unmap();
        m_Data.m_Outputs[0]->Unmap();
        ++Executions();
    }
    static int& Executions() { static int n = 0; return n; }
private:
    size_t m_Bytes;
};

class ConstantWorkload : public BaseWorkload<ConstantQueueDescriptor>
{
public:
    using BaseWorkload<ConstantQueueDescriptor>::BaseWorkload;
    void Execute() const override { m_Data.m_Outputs[0]->CopyInFrom(m_Data.m_LayerOutput->Map(true)); }
};

class Factory : public IWorkloadFactory
{
public:
    const BackendId& GetBackendId() const override { return Id(); }
    bool SupportsSubTensors() const override { return false; }
    std::unique_ptr<ITensorHandle> CreateSubTensorHandle(ITensorHandle&, TensorShape const&, unsigned int const*) const override { return nullptr; }
    std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& info, const bool) const override { return std::make_unique<HostHandle>(info); }
    std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& info, DataLayout, const bool) const override { return std::make_unique<HostHandle>(info); }
    std::unique_ptr<IWorkload> CreateWorkload(LayerType type, const QueueDescriptor& d, const WorkloadInfo& info) const override
    {
        switch (type)
        {
            case LayerType::Activation: return std::make_unique<CopyActivationWorkload>(*PolymorphicDowncast<const ActivationQueueDescriptor*>(&d), info);
            case LayerType::Constant: return std::make_unique<ConstantWorkload>(*PolymorphicDowncast<const ConstantQueueDescriptor*>(&d), info);
            case LayerType::MemCopy: case LayerType::Input: case LayerType::Output:
                return std::make_unique<CopyMemGenericWorkload>(*PolymorphicDowncast<const MemCopyQueueDescriptor*>(&d), info);
            default: return nullptr;
        }
    }
};

class Support : public ILayerSupport
{
public:
    bool IsLayerSupported(const LayerType& type, const std::vector<TensorInfo>& infos, const BaseDescriptor& descriptor,
                          const Optional<LstmInputParamsInfo>&, const Optional<QuantizedLstmInputParamsInfo>&,
                          Optional<std::string&> reason) const override
    {
        switch (type)
        {
            case LayerType::Input: case LayerType::Output: case LayerType::MemCopy: case LayerType::Constant: return true;
            case LayerType::Activation:
            {
                const auto& d = static_cast<const ActivationDescriptor&>(descriptor);
                if (d.m_Function == ActivationFunction::Linear && d.m_A == 1.0f && d.m_B == 0.0f && infos[0] == infos[1]) return true;
                if (reason.has_value()) reason.value() = "TestHost: only the identity Linear activation";
                return false;
            }
            default:
                if (reason.has_value()) reason.value() = "TestHost: not implemented";
                return false;
        }
    }
};

class Backend : public IBackendInternal
{
public:
    const BackendId& GetId() const override { return Id(); }
    IWorkloadFactoryPtr CreateWorkloadFactory(const IMemoryManagerSharedPtr&) const override { return std::make_unique<Factory>(); }
    ILayerSupportSharedPtr GetLayerSupport() const override { static ILayerSupportSharedPtr s{new Support}; return s; }
};

// The same backend under a second id, with the capability that lets the runtime plan its tensors' memory; its default
// allocator counts what it hands out.
inline const BackendId& PlannedId() { static const BackendId id("TestHostPlanned"); return id; }
struct AllocatorLog
{
    int allocations = 0, frees = 0;
    size_t bytes = 0;
    static AllocatorLog& Default() { static AllocatorLog log; return log; }
};
class CountingAllocator : public ICustomAllocator
{
public:
    explicit CountingAllocator(AllocatorLog& log, MemorySource source = MemorySource::Malloc) : m_Log(log), m_Source(source) {}
    void* allocate(size_t size, size_t) override { ++m_Log.allocations; m_Log.bytes += size; return ::operator new(size ? size : 1); }
    void free(void* p) override { ++m_Log.frees; ::operator delete(p); }
    MemorySource GetMemorySourceType() override { return m_Source; }
    void* GetMemoryRegionAtOffset(void* buffer, size_t offset, size_t = 0) override { return static_cast<char*>(buffer) + offset; }
private:
    AllocatorLog& m_Log;
    MemorySource m_Source;
};
class PlannedFactory : public Factory
{
public:
    const BackendId& GetBackendId() const override { return PlannedId(); }
};
class PlannedBackend : public Backend
{
public:
    const BackendId& GetId() const override { return PlannedId(); }
    IWorkloadFactoryPtr CreateWorkloadFactory(const IMemoryManagerSharedPtr&) const override { return std::make_unique<PlannedFactory>(); }
    BackendCapabilities GetCapabilities() const override { return BackendCapabilities(PlannedId(), {{"ExternallyManagedMemory", true}}); }
    std::unique_ptr<ICustomAllocator> GetDefaultAllocator() const override { return std::make_unique<CountingAllocator>(AllocatorLog::Default()); }
    bool UseCustomMemoryAllocator(std::shared_ptr<ICustomAllocator> allocator, armnn::Optional<std::string&> err) override
    {
        if (allocator->GetMemorySourceType() == MemorySource::Malloc) return true;
        if (err) err.value() = "TestHostPlanned: only MemorySource::Malloc";
        return false;
    }
};

// Packs blocks into one bin: each block goes to the lowest 256-byte aligned offset where it meets no block placed
// before it whose lifetime overlaps its own.
class PackingStrategy : public IMemoryOptimizerStrategy
{
public:
    std::string GetName() const override { return "TestPacking"; }
    MemBlockStrategyType GetMemBlockStrategyType() const override { return MemBlockStrategyType::SingleAxisPacking; }
    std::vector<MemBin> Optimize(std::vector<MemBlock>& blocks) override
    {
        MemBin bin;
        bin.m_MemSize = 0;
        for (MemBlock& b : blocks)
        {
            size_t offset = 0;
            for (bool moved = true; moved;)
            {
                moved = false;
                for (const MemBlock& placed : bin.m_MemBlocks)
                {
                    const bool alive = placed.m_StartOfLife <= b.m_EndOfLife && b.m_StartOfLife <= placed.m_EndOfLife;
                    const bool meets = placed.m_Offset < offset + b.m_MemSize && offset < placed.m_Offset + placed.m_MemSize;
                    if (alive && meets) { offset = (placed.m_Offset + placed.m_MemSize + 255) / 256 * 256; moved = true; }
                }
            }
            b.m_Offset = offset;
            bin.m_MemBlocks.push_back(b);
            bin.m_MemSize = std::max(bin.m_MemSize, offset + b.m_MemSize);
        }
        return {bin};
    }
};

inline void RegisterPlanned()
{
    if (!BackendRegistryInstance().IsBackendRegistered(PlannedId()))
        BackendRegistryInstance().Register(PlannedId(), [] { return IBackendInternalUniquePtr(new PlannedBackend); });
}

inline void Register()
{
    if (!BackendRegistryInstance().IsBackendRegistered(Id()))
        BackendRegistryInstance().Register(Id(), [] { return IBackendInternalUniquePtr(new Backend); });
}
} // namespace testhost
