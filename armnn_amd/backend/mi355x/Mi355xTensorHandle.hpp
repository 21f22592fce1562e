// ITensorHandle / ITensorHandleFactory of the Mi355x backend: dense device tensors.
//
//   managed handles   live in the memory manager's arena (Manage() reserves, Allocate() ends the lifetime);
//   unmanaged handles (constants, network inputs) own a device allocation made by Allocate().
//
// Map() gives the host a pinned staging copy: it downloads the tensor if kernels may have written it since the
// last upload, and Unmap() uploads the staging copy again -- so the Map/memcpy/Unmap sequence of
// CopyMemGenericWorkload and of the runtime's input/output binding works unchanged
// (RefTensorHandle::Map/CopyInFrom/CopyOutTo, src/backends/reference/RefTensorHandle.cpp:45-133, are the host-memory
// counterparts).  Workloads call MarkDeviceWritten() on their outputs.
//
// An unmanaged handle can instead adopt caller memory the copy engines reach directly -- pinned host memory or device
// memory (Import with MemorySource::Malloc; pageable memory is refused).  The caller's buffer then takes the place of the
// staging copy: a workload that reads the tensor before any workload wrote it gets the buffer's current contents by one
// asynchronous transfer, and Map() brings results back into the buffer and waits -- no host-side memcpy on either side
// (RefTensorHandle::Import, src/backends/reference/RefTensorHandle.cpp:135-165, is the host-memory counterpart).
// Kernels do not read pinned host memory in place: a convolution reading its input across the bus proved slower than
// the transfer.  Adopted device memory is used in place: kernels read and write it, and Map() stages it through a pinned
// copy like a tensor of the backend's own.  That is also how a caller-side memory plan reaches the backend: the runtime
// creates every tensor unmanaged and hands each its place in a buffer from the backend's allocator
// (LoadedNetwork.cpp:1176-1184 with ExternallyManagedMemory).
#pragma once
#include "Mi355xBackendId.hpp"
#include "Mi355xMemoryManager.hpp"

#include <armnn/backends/ITensorHandle.hpp>
#include <armnn/backends/ITensorHandleFactory.hpp>

#include <memory>

namespace armnn
{
class Mi355xTensorHandle : public ITensorHandle
{
public:
    Mi355xTensorHandle(const TensorInfo& info, std::shared_ptr<Mi355xMemoryManager> memoryManager, bool managed);
    ~Mi355xTensorHandle() override;

    void Manage() override;
    void Allocate() override;
    ITensorHandle* GetParent() const override { return nullptr; }
    const void* Map(bool blocking = true) const override;
    void Unmap() const override;
    TensorShape GetStrides() const override;
    TensorShape GetShape() const override { return m_Info.GetShape(); }
    void CopyOutTo(void* memory) const override;
    void CopyInFrom(const void* memory) override;
    unsigned int GetImportFlags() const override { return static_cast<unsigned int>(MemorySource::Malloc); }
    bool CanBeImported(void* memory, MemorySource source) override;
    bool Import(void* memory, MemorySource source) override;
    void Unimport() override;

    const TensorInfo& GetTensorInfo() const { return m_Info; }
    /// device address; throws NullPointerException when the tensor has no memory yet
    void* GetDevicePointer() const;
    /// device address for a workload that reads the tensor: refreshes an adopted buffer's device copy first
    const void* GetDevicePointerForRead() const;
    void MarkDeviceWritten() const { m_DeviceNewer = true; }
    bool IsManaged() const { return m_Managed; }

private:
    unsigned int UploadLanes() const;
    TensorInfo m_Info;
    std::shared_ptr<Mi355xMemoryManager> m_MemoryManager;
    const bool m_Managed;
    bool m_Reserved = false;
    bool m_Retired = false;
    size_t m_Offset = 0;
    void* m_Owned = nullptr;            // unmanaged handles
    void* m_ImportedHost = nullptr;     // caller memory adopted by Import(), as the caller addresses it ...
    void* m_ImportedDevice = nullptr;   // ... and as the device does
    bool m_ImportedIsDeviceMemory = false;   // adopted device memory is used in place, without transfers
    bool m_ImportedOverlaps = false;         // ... and shares addresses with another adopted tensor
    mutable bool m_MappedToRead = false;     // the current Map() downloaded the tensor: Unmap() has nothing to upload
    mutable void* m_Staging = nullptr;  // pinned host copy, created by the first Map()
    mutable bool m_DeviceNewer = false;
    mutable bool m_UploadInFlight = false;
    mutable unsigned long long m_FetchedInEpoch = 0;   // mi355x::SyncEpoch() when an adopted input was last brought over
    mutable int m_MapCount = 0;
};

class Mi355xTensorHandleFactory : public ITensorHandleFactory
{
public:
    explicit Mi355xTensorHandleFactory(std::shared_ptr<Mi355xMemoryManager> mgr) : m_MemoryManager(std::move(mgr)) {}
    std::unique_ptr<ITensorHandle> CreateSubTensorHandle(ITensorHandle& parent, TensorShape const& subTensorShape,
                                                         unsigned int const* subTensorOrigin) const override;
    std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo) const override;
    std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo, DataLayout dataLayout) const override;
    std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo, const bool IsMemoryManaged) const override;
    std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo, DataLayout dataLayout,
                                                      const bool IsMemoryManaged) const override;
    static const FactoryId& GetIdStatic();
    const FactoryId& GetId() const override { return GetIdStatic(); }
    bool SupportsSubTensors() const override { return false; }
    MemorySourceFlags GetExportFlags() const override { return static_cast<MemorySourceFlags>(MemorySource::Malloc); }
    MemorySourceFlags GetImportFlags() const override { return static_cast<MemorySourceFlags>(MemorySource::Malloc); }
    const std::shared_ptr<Mi355xMemoryManager>& GetMemoryManager() const { return m_MemoryManager; }
private:
    std::shared_ptr<Mi355xMemoryManager> m_MemoryManager;
};
} // namespace armnn
