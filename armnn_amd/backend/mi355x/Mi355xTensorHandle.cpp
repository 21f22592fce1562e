#include "Mi355xTensorHandle.hpp"
#include "Mi355xDevice.hpp"

#include <armnn/backends/TensorHandle.hpp>

#include <cstdint>
#include <cstring>

namespace armnn
{
Mi355xTensorHandle::Mi355xTensorHandle(const TensorInfo& info, std::shared_ptr<Mi355xMemoryManager> memoryManager, bool managed)
    : m_Info(info), m_MemoryManager(std::move(memoryManager)), m_Managed(managed && m_MemoryManager)
{
}

Mi355xTensorHandle::~Mi355xTensorHandle()
{
    if (m_ImportedDevice && m_ImportedIsDeviceMemory) mi355x::ForgetAdoptedRange(m_ImportedDevice, m_Info.GetNumBytes(), m_ImportedOverlaps);
    if (m_Owned) mi355x_free(m_Owned);
    if (m_Staging) mi355x_host_free(m_Staging);
}

void Mi355xTensorHandle::Manage()
{
    if (!m_Managed) return;
    if (m_Reserved) throw InvalidArgumentException("Mi355xTensorHandle::Manage() called twice");
    m_Offset = m_MemoryManager->Reserve(m_Info.GetNumBytes());
    m_Reserved = true;
}

void Mi355xTensorHandle::Allocate()
{
    // Allocate() without a lifetime opened by Manage() asks for memory that lasts: the runtime does that for the outputs
    // of Constant layers (Graph::AllocateDynamicBuffers, src/armnn/Graph.cpp:237-252; RefTensorHandle::Allocate,
    // src/backends/reference/RefTensorHandle.cpp:45-66, allocates directly in that case)
    if (m_Managed && m_Reserved)
    {
        if (m_Retired) throw InvalidArgumentException("Mi355xTensorHandle::Allocate() called twice");
        m_MemoryManager->Retire(m_Offset, m_Info.GetNumBytes());
        m_Retired = true;
        return;
    }
    if (m_Owned) throw InvalidArgumentException("Mi355xTensorHandle::Allocate() called on a tensor that already has memory");
    mi355x::EnsureDevice();
    const size_t bytes = m_Info.GetNumBytes() ? m_Info.GetNumBytes() : 1;
    mi355x::Check(mi355x_malloc(&m_Owned, bytes), "mi355x_malloc");
}

bool Mi355xTensorHandle::CanBeImported(void* memory, MemorySource source)
{
    if (source != MemorySource::Malloc || m_Managed || !memory) return false;
    if (reinterpret_cast<uintptr_t>(memory) % 16 != 0) return false;          // the kernels' vector loads and stores
    if (mi355x::DeviceCount() == 0) return false;
    void* device = nullptr;
    int isDevice = 0;
    return mi355x_host_device_pointer(memory, &device, &isDevice) == 0 && device != nullptr;
}

bool Mi355xTensorHandle::Import(void* memory, MemorySource source)
{
    if (m_Managed) throw MemoryImportException("Mi355xTensorHandle::Import: a tensor that lives in the arena cannot adopt caller memory");
    if (source != MemorySource::Malloc) return false;
    if (!memory) throw MemoryImportException("Mi355xTensorHandle::Import: null memory");
    if (reinterpret_cast<uintptr_t>(memory) % 16 != 0) throw MemoryImportException("Mi355xTensorHandle::Import: memory is not 16-byte aligned");
    mi355x::EnsureDevice();
    void* device = nullptr;
    int isDevice = 0;
    if (mi355x_host_device_pointer(memory, &device, &isDevice) != 0 || !device) return false;
    if (m_ImportedDevice) Unimport();
    m_ImportedIsDeviceMemory = isDevice != 0;
    m_ImportedOverlaps = m_ImportedIsDeviceMemory && mi355x::NoteAdoptedRange(device, m_Info.GetNumBytes());
    if (!m_Owned && !m_ImportedIsDeviceMemory) mi355x::Check(mi355x_malloc(&m_Owned, m_Info.GetNumBytes() ? m_Info.GetNumBytes() : 1), "mi355x_malloc");
    m_ImportedHost = memory;
    m_ImportedDevice = device;
    m_DeviceNewer = false;
    m_FetchedInEpoch = 0;
    return true;
}

void Mi355xTensorHandle::Unimport()
{
    if (m_ImportedDevice) mi355x::Synchronize();       // no kernel may still be using the caller's memory
    if (m_ImportedDevice && m_ImportedIsDeviceMemory) mi355x::ForgetAdoptedRange(m_ImportedDevice, m_Info.GetNumBytes(), m_ImportedOverlaps);
    m_ImportedOverlaps = false;
    m_ImportedHost = nullptr;
    m_ImportedDevice = nullptr;
    m_ImportedIsDeviceMemory = false;
}

const void* Mi355xTensorHandle::GetDevicePointerForRead() const
{
    void* dev = GetDevicePointer();
    // adopted buffer, not written by a workload since the caller last saw it: it is an input, and whatever the caller
    // has put there is what this inference reads -- fetched once per inference, however many workloads read the tensor
    if (m_ImportedDevice && !m_ImportedIsDeviceMemory && !m_DeviceNewer && m_Info.GetNumBytes() && m_FetchedInEpoch != mi355x::SyncEpoch())
    {
        mi355x::UploadInLanes(dev, m_ImportedDevice, m_Info.GetNumBytes(), UploadLanes());
        m_FetchedInEpoch = mi355x::SyncEpoch();
    }
    return dev;
}

// A batch of images large enough to be worth it goes up slice by slice, so that the first lane starts computing while
// the later slices are still on the bus.
unsigned int Mi355xTensorHandle::UploadLanes() const
{
    if (m_Info.IsConstant() || m_Info.GetNumDimensions() < 2 || m_Info.GetNumBytes() < (1u << 20)) return 1;
    return mi355x::LanesFor(m_Info.GetShape()[0]);
}

void* Mi355xTensorHandle::GetDevicePointer() const
{
    if (m_ImportedDevice && m_ImportedIsDeviceMemory) return m_ImportedDevice;
    if (m_Managed && m_Reserved) return m_MemoryManager->Resolve(m_Offset);
    if (!m_Owned) throw NullPointerException("Mi355xTensorHandle: tensor has no memory (Allocate was not called)");
    return m_Owned;
}

TensorShape Mi355xTensorHandle::GetStrides() const { return GetUnpaddedTensorStrides(m_Info); }

const void* Mi355xTensorHandle::Map(bool /*blocking*/) const
{
    if (m_ImportedDevice && !m_ImportedIsDeviceMemory)
    {
        // results go straight into the caller's buffer; either way the host waits for what is queued
        if (m_MapCount++ == 0)
        {
            if (m_DeviceNewer && !m_ImportedIsDeviceMemory && m_Info.GetNumBytes())
                mi355x::Check(mi355x_memcpy_d2h(m_ImportedDevice, GetDevicePointer(), m_Info.GetNumBytes(), mi355x::Stream()), "mi355x_memcpy_d2h (adopted buffer)");
            mi355x::Synchronize();
            m_DeviceNewer = false;
        }
        return m_ImportedHost;
    }
    void* dev = GetDevicePointer();
    const size_t bytes = m_Info.GetNumBytes();
    if (!m_Staging) mi355x::Check(mi355x_host_alloc(&m_Staging, bytes ? bytes : 1), "mi355x_host_alloc");
    if (m_MapCount == 0 && m_UploadInFlight)
    {
        // the host is about to touch the staging copy again: the previous upload must have left it
        mi355x::Synchronize();
        m_UploadInFlight = false;
    }
    if (m_MapCount++ == 0)
    {
        // A tensor has one producer.  If that is a kernel, the host maps the tensor to read it (a network output, a copy
        // to another backend) and Unmap() has nothing to bring back; if it is the host, no kernel ever makes the device
        // copy the newer one.
        m_MappedToRead = m_DeviceNewer;
        if (m_DeviceNewer && bytes)
        {
            mi355x::Check(mi355x_memcpy_d2h(m_Staging, dev, bytes, mi355x::Stream()), "mi355x_memcpy_d2h");
            mi355x::Synchronize();
            m_DeviceNewer = false;
        }
        else if (m_ImportedDevice)
        {
            mi355x::Synchronize();      // adopted device memory: mapping it is also how the runtime waits for the results
        }
    }
    return m_Staging;
}

void Mi355xTensorHandle::Unmap() const
{
    if (m_MapCount == 0) return;
    if (--m_MapCount != 0) return;
    if (m_ImportedDevice && !m_ImportedIsDeviceMemory) return;
    const size_t bytes = m_Info.GetNumBytes();
    if (!bytes || m_MappedToRead) return;
    // the pinned copy stays alive with the handle, so the upload may complete asynchronously in stream order
    mi355x::UploadInLanes(GetDevicePointer(), m_Staging, bytes, UploadLanes());
    m_UploadInFlight = true;
}

void Mi355xTensorHandle::CopyOutTo(void* memory) const
{
    const void* p = Map(true);
    std::memcpy(memory, p, m_Info.GetNumBytes());
    // nothing was modified: skip the upload Unmap() would do
    --m_MapCount;
}

void Mi355xTensorHandle::CopyInFrom(const void* memory)
{
    const size_t bytes = m_Info.GetNumBytes();
    if (!m_Staging) mi355x::Check(mi355x_host_alloc(&m_Staging, bytes ? bytes : 1), "mi355x_host_alloc");
    if (m_UploadInFlight) mi355x::Synchronize();
    std::memcpy(m_Staging, memory, bytes);
    if (bytes) mi355x::UploadInLanes(GetDevicePointer(), m_Staging, bytes, UploadLanes());
    m_UploadInFlight = bytes != 0;
    m_DeviceNewer = false;
}

// ---- factory ---------------------------------------------------------------------------------------------------------
const ITensorHandleFactory::FactoryId& Mi355xTensorHandleFactory::GetIdStatic()
{
    static const FactoryId id(Mi355xTensorHandleFactoryId());
    return id;
}

std::unique_ptr<ITensorHandle> Mi355xTensorHandleFactory::CreateSubTensorHandle(ITensorHandle&, TensorShape const&, unsigned int const*) const
{
    return nullptr;
}
std::unique_ptr<ITensorHandle> Mi355xTensorHandleFactory::CreateTensorHandle(const TensorInfo& info) const
{
    return std::make_unique<Mi355xTensorHandle>(info, m_MemoryManager, true);
}
std::unique_ptr<ITensorHandle> Mi355xTensorHandleFactory::CreateTensorHandle(const TensorInfo& info, DataLayout) const
{
    return std::make_unique<Mi355xTensorHandle>(info, m_MemoryManager, true);
}
std::unique_ptr<ITensorHandle> Mi355xTensorHandleFactory::CreateTensorHandle(const TensorInfo& info, const bool managed) const
{
    return std::make_unique<Mi355xTensorHandle>(info, m_MemoryManager, managed);
}
std::unique_ptr<ITensorHandle> Mi355xTensorHandleFactory::CreateTensorHandle(const TensorInfo& info, DataLayout, const bool managed) const
{
    return std::make_unique<Mi355xTensorHandle>(info, m_MemoryManager, managed);
}
} // namespace armnn
