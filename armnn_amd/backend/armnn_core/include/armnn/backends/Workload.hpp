// Minimal host core: BaseWorkload (include/armnn/backends/Workload.hpp:31-77): copies the descriptor and
// validates it in the constructor.
#pragma once
#include "IWorkload.hpp"
#include "WorkloadData.hpp"
#include "WorkloadInfo.hpp"
#include "../utility/IgnoreUnused.hpp"

namespace armnn
{
template <typename QueueDescriptor>
class BaseWorkload : public IWorkload
{
public:
    BaseWorkload(const QueueDescriptor& descriptor, const WorkloadInfo& info)
        : m_Data(descriptor), m_Guid(arm::pipe::IProfilingService::GetNextGuid()), m_Name(info.m_Name)
    {
        m_Data.Validate(info);
    }
    const std::string& GetName() const override { return m_Name; }
    void PostAllocationConfigure() override {}
    const QueueDescriptor& GetData() const { return m_Data; }
    arm::pipe::ProfilingGuid GetGuid() const final { return m_Guid; }
    bool SupportsTensorHandleReplacement() const override { return false; }
    void ReplaceInputTensorHandle(ITensorHandle* tensorHandle, unsigned int slot) override
    {
        IgnoreUnused(tensorHandle, slot);
        throw UnimplementedException("ReplaceInputTensorHandle not implemented for this workload");
    }
    void ReplaceOutputTensorHandle(ITensorHandle* tensorHandle, unsigned int slot) override
    {
        IgnoreUnused(tensorHandle, slot);
        throw UnimplementedException("ReplaceOutputTensorHandle not implemented for this workload");
    }
protected:
    QueueDescriptor m_Data;
    const arm::pipe::ProfilingGuid m_Guid;
    const std::string m_Name;
};
} // namespace armnn
