// Minimal host core: the generic Map/memcpy/Unmap copy workload used for Input, Output and MemCopy layers
// (src/backends/backendsCommon/MemCopyWorkload.cpp:44-64).
#pragma once
#include "Workload.hpp"
namespace armnn
{
class CopyMemGenericWorkload : public BaseWorkload<MemCopyQueueDescriptor>
{
public:
    CopyMemGenericWorkload(const MemCopyQueueDescriptor& descriptor, const WorkloadInfo& info);
    void Execute() const override;
};
} // namespace armnn
