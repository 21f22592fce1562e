// Minimal host core: include/armnn/backends/IWorkload.hpp:14-43.
#pragma once
#include "ITensorHandle.hpp"
#include "WorkloadInfo.hpp"
#include <cstdint>
#include <string>
namespace arm { namespace pipe {
// the profiling GUID of the real library reduced to its value
class ProfilingGuid
{
public:
    ProfilingGuid(uint64_t guid = 0) : m_Guid(guid) {}
    operator uint64_t() const { return m_Guid; }
private:
    uint64_t m_Guid;
};
struct IProfilingService { static ProfilingGuid GetNextGuid(); };
}} // namespace arm::pipe

namespace armnn
{
class IWorkload
{
public:
    virtual ~IWorkload() {}
    virtual void PostAllocationConfigure() = 0;
    virtual void Execute() const = 0;
    virtual arm::pipe::ProfilingGuid GetGuid() const = 0;
    virtual bool SupportsTensorHandleReplacement() const = 0;
    virtual void ReplaceInputTensorHandle(ITensorHandle*, unsigned int) = 0;
    virtual const std::string& GetName() const = 0;
    virtual void ReplaceOutputTensorHandle(ITensorHandle*, unsigned int) = 0;
    virtual armnn::Optional<armnn::MemoryRequirements> GetMemoryRequirements() { return armnn::EmptyOptional(); }
};
} // namespace armnn
