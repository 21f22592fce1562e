// Minimal host core: the per-network profiler with the public names of include/armnn/IProfiler.hpp:21-80.
#pragma once
#include "BackendId.hpp"
#include "Optional.hpp"
#include "backends/IWorkload.hpp"
#include "backends/WorkloadInfo.hpp"
#include <iosfwd>
#include <memory>
#include <string>
#include <vector>

namespace armnn
{
class Instrument;
class Event;
class ProfilerImpl;

class IProfiler
{
public:
    IProfiler();
    ~IProfiler();
    /// events are recorded only while this is on
    void EnableProfiling(bool enableProfiling);
    bool IsProfilingEnabled();
    /// one line per event: name, backend, every measurement of every instrument
    void AnalyzeEventsAndWriteResults(std::ostream& outStream) const;
    /// the event tree as JSON (events nest as they were open inside each other), then forgets the events
    void Print(std::ostream& outStream) const;
    /// what a workload reported about itself when it was built (ARMNN_REPORT_PROFILING_WORKLOAD_DESC)
    void AddLayerDetails(const std::string& name, const std::string& descriptorText, const WorkloadInfo& infos,
                         const arm::pipe::ProfilingGuid guid);
    /// the events recorded since the last Print(), outermost first
    const std::vector<std::unique_ptr<Event>>& GetEvents() const;

    Event* BeginEvent(const BackendId& backendId, const std::string& name, std::vector<std::unique_ptr<Instrument>>&& instruments,
                      const Optional<arm::pipe::ProfilingGuid>& guid);
    std::unique_ptr<ProfilerImpl> pProfilerImpl;
};
} // namespace armnn
