// Minimal host core: scoped profiling events (src/armnn/Profiling.hpp:108-260).  The thread's current profiler is the
// one of the network being executed; an event exists only while that profiler is enabled.
#pragma once
#include "Instrument.hpp"
#include "WallClockTimer.hpp"
#include <armnn/Descriptors.hpp>
#include <armnn/IProfiler.hpp>

#include <memory>
#include <sstream>
#include <string>
#include <utility>
#include <vector>

namespace armnn
{
/// one timed region: its instruments are started when it opens and stopped when it closes
class Event
{
public:
    Event(const std::string& name, const BackendId& backendId, Event* parent, std::vector<std::unique_ptr<Instrument>>&& instruments,
          const Optional<arm::pipe::ProfilingGuid>& guid)
        : m_Name(name), m_BackendId(backendId), m_Parent(parent), m_Instruments(std::move(instruments)), m_Guid(guid) {}
    void Start() { for (auto& i : m_Instruments) i->Start(); }
    void Stop() { for (auto& i : m_Instruments) i->Stop(); }
    const std::string& GetName() const { return m_Name; }
    const BackendId& GetBackendId() const { return m_BackendId; }
    const Event* GetParentEvent() const { return m_Parent; }
    Optional<arm::pipe::ProfilingGuid> GetProfilingGuid() const { return m_Guid; }
    const std::vector<std::unique_ptr<Instrument>>& GetInstruments() const { return m_Instruments; }
    std::vector<Measurement> GetMeasurements() const
    {
        std::vector<Measurement> all;
        for (const auto& i : m_Instruments)
            for (const Measurement& m : i->GetMeasurements()) all.push_back(m);
        return all;
    }
private:
    std::string m_Name;
    BackendId m_BackendId;
    Event* m_Parent;
    std::vector<std::unique_ptr<Instrument>> m_Instruments;
    Optional<arm::pipe::ProfilingGuid> m_Guid;
};

class ProfilerImpl
{
public:
    Event* BeginEvent(const BackendId& backendId, const std::string& name, std::vector<std::unique_ptr<Instrument>>&& instruments,
                      const Optional<arm::pipe::ProfilingGuid>& guid);
    void EndEvent(Event* event);
    struct Details { std::string name, descriptor; WorkloadInfo infos; uint64_t guid; };
    bool m_Enabled = false;
    std::vector<Event*> m_Open;
    std::vector<std::unique_ptr<Event>> m_Events;
    std::vector<Details> m_Details;
};

/// the profiler of the network the calling thread is executing (LoadedNetwork registers it around EnqueueWorkload)
class ProfilerManager
{
public:
    void RegisterProfiler(IProfiler* profiler);
    IProfiler* GetProfiler();
    static ProfilerManager& GetInstance();
private:
    ProfilerManager() {}
};

class ScopedProfilingEvent
{
public:
    template <typename... Args>
    ScopedProfilingEvent(const BackendId& backendId, const Optional<arm::pipe::ProfilingGuid>& guid, const std::string& name, Args&&... args)
        : m_Event(nullptr), m_Profiler(ProfilerManager::GetInstance().GetProfiler())
    {
        if (m_Profiler && m_Profiler->IsProfilingEnabled())
        {
            std::vector<std::unique_ptr<Instrument>> instruments;
            instruments.reserve(sizeof...(args));
            (instruments.emplace_back(std::make_unique<std::decay_t<Args>>(std::forward<Args>(args))), ...);
            m_Event = m_Profiler->BeginEvent(backendId, name, std::move(instruments), guid);
        }
    }
    ~ScopedProfilingEvent()
    {
        if (m_Profiler && m_Event) m_Profiler->pProfilerImpl->EndEvent(m_Event);
    }
    ScopedProfilingEvent(const ScopedProfilingEvent&) = delete;
    ScopedProfilingEvent& operator=(const ScopedProfilingEvent&) = delete;
private:
    Event* m_Event;
    IProfiler* m_Profiler;
};

/// text of a descriptor for the details record; backends' descriptors are the ones of Descriptors.hpp
std::string DescribeParameters(const BaseDescriptor& descriptor);

template <typename DescriptorType>
inline void ProfilingUpdateDescriptions(const std::string& name, const DescriptorType& desc, const WorkloadInfo& infos,
                                        const arm::pipe::ProfilingGuid guid)
{
    IProfiler* profiler = ProfilerManager::GetInstance().GetProfiler();
    if (profiler && profiler->IsProfilingEnabled()) profiler->AddLayerDetails(name, DescribeParameters(desc), infos, guid);
}
} // namespace armnn

#define ARMNN_PROFILING_CONCAT_INNER(a, b) a##b
#define ARMNN_PROFILING_CONCAT(a, b) ARMNN_PROFILING_CONCAT_INNER(a, b)
#define ARMNN_SCOPED_PROFILING_EVENT_WITH_INSTRUMENTS(backendId, guid, /*name,*/...) \
    armnn::ScopedProfilingEvent ARMNN_PROFILING_CONCAT(e_, __LINE__)(backendId, guid, /*name,*/ __VA_ARGS__);
#define ARMNN_SCOPED_PROFILING_EVENT(backendId, name) \
    ARMNN_SCOPED_PROFILING_EVENT_WITH_INSTRUMENTS(backendId, armnn::EmptyOptional(), name, armnn::WallClockTimer())
#define ARMNN_SCOPED_PROFILING_EVENT_GUID(backendId, name, guid) \
    ARMNN_SCOPED_PROFILING_EVENT_WITH_INSTRUMENTS(backendId, guid, name, armnn::WallClockTimer())
#define ARMNN_REPORT_PROFILING_WORKLOAD_DESC(name, desc, infos, guid) armnn::ProfilingUpdateDescriptions(name, desc, infos, guid);
