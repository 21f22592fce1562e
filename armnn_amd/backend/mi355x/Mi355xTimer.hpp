// Device time of what a workload puts on the backend's stream between Start() and Stop(), measured with a pair of HIP
// events through the C ABI.  The counterpart of OpenClTimer (src/backends/cl/OpenClTimer.hpp:22-66) for the profiler's
// scoped events; unlike it, one measurement covers all launches of the region (a workload here is one launch).
#pragma once
#include "Mi355xDevice.hpp"

#include <Instrument.hpp>

#include <memory>

namespace armnn
{
class Mi355xTimer : public Instrument
{
public:
    Mi355xTimer() = default;
    /// records the start event on the backend's stream (events are created on first use)
    void Start() override;
    /// records the stop event; does not wait
    void Stop() override;
    bool HasKernelMeasurements() const override { return true; }
    const char* GetName() const override { return "Mi355xKernelTimer"; }
    /// waits for the stop event, then reports the device time between the two events in microseconds
    std::vector<Measurement> GetMeasurements() const override;
private:
    struct Events
    {
        mi355x_event_t start = nullptr, stop = nullptr;
        bool stopped = false;
        ~Events();
    };
    std::shared_ptr<Events> m_Events;      // shared so that the copies the profiler makes refer to one pair
};

/// Profiling event for a workload's Execute(), named and keyed like ARMNN_SCOPED_PROFILING_EVENT_CL_NAME_GUID
/// (src/backends/cl/workloads/ClWorkloadUtils.hpp:35-41): device time and host time of the region.
#define ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID(label) \
    ARMNN_SCOPED_PROFILING_EVENT_WITH_INSTRUMENTS(armnn::BackendId(armnn::Mi355xBackendId()), this->GetGuid(), this->GetName() + "_" + label, \
                                                  armnn::Mi355xTimer(), armnn::WallClockTimer())
} // namespace armnn
