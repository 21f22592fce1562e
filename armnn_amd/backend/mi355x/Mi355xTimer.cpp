#include "Mi355xTimer.hpp"

namespace armnn
{
Mi355xTimer::Events::~Events()
{
    if (start) mi355x_event_destroy(start);
    if (stop) mi355x_event_destroy(stop);
}

void Mi355xTimer::Start()
{
    if (!m_Events)
    {
        auto events = std::make_shared<Events>();
        mi355x::Check(mi355x_event_create(&events->start), "mi355x_event_create");
        mi355x::Check(mi355x_event_create(&events->stop), "mi355x_event_create");
        m_Events = std::move(events);
    }
    m_Events->stopped = false;
    mi355x::Check(mi355x_event_record(m_Events->start, mi355x::Stream()), "mi355x_event_record");
}

void Mi355xTimer::Stop()
{
    if (!m_Events) return;
    mi355x::Check(mi355x_event_record(m_Events->stop, mi355x::Stream()), "mi355x_event_record");
    m_Events->stopped = true;
}

std::vector<Measurement> Mi355xTimer::GetMeasurements() const
{
    if (!m_Events || !m_Events->stopped) return {};
    mi355x::Check(mi355x_event_synchronize(m_Events->stop), "mi355x_event_synchronize");
    float ms = 0.0f;
    mi355x::Check(mi355x_event_elapsed_ms(m_Events->start, m_Events->stop, &ms), "mi355x_event_elapsed_ms");
    return {Measurement("Device time", static_cast<double>(ms) * 1000.0, Measurement::TIME_US)};
}
} // namespace armnn
