// Minimal host core: host time between Start() and Stop() (src/armnn/WallClockTimer.hpp:38-88).
#pragma once
#include "Instrument.hpp"
#include <chrono>

namespace armnn
{
class WallClockTimer : public Instrument
{
public:
    using clock = std::chrono::steady_clock;
    void Start() override { m_Start = clock::now(); }
    void Stop() override { m_Stop = clock::now(); }
    const char* GetName() const override { return "WallClockTimer"; }
    std::vector<Measurement> GetMeasurements() const override
    {
        const double us = std::chrono::duration<double, std::micro>(m_Stop - m_Start).count();
        return {Measurement("Wall clock time", us, Measurement::TIME_US)};
    }
private:
    clock::time_point m_Start, m_Stop;
};
} // namespace armnn
