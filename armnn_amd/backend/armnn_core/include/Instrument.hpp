// Minimal host core: what a profiling event measures with (src/armnn/Instrument.hpp:14-66).
#pragma once
#include <string>
#include <vector>

namespace armnn
{
struct Measurement
{
    enum Unit { TIME_NS, TIME_US, TIME_MS };
    static const char* ToString(Unit unit) { return unit == TIME_NS ? "ns" : unit == TIME_US ? "us" : unit == TIME_MS ? "ms" : ""; }
    Measurement(const std::string& name, double value, Unit unit) : m_Name(name), m_Value(value), m_Unit(unit) {}
    std::string m_Name;
    double m_Value;
    Unit m_Unit;
};

class Instrument
{
public:
    virtual ~Instrument() {}
    virtual void Start() = 0;
    virtual void Stop() = 0;
    virtual std::vector<Measurement> GetMeasurements() const = 0;
    virtual const char* GetName() const = 0;
    virtual bool HasKernelMeasurements() const { return false; }
};
} // namespace armnn
