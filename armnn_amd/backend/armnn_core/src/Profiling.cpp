// Minimal host core: event recording and reporting behind IProfiler (src/armnn/Profiling.cpp:180-620 is the reference's;
// the JSON here keeps its nesting -- an event is an object holding its measurements and the events opened inside it).
#include <Profiling.hpp>

#include <iomanip>
#include <map>
#include <ostream>

namespace armnn
{
namespace
{
std::string Quote(const std::string& s)
{
    std::string out = "\"";
    for (char c : s)
    {
        if (c == '"' || c == '\\') out += '\\';
        out += c;
    }
    return out + "\"";
}

std::string ShapeText(const TensorInfo& info)
{
    std::ostringstream os;
    os << "[";
    for (unsigned int i = 0; i < info.GetNumDimensions(); ++i) os << (i ? "," : "") << info.GetShape()[i];
    os << "] " << GetDataTypeName(info.GetDataType());
    if (IsQuantizedType(info.GetDataType()))
    {
        os << " scale " << (info.HasMultipleQuantizationScales() ? std::string("per-axis") : std::to_string(info.GetQuantizationScale()))
           << " offset " << info.GetQuantizationOffset();
    }
    return os.str();
}

void PrintEvent(std::ostream& os, const Event* e, const std::multimap<const Event*, const Event*>& children, int depth, size_t& counter)
{
    const std::string pad(static_cast<size_t>(depth) * 2, ' ');
    os << pad << Quote(e->GetName() + "_#" + std::to_string(counter++)) << ": {\n";
    os << pad << "  \"type\": \"Event\"";
    if (e->GetBackendId() != BackendId()) os << ",\n" << pad << "  \"backendId\": " << Quote(e->GetBackendId().Get());
    if (e->GetProfilingGuid().has_value()) os << ",\n" << pad << "  \"GUID\": " << static_cast<uint64_t>(e->GetProfilingGuid().value());
    size_t m = 0;
    for (const Measurement& meas : e->GetMeasurements())
    {
        os << ",\n" << pad << "  " << Quote(meas.m_Name + "_#" + std::to_string(m++)) << ": {\"type\": \"Measurement\", \"raw\": ["
           << std::fixed << std::setprecision(3) << meas.m_Value << "], \"unit\": " << Quote(Measurement::ToString(meas.m_Unit)) << "}";
    }
    auto range = children.equal_range(e);
    for (auto it = range.first; it != range.second; ++it)
    {
        os << ",\n";
        PrintEvent(os, it->second, children, depth + 1, counter);
    }
    os << "\n" << pad << "}";
}
} // namespace

std::string DescribeParameters(const BaseDescriptor& descriptor)
{
    std::ostringstream os;
    auto conv = [&](const auto& d) {
        os << "pad (l,r,t,b) " << d.m_PadLeft << "," << d.m_PadRight << "," << d.m_PadTop << "," << d.m_PadBottom << " stride " << d.m_StrideX << "x"
           << d.m_StrideY << " dilation " << d.m_DilationX << "x" << d.m_DilationY << " bias " << d.m_BiasEnabled
           << (d.m_DataLayout == DataLayout::NHWC ? " NHWC" : " NCHW");
    };
    if (auto* c = dynamic_cast<const Convolution2dDescriptor*>(&descriptor)) conv(*c);
    else if (auto* dw = dynamic_cast<const DepthwiseConvolution2dDescriptor*>(&descriptor)) conv(*dw);
    else if (auto* fc = dynamic_cast<const FullyConnectedDescriptor*>(&descriptor))
        os << "bias " << fc->m_BiasEnabled << " transposed weights " << fc->m_TransposeWeightMatrix;
    else if (auto* p = dynamic_cast<const Pooling2dDescriptor*>(&descriptor))
        os << (p->m_PoolType == PoolingAlgorithm::Max ? "max " : p->m_PoolType == PoolingAlgorithm::Average ? "average " : "l2 ") << p->m_PoolWidth << "x"
           << p->m_PoolHeight << " stride " << p->m_StrideX << "x" << p->m_StrideY << " pad (l,r,t,b) " << p->m_PadLeft << "," << p->m_PadRight << ","
           << p->m_PadTop << "," << p->m_PadBottom << (p->m_PaddingMethod == PaddingMethod::Exclude ? " exclude" : " ignore-value");
    else if (auto* a = dynamic_cast<const ActivationDescriptor*>(&descriptor))
        os << "function " << static_cast<int>(a->m_Function) << " a " << a->m_A << " b " << a->m_B;
    else if (auto* s = dynamic_cast<const SoftmaxDescriptor*>(&descriptor)) os << "beta " << s->m_Beta << " axis " << s->m_Axis;
    else if (auto* pd = dynamic_cast<const PadDescriptor*>(&descriptor))
    {
        os << "value " << pd->m_PadValue << " list";
        for (const auto& pr : pd->m_PadList) os << " (" << pr.first << "," << pr.second << ")";
    }
    else if (auto* e = dynamic_cast<const ElementwiseBinaryDescriptor*>(&descriptor)) os << "operation " << static_cast<int>(e->m_Operation);
    return os.str();
}

// ---- ProfilerImpl ----------------------------------------------------------------------------------------------------
Event* ProfilerImpl::BeginEvent(const BackendId& backendId, const std::string& name, std::vector<std::unique_ptr<Instrument>>&& instruments,
                                const Optional<arm::pipe::ProfilingGuid>& guid)
{
    Event* parent = m_Open.empty() ? nullptr : m_Open.back();
    m_Events.push_back(std::make_unique<Event>(name, backendId, parent, std::move(instruments), guid));
    Event* e = m_Events.back().get();
    m_Open.push_back(e);
    e->Start();
    return e;
}

void ProfilerImpl::EndEvent(Event* event)
{
    event->Stop();
    // events close in the reverse order of opening; anything else is a scoping error in the caller
    if (m_Open.empty() || m_Open.back() != event) throw RuntimeException("profiling events were closed out of order");
    m_Open.pop_back();
}

// ---- IProfiler -------------------------------------------------------------------------------------------------------
IProfiler::IProfiler() : pProfilerImpl(new ProfilerImpl) {}
IProfiler::~IProfiler() = default;
void IProfiler::EnableProfiling(bool enableProfiling) { pProfilerImpl->m_Enabled = enableProfiling; }
bool IProfiler::IsProfilingEnabled() { return pProfilerImpl->m_Enabled; }
const std::vector<std::unique_ptr<Event>>& IProfiler::GetEvents() const { return pProfilerImpl->m_Events; }

Event* IProfiler::BeginEvent(const BackendId& backendId, const std::string& name, std::vector<std::unique_ptr<Instrument>>&& instruments,
                             const Optional<arm::pipe::ProfilingGuid>& guid)
{
    return pProfilerImpl->BeginEvent(backendId, name, std::move(instruments), guid);
}

void IProfiler::AddLayerDetails(const std::string& name, const std::string& descriptorText, const WorkloadInfo& infos,
                                const arm::pipe::ProfilingGuid guid)
{
    pProfilerImpl->m_Details.push_back({name, descriptorText, infos, static_cast<uint64_t>(guid)});
}

void IProfiler::AnalyzeEventsAndWriteResults(std::ostream& os) const
{
    os << std::left << std::setw(64) << "Event" << std::setw(12) << "Backend" << "Measurements\n";
    for (const auto& e : pProfilerImpl->m_Events)
    {
        int depth = 0;
        for (const Event* p = e->GetParentEvent(); p; p = p->GetParentEvent()) ++depth;
        os << std::left << std::setw(64) << (std::string(static_cast<size_t>(depth) * 2, ' ') + e->GetName()) << std::setw(12)
           << (e->GetBackendId() != BackendId() ? e->GetBackendId().Get() : std::string("-"));
        for (const Measurement& m : e->GetMeasurements())
            os << m.m_Name << " " << std::fixed << std::setprecision(3) << m.m_Value << " " << Measurement::ToString(m.m_Unit) << "; ";
        os << "\n";
    }
}

void IProfiler::Print(std::ostream& os) const
{
    std::multimap<const Event*, const Event*> children;
    for (const auto& e : pProfilerImpl->m_Events) children.emplace(e->GetParentEvent(), e.get());
    os << "{\n  \"ArmNN\": {\n";
    size_t counter = 0;
    bool first = true;
    if (!pProfilerImpl->m_Details.empty())
    {
        os << "    \"layer_details\": {\n";
        for (size_t i = 0; i < pProfilerImpl->m_Details.size(); ++i)
        {
            const auto& d = pProfilerImpl->m_Details[i];
            os << "      " << Quote(d.name + "_#" + std::to_string(i)) << ": {\"GUID\": " << d.guid << ", \"Name\": " << Quote(d.infos.m_Name)
               << ", \"Parameters\": " << Quote(d.descriptor);
            for (size_t k = 0; k < d.infos.m_InputTensorInfos.size(); ++k) os << ", " << Quote("Input_" + std::to_string(k)) << ": " << Quote(ShapeText(d.infos.m_InputTensorInfos[k]));
            for (size_t k = 0; k < d.infos.m_OutputTensorInfos.size(); ++k) os << ", " << Quote("Output_" + std::to_string(k)) << ": " << Quote(ShapeText(d.infos.m_OutputTensorInfos[k]));
            if (d.infos.m_WeightsTensorInfo.has_value()) os << ", \"Weights\": " << Quote(ShapeText(d.infos.m_WeightsTensorInfo.value()));
            if (d.infos.m_BiasTensorInfo.has_value()) os << ", \"Bias\": " << Quote(ShapeText(d.infos.m_BiasTensorInfo.value()));
            if (d.infos.m_ConvolutionMethod.has_value()) os << ", \"ConvolutionMethod\": " << Quote(d.infos.m_ConvolutionMethod.value());
            os << "}" << (i + 1 < pProfilerImpl->m_Details.size() ? "," : "") << "\n";
        }
        os << "    }";
        first = false;
    }
    auto roots = children.equal_range(nullptr);
    for (auto it = roots.first; it != roots.second; ++it)
    {
        os << (first ? "" : ",\n");
        first = false;
        PrintEvent(os, it->second, children, 2, counter);
    }
    os << "\n  }\n}\n";
    pProfilerImpl->m_Events.clear();
    pProfilerImpl->m_Open.clear();
}

// ---- ProfilerManager -------------------------------------------------------------------------------------------------
namespace
{
thread_local IProfiler* t_Profiler = nullptr;
}
ProfilerManager& ProfilerManager::GetInstance()
{
    static ProfilerManager instance;
    return instance;
}
void ProfilerManager::RegisterProfiler(IProfiler* profiler) { t_Profiler = profiler; }
IProfiler* ProfilerManager::GetProfiler() { return t_Profiler; }
} // namespace armnn
