// Minimal host core: Optimize() -- backend assignment with fallback, per-backend sub-graph substitution, and copy
// layers on edges that cross backends (the parts of src/armnn/Network.cpp:1127-1420 and :2026-2271 a backend sees).
#include <Layer.hpp>
#include <armnn/BackendRegistry.hpp>
#include <armnn/backends/IBackendInternal.hpp>
#include <armnn/backends/WorkloadFactory.hpp>

#include <algorithm>
#include <map>
#include <set>

namespace armnn
{
namespace
{
void Report(Optional<std::vector<std::string>&> messages, const std::string& text)
{
    if (messages.has_value()) messages.value().push_back(text);
}

// the layers a backend owns, as one view: boundary = slots whose other end lies outside the set.  Input and Output
// layers stay out of the view, as SubgraphViewSelector leaves them out (src/armnn/Network.cpp:1283-1291).
SubgraphView MakeBackendView(const std::vector<Layer*>& order, const BackendId& backend)
{
    std::set<const Layer*> members;
    SubgraphView::IConnectableLayers layers;
    for (Layer* l : order)
        if (l->GetBackendId() == backend && l->GetType() != LayerType::Input && l->GetType() != LayerType::Output)
        {
            members.insert(l);
            layers.push_back(l);
        }
    SubgraphView::IInputSlots ins;
    SubgraphView::IOutputSlots outs;
    for (IConnectableLayer* il : layers)
    {
        Layer* l = PolymorphicDowncast<Layer*>(il);
        for (unsigned int i = 0; i < l->GetNumInputSlots(); ++i)
            if (!members.count(&l->In(i).GetConnectedOutputSlot()->GetOwningLayer())) ins.push_back(&l->In(i));
        for (unsigned int i = 0; i < l->GetNumOutputSlots(); ++i)
        {
            bool leaves = false;
            for (InputSlot* c : l->Out(i).GetConnections()) leaves |= !members.count(&c->GetOwningLayer());
            if (leaves) outs.push_back(&l->Out(i));
        }
    }
    return SubgraphView(std::move(layers), std::move(ins), std::move(outs));
}

// Graph::SubstituteSubgraph (src/armnn/Graph.cpp:475-519): input slot i of the old view is re-fed into input slot i of
// the replacement, consumers of output slot i move to the replacement's output slot i, the old layers are erased.
void ApplySubstitution(Graph& graph, Graph& replacementOwner, const OptimizationViews::SubstitutionPair& s, const BackendId& backend)
{
    const SubgraphView& oldView = s.m_SubstitutableSubgraph;
    const SubgraphView& newView = s.m_ReplacementSubgraph;
    for (IConnectableLayer* il : newView.GetIConnectableLayers())
    {
        Layer* l = graph.Adopt(replacementOwner, PolymorphicDowncast<Layer*>(il));
        l->SetBackendId(backend);
    }
    for (size_t i = 0; i < oldView.GetIInputSlots().size(); ++i)
    {
        InputSlot* oldIn = PolymorphicDowncast<InputSlot*>(oldView.GetIInputSlots()[i]);
        OutputSlot* src = oldIn->GetConnectedOutputSlot();
        if (!src) throw GraphValidationException("substitution: boundary input slot is not connected");
        src->Disconnect(*oldIn);
        src->Connect(*newView.GetIInputSlots()[i]);
    }
    for (size_t i = 0; i < oldView.GetIOutputSlots().size(); ++i)
    {
        OutputSlot* oldOut = PolymorphicDowncast<OutputSlot*>(oldView.GetIOutputSlots()[i]);
        OutputSlot* newOut = PolymorphicDowncast<OutputSlot*>(newView.GetIOutputSlots()[i]);
        if (!newOut->IsTensorInfoSet()) newOut->SetTensorInfo(oldOut->GetTensorInfo());
        oldOut->MoveAllConnections(*newOut);
    }
    for (IConnectableLayer* il : oldView.GetIConnectableLayers()) graph.EraseLayer(PolymorphicDowncast<Layer*>(il));
}
} // namespace

IOptimizedNetworkPtr Optimize(const INetwork& network, const std::vector<BackendId>& backendPreferences, const IDeviceSpec& deviceSpec,
                              const OptimizerOptionsOpaque& options, Optional<std::vector<std::string>&> messages)
{
    if (backendPreferences.empty()) throw InvalidArgumentException("Invoked Optimize with no backends specified");
    std::unique_ptr<Graph> graph = network.GetGraph().Clone();
    std::vector<Layer*> order = graph->TopologicalSort();

    // every produced tensor must be described (Graph::VerifyConstantLayerSetTensorInfo / InferTensorInfos)
    for (Layer* l : order)
        for (unsigned int i = 0; i < l->GetNumOutputSlots(); ++i)
            if (!l->Out(i).IsTensorInfoSet())
                throw LayerValidationException(std::string("Output slot TensorInfo not set on ") + GetLayerTypeAsCString(l->GetType()) +
                                               " layer \"" + l->GetName() + "\"");

    // preferred backends the device actually has (src/armnn/Network.cpp:2081-2099)
    std::vector<BackendId> available;
    const BackendIdSet& supported = deviceSpec.GetSupportedBackends();
    for (const BackendId& b : backendPreferences)
    {
        if (supported.count(b)) available.push_back(b);
        else Report(messages, "WARNING: backend " + b.Get() + " is not available on this device and is ignored");
    }
    if (available.empty())
    {
        const std::string text = "None of the preferred backends " + [&] { std::string s = "["; for (auto& b : backendPreferences) s += b.Get() + " "; return s + "]"; }() +
                                 " are supported. Current platform provides " + BackendRegistryInstance().GetBackendIdsAsString();
        Report(messages, "ERROR: " + text);
        throw InvalidArgumentException(text);
    }

    // first available backend that supports the layer wins (AssignBackends, src/armnn/Network.cpp:1127-1268)
    for (Layer* l : order)
    {
        bool assigned = false;
        std::string reasons;
        for (const BackendId& b : available)
        {
            std::string reason;
            if (IWorkloadFactory::IsLayerSupported(b, *l, EmptyOptional(), reason, options.GetModelOptions()))
            {
                l->SetBackendId(b);
                assigned = true;
                break;
            }
            Report(messages, std::string("WARNING: Layer of type ") + GetLayerTypeAsCString(l->GetType()) + " is not supported on requested backend " +
                                 b.Get() + " (reason: " + reason + "), falling back to the next backend.");
            reasons += " " + b.Get() + ": " + reason + ";";
        }
        if (!assigned)
        {
            const std::string text = std::string("Layer of type ") + GetLayerTypeAsCString(l->GetType()) + " \"" + l->GetName() +
                                     "\" is not supported on any preferred backend:" + reasons;
            Report(messages, "ERROR: " + text);
            throw InvalidArgumentException(text);
        }
    }

    // per-backend optimisation (ApplyBackendOptimizations, src/armnn/Network.cpp:1271-1420)
    for (const BackendId& b : available)
    {
        order = graph->TopologicalSort();
        SubgraphView view = MakeBackendView(order, b);
        if (view.GetIConnectableLayers().empty()) continue;
        auto backend = BackendRegistryInstance().GetFactory(b)();
        OptimizationViews views = backend->OptimizeSubgraphView(view, options.GetModelOptions());
        if (!views.Validate(view)) throw GraphValidationException("backend " + b.Get() + " returned inconsistent OptimizationViews");
        for (const auto& s : views.GetSubstitutions()) ApplySubstitution(*graph, views.GetINetwork()->GetGraph(), s, b);
        for (const auto& d : views.GetDeletedSubgraphs())
            for (IConnectableLayer* il : d.GetIConnectableLayers()) graph->EraseLayer(PolymorphicDowncast<Layer*>(il));
        if (!views.GetFailedSubgraphs().empty())
            throw InvalidArgumentException("backend " + b.Get() + " failed to optimise a sub-graph it had accepted");
    }

    // MemCopy on every edge between two backends, owned by the consumer's backend (AddCompatibilityLayers,
    // src/armnn/Graph.cpp:330-472)
    order = graph->TopologicalSort();
    for (Layer* l : order)
    {
        if (l->GetType() == LayerType::MemCopy) continue;
        for (unsigned int o = 0; o < l->GetNumOutputSlots(); ++o)
        {
            std::map<BackendId, Layer*> copies;
            const std::vector<InputSlot*> consumers = l->Out(o).GetConnections();
            for (InputSlot* in : consumers)
            {
                Layer& dst = in->GetOwningLayer();
                if (dst.GetBackendId() == l->GetBackendId() || dst.GetType() == LayerType::MemCopy) continue;
                Layer*& copy = copies[dst.GetBackendId()];
                if (!copy)
                {
                    const std::string name = std::string("[ ") + l->GetName() + " (" + std::to_string(o) + ") -> " + dst.GetBackendId().Get() + " ]";
                    copy = graph->AddLayer(LayerType::MemCopy, name.c_str(), 1, 1, nullptr);
                    copy->SetBackendId(dst.GetBackendId());
                    copy->Out(0).SetTensorInfo(l->Out(o).GetTensorInfo());
                    l->Out(o).Connect(copy->In(0));
                }
                l->Out(o).Disconnect(*in);
                copy->Out(0).Connect(*in);
            }
        }
    }
    graph->TopologicalSort();
    return IOptimizedNetworkPtr(new IOptimizedNetwork(std::move(graph), options.GetModelOptions()), &IOptimizedNetwork::Destroy);
}
} // namespace armnn
