// Minimal host core: graph nodes, slots, the Graph container and the INetwork builder on top of it.
#include <Layer.hpp>
#include <armnn/INetwork.hpp>
#include <armnn/backends/SubgraphView.hpp>

#include <algorithm>
#include <atomic>
#include <map>

namespace armnn
{
namespace
{
std::atomic<uint64_t> g_NextGuid{1};
}

// ---- slots ---------------------------------------------------------------------------------------------------
const IOutputSlot* InputSlot::GetConnection() const { return m_Connection; }
IOutputSlot* InputSlot::GetConnection() { return m_Connection; }
const IConnectableLayer& InputSlot::GetOwningIConnectableLayer() const { return m_Owner; }
IConnectableLayer& InputSlot::GetOwningIConnectableLayer() { return m_Owner; }

const IInputSlot* OutputSlot::GetConnection(unsigned int index) const { return m_Connections.at(index); }
IInputSlot* OutputSlot::GetConnection(unsigned int index) { return m_Connections.at(index); }
LayerGuid OutputSlot::GetOwningLayerGuid() const { return m_Owner.GetGuid(); }
const IConnectableLayer& OutputSlot::GetOwningIConnectableLayer() const { return m_Owner; }
IConnectableLayer& OutputSlot::GetOwningIConnectableLayer() { return m_Owner; }
void OutputSlot::SetTensorHandle(std::unique_ptr<ITensorHandle> h) { m_Handle = std::move(h); }

int OutputSlot::Connect(IInputSlot& destination)
{
    InputSlot& in = *PolymorphicDowncast<InputSlot*>(&destination);
    if (in.GetConnectedOutputSlot() != nullptr) throw InvalidArgumentException("Connect: the input slot is already connected");
    in.SetConnection(this);
    m_Connections.push_back(&in);
    return static_cast<int>(m_Connections.size()) - 1;
}

void OutputSlot::Disconnect(IInputSlot& slot)
{
    InputSlot& in = *PolymorphicDowncast<InputSlot*>(&slot);
    auto it = std::find(m_Connections.begin(), m_Connections.end(), &in);
    if (it == m_Connections.end()) return;
    m_Connections.erase(it);
    in.SetConnection(nullptr);
}

void OutputSlot::MoveAllConnections(OutputSlot& destination)
{
    while (!m_Connections.empty())
    {
        InputSlot* in = m_Connections.front();
        Disconnect(*in);
        destination.Connect(*in);
    }
}

// ---- Layer -----------------------------------------------------------------------------------------------------
Layer::Layer(LayerType type, const char* name, unsigned int numInputs, unsigned int numOutputs, std::shared_ptr<BaseDescriptor> params)
    : m_Type(type), m_Name(name ? name : ""), m_Params(params ? std::move(params) : std::make_shared<NullDescriptor>()),
      m_Guid(g_NextGuid.fetch_add(1))
{
    for (unsigned int i = 0; i < numInputs; ++i) m_InputSlots.emplace_back(new InputSlot(*this, i));
    for (unsigned int i = 0; i < numOutputs; ++i) m_OutputSlots.emplace_back(new OutputSlot(*this, i));
}

// ---- Graph -----------------------------------------------------------------------------------------------------
Layer* Graph::AddLayer(LayerType type, const char* name, unsigned int numInputs, unsigned int numOutputs,
                       std::shared_ptr<BaseDescriptor> params)
{
    m_Layers.emplace_back(new Layer(type, name, numInputs, numOutputs, std::move(params)));
    return m_Layers.back().get();
}

Layer* Graph::Adopt(Graph& other, Layer* layer)
{
    for (auto it = other.m_Layers.begin(); it != other.m_Layers.end(); ++it)
    {
        if (it->get() == layer)
        {
            m_Layers.push_back(std::move(*it));
            other.m_Layers.erase(it);
            return layer;
        }
    }
    throw InvalidArgumentException("Graph::Adopt: the layer does not belong to the source graph");
}

void Graph::EraseLayer(Layer* layer)
{
    for (unsigned int i = 0; i < layer->GetNumInputSlots(); ++i)
        if (OutputSlot* src = layer->In(i).GetConnectedOutputSlot()) src->Disconnect(layer->In(i));
    for (unsigned int i = 0; i < layer->GetNumOutputSlots(); ++i)
        while (layer->Out(i).GetNumConnections() > 0) layer->Out(i).Disconnect(*layer->Out(i).GetConnections().front());
    auto it = std::find_if(m_Layers.begin(), m_Layers.end(), [&](const std::unique_ptr<Layer>& p) { return p.get() == layer; });
    if (it != m_Layers.end()) m_Layers.erase(it);
}

std::unique_ptr<Graph> Graph::Clone() const
{
    auto g = std::make_unique<Graph>();
    std::map<const Layer*, Layer*> twin;
    for (const auto& l : m_Layers)
    {
        Layer* c = g->AddLayer(l->GetType(), l->GetName(), l->GetNumInputSlots(), l->GetNumOutputSlots(), l->GetParametersPtr());
        c->SetBackendId(l->GetBackendId());
        c->SetBindingId(l->GetBindingId());
        c->m_LayerOutput = l->m_LayerOutput;
        c->SetAdditionalInfoForObject(l->GetAdditionalInformation<void>());
        for (unsigned int i = 0; i < l->GetNumOutputSlots(); ++i)
            if (l->Out(i).IsTensorInfoSet()) c->Out(i).SetTensorInfo(l->Out(i).GetTensorInfo());
        twin[l.get()] = c;
    }
    for (const auto& l : m_Layers)
        for (unsigned int i = 0; i < l->GetNumInputSlots(); ++i)
            if (const OutputSlot* src = l->In(i).GetConnectedOutputSlot())
                twin[&src->GetOwningLayer()]->Out(src->CalculateIndexOnOwner()).Connect(twin[l.get()]->In(i));
    return g;
}

std::vector<Layer*> Graph::TopologicalSort() const
{
    std::map<const Layer*, unsigned int> pending;
    std::vector<Layer*> ready, order;
    for (const auto& l : m_Layers)
    {
        unsigned int n = 0;
        for (unsigned int i = 0; i < l->GetNumInputSlots(); ++i)
        {
            if (l->In(i).GetConnectedOutputSlot() == nullptr)
                throw GraphValidationException(std::string("Layer '") + l->GetName() + "' has an unconnected input slot");
            ++n;
        }
        pending[l.get()] = n;
        if (n == 0) ready.push_back(l.get());
    }
    size_t head = 0;
    while (head < ready.size())
    {
        Layer* l = ready[head++];
        order.push_back(l);
        for (unsigned int i = 0; i < l->GetNumOutputSlots(); ++i)
            for (InputSlot* in : l->Out(i).GetConnections())
                if (--pending[&in->GetOwningLayer()] == 0) ready.push_back(&in->GetOwningLayer());
    }
    if (order.size() != m_Layers.size()) throw GraphValidationException("Graph contains a cycle");
    return order;
}

// ---- SubgraphView of a single layer ------------------------------------------------------------------------
SubgraphView::SubgraphView(IConnectableLayer* layer)
{
    m_Layers.push_back(layer);
    for (unsigned int i = 0; i < layer->GetNumInputSlots(); ++i) m_InputSlots.push_back(&layer->GetInputSlot(i));
    for (unsigned int i = 0; i < layer->GetNumOutputSlots(); ++i) m_OutputSlots.push_back(&layer->GetOutputSlot(i));
}

// ---- INetwork ----------------------------------------------------------------------------------------------
INetwork::INetwork(const NetworkOptions&) : m_Graph(new Graph) {}
INetwork::~INetwork() = default;
INetwork* INetwork::CreateRaw(const NetworkOptions& o) { return new INetwork(o); }
INetworkPtr INetwork::Create(const NetworkOptions& o) { return INetworkPtr(CreateRaw(o), &INetwork::Destroy); }
void INetwork::Destroy(INetwork* n) { delete n; }
Graph& INetwork::GetGraph() { return *m_Graph; }
const Graph& INetwork::GetGraph() const { return *m_Graph; }

IConnectableLayer* INetwork::AddInputLayer(LayerBindingId id, const char* name)
{
    Layer* l = m_Graph->AddLayer(LayerType::Input, name, 0, 1, nullptr);
    l->SetBindingId(id);
    return l;
}
IConnectableLayer* INetwork::AddOutputLayer(LayerBindingId id, const char* name)
{
    Layer* l = m_Graph->AddLayer(LayerType::Output, name, 1, 0, nullptr);
    l->SetBindingId(id);
    return l;
}
IConnectableLayer* INetwork::AddConstantLayer(const ConstTensor& input, const char* name)
{
    Layer* l = m_Graph->AddLayer(LayerType::Constant, name, 0, 1, nullptr);
    l->m_LayerOutput = std::make_shared<ScopedTensorHandle>(input);
    l->Out(0).SetTensorInfo(input.GetInfo());
    return l;
}
IConnectableLayer* INetwork::AddConvolution2dLayer(const Convolution2dDescriptor& d, const char* name)
{
    return m_Graph->AddLayer(LayerType::Convolution2d, name, d.GetNumInputs(), 1, std::make_shared<Convolution2dDescriptor>(d));
}
IConnectableLayer* INetwork::AddDepthwiseConvolution2dLayer(const DepthwiseConvolution2dDescriptor& d, const char* name)
{
    return m_Graph->AddLayer(LayerType::DepthwiseConvolution2d, name, d.GetNumInputs(), 1, std::make_shared<DepthwiseConvolution2dDescriptor>(d));
}
IConnectableLayer* INetwork::AddFullyConnectedLayer(const FullyConnectedDescriptor& d, const char* name)
{
    return m_Graph->AddLayer(LayerType::FullyConnected, name, d.GetNumInputs(), 1, std::make_shared<FullyConnectedDescriptor>(d));
}
IConnectableLayer* INetwork::AddActivationLayer(const ActivationDescriptor& d, const char* name)
{
    return m_Graph->AddLayer(LayerType::Activation, name, 1, 1, std::make_shared<ActivationDescriptor>(d));
}
IConnectableLayer* INetwork::AddPooling2dLayer(const Pooling2dDescriptor& d, const char* name)
{
    return m_Graph->AddLayer(LayerType::Pooling2d, name, 1, 1, std::make_shared<Pooling2dDescriptor>(d));
}
IConnectableLayer* INetwork::AddMeanLayer(const MeanDescriptor& d, const char* name)
{
    return m_Graph->AddLayer(LayerType::Mean, name, 1, 1, std::make_shared<MeanDescriptor>(d));
}
IConnectableLayer* INetwork::AddPadLayer(const PadDescriptor& d, const char* name)
{
    return m_Graph->AddLayer(LayerType::Pad, name, 1, 1, std::make_shared<PadDescriptor>(d));
}
IConnectableLayer* INetwork::AddSoftmaxLayer(const SoftmaxDescriptor& d, const char* name)
{
    return m_Graph->AddLayer(LayerType::Softmax, name, 1, 1, std::make_shared<SoftmaxDescriptor>(d));
}
IConnectableLayer* INetwork::AddElementwiseBinaryLayer(const ElementwiseBinaryDescriptor& d, const char* name)
{
    return m_Graph->AddLayer(LayerType::ElementwiseBinary, name, 2, 1, std::make_shared<ElementwiseBinaryDescriptor>(d));
}
IConnectableLayer* INetwork::AddReshapeLayer(const ReshapeDescriptor& d, const char* name)
{
    return m_Graph->AddLayer(LayerType::Reshape, name, 1, 1, std::make_shared<ReshapeDescriptor>(d));
}

IOptimizedNetwork::IOptimizedNetwork(std::unique_ptr<Graph> graph, const ModelOptions& modelOptions)
    : m_Graph(std::move(graph)), m_ModelOptions(modelOptions) {}
IOptimizedNetwork::~IOptimizedNetwork() = default;
void IOptimizedNetwork::Destroy(IOptimizedNetwork* n) { delete n; }
Graph& IOptimizedNetwork::GetGraph() { return *m_Graph; }
const Graph& IOptimizedNetwork::GetGraph() const { return *m_Graph; }
Graph& GetGraphForTesting(IOptimizedNetwork* optNetPtr) { return optNetPtr->GetGraph(); }
size_t IOptimizedNetwork::GetNumInputs() const
{
    size_t n = 0;
    for (const auto& l : m_Graph->GetLayers()) n += l->GetType() == LayerType::Input;
    return n;
}
size_t IOptimizedNetwork::GetNumOutputs() const
{
    size_t n = 0;
    for (const auto& l : m_Graph->GetLayers()) n += l->GetType() == LayerType::Output;
    return n;
}
} // namespace armnn
