// Minimal host core: the slice of a graph handed to IBackendInternal::OptimizeSubgraphView
// (include/armnn/backends/SubgraphView.hpp), reduced to layer lists and boundary slots.
#pragma once
#include "../INetwork.hpp"
#include <list>
#include <memory>
#include <vector>

namespace armnn
{
class SubgraphView final
{
public:
    using IConnectableLayers = std::list<IConnectableLayer*>;
    using IInputSlots = std::vector<IInputSlot*>;
    using IOutputSlots = std::vector<IOutputSlot*>;
    using SubgraphViewPtr = std::shared_ptr<SubgraphView>;

    SubgraphView() = default;
    SubgraphView(IConnectableLayers&& layers, IInputSlots&& inputs, IOutputSlots&& outputs)
        : m_Layers(std::move(layers)), m_InputSlots(std::move(inputs)), m_OutputSlots(std::move(outputs)) {}
    /// a view of one layer: all of its input slots and output slots are the boundary
    SubgraphView(IConnectableLayer* layer);

    const IConnectableLayers& GetIConnectableLayers() const { return m_Layers; }
    const IInputSlots& GetIInputSlots() const { return m_InputSlots; }
    const IOutputSlots& GetIOutputSlots() const { return m_OutputSlots; }
    unsigned int GetNumInputSlots() const { return static_cast<unsigned int>(m_InputSlots.size()); }
    unsigned int GetNumOutputSlots() const { return static_cast<unsigned int>(m_OutputSlots.size()); }
    IConnectableLayers::const_iterator begin() const { return m_Layers.begin(); }
    IConnectableLayers::const_iterator end() const { return m_Layers.end(); }
private:
    IConnectableLayers m_Layers;
    IInputSlots m_InputSlots;
    IOutputSlots m_OutputSlots;
};
} // namespace armnn
