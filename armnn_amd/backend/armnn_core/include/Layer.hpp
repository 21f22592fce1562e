// Minimal host core: the concrete graph node behind IConnectableLayer.  Backends reach it the way the reference's
// backends reach src/armnn/Layer.hpp: PolymorphicDowncast<Layer*>(iconnectableLayer), to attach an "additional info"
// object (e.g. the ActivationDescriptor fused into a convolution, src/armnn/Layer.hpp:429-433).
#pragma once
#include <armnn/INetwork.hpp>
#include <armnn/backends/TensorHandle.hpp>
#include <armnn/utility/PolymorphicDowncast.hpp>
#include <memory>
#include <string>
#include <vector>

namespace armnn
{
class Layer;
class ITensorHandle;
using AdditionalInfoObjectPtr = std::shared_ptr<void>;

class OutputSlot;
class InputSlot final : public IInputSlot
{
public:
    InputSlot(Layer& owner, unsigned int index) : m_Owner(owner), m_Index(index) {}
    const IOutputSlot* GetConnection() const override;
    IOutputSlot* GetConnection() override;
    const IConnectableLayer& GetOwningIConnectableLayer() const override;
    IConnectableLayer& GetOwningIConnectableLayer() override;
    unsigned int GetSlotIndex() const override { return m_Index; }
    OutputSlot* GetConnectedOutputSlot() const { return m_Connection; }
    void SetConnection(OutputSlot* source) { m_Connection = source; }
    Layer& GetOwningLayer() const { return m_Owner; }
private:
    Layer& m_Owner;
    unsigned int m_Index;
    OutputSlot* m_Connection = nullptr;
};

class OutputSlot final : public IOutputSlot
{
public:
    OutputSlot(Layer& owner, unsigned int index) : m_Owner(owner), m_Index(index) {}
    unsigned int GetNumConnections() const override { return static_cast<unsigned int>(m_Connections.size()); }
    const IInputSlot* GetConnection(unsigned int index) const override;
    IInputSlot* GetConnection(unsigned int index) override;
    void SetTensorInfo(const TensorInfo& tensorInfo) override { m_TensorInfo = tensorInfo; m_InfoSet = true; }
    const TensorInfo& GetTensorInfo() const override { return m_TensorInfo; }
    bool IsTensorInfoSet() const override { return m_InfoSet; }
    int Connect(IInputSlot& destination) override;
    void Disconnect(IInputSlot& slot) override;
    unsigned int CalculateIndexOnOwner() const override { return m_Index; }
    LayerGuid GetOwningLayerGuid() const override;
    const IConnectableLayer& GetOwningIConnectableLayer() const override;
    IConnectableLayer& GetOwningIConnectableLayer() override;
    Layer& GetOwningLayer() const { return m_Owner; }
    const std::vector<InputSlot*>& GetConnections() const { return m_Connections; }
    /// move every consumer of this slot over to `destination`
    void MoveAllConnections(OutputSlot& destination);
    ITensorHandle* GetTensorHandle() const { return m_Handle.get(); }
    void SetTensorHandle(std::unique_ptr<ITensorHandle> h);
private:
    Layer& m_Owner;
    unsigned int m_Index;
    std::vector<InputSlot*> m_Connections;
    TensorInfo m_TensorInfo;
    bool m_InfoSet = false;
    std::shared_ptr<ITensorHandle> m_Handle;
};

class Layer final : public IConnectableLayer
{
public:
    Layer(LayerType type, const char* name, unsigned int numInputs, unsigned int numOutputs,
          std::shared_ptr<BaseDescriptor> params);
    const char* GetName() const override { return m_Name.c_str(); }
    const std::string& GetNameStr() const { return m_Name; }
    unsigned int GetNumInputSlots() const override { return static_cast<unsigned int>(m_InputSlots.size()); }
    unsigned int GetNumOutputSlots() const override { return static_cast<unsigned int>(m_OutputSlots.size()); }
    // covariant returns, as in src/armnn/Layer.hpp:339-342: code holding a Layer gets the concrete slot types
    const InputSlot& GetInputSlot(unsigned int index) const override { return *m_InputSlots.at(index); }
    InputSlot& GetInputSlot(unsigned int index) override { return *m_InputSlots.at(index); }
    const OutputSlot& GetOutputSlot(unsigned int index = 0) const override { return *m_OutputSlots.at(index); }
    OutputSlot& GetOutputSlot(unsigned int index = 0) override { return *m_OutputSlots.at(index); }
    InputSlot& In(unsigned int i) { return *m_InputSlots.at(i); }
    OutputSlot& Out(unsigned int i) { return *m_OutputSlots.at(i); }
    const InputSlot& In(unsigned int i) const { return *m_InputSlots.at(i); }
    const OutputSlot& Out(unsigned int i) const { return *m_OutputSlots.at(i); }
    LayerGuid GetGuid() const override { return m_Guid; }
    void BackendSelectionHint(Optional<BackendId> backend) override { m_Hint = backend; }
    LayerType GetType() const override { return m_Type; }
    const BaseDescriptor& GetParameters() const override { return *m_Params; }
    std::shared_ptr<BaseDescriptor> GetParametersPtr() const { return m_Params; }
    void SetBackendId(const BackendId& id) override { m_BackendId = id; }
    const BackendId& GetBackendId() const { return m_BackendId; }

    template <typename T>
    std::shared_ptr<T> GetAdditionalInformation() const { return std::static_pointer_cast<T>(m_AdditionalInfoObject); }
    void SetAdditionalInfoForObject(const AdditionalInfoObjectPtr& additionalInfo) { m_AdditionalInfoObject = additionalInfo; }

    // Input / Output layers
    LayerBindingId GetBindingId() const { return m_BindingId; }
    void SetBindingId(LayerBindingId id) { m_BindingId = id; }
    // Constant layers
    std::shared_ptr<ConstTensorHandle> m_LayerOutput;
private:
    LayerType m_Type;
    std::string m_Name;
    std::vector<std::unique_ptr<InputSlot>> m_InputSlots;
    std::vector<std::unique_ptr<OutputSlot>> m_OutputSlots;
    std::shared_ptr<BaseDescriptor> m_Params;
    BackendId m_BackendId;
    Optional<BackendId> m_Hint;
    AdditionalInfoObjectPtr m_AdditionalInfoObject;
    LayerBindingId m_BindingId = 0;
    LayerGuid m_Guid;
};

/// Owns the layers of a network.
class Graph
{
public:
    Graph() = default;
    Layer* AddLayer(LayerType type, const char* name, unsigned int numInputs, unsigned int numOutputs,
                    std::shared_ptr<BaseDescriptor> params);
    /// take ownership of a layer created in another graph (substitution replacements)
    Layer* Adopt(Graph& other, Layer* layer);
    void EraseLayer(Layer* layer);
    std::unique_ptr<Graph> Clone() const;
    /// layers with every producer before its consumers; throws GraphValidationException on a cycle or a dangling input
    std::vector<Layer*> TopologicalSort() const;
    const std::vector<std::unique_ptr<Layer>>& GetLayers() const { return m_Layers; }
    /// `for (auto&& layer : graph)` as with the reference's Graph (src/armnn/Graph.hpp:169-186); elements act as Layer*
    auto begin() const { return m_Layers.begin(); }
    auto end() const { return m_Layers.end(); }
    size_t GetNumLayers() const { return m_Layers.size(); }
private:
    std::vector<std::unique_ptr<Layer>> m_Layers;
};
} // namespace armnn
