// Minimal host core: the graph-building API with the names of include/armnn/INetwork.hpp
// (IInputSlot/IOutputSlot :29-78, IConnectableLayer :80-156, INetwork::AddXxxLayer :361-684, Optimize :956-985).
#pragma once
#include "BackendId.hpp"
#include "BackendOptions.hpp"
#include "Descriptors.hpp"
#include "Optional.hpp"
#include "Tensor.hpp"
#include "Types.hpp"
#include <memory>
#include <string>
#include <vector>

namespace armnn
{
class IConnectableLayer;
class IOutputSlot;

class IInputSlot
{
public:
    virtual const IOutputSlot* GetConnection() const = 0;
    virtual IOutputSlot* GetConnection() = 0;
    virtual const IConnectableLayer& GetOwningIConnectableLayer() const = 0;
    virtual IConnectableLayer& GetOwningIConnectableLayer() = 0;
    virtual unsigned int GetSlotIndex() const = 0;
protected:
    ~IInputSlot() {}
};

class IOutputSlot
{
public:
    virtual unsigned int GetNumConnections() const = 0;
    virtual const IInputSlot* GetConnection(unsigned int index) const = 0;
    virtual IInputSlot* GetConnection(unsigned int outputindex) = 0;
    virtual void SetTensorInfo(const TensorInfo& tensorInfo) = 0;
    virtual const TensorInfo& GetTensorInfo() const = 0;
    virtual bool IsTensorInfoSet() const = 0;
    virtual int Connect(IInputSlot& destination) = 0;
    virtual void Disconnect(IInputSlot& slot) = 0;
    virtual unsigned int CalculateIndexOnOwner() const = 0;
    virtual LayerGuid GetOwningLayerGuid() const = 0;
    virtual const IConnectableLayer& GetOwningIConnectableLayer() const = 0;
    virtual IConnectableLayer& GetOwningIConnectableLayer() = 0;
protected:
    ~IOutputSlot() {}
};

class IConnectableLayer
{
public:
    virtual const char* GetName() const = 0;
    virtual unsigned int GetNumInputSlots() const = 0;
    virtual unsigned int GetNumOutputSlots() const = 0;
    virtual const IInputSlot& GetInputSlot(unsigned int index) const = 0;
    virtual IInputSlot& GetInputSlot(unsigned int index) = 0;
    virtual const IOutputSlot& GetOutputSlot(unsigned int index) const = 0;
    virtual IOutputSlot& GetOutputSlot(unsigned int index) = 0;
    virtual LayerGuid GetGuid() const = 0;
    virtual void BackendSelectionHint(Optional<BackendId> backend) = 0;
    virtual LayerType GetType() const = 0;
    virtual const BaseDescriptor& GetParameters() const = 0;
    virtual void SetBackendId(const BackendId& id) = 0;
protected:
    ~IConnectableLayer() {}
};

struct OptimizerOptionsOpaque
{
    bool m_ReduceFp32ToFp16 = false;
    bool m_Debug = false;
    ModelOptions m_ModelOptions;
    void AddModelOption(const BackendOptions& o) { m_ModelOptions.push_back(o); }
    const ModelOptions& GetModelOptions() const { return m_ModelOptions; }
};

class Graph;
class INetwork;
using INetworkPtr = std::unique_ptr<INetwork, void (*)(INetwork* network)>;

class INetwork
{
public:
    static INetwork* CreateRaw(const NetworkOptions& networkOptions = {});
    static INetworkPtr Create(const NetworkOptions& networkOptions = {});
    static void Destroy(INetwork* network);

    IConnectableLayer* AddInputLayer(LayerBindingId id, const char* name = nullptr);
    IConnectableLayer* AddOutputLayer(LayerBindingId id, const char* name = nullptr);
    IConnectableLayer* AddConstantLayer(const ConstTensor& input, const char* name = nullptr);
    /// weights are input slot 1 and biases input slot 2, normally fed by Constant layers
    IConnectableLayer* AddConvolution2dLayer(const Convolution2dDescriptor& descriptor, const char* name = nullptr);
    IConnectableLayer* AddDepthwiseConvolution2dLayer(const DepthwiseConvolution2dDescriptor& descriptor, const char* name = nullptr);
    IConnectableLayer* AddFullyConnectedLayer(const FullyConnectedDescriptor& descriptor, const char* name = nullptr);
    IConnectableLayer* AddActivationLayer(const ActivationDescriptor& descriptor, const char* name = nullptr);
    IConnectableLayer* AddPooling2dLayer(const Pooling2dDescriptor& descriptor, const char* name = nullptr);
    IConnectableLayer* AddMeanLayer(const MeanDescriptor& descriptor, const char* name = nullptr);
    IConnectableLayer* AddPadLayer(const PadDescriptor& descriptor, const char* name = nullptr);
    IConnectableLayer* AddSoftmaxLayer(const SoftmaxDescriptor& descriptor, const char* name = nullptr);
    IConnectableLayer* AddElementwiseBinaryLayer(const ElementwiseBinaryDescriptor& descriptor, const char* name = nullptr);
    IConnectableLayer* AddReshapeLayer(const ReshapeDescriptor& descriptor, const char* name = nullptr);

    Graph& GetGraph();
    const Graph& GetGraph() const;
    ~INetwork();
protected:
    INetwork(const NetworkOptions& networkOptions);
private:
    std::unique_ptr<Graph> m_Graph;
};

class IOptimizedNetwork;
using IOptimizedNetworkPtr = std::unique_ptr<IOptimizedNetwork, void (*)(IOptimizedNetwork* network)>;

class IOptimizedNetwork
{
public:
    static void Destroy(IOptimizedNetwork* network);
    Graph& GetGraph();
    const Graph& GetGraph() const;
    const ModelOptions& GetModelOptions() const { return m_ModelOptions; }
    size_t GetNumInputs() const;
    size_t GetNumOutputs() const;
    ~IOptimizedNetwork();
    IOptimizedNetwork(std::unique_ptr<Graph> graph, const ModelOptions& modelOptions);
private:
    std::unique_ptr<Graph> m_Graph;
    ModelOptions m_ModelOptions;
};

/// The optimized graph, for tests and tools that count or inspect its layers (declared a friend of IOptimizedNetwork in
/// include/armnn/INetwork.hpp:929 and defined by the test utilities, src/armnnTestUtils/TestUtils.cpp:49-52).
Graph& GetGraphForTesting(IOptimizedNetwork* optNetPtr);

/// Assign every layer to the first backend of `backendPreferences` that is available and supports it, let each
/// backend substitute sub-graphs it can fuse, and return the result (src/armnn/Network.cpp:2026-2271).
/// Throws InvalidArgumentException when a layer is supported by none of the preferred backends.
IOptimizedNetworkPtr Optimize(const INetwork& network, const std::vector<BackendId>& backendPreferences,
                              const IDeviceSpec& deviceSpec, const OptimizerOptionsOpaque& options = OptimizerOptionsOpaque(),
                              Optional<std::vector<std::string>&> messages = EmptyOptional());
} // namespace armnn
