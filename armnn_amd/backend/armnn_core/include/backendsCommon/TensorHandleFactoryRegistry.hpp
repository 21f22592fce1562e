// Minimal host core: src/backends/backendsCommon/TensorHandleFactoryRegistry.hpp:23-67.
#pragma once
#include <armnn/backends/IMemoryManager.hpp>
#include <armnn/backends/ITensorHandleFactory.hpp>
#include <map>
#include <memory>
#include <vector>

namespace armnn
{
class TensorHandleFactoryRegistry
{
public:
    TensorHandleFactoryRegistry() = default;
    TensorHandleFactoryRegistry(const TensorHandleFactoryRegistry&) = delete;
    TensorHandleFactoryRegistry(TensorHandleFactoryRegistry&&) = delete;
    void RegisterFactory(std::unique_ptr<ITensorHandleFactory> allocator);
    void RegisterMemoryManager(std::shared_ptr<IMemoryManager> memoryManger);
    ITensorHandleFactory* GetFactory(ITensorHandleFactory::FactoryId id) const;
    void RegisterCopyAndImportFactoryPair(ITensorHandleFactory::FactoryId copyFactoryId, ITensorHandleFactory::FactoryId importFactoryId);
    ITensorHandleFactory::FactoryId GetMatchingImportFactoryId(ITensorHandleFactory::FactoryId copyFactoryId);
    void AquireMemory();
    void ReleaseMemory();
    std::vector<std::shared_ptr<IMemoryManager>>& GetMemoryManagers() { return m_MemoryManagers; }
private:
    std::vector<std::unique_ptr<ITensorHandleFactory>> m_Factories;
    std::vector<std::shared_ptr<IMemoryManager>> m_MemoryManagers;
    std::map<ITensorHandleFactory::FactoryId, ITensorHandleFactory::FactoryId> m_FactoryMappings;
};
} // namespace armnn
