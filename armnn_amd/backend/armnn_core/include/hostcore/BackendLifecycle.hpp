// Minimal host core: how a backend enters the process and follows the runtime's life -- the process-wide registry
// (include/armnn/BackendRegistry.hpp:35-89, behaviour of src/armnn/BackendRegistry.cpp:21-60) and the per-runtime
// context with its load / unload / enqueue hooks (include/armnn/backends/IBackendContext.hpp:14-32).  The Arm NN-named
// headers forward here.
#pragma once
#include <armnn/BackendId.hpp>
#include <armnn/IRuntime.hpp>
#include <functional>
#include <memory>
#include <string>
#include <unordered_map>

namespace armnn
{
// ---- registry ------------------------------------------------------------------------------------------------------
class IBackendInternal;
using IBackendInternalUniquePtr = std::unique_ptr<IBackendInternal>;

class BackendRegistry
{
public:
    using PointerType = IBackendInternalUniquePtr;
    using FactoryFunction = std::function<PointerType()>;

    void Register(const BackendId& id, FactoryFunction factory);      ///< throws InvalidArgumentException on a duplicate id
    bool IsBackendRegistered(const BackendId& id) const;
    FactoryFunction GetFactory(const BackendId& id) const;            ///< throws InvalidArgumentException when unknown
    size_t Size() const;
    BackendIdSet GetBackendIds() const;
    std::string GetBackendIdsAsString() const;
    void Deregister(const BackendId& id);
    /// allocators and memory optimizer strategies callers chose per backend (BackendRegistry.hpp:48-58)
    void RegisterAllocator(const BackendId& id, std::shared_ptr<ICustomAllocator> alloc);
    std::unordered_map<BackendId, std::shared_ptr<ICustomAllocator>> GetAllocators();
    void DeregisterAllocator(const BackendId& id);
    void RegisterMemoryOptimizerStrategy(const BackendId& id, std::shared_ptr<IMemoryOptimizerStrategy> strategy);
    std::unordered_map<BackendId, std::shared_ptr<IMemoryOptimizerStrategy>> GetMemoryOptimizerStrategies();
    void DeregisterMemoryOptimizerStrategy(const BackendId& id);

    BackendRegistry() {}
    virtual ~BackendRegistry() {}

    struct StaticRegistryInitializer
    {
        StaticRegistryInitializer(BackendRegistry& instance, const BackendId& id, FactoryFunction factory)
        {
            instance.Register(id, factory);
        }
    };
private:
    BackendRegistry(const BackendRegistry&) = delete;
    BackendRegistry& operator=(const BackendRegistry&) = delete;
    std::unordered_map<BackendId, FactoryFunction> m_Factories;
    std::unordered_map<BackendId, std::shared_ptr<ICustomAllocator>> m_CustomMemoryAllocatorMap;
    std::unordered_map<BackendId, std::shared_ptr<IMemoryOptimizerStrategy>> m_MemoryOptimizerStrategyMap;
};

BackendRegistry& BackendRegistryInstance();

// ---- per-runtime context -------------------------------------------------------------------------------------------
class IBackendContext
{
protected:
    IBackendContext(const IRuntime::CreationOptions&) {}
public:
    virtual bool BeforeLoadNetwork(NetworkId networkId) = 0;
    virtual bool AfterLoadNetwork(NetworkId networkId) = 0;
    virtual bool BeforeUnloadNetwork(NetworkId networkId) = 0;
    virtual bool AfterUnloadNetwork(NetworkId networkId) = 0;
    virtual bool AfterEnqueueWorkload(NetworkId networkId) = 0;
    virtual ~IBackendContext() {}
};
using IBackendContextUniquePtr = std::unique_ptr<IBackendContext>;
class IBackendModelContext
{
public:
    virtual ~IBackendModelContext() {}
};
} // namespace armnn
