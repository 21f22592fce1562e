// Minimal host core: the process-wide backend registry (include/armnn/BackendRegistry.hpp:35-89,
// behaviour of src/armnn/BackendRegistry.cpp:21-60).
#pragma once
#include "BackendId.hpp"
#include <functional>
#include <memory>
#include <string>
#include <unordered_map>

namespace armnn
{
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
};

BackendRegistry& BackendRegistryInstance();
} // namespace armnn
