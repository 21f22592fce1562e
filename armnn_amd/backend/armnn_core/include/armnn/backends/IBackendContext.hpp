// Minimal host core: include/armnn/backends/IBackendContext.hpp:14-32.
#pragma once
#include "../IRuntime.hpp"
#include <memory>
namespace armnn
{
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
