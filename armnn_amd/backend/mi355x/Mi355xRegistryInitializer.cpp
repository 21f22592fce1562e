// Static registration, as every in-tree backend does (src/backends/reference/RefRegistryInitializer.cpp:13-22):
// linking this object into the Arm NN library makes "Mi355x" known to BackendRegistryInstance() before main().
#include "Mi355xBackend.hpp"

#include <armnn/BackendRegistry.hpp>

namespace
{
using namespace armnn;
static BackendRegistry::StaticRegistryInitializer g_RegisterHelper{
    BackendRegistryInstance(), Mi355xBackend::GetIdStatic(),
    []() { return IBackendInternalUniquePtr(new Mi355xBackend); }};
} // namespace
