// Minimal host core: the C ABI of a dynamically loaded backend (include/armnn/backends/DynamicBackend.hpp:41-43):
//   extern "C" const char* GetBackendId();  void GetVersion(uint32_t* major, uint32_t* minor);  void* BackendFactory();
// BackendFactory returns a heap IBackendInternal*; ownership passes to the runtime.
#pragma once
#include "IBackendInternal.hpp"
#include <string>
#include <vector>

namespace armnn
{
class DynamicBackendUtils
{
public:
    /// file names matching ^[a-zA-Z0-9]+_[a-zA-Z0-9]+_backend.so(\.[0-9]+)*$ in `path`
    /// (src/backends/backendsCommon/DynamicBackendUtils.cpp:228-231)
    static std::vector<std::string> GetSharedObjects(const std::string& path);
    static bool IsBackendCompatible(const BackendVersion& backendVersion);
    /// dlopen each object, check symbols and version, register the factory; returns the ids registered
    static BackendIdSet RegisterDynamicBackends(const std::vector<std::string>& sharedObjects);
};
} // namespace armnn
