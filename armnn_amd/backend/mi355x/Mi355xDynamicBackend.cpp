// The three C symbols the runtime's dynamic backend loader looks up in <vendor>_<name>_backend.so
// (include/armnn/backends/DynamicBackend.hpp:41-43, src/backends/backendsCommon/DynamicBackendUtils.cpp).
#include "Mi355xBackend.hpp"
#include "Mi355xBackendId.hpp"

extern "C"
{
const char* GetBackendId() { return armnn::Mi355xBackendId(); }

void GetVersion(uint32_t* outMajor, uint32_t* outMinor)
{
    if (!outMajor || !outMinor) return;
    const armnn::BackendVersion v = armnn::IBackendInternal::GetApiVersion();
    *outMajor = v.m_Major;
    *outMinor = v.m_Minor;
}

void* BackendFactory() { return new armnn::Mi355xBackend(); }
}
