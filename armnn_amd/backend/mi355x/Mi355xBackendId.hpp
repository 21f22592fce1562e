// Backend id, as RefBackendId.hpp does for "CpuRef" (src/backends/reference/RefBackendId.hpp:10).
#pragma once
namespace armnn
{
constexpr const char* Mi355xBackendId() { return "Mi355x"; }
constexpr const char* Mi355xTensorHandleFactoryId() { return "Amd/Mi355x/TensorHandleFactory"; }
} // namespace armnn
