// Minimal host core: include/armnn/backends/WorkloadInfo.hpp:16-36.
#pragma once
#include "../Optional.hpp"
#include "../Tensor.hpp"
#include <string>
#include <vector>
namespace armnn
{
struct WorkloadInfo
{
    std::vector<TensorInfo> m_InputTensorInfos;
    std::vector<TensorInfo> m_OutputTensorInfos;
    std::string m_Name;
    Optional<TensorInfo> m_WeightsTensorInfo = EmptyOptional();
    Optional<TensorInfo> m_BiasTensorInfo = EmptyOptional();
    Optional<std::string> m_ConvolutionMethod = EmptyOptional();
};
/// scratch memory a workload needs besides its tensors, for a memory plan made outside the backend
struct MemoryInfo
{
    unsigned int m_OutputSlotIndex;
    size_t m_Size{0};
    size_t m_Alignment{64};
};
struct MemoryRequirements
{
    Optional<std::vector<MemoryInfo>> m_IntraLayerTensors;
};
} // namespace armnn
