#include "Mi355xWorkloadFactory.hpp"
#include "Mi355xBackendId.hpp"
#include "Mi355xTensorHandle.hpp"
#include "Mi355xWorkloads.hpp"

#include <armnn/backends/MemCopyWorkload.hpp>
#include <armnn/utility/PolymorphicDowncast.hpp>

#include <functional>
#include <mutex>

namespace armnn
{
namespace
{
const BackendId s_Id{Mi355xBackendId()};

}

struct Mi355xWorkloadFactory::Candidate
{
    std::mutex mutex;
    Mi355xConvolution2dWorkload* convolution = nullptr;
    Mi355xConvolution2dWorkload* Take()
    {
        std::lock_guard<std::mutex> lock(mutex);
        Mi355xConvolution2dWorkload* w = convolution;
        convolution = nullptr;
        return w;
    }
    // the depthwise workload created last, while it is marked as feeding one pointwise convolution only
    Mi355xDepthwiseConvolution2dWorkload* depthwise = nullptr;
    Mi355xDepthwiseConvolution2dWorkload* TakeDepthwise()
    {
        std::lock_guard<std::mutex> lock(mutex);
        Mi355xDepthwiseConvolution2dWorkload* w = depthwise;
        depthwise = nullptr;
        return w;
    }
};

namespace
{
// the convolution workload the factory hands out: its destructor withdraws it as its factory's candidate, should it still be one
class CandidateConvolution final : public Mi355xConvolution2dWorkload
{
public:
    template <typename C>
    CandidateConvolution(const Convolution2dQueueDescriptor& d, const WorkloadInfo& info, std::shared_ptr<C> slot)
        : Mi355xConvolution2dWorkload(d, info), m_Withdraw([slot](Mi355xConvolution2dWorkload* self) {
              std::lock_guard<std::mutex> lock(slot->mutex);
              if (slot->convolution == self) slot->convolution = nullptr;
          })
    {
    }
    ~CandidateConvolution() override { m_Withdraw(this); }
private:
    std::function<void(Mi355xConvolution2dWorkload*)> m_Withdraw;
};

// the same for the depthwise workload
class CandidateDepthwise final : public Mi355xDepthwiseConvolution2dWorkload
{
public:
    template <typename C>
    CandidateDepthwise(const DepthwiseConvolution2dQueueDescriptor& d, const WorkloadInfo& info, std::shared_ptr<C> slot)
        : Mi355xDepthwiseConvolution2dWorkload(d, info), m_Withdraw([slot](Mi355xDepthwiseConvolution2dWorkload* self) {
              std::lock_guard<std::mutex> lock(slot->mutex);
              if (slot->depthwise == self) slot->depthwise = nullptr;
          })
    {
    }
    ~CandidateDepthwise() override { m_Withdraw(this); }
private:
    std::function<void(Mi355xDepthwiseConvolution2dWorkload*)> m_Withdraw;
};
}

Mi355xWorkloadFactory::Mi355xWorkloadFactory(const std::shared_ptr<Mi355xMemoryManager>& memoryManager)
    : m_MemoryManager(memoryManager), m_Candidate(std::make_shared<Candidate>()) {}
Mi355xWorkloadFactory::Mi355xWorkloadFactory() : m_MemoryManager(new Mi355xMemoryManager()), m_Candidate(std::make_shared<Candidate>()) {}

const BackendId& Mi355xWorkloadFactory::GetBackendId() const { return s_Id; }

bool Mi355xWorkloadFactory::IsLayerSupported(const IConnectableLayer& layer, Optional<DataType> dataType, std::string& outReasonIfUnsupported)
{
    return IWorkloadFactory::IsLayerSupported(s_Id, layer, dataType, outReasonIfUnsupported);
}

std::unique_ptr<ITensorHandle> Mi355xWorkloadFactory::CreateTensorHandle(const TensorInfo& info, const bool managed) const
{
    return std::make_unique<Mi355xTensorHandle>(info, m_MemoryManager, managed);
}
std::unique_ptr<ITensorHandle> Mi355xWorkloadFactory::CreateTensorHandle(const TensorInfo& info, DataLayout, const bool managed) const
{
    return std::make_unique<Mi355xTensorHandle>(info, m_MemoryManager, managed);
}

std::unique_ptr<IWorkload> Mi355xWorkloadFactory::CreateWorkload(LayerType type, const QueueDescriptor& descriptor, const WorkloadInfo& info) const
{
    // constants write no tensor another workload's operand could share an address with: they leave the candidate alone
    Mi355xConvolution2dWorkload* candidate = type == LayerType::Constant ? nullptr : m_Candidate->Take();
    Mi355xDepthwiseConvolution2dWorkload* depthwise = type == LayerType::Constant ? nullptr : m_Candidate->TakeDepthwise();
    switch (type)
    {
        case LayerType::Convolution2d:
        {
            auto w = std::make_unique<CandidateConvolution>(*PolymorphicDowncast<const Convolution2dQueueDescriptor*>(&descriptor), info, m_Candidate);
            // the depthwise layer created just before, marked as feeding only this kind of convolution: the two run as a pair
            w->TakeOver(depthwise);
            if (w->FeedsOnlyAnAddition() || w->OnlyConsumerIsAGlobalPooling())
            {
                std::lock_guard<std::mutex> lock(m_Candidate->mutex);
                m_Candidate->convolution = w.get();
            }
            return w;
        }
        case LayerType::DepthwiseConvolution2d:
        {
            auto w = std::make_unique<CandidateDepthwise>(*PolymorphicDowncast<const DepthwiseConvolution2dQueueDescriptor*>(&descriptor), info, m_Candidate);
            if (w->OnlyConsumerIsAPointwiseConvolution())
            {
                std::lock_guard<std::mutex> lock(m_Candidate->mutex);
                m_Candidate->depthwise = w.get();
            }
            return w;
        }
        case LayerType::FullyConnected:
            return std::make_unique<Mi355xFullyConnectedWorkload>(*PolymorphicDowncast<const FullyConnectedQueueDescriptor*>(&descriptor), info);
        case LayerType::Activation:
            return std::make_unique<Mi355xActivationWorkload>(*PolymorphicDowncast<const ActivationQueueDescriptor*>(&descriptor), info);
        case LayerType::Pooling2d:
        {
            auto w = std::make_unique<Mi355xPooling2dWorkload>(*PolymorphicDowncast<const Pooling2dQueueDescriptor*>(&descriptor), info);
            w->TakeOver(candidate);
            return w;
        }
        case LayerType::Mean:
            return std::make_unique<Mi355xMeanWorkload>(*PolymorphicDowncast<const MeanQueueDescriptor*>(&descriptor), info);
        case LayerType::Pad:
            return std::make_unique<Mi355xPadWorkload>(*PolymorphicDowncast<const PadQueueDescriptor*>(&descriptor), info);
        case LayerType::Softmax:
            return std::make_unique<Mi355xSoftmaxWorkload>(*PolymorphicDowncast<const SoftmaxQueueDescriptor*>(&descriptor), info);
        case LayerType::ElementwiseBinary:
        {
            auto w = std::make_unique<Mi355xAdditionWorkload>(*PolymorphicDowncast<const ElementwiseBinaryQueueDescriptor*>(&descriptor), info);
            w->TakeOver(candidate);
            return w;
        }
        case LayerType::Reshape:
            return std::make_unique<Mi355xReshapeWorkload>(*PolymorphicDowncast<const ReshapeQueueDescriptor*>(&descriptor), info);
        case LayerType::Constant:
            return std::make_unique<Mi355xConstantWorkload>(*PolymorphicDowncast<const ConstantQueueDescriptor*>(&descriptor), info);
        case LayerType::Input:
        case LayerType::Output:
        case LayerType::MemCopy:
        {
            // Map / memcpy / Unmap between any two handle types; the device handle's Map() and Unmap() do the transfers
            const auto* d = PolymorphicDowncast<const MemCopyQueueDescriptor*>(&descriptor);
            if (d->m_Inputs.empty() || !d->m_Inputs[0]) throw InvalidArgumentException("Mi355xWorkloadFactory: copy workload without an input handle");
            return std::make_unique<CopyMemGenericWorkload>(*d, info);
        }
        default:
            return nullptr;
    }
}
} // namespace armnn
