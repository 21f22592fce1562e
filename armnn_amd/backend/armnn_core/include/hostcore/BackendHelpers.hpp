// Minimal host core: two helpers every backend leans on.
//   OptimizationViews       what OptimizeSubgraphView returns (include/armnn/backends/OptimizationViews.hpp:17-81): every
//                           layer of the incoming view must end up in exactly one of a substitution's substitutable side,
//                           the failed list, the untouched list or the deleted list
//                           (src/backends/backendsCommon/OptimizationViews.cpp:11-75).
//   CopyMemGenericWorkload  the Map / memcpy / Unmap workload behind Input, Output and MemCopy layers
//                           (src/backends/backendsCommon/MemCopyWorkload.cpp:44-64).
// The Arm NN-named headers forward here.
#pragma once
#include <armnn/INetwork.hpp>
#include <armnn/backends/SubgraphView.hpp>
#include <armnn/backends/Workload.hpp>
#include <vector>

namespace armnn
{
class OptimizationViews
{
public:
    OptimizationViews(const NetworkOptions& networkOptions = {}) : m_INetwork(INetwork::Create(networkOptions)) {}
    OptimizationViews(const OptimizationViews&) = delete;
    OptimizationViews& operator=(const OptimizationViews&) = delete;
    OptimizationViews(OptimizationViews&&) = default;
    OptimizationViews& operator=(OptimizationViews&&) = default;

    struct SubstitutionPair
    {
        SubgraphView m_SubstitutableSubgraph;   ///< layers of the original graph to take out
        SubgraphView m_ReplacementSubgraph;     ///< layers created through GetINetwork() to put in their place
    };
    using Subgraphs = std::vector<SubgraphView>;
    using Substitutions = std::vector<SubstitutionPair>;

    void AddSubstitution(SubstitutionPair&& substitution) { m_SuccesfulOptimizations.emplace_back(std::move(substitution)); }
    void AddFailedSubgraph(SubgraphView&& subgraph) { m_FailedOptimizations.emplace_back(std::move(subgraph)); }
    void AddUntouchedSubgraph(SubgraphView&& subgraph) { m_UntouchedSubgraphs.emplace_back(std::move(subgraph)); }
    void AddDeletedSubgraph(SubgraphView&& subgraph) { m_DeletedSubgraphs.emplace_back(std::move(subgraph)); }
    const Substitutions& GetSubstitutions() const { return m_SuccesfulOptimizations; }
    const Subgraphs& GetFailedSubgraphs() const { return m_FailedOptimizations; }
    const Subgraphs& GetUntouchedSubgraphs() const { return m_UntouchedSubgraphs; }
    const Subgraphs& GetDeletedSubgraphs() const { return m_DeletedSubgraphs; }
    Substitutions& GetSubstitutions() { return m_SuccesfulOptimizations; }
    bool Validate(const SubgraphView& originalSubgraph) const;
    INetwork* GetINetwork() { return m_INetwork.get(); }
    INetwork& GetINetworkRef() { return *m_INetwork; }
private:
    Substitutions m_SuccesfulOptimizations;
    Subgraphs m_FailedOptimizations;
    Subgraphs m_UntouchedSubgraphs;
    Subgraphs m_DeletedSubgraphs;
    INetworkPtr m_INetwork = INetworkPtr(nullptr, &INetwork::Destroy);
};

class CopyMemGenericWorkload : public BaseWorkload<MemCopyQueueDescriptor>
{
public:
    CopyMemGenericWorkload(const MemCopyQueueDescriptor& descriptor, const WorkloadInfo& info);
    void Execute() const override;
};
} // namespace armnn
