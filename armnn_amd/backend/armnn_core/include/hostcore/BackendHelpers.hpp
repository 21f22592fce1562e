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
// Result of IBackendInternal::OptimizeSubgraphView.  A backend sorts the layers of the view it was given into four bins;
// replacement layers are created through the private network the object owns, so they outlive the call.
class OptimizationViews
{
public:
    /// layers of the original graph to take out, and the layers (made through GetINetwork()) that go in their place
    struct SubstitutionPair
    {
        SubgraphView m_SubstitutableSubgraph;
        SubgraphView m_ReplacementSubgraph;
    };
    using Substitutions = std::vector<SubstitutionPair>;
    using Subgraphs = std::vector<SubgraphView>;

    explicit OptimizationViews(const NetworkOptions& networkOptions = {});
    OptimizationViews(OptimizationViews&&) = default;
    OptimizationViews& operator=(OptimizationViews&&) = default;
    OptimizationViews(const OptimizationViews&) = delete;
    OptimizationViews& operator=(const OptimizationViews&) = delete;

    // the four bins
    void AddSubstitution(SubstitutionPair&& substitution);
    void AddFailedSubgraph(SubgraphView&& subgraph);
    void AddUntouchedSubgraph(SubgraphView&& subgraph);
    void AddDeletedSubgraph(SubgraphView&& subgraph);
    Substitutions& GetSubstitutions();
    const Substitutions& GetSubstitutions() const;
    const Subgraphs& GetFailedSubgraphs() const;
    const Subgraphs& GetUntouchedSubgraphs() const;
    const Subgraphs& GetDeletedSubgraphs() const;

    /// true when every layer of `originalSubgraph` sits in exactly one bin and every substitution keeps its slot counts
    bool Validate(const SubgraphView& originalSubgraph) const;

    /// where replacement layers are created
    INetwork* GetINetwork();
    INetwork& GetINetworkRef();

private:
    INetworkPtr m_INetwork;
    Substitutions m_SuccesfulOptimizations;
    Subgraphs m_FailedOptimizations, m_UntouchedSubgraphs, m_DeletedSubgraphs;
};

class CopyMemGenericWorkload : public BaseWorkload<MemCopyQueueDescriptor>
{
public:
    CopyMemGenericWorkload(const MemCopyQueueDescriptor& descriptor, const WorkloadInfo& info);
    void Execute() const override;
};
} // namespace armnn
