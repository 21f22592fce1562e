// For builds against an Arm NN source tree only: the accessor that include/armnn/INetwork.hpp:929 declares a friend of
// IOptimizedNetwork and that the tree's test utilities define (src/armnnTestUtils/TestUtils.cpp:49-52), which libarmnn.so
// does not contain.
#include <armnn/INetwork.hpp>
#include <Graph.hpp>
#include <OptimizedNetworkImpl.hpp>

namespace armnn
{
Graph& GetGraphForTesting(IOptimizedNetwork* optNetPtr) { return optNetPtr->pOptimizedNetworkImpl->GetGraph(); }
} // namespace armnn
