// Minimal host core: small utilities the Arm NN-named headers under armnn/utility/ forward to.
#pragma once

namespace armnn
{
// swallows values that are unused on purpose (armnn::IgnoreUnused, include/armnn/utility/IgnoreUnused.hpp)
template <typename... Ts>
inline void IgnoreUnused(Ts&&...) {}
} // namespace armnn
