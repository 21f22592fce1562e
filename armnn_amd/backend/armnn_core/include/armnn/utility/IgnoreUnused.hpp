#pragma once
namespace armnn
{
template <typename... Ts>
inline void IgnoreUnused(Ts&&...) {}
} // namespace armnn
