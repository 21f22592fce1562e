#pragma once
namespace armnn
{
template <typename Dest, typename Source>
constexpr Dest numeric_cast(Source s) { return static_cast<Dest>(s); }
} // namespace armnn
