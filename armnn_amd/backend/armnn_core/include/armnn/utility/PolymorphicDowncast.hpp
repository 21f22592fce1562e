// PolymorphicDowncast: static_cast checked with dynamic_cast (include/armnn/utility/PolymorphicDowncast.hpp).
#pragma once
#include "../Exceptions.hpp"
#include <type_traits>
namespace armnn
{
template <typename DestType, typename SourceType>
DestType PolymorphicDowncast(SourceType* value)
{
    static_assert(std::is_pointer<DestType>::value, "PolymorphicDowncast: destination must be a pointer type");
    if (value != nullptr && dynamic_cast<DestType>(value) == nullptr)
        throw InvalidArgumentException("PolymorphicDowncast: value is not of the destination type");
    return static_cast<DestType>(value);
}
} // namespace armnn
