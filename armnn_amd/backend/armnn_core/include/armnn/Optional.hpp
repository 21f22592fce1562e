// Minimal host core: armnn::Optional / EmptyOptional (include/armnn/Optional.hpp), values and references.
#pragma once
#include "Exceptions.hpp"
#include <utility>

namespace armnn
{
struct EmptyOptional {};

template <typename T>
class Optional
{
public:
    Optional() noexcept = default;
    Optional(EmptyOptional) noexcept {}
    Optional(const T& v) : m_Value(v), m_Has(true) {}
    Optional(T&& v) : m_Value(std::move(v)), m_Has(true) {}
    Optional& operator=(EmptyOptional) { m_Has = false; return *this; }
    bool has_value() const noexcept { return m_Has; }
    explicit operator bool() const noexcept { return m_Has; }
    const T& value() const { if (!m_Has) throw BadOptionalAccessException("Optional has no value"); return m_Value; }
    T& value() { if (!m_Has) throw BadOptionalAccessException("Optional has no value"); return m_Value; }
    void reset() { m_Has = false; }
private:
    T m_Value{};
    bool m_Has = false;
};

template <typename T>
class Optional<T&>
{
public:
    Optional() noexcept = default;
    Optional(EmptyOptional) noexcept {}
    Optional(T& v) : m_Ptr(&v) {}
    bool has_value() const noexcept { return m_Ptr != nullptr; }
    explicit operator bool() const noexcept { return m_Ptr != nullptr; }
    T& value() const { if (!m_Ptr) throw BadOptionalAccessException("Optional has no value"); return *m_Ptr; }
private:
    T* m_Ptr = nullptr;
};

template <typename T>
Optional<T> MakeOptional(const T& v) { return Optional<T>(v); }
} // namespace armnn
