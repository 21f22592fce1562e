// Minimal host core: BackendId is a string wrapper (include/armnn/BackendId.hpp:78-148).
#pragma once
#include <ostream>
#include <string>
#include <unordered_set>
#include <vector>

namespace armnn
{
class BackendId final
{
public:
    BackendId() : m_Id("Undefined") {}
    BackendId(const std::string& id) : m_Id{id} {}
    BackendId(const char* id) : m_Id{id} {}
    BackendId(const BackendId&) = default;
    BackendId(BackendId&&) = default;
    BackendId& operator=(const BackendId&) = default;
    BackendId& operator=(BackendId&&) = default;
    bool operator==(const BackendId& other) const { return m_Id == other.m_Id; }
    bool operator!=(const BackendId& other) const { return m_Id != other.m_Id; }
    bool operator<(const BackendId& other) const { return m_Id < other.m_Id; }
    operator std::string() const { return m_Id; }
    const std::string& Get() const { return m_Id; }
    bool IsEmpty() const { return m_Id.empty(); }
    bool IsUndefined() const { return m_Id == "Undefined"; }
private:
    std::string m_Id;
};
inline std::ostream& operator<<(std::ostream& os, const BackendId& id) { return os << id.Get(); }
} // namespace armnn

namespace std
{
template <>
struct hash<armnn::BackendId>
{
    size_t operator()(const armnn::BackendId& id) const noexcept { return std::hash<std::string>()(id.Get()); }
};
} // namespace std

namespace armnn
{
using BackendIdVector = std::vector<BackendId>;
using BackendIdSet = std::unordered_set<BackendId>;
} // namespace armnn
