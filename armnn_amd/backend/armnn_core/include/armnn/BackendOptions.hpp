// Minimal host core: named option bags (include/armnn/BackendOptions.hpp:22-339) -- also used for capabilities.
#pragma once
#include "BackendId.hpp"
#include <string>
#include <vector>

namespace armnn
{
struct BackendOptions
{
    class Var
    {
    public:
        Var(int v) : m_Kind(Kind::Int) { m_I = v; }
        Var(unsigned int v) : m_Kind(Kind::UInt) { m_U = v; }
        Var(float v) : m_Kind(Kind::Float) { m_F = v; }
        Var(bool v) : m_Kind(Kind::Bool) { m_B = v; }
        Var(const char* v) : m_Kind(Kind::String), m_S(v) {}
        Var(std::string v) : m_Kind(Kind::String), m_S(std::move(v)) {}
        bool IsBool() const { return m_Kind == Kind::Bool; }
        bool IsInt() const { return m_Kind == Kind::Int; }
        bool IsUnsignedInt() const { return m_Kind == Kind::UInt; }
        bool IsFloat() const { return m_Kind == Kind::Float; }
        bool IsString() const { return m_Kind == Kind::String; }
        bool AsBool() const { return m_B; }
        int AsInt() const { return m_I; }
        unsigned int AsUnsignedInt() const { return m_U; }
        float AsFloat() const { return m_F; }
        std::string AsString() const { return m_S; }
    private:
        enum class Kind { Int, UInt, Float, Bool, String } m_Kind;
        union { int m_I; unsigned int m_U; float m_F; bool m_B; };
        std::string m_S;
    };

    class BackendOption
    {
    public:
        BackendOption(std::string name, Var value) : m_Name(std::move(name)), m_Value(std::move(value)) {}
        const std::string& GetName() const { return m_Name; }
        const Var& GetValue() const { return m_Value; }
    private:
        std::string m_Name;
        Var m_Value;
    };

    explicit BackendOptions(BackendId backend) : m_TargetBackend(std::move(backend)) {}
    BackendOptions(BackendId backend, std::initializer_list<BackendOption> options)
        : m_TargetBackend(std::move(backend)), m_Options(options) {}
    void AddOption(const BackendOption& option) { m_Options.push_back(option); }
    const BackendId& GetBackendId() const noexcept { return m_TargetBackend; }
    size_t GetOptionCount() const noexcept { return m_Options.size(); }
    const BackendOption& GetOption(size_t idx) const { return m_Options[idx]; }
private:
    BackendId m_TargetBackend;
    std::vector<BackendOption> m_Options;
};

using ModelOptions = std::vector<BackendOptions>;
using NetworkOptions = std::vector<BackendOptions>;
using BackendCapabilities = BackendOptions;

template <typename F>
void ParseOptions(const std::vector<BackendOptions>& options, BackendId backend, F f)
{
    for (const auto& group : options)
        if (group.GetBackendId() == backend)
            for (size_t i = 0; i < group.GetOptionCount(); ++i) f(group.GetOption(i).GetName(), group.GetOption(i).GetValue());
}

inline bool HasCapability(const std::string& name, const BackendCapabilities& capabilities)
{
    for (size_t i = 0; i < capabilities.GetOptionCount(); ++i)
        if (capabilities.GetOption(i).GetName() == name) return true;
    return false;
}
} // namespace armnn
