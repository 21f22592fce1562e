// A very small test harness: TEST_CASE registers a function; the runner executes the cases whose tag matches.
//   ./backend_tests --tag cpu|gpu [--filter substring] [--list]
// A failed CHECK is recorded and the case continues; REQUIRE ends the case.
#pragma once
#include <cstdio>
#include <cstring>
#include <exception>
#include <functional>
#include <string>
#include <vector>

namespace minitest
{
struct Case { std::string name, tag; std::function<void()> fn; };
inline std::vector<Case>& Cases() { static std::vector<Case> c; return c; }
inline int& Failures() { static int f = 0; return f; }
struct Abort {};
struct Registrar { Registrar(const char* n, const char* t, std::function<void()> f) { Cases().push_back({n, t, std::move(f)}); } };

inline void Fail(const char* file, int line, const std::string& what)
{
    ++Failures();
    std::printf("    FAILED %s:%d: %s\n", file, line, what.c_str());
    std::fflush(stdout);
}

inline int Run(int argc, char** argv)
{
    std::string tag, filter;
    bool list = false;
    for (int i = 1; i < argc; ++i)
    {
        if (!std::strcmp(argv[i], "--tag") && i + 1 < argc) tag = argv[++i];
        else if (!std::strcmp(argv[i], "--filter") && i + 1 < argc) filter = argv[++i];
        else if (!std::strcmp(argv[i], "--list")) list = true;
    }
    int ran = 0, failedCases = 0;
    for (const Case& c : Cases())
    {
        if (!tag.empty() && c.tag != tag) continue;
        if (!filter.empty() && c.name.find(filter) == std::string::npos) continue;
        if (list) { std::printf("%s [%s]\n", c.name.c_str(), c.tag.c_str()); continue; }
        std::printf("[ RUN  ] %s\n", c.name.c_str());
        std::fflush(stdout);
        const int before = Failures();
        try { c.fn(); }
        catch (const Abort&) {}
        catch (const std::exception& e) { Fail(__FILE__, __LINE__, std::string("unexpected exception: ") + e.what()); }
        ++ran;
        if (Failures() != before) { ++failedCases; std::printf("[ FAIL ] %s\n", c.name.c_str()); }
        else std::printf("[  OK  ] %s\n", c.name.c_str());
        std::fflush(stdout);
    }
    if (!list) std::printf("%d case(s) run, %d failed\n", ran, failedCases);
    return failedCases ? 1 : 0;
}
} // namespace minitest

#define MT_CAT2(a, b) a##b
#define MT_CAT(a, b) MT_CAT2(a, b)
#define TEST_CASE(name, tag)                                                         \
    static void MT_CAT(mt_fn_, __LINE__)();                                          \
    static minitest::Registrar MT_CAT(mt_reg_, __LINE__)(name, tag, MT_CAT(mt_fn_, __LINE__)); \
    static void MT_CAT(mt_fn_, __LINE__)()
#define CHECK(cond) do { if (!(cond)) minitest::Fail(__FILE__, __LINE__, #cond); } while (0)
#define CHECK_MSG(cond, msg) do { if (!(cond)) minitest::Fail(__FILE__, __LINE__, std::string(#cond) + ": " + (msg)); } while (0)
#define REQUIRE(cond) do { if (!(cond)) { minitest::Fail(__FILE__, __LINE__, #cond); throw minitest::Abort(); } } while (0)
#define CHECK_THROWS_AS(expr, type)                                                   \
    do { bool mt_ok = false; try { expr; } catch (const type&) { mt_ok = true; } catch (...) {} \
         if (!mt_ok) minitest::Fail(__FILE__, __LINE__, #expr " did not throw " #type); } while (0)
#define CHECK_NOTHROW(expr) \
    do { try { expr; } catch (const std::exception& e) { minitest::Fail(__FILE__, __LINE__, std::string(#expr " threw: ") + e.what()); } } while (0)
