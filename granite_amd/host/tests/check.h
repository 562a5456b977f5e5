// Tiny test harness: named cases, CHECK macros, non-zero exit on any failure.
#pragma once

#include <cstdio>
#include <cstdlib>
#include <functional>
#include <string>
#include <vector>

namespace hosttest {

struct Case {
    const char* name;
    std::function<void()> body;
};

inline std::vector<Case>& cases() {
    static std::vector<Case> all;
    return all;
}
inline int& failures() {
    static int n = 0;
    return n;
}
struct Register {
    Register(const char* name, std::function<void()> body) { cases().push_back({name, std::move(body)}); }
};

inline int run_all(int argc, char** argv) {
    const std::string only = argc > 1 ? argv[1] : "";
    int ran = 0;
    for (auto& c : cases()) {
        if (!only.empty() && only != c.name) continue;
        std::printf("[ RUN  ] %s\n", c.name);
        std::fflush(stdout);
        const int before = failures();
        c.body();
        std::printf("[ %s ] %s\n", failures() == before ? " OK " : "FAIL", c.name);
        std::fflush(stdout);
        ++ran;
    }
    std::printf("%d cases, %d failed checks\n", ran, failures());
    return failures() == 0 && ran > 0 ? 0 : 1;
}

}  // namespace hosttest

#define TEST_CASE(id)                                               \
    static void id();                                               \
    static hosttest::Register _reg_##id(#id, id);                   \
    static void id()

#define CHECK(cond)                                                                  \
    do {                                                                             \
        if (!(cond)) {                                                               \
            std::printf("  CHECK failed %s:%d: %s\n", __FILE__, __LINE__, #cond);    \
            ++hosttest::failures();                                                  \
        }                                                                            \
    } while (0)

#define REQUIRE(cond)                                                                \
    do {                                                                             \
        if (!(cond)) {                                                               \
            std::printf("  REQUIRE failed %s:%d: %s\n", __FILE__, __LINE__, #cond);  \
            ++hosttest::failures();                                                  \
            return;                                                                  \
        }                                                                            \
    } while (0)

#define CHECK_OK(expr)                                                               \
    do {                                                                             \
        auto _r = (expr);                                                            \
        if (!_r.ok()) {                                                              \
            std::printf("  CHECK_OK failed %s:%d: %s -> %s\n", __FILE__, __LINE__, #expr, \
                        _r.error().to_string().c_str());                             \
            ++hosttest::failures();                                                  \
        }                                                                            \
    } while (0)

#define CHECK_CODE(expr, expected)                                                   \
    do {                                                                             \
        auto _r = (expr);                                                            \
        if (_r.ok() || _r.error().code() != (expected)) {                            \
            std::printf("  CHECK_CODE failed %s:%d: %s (got %s)\n", __FILE__, __LINE__, #expr, \
                        _r.ok() ? "ok" : granite::error_code_name(_r.error().code())); \
            ++hosttest::failures();                                                  \
        }                                                                            \
    } while (0)
