// Minimal test harness (GoogleTest is not available in this image).
#ifndef NZ_MINI_TEST_HPP
#define NZ_MINI_TEST_HPP
#include <cstdio>
#include <functional>
#include <string>
#include <vector>

namespace mini {
    struct Case {
        const char* name;
        std::function<void()> body;
    };
    inline std::vector<Case>& registry() {
        static std::vector<Case> r;
        return r;
    }
    inline int& failures() {
        static int f = 0;
        return f;
    }
    struct Registrar {
        Registrar(const char* name, std::function<void()> body) { registry().push_back({name, std::move(body)}); }
    };
    inline int run_all(const char* filter = nullptr) {
        int ran = 0;
        for (auto& c : registry()) {
            if (filter && std::string(c.name).find(filter) == std::string::npos) continue;
            const int before = failures();
            std::printf("[ RUN  ] %s\n", c.name);
            std::fflush(stdout);
            try {
                c.body();
            } catch (const std::exception& e) {
                std::printf("  unexpected exception: %s\n", e.what());
                failures()++;
            }
            std::printf("[ %s ] %s\n", failures() == before ? " OK " : "FAIL", c.name);
            std::fflush(stdout);
            ran++;
        }
        std::printf("%d tests, %d failures\n", ran, failures());
        return failures() ? 1 : 0;
    }
}

#define TEST(suite, name)                                                        \
    static void suite##_##name();                                                \
    static mini::Registrar reg_##suite##_##name(#suite "." #name, suite##_##name); \
    static void suite##_##name()

#define EXPECT_TRUE(cond)                                                                  \
    do {                                                                                   \
        if (!(cond)) {                                                                     \
            std::printf("  %s:%d: EXPECT_TRUE(%s) failed\n", __FILE__, __LINE__, #cond);   \
            mini::failures()++;                                                            \
        }                                                                                  \
    } while (0)
#define EXPECT_EQ(a, b) EXPECT_TRUE((a) == (b))
#define EXPECT_THROW(stmt, ex)                                                             \
    do {                                                                                   \
        bool caught__ = false;                                                             \
        try {                                                                              \
            stmt;                                                                          \
        } catch (const ex&) {                                                              \
            caught__ = true;                                                               \
        } catch (...) {                                                                    \
        }                                                                                  \
        if (!caught__) {                                                                   \
            std::printf("  %s:%d: expected %s from %s\n", __FILE__, __LINE__, #ex, #stmt); \
            mini::failures()++;                                                            \
        }                                                                                  \
    } while (0)
#endif
