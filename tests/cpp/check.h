// Minimal assertion helpers for the C++ test programs (each program exits non-zero on the first failed suite).
#pragma once
#include <cstdio>
#include <cstdlib>
#include <exception>
#include <functional>
#include <string>

static int g_failed = 0;
static int g_checks = 0;

#define CHECK(cond)                                                                  \
    do {                                                                             \
        ++g_checks;                                                                  \
        if (!(cond)) {                                                               \
            ++g_failed;                                                              \
            printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);                 \
        }                                                                            \
    } while (0)

#define CHECK_EQ(a, b) CHECK((a) == (b))

template <typename E> static void checkThrows(const char* what, const std::function<void()>& fn)
{
    ++g_checks;
    try {
        fn();
    } catch (const E&) {
        return;
    } catch (const std::exception& e) {
        ++g_failed;
        printf("FAILED %s: wrong exception type: %s\n", what, e.what());
        return;
    }
    ++g_failed;
    printf("FAILED %s: no exception\n", what);
}

static int finish(const char* name)
{
    printf("%s: %d checks, %d failed\n", name, g_checks, g_failed);
    fflush(stdout);
    return g_failed ? 1 : 0;
}
