// Minimal assertion helpers for the host-layer test programs (run by pytest as subprocesses).
#pragma once
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

static int g_checks = 0;

#define CHECK(cond)                                                                   \
    do {                                                                              \
        g_checks++;                                                                   \
        if (!(cond)) {                                                                \
            std::fprintf(stderr, "%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond); \
            std::exit(1);                                                             \
        }                                                                             \
    } while (0)

#define CHECK_MSG(cond, ...)                                                          \
    do {                                                                              \
        g_checks++;                                                                   \
        if (!(cond)) {                                                                \
            std::fprintf(stderr, "%s:%d: CHECK failed: %s: ", __FILE__, __LINE__, #cond); \
            std::fprintf(stderr, __VA_ARGS__);                                        \
            std::fprintf(stderr, "\n");                                               \
            std::exit(1);                                                             \
        }                                                                             \
    } while (0)

static inline void say(const std::string &s) {
    std::printf("[case] %s\n", s.c_str());
    std::fflush(stdout);
}

static inline uint32_t bits_of(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}
