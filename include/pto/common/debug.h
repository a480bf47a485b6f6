// Run-time assertions of kernel sources (the reference's include/pto/common/debug.h:19-35): PTO_ASSERT(condition, message)
// checks only in _DEBUG builds, where a failing condition prints the message with its place and stops the wave;
// otherwise it evaluates nothing.  DEBUG_CHECK always checks.
#pragma once
#include <cstdio>

#define DEBUG_CHECK(condition, message)                                                                            \
    do {                                                                                                           \
        if (!(condition)) {                                                                                        \
            printf("[PTO][ASSERT] %s\n  Condition: %s\n  Location: %s:%d\n", (message), #condition, __FILE__, __LINE__); \
            __builtin_trap();                                                                                      \
        }                                                                                                          \
    } while (0)

#if defined(_DEBUG)
#define PTO_ASSERT(condition, message) DEBUG_CHECK(condition, message)
#else
#define PTO_ASSERT(condition, message) ((void)0)
#endif
