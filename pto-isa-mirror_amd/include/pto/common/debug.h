// PTO_ASSERT / DEBUG_CHECK for kernel sources that include <pto/common/debug.h> (reference:
// include/pto/common/debug.h:14-33).  A failed DEBUG_CHECK prints the message, the condition and the place, and raises
// the core's status word (what the launcher's *_status() call returns); it does not trap, since a trapping wave takes
// the whole device context with it.  PTO_ASSERT is DEBUG_CHECK in _DEBUG builds and nothing otherwise.
#pragma once
#include <cstdio>

#include "../amd/tile.hpp"

#define DEBUG_CHECK(condition, message)                                                                              \
    do {                                                                                                             \
        if (!(condition)) {                                                                                          \
            printf("[PTO][ASSERT] %s\n  Condition: %s\n  Location: %s:%d\n", (message), #condition, __FILE__, __LINE__); \
            ::pto::amd::report(2);                                                                                   \
        }                                                                                                            \
    } while (0)

#ifdef _DEBUG
#define PTO_ASSERT(condition, message) DEBUG_CHECK(condition, message)
#else
#define PTO_ASSERT(condition, message) ((void)0)
#endif
