// Status codes, checking macros and small helpers shared by the host classes.
// Interface-compatible with the reference's include/util/common.h:7-61 (same enum, same macro
// names, same helper signatures) without its glog dependency: messages go to stderr.
#pragma once
#include <cstdio>
#include <cstdlib>
#include <exception>
#include <iostream>

// Same enumerators, same order, global namespace (reference include/util/common.h:16-23).
enum Status { Succ, Fail, Timeout, NotFound, OutOfRange, Full };

inline const char *status_name(Status s) {
    static const char *names[] = {"Succ", "Fail", "Timeout", "NotFound", "OutOfRange", "Full"};
    return (int)s >= 0 && (int)s < 6 ? names[(int)s] : "?";
}

#define div_ceil(a, b) (((a) + (b)-1) / (b))

// exit(1) on failure (reference common.h:7-14)
#define CHECK_STATUS(cmd)                                                                       \
    do {                                                                                        \
        Status gp_s_ = (cmd);                                                                   \
        if (gp_s_ != Status::Succ) {                                                            \
            std::fprintf(stderr, "%s -> %s at %s:%d\n", #cmd, status_name(gp_s_), __FILE__, __LINE__); \
            std::exit(1);                                                                       \
        }                                                                                       \
    } while (0)

// The reference logs and then calls std::terminate() (common.h:26-34).  Here the status is
// handed back to the caller after logging, so an error path can be tested without killing the
// process; define GPREEMPT_TERMINATE_ON_ERROR to get the reference's behaviour.
#ifdef GPREEMPT_TERMINATE_ON_ERROR
#define GP_ON_ERROR_ std::terminate()
#else
#define GP_ON_ERROR_ (void)0
#endif
#define RETURN_STATUS(cmd)                                                                      \
    do {                                                                                        \
        Status gp_s_ = (cmd);                                                                   \
        if (gp_s_ != Status::Succ) {                                                            \
            std::fprintf(stderr, "%s -> %s at %s:%d\n", #cmd, status_name(gp_s_), __FILE__, __LINE__); \
            GP_ON_ERROR_;                                                                       \
            return gp_s_;                                                                       \
        }                                                                                       \
    } while (0)

#define ASSERT(condition)                                                                       \
    do {                                                                                        \
        if (!(condition)) {                                                                     \
            std::cerr << "Assertion `" #condition "` failed in " << __FILE__ << ":" << __LINE__ << std::endl; \
            std::terminate();                                                                   \
        }                                                                                       \
    } while (false)

template <typename T> T align_up(T value, T alignment) {
    T rem = value % alignment;
    return rem == 0 ? value : value + (alignment - rem);
}
template <typename T> T align_down(T value, T alignment) { return value - value % alignment; }

// Pins the calling thread to one core (reference src/util/util.cpp:3-10).
void bind_core(int core_id);
