// Timing and error macros for harness code written against the reference's src/gemm/common.h:
// same macro names and argument order, so a main() shaped like the reference's test.cc / benchmark.cc
// compiles against this header unchanged.
//
// Differences from the reference (src/gemm/common.h:4-24):
//   - GPU_TIMER_END reports seconds, as there, but the events are destroyed after use;
//   - HIP_CHECK exits with status 1, not 0, so a failed run is visible to scripts.
#ifndef MMBO_HOST_COMMON_H
#define MMBO_HOST_COMMON_H

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define GPU_TIMER_START(elapsed_time, event_start, event_stop)                  \
    do {                                                                        \
        (elapsed_time) = 0.0f;                                                  \
        (void)hipEventCreateWithFlags(&(event_start), hipEventBlockingSync);    \
        (void)hipEventCreateWithFlags(&(event_stop), hipEventBlockingSync);     \
        (void)hipEventRecord((event_start), NULL);                              \
    } while (0)

#define GPU_TIMER_END(elapsed_time, event_start, event_stop)                    \
    do {                                                                        \
        (void)hipEventRecord((event_stop), NULL);                               \
        (void)hipEventSynchronize((event_stop));                                \
        (void)hipEventElapsedTime(&(elapsed_time), (event_start), (event_stop)); \
        (elapsed_time) /= 1000.0f;                                              \
        (void)hipEventDestroy((event_start));                                   \
        (void)hipEventDestroy((event_stop));                                    \
    } while (0)

#define HIP_CHECK(status)                                                                       \
    do {                                                                                        \
        hipError_t mmbo_hip_status_ = (status);                                                 \
        if (mmbo_hip_status_ != hipSuccess) {                                                   \
            std::fprintf(stderr, "HIP error %d (%s) at %s:%d\n", (int)mmbo_hip_status_,         \
                         hipGetErrorString(mmbo_hip_status_), __FILE__, __LINE__);              \
            std::exit(1);                                                                       \
        }                                                                                       \
    } while (0)

#define MMBO_CHECK(status)                                                                      \
    do {                                                                                        \
        int mmbo_status_ = (status);                                                            \
        if (mmbo_status_ != 0) {                                                                \
            std::fprintf(stderr, "mmbo_gemm error %d (%s) at %s:%d\n", mmbo_status_,            \
                         mmbo_status_string(mmbo_status_), __FILE__, __LINE__);                 \
            std::exit(1);                                                                       \
        }                                                                                       \
    } while (0)

#endif
