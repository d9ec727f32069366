// Stage timestamps inside the attention kernels, for the measurement build only.
//
// The library proper compiles ITAK_MARK* to nothing. Built with -DITAK_TIMELINE
// (`python build.py --timeline` writes lib/libitak_hip_kv_timeline.so) every wavefront of a
// marked kernel records the constant 100 MHz clock at its numbered marks and leaves them in a
// buffer in device memory, which `bench.py --timeline` reads back through the reader function
// the kernel's file exports and turns into a table of stage times. Each source file that uses
// marks has its own buffer and reader (device symbols are private to a file here).
#pragma once

#include <hip/hip_runtime.h>

#ifdef ITAK_TIMELINE

#define ITAK_TIMELINE_MARKS 12
#define ITAK_TIMELINE_WAVES 8192  // wavefront records kept (8 per workgroup of the first 1024)

static __device__ unsigned long long itak_timeline_buf[ITAK_TIMELINE_WAVES * ITAK_TIMELINE_MARKS];

// Defines `extern "C" int NAME(unsigned long long *host, unsigned long long count)`: copies the
// first `count` words of this file's buffer to host memory and clears nothing.
#define ITAK_TIMELINE_READER(NAME)                                                            \
    extern "C" __attribute__((visibility("default"))) int NAME(unsigned long long *host,      \
                                                               unsigned long long count) {    \
        return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(itak_timeline_buf), count * 8);      \
    }

#define ITAK_MARK_BEGIN                                \
    unsigned long long tm_[ITAK_TIMELINE_MARKS];       \
    _Pragma("unroll") for (int i_ = 0; i_ < ITAK_TIMELINE_MARKS; ++i_) tm_[i_] = 0;
#define ITAK_MARK(i)                             \
    {                                            \
        __builtin_amdgcn_sched_barrier(0);       \
        tm_[i] = wall_clock64();                 \
        __builtin_amdgcn_sched_barrier(0);       \
    }
// The last mark waits for everything the wavefront has in flight (stores included), then the
// record of wavefront w of workgroup b goes to slot b*8 + w (+ `base` for a second kernel).
#define ITAK_MARK_END_AT(base)                                                                 \
    {                                                                                          \
        __builtin_amdgcn_s_waitcnt(0);                                                         \
        tm_[ITAK_TIMELINE_MARKS - 1] = wall_clock64();                                         \
        if ((threadIdx.x & 63) == 0) {                                                         \
            const unsigned w_ = (base) + blockIdx.x * 8 + (threadIdx.x >> 6);                  \
            if (w_ < ITAK_TIMELINE_WAVES) {                                                    \
                _Pragma("unroll") for (int i_ = 0; i_ < ITAK_TIMELINE_MARKS; ++i_)             \
                    itak_timeline_buf[w_ * ITAK_TIMELINE_MARKS + i_] = tm_[i_];                \
            }                                                                                  \
        }                                                                                      \
    }
#define ITAK_MARK_END ITAK_MARK_END_AT(0)

#else

#define ITAK_TIMELINE_READER(NAME)
#define ITAK_MARK_BEGIN
#define ITAK_MARK(i)
#define ITAK_MARK_END_AT(base)
#define ITAK_MARK_END

#endif
