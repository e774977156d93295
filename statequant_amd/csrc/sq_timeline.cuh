// Optional instrumentation, compiled in with -DSQ_TIMELINE only (build.py --timeline writes a library of its own):
// every wavefront of a marked kernel records the 100 MHz real-time counter at fixed points of its life, 16 x 8 bytes
// per wavefront, workgroup-major, into the buffer that the environment variable SQ_TIMELINE_BUF names at the time
// of the launch as "<device address>:<capacity in wavefronts>" (decimal); wavefronts beyond the capacity record
// nothing.  A launch can then be laid out as a timeline of its workgroups (profile_timeline.py).  A mark waits for the scalar loads and LDS operations in flight, so the marks cost a
// wavefront about a microsecond altogether.  Without the define they compile to nothing.  A marked kernel takes the
// buffer as `SQ_TL_PARAM` ahead of its parameter struct; its launcher passes `sq_timeline_buffer()`.
#pragma once
#ifdef SQ_TIMELINE
#include <stdint.h>
#include <stdlib.h>
#define SQ_TL_PARAM uint64_t* tl, uint32_t tl_cap,
#define SQ_MARK(k)                                                                                                 \
    do {                                                                                                           \
        if (tl) {                                                                                                  \
            uint64_t t_;                                                                                           \
            asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t_)::"memory");                         \
            const uint32_t wv_ = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);                             \
            if ((threadIdx.x & 63) == 0 && wv_ < tl_cap) tl[uint64_t(wv_) * 16 + (k)] = t_;                        \
        }                                                                                                          \
    } while (0)
struct SqTimelineBuf { uint64_t* p; uint32_t cap; };
inline SqTimelineBuf sq_timeline_buffer() {
    const char* e = getenv("SQ_TIMELINE_BUF");
    if (!e) return {nullptr, 0u};
    char* end = nullptr;
    uint64_t* p = reinterpret_cast<uint64_t*>(strtoull(e, &end, 10));
    const uint32_t cap = (end && *end == ':') ? uint32_t(strtoul(end + 1, nullptr, 10)) : 0u;
    return {cap ? p : nullptr, cap};
}
#else
#define SQ_TL_PARAM
#define SQ_MARK(k) do { } while (0)
#endif
