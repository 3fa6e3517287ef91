// Host-side helpers shared by the C-ABI front ends (pools, one-shot GEMV): monotonic clock, bounded error text, whole-range
// pread, grow-only device buffers.
#pragma once
#include <errno.h>
#include <limits.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <time.h>
#include <unistd.h>

#include <hip/hip_runtime.h>

namespace redhip {

inline double now_ms() {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec * 1000.0 + (double)ts.tv_nsec / 1.0e6;
}

inline void set_err(char *dst, size_t cap, const char *fmt, ...) {
    if (!dst || !cap) return;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(dst, cap, fmt, ap);
    va_end(ap);
}

// whole-range pread with EINTR retry; counts calls and bytes
inline bool pread_range(int fd, uint64_t file_size, uint64_t offset, uint64_t len, uint8_t *dst, uint64_t *bytes, uint64_t *calls,
                        char *err, size_t cap) {
    if (!dst || offset > file_size || len > file_size - offset) {
        set_err(err, cap, "invalid pread range offset=%llu len=%llu file_size=%llu", (unsigned long long)offset,
                (unsigned long long)len, (unsigned long long)file_size);
        return false;
    }
    uint64_t pos = 0;
    while (pos < len) {
        const uint64_t rem = len - pos;
        const size_t want = rem > (uint64_t)SSIZE_MAX ? (size_t)SSIZE_MAX : (size_t)rem;
        ssize_t n;
        do { n = pread(fd, dst + pos, want, (off_t)(offset + pos)); } while (n < 0 && errno == EINTR);
        if (calls) ++*calls;
        if (n <= 0) {
            set_err(err, cap, n < 0 ? "pread failed: %s" : "unexpected end of file%s", n < 0 ? strerror(errno) : "");
            return false;
        }
        pos += (uint64_t)n;
    }
    if (bytes) *bytes += len;
    return true;
}

struct DevBuf {                       // grow-only device scratch
    void *p = nullptr;
    size_t cap = 0;
    bool reserve(size_t n) {
        if (n <= cap) return true;
        if (p) (void)hipFree(p);
        p = nullptr;
        cap = 0;
        if (hipMalloc(&p, n) != hipSuccess) { p = nullptr; return false; }
        cap = n;
        return true;
    }
    ~DevBuf() { if (p) (void)hipFree(p); }
};

inline bool sizes_overflow(uint64_t a, uint64_t b, uint64_t c) { return a > UINT64_MAX - b || a + b > UINT64_MAX - c; }

}  // namespace redhip
