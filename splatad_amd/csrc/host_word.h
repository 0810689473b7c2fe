// A 64-bit word that a kernel hands to the waiting host without draining the stream.
//
// Two-call entry points (count, then fill) need one number on the host between the calls: the
// size of the outputs the caller has to allocate.  A device-to-host copy plus a stream
// synchronisation would make the host wait for everything enqueued so far and leave the GPU
// idle until the next launch arrives.  Instead the producing kernel stores the number into a
// pinned host word (relaxed, system scope), the host polls that word, and whatever was enqueued
// behind the kernel keeps the GPU busy meanwhile.
#pragma once

#include <hip/hip_runtime.h>

#include <mutex>

#include "common.h"

namespace { // one private copy per translation unit

constexpr unsigned long long kHostWordPending = ~0ull;

// One pinned word, created at a device's first use and kept for the life of the process.  The
// owner serialises the sequences that use it.
struct HostWord {
    unsigned long long *host = nullptr, *device = nullptr; // host address, address for kernels
};

static inline int host_word_create(HostWord *w) {
    SPLATAD_CHECK_HIP(hipHostMalloc((void **)&w->host, 64, hipHostMallocDefault));
    SPLATAD_CHECK_HIP(hipHostGetDevicePointer((void **)&w->device, w->host, 0));
    return 0;
}

// A stream under graph capture would never deliver the word.
static inline int host_word_refuse_capture(hipStream_t stream, const char *what) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    SPLATAD_CHECK_HIP(hipStreamIsCapturing(stream, &capturing));
    SPLATAD_REQUIRE(capturing == hipStreamCaptureStatusNone,
                    "%s: the counting call returns a number to the host and cannot be captured in a graph",
                    what);
    return 0;
}

// Publishes *src (a kernel launched behind the one that wrote it, on the same stream).
__global__ void host_word_publish_kernel(const int64_t *__restrict__ src,
                                         unsigned long long *__restrict__ word) {
    if (blockIdx.x == 0 && threadIdx.x == 0)
        __hip_atomic_store(word, (unsigned long long)*src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Waits for the word only, not for the work behind it; now and then asks the stream, so that a
// failed launch or a fault ends the wait with its error.
static inline int host_word_wait(HostWord *w, hipStream_t stream, const char *what,
                                 unsigned long long *out) {
    volatile unsigned long long *slot = w->host;
    unsigned long long n = kHostWordPending;
    for (uint32_t spin = 1; (n = *slot) == kHostWordPending; ++spin) {
        __builtin_ia32_pause();
        if ((spin & 0xFFFFu) == 0) {
            const hipError_t q = hipStreamQuery(stream);
            if (q == hipErrorNotReady) { (void)hipGetLastError(); continue; }
            SPLATAD_CHECK_HIP(q);
            n = *slot; // the stream has drained: the word is there, or never will be
            SPLATAD_REQUIRE(n != kHostWordPending, "%s: the counting kernel left no result", what);
            break;
        }
    }
    *out = n;
    return 0;
}

} // namespace
