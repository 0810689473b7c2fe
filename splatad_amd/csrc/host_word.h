// A 64-bit word that a kernel hands to the waiting host without draining the stream.
//
// Two-call entry points (count, then fill) need one number on the host between the calls: the
// size of the outputs the caller has to allocate.  A device-to-host copy plus a stream
// synchronisation would make the host wait for everything enqueued so far and leave the GPU
// idle until the next launch arrives.  Instead the producing kernel stores the number into a
// pinned host word (relaxed, system scope), the host polls that word, and whatever was enqueued
// behind the kernel keeps the GPU busy meanwhile.
//
// Calls from several host threads (each on a stream of its own) overlap: a device owns a small
// pool of such words, a call leases one for as long as a kernel may still write it, and no lock
// is held while a call waits for its word.
#pragma once

#include <hip/hip_runtime.h>

#include <mutex>
#include <thread>

#include "common.h"

namespace { // one private copy per translation unit

constexpr unsigned long long kHostWordPending = ~0ull;
constexpr int kHostWordSlots = 16;      // concurrent counting calls per device and pool
constexpr int kHostWordStride = 8;      // words between slots: a 64-byte line each
constexpr int kHostWordDevices = 64;

// The pinned words of one device, created at the device's first use and kept for the life of
// the process (1 KiB of pinned host memory).
struct HostWordPool {
    unsigned long long *host = nullptr, *device = nullptr; // host address, address for kernels
    uint32_t busy = 0;                                      // bit per leased slot
    std::mutex guard;                                       // protects `busy` and the creation
};

struct HostWord {
    unsigned long long *host = nullptr, *device = nullptr;
    HostWordPool *pool = nullptr;
    int slot = -1;
};

static inline int host_word_pool(HostWordPool **out) {
    static HostWordPool pools[kHostWordDevices];
    int dev = 0;
    SPLATAD_CHECK_HIP(hipGetDevice(&dev));
    SPLATAD_REQUIRE(dev >= 0 && dev < kHostWordDevices, "device index %d out of range", dev);
    HostWordPool *p = &pools[dev];
    std::lock_guard<std::mutex> lock(p->guard);
    if (p->host == nullptr) {
        unsigned long long *h = nullptr, *d = nullptr;
        SPLATAD_CHECK_HIP(hipHostMalloc((void **)&h, kHostWordSlots * kHostWordStride * 8, hipHostMallocDefault));
        SPLATAD_CHECK_HIP(hipHostGetDevicePointer((void **)&d, h, 0));
        p->device = d;
        p->host = h;
    }
    *out = p;
    return 0;
}

// Leases a word of the current device's pool and marks it pending.  With every slot leased
// (more than kHostWordSlots counting calls in flight on one device) the caller yields until one
// is returned.
static inline int host_word_acquire(HostWord *w) {
    HostWordPool *p = nullptr;
    if (int rc = host_word_pool(&p)) return rc;
    for (;;) {
        {
            std::lock_guard<std::mutex> lock(p->guard);
            for (int s = 0; s < kHostWordSlots; ++s) {
                if (p->busy & (1u << s)) continue;
                p->busy |= 1u << s;
                w->pool = p;
                w->slot = s;
                w->host = p->host + s * kHostWordStride;
                w->device = p->device + s * kHostWordStride;
                *(volatile unsigned long long *)w->host = kHostWordPending;
                return 0;
            }
        }
        std::this_thread::yield();
    }
}

// Returns the word to its pool.  `delivered` says that the kernel's store has been seen; if it
// has not (an error between the launch and the wait), the stream is drained first, so that a
// late store cannot land in the word's next lease.
static inline void host_word_release(HostWord *w, hipStream_t stream, bool delivered) {
    if (w->pool == nullptr) return;
    if (!delivered) {
        (void)hipStreamSynchronize(stream);
        (void)hipGetLastError();
    }
    std::lock_guard<std::mutex> lock(w->pool->guard);
    w->pool->busy &= ~(1u << w->slot);
    w->pool = nullptr;
}

// Scope of a lease: released (after draining the stream, unless the word was delivered) when the
// call returns, whichever way.
struct HostWordLease {
    HostWord word;
    hipStream_t stream;
    bool delivered = false;
    explicit HostWordLease(hipStream_t s) : stream(s) {}
    HostWordLease(const HostWordLease &) = delete;
    HostWordLease &operator=(const HostWordLease &) = delete;
    ~HostWordLease() { host_word_release(&word, stream, delivered); }
};

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
static inline int host_word_wait(HostWordLease *lease, const char *what, unsigned long long *out) {
    volatile unsigned long long *slot = lease->word.host;
    unsigned long long n = kHostWordPending;
    for (uint32_t spin = 1; (n = *slot) == kHostWordPending; ++spin) {
        __builtin_ia32_pause();
        if ((spin & 0xFFFFu) == 0) {
            const hipError_t q = hipStreamQuery(lease->stream);
            if (q == hipErrorNotReady) { (void)hipGetLastError(); continue; }
            SPLATAD_CHECK_HIP(q);
            n = *slot; // the stream has drained: the word is there, or never will be
            lease->delivered = true; // nothing is left that could still write it
            SPLATAD_REQUIRE(n != kHostWordPending, "%s: the counting kernel left no result", what);
            break;
        }
    }
    lease->delivered = true;
    *out = n;
    return 0;
}

} // namespace
