// Shared host/device helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/splatad_hip.h"

#define SPLATAD_WAVE 64
#define SPLATAD_THREADS 256

void splatad_set_error(const char *fmt, ...);

#define SPLATAD_CHECK_HIP(expr)                                                              \
    do {                                                                                     \
        hipError_t _e = (expr);                                                              \
        if (_e != hipSuccess) {                                                              \
            splatad_set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e),         \
                              __FILE__, __LINE__);                                           \
            return -2;                                                                       \
        }                                                                                    \
    } while (0)

#define SPLATAD_REQUIRE(cond, ...)                                                           \
    do {                                                                                     \
        if (!(cond)) {                                                                       \
            splatad_set_error(__VA_ARGS__);                                                  \
            return -1;                                                                       \
        }                                                                                    \
    } while (0)

#define SPLATAD_LAUNCH_CHECK() SPLATAD_CHECK_HIP(hipGetLastError())

static inline uint32_t splatad_bit_width(uint32_t v) {
    uint32_t b = 0;
    while (v) {
        ++b;
        v >>= 1;
    }
    return b;
}

static inline size_t splatad_align256(size_t v) { return (v + 255) & ~(size_t)255; }

#ifdef __HIPCC__

struct Mat3 {
    float m[9]; // row-major
};

__device__ __forceinline__ Mat3 mat3_mul(const Mat3 &A, const Mat3 &B) {
    Mat3 C;
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j)
            C.m[i * 3 + j] = A.m[i * 3] * B.m[j] + A.m[i * 3 + 1] * B.m[3 + j] + A.m[i * 3 + 2] * B.m[6 + j];
    return C;
}

// A * B^T
__device__ __forceinline__ Mat3 mat3_mul_bt(const Mat3 &A, const Mat3 &B) {
    Mat3 C;
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j)
            C.m[i * 3 + j] = A.m[i * 3] * B.m[j * 3] + A.m[i * 3 + 1] * B.m[j * 3 + 1] + A.m[i * 3 + 2] * B.m[j * 3 + 2];
    return C;
}

// A^T * B
__device__ __forceinline__ Mat3 mat3_mul_at(const Mat3 &A, const Mat3 &B) {
    Mat3 C;
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j)
            C.m[i * 3 + j] = A.m[i] * B.m[j] + A.m[3 + i] * B.m[3 + j] + A.m[6 + i] * B.m[6 + j];
    return C;
}

__device__ __forceinline__ Mat3 mat3_transpose(const Mat3 &A) {
    Mat3 C;
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) C.m[i * 3 + j] = A.m[j * 3 + i];
    return C;
}

__device__ __forceinline__ Mat3 mat3_zero() {
    Mat3 C;
#pragma unroll
    for (int i = 0; i < 9; ++i) C.m[i] = 0.f;
    return C;
}

// Rotation matrix of the (w, x, y, z) quaternion, normalised here.
__device__ __forceinline__ Mat3 quat_to_rotmat(float w, float x, float y, float z) {
    float inv = rsqrtf(w * w + x * x + y * y + z * z);
    w *= inv; x *= inv; y *= inv; z *= inv;
    float x2 = x * x, y2 = y * y, z2 = z * z;
    float xy = x * y, xz = x * z, yz = y * z;
    float wx = w * x, wy = w * y, wz = w * z;
    Mat3 R;
    R.m[0] = 1.f - 2.f * (y2 + z2); R.m[1] = 2.f * (xy - wz); R.m[2] = 2.f * (xz + wy);
    R.m[3] = 2.f * (xy + wz); R.m[4] = 1.f - 2.f * (x2 + z2); R.m[5] = 2.f * (yz - wx);
    R.m[6] = 2.f * (xz - wy); R.m[7] = 2.f * (yz + wx); R.m[8] = 1.f - 2.f * (x2 + y2);
    return R;
}

// Sum over the 64 lanes of a wavefront; every lane gets the total.
// Lane mask of a predicate.  Unlike __ballot(int) this takes the condition as it is held
// (one bit per lane in a scalar register pair), without a round trip through a vector register.
__device__ __forceinline__ uint64_t wave_ballot(bool pred) {
    return __builtin_amdgcn_ballot_w64(pred);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, SPLATAD_WAVE);
    return v;
}

// Sums NV (a power of two, 2..64) per-lane values over the 64 lanes of a wavefront with
// NV - 1 + log2(64 / NV) shuffles instead of 6 NV: at every step a lane hands half of its
// values to the partner that keeps accumulating them.  Afterwards every lane holds, in
// v[0], the wavefront total of value `wave_reduce_slot<NV>(lane)`; 64 / NV lanes hold each.
template <int NV>
__device__ __forceinline__ void wave_reduce_scatter(float (&v)[NV], int lane) {
    int off = 32;
#pragma unroll
    for (int half = NV / 2; half >= 1; half /= 2) {
        // bit masks instead of selects: a select between two array elements would be turned
        // into a dynamically indexed access, i.e. a compare-and-select chain over the array
        const uint32_t m = (lane & off) != 0 ? 0xFFFFFFFFu : 0u; // upper half of the pair
#pragma unroll
        for (int k = 0; k < half; ++k) {
            const uint32_t lo = __float_as_uint(v[k]), hi = __float_as_uint(v[k + half]);
            const float send = __uint_as_float((lo & m) | (hi & ~m));
            const float keep = __uint_as_float((hi & m) | (lo & ~m));
            v[k] = keep + __shfl_xor(send, off, SPLATAD_WAVE);
        }
        off >>= 1;
    }
#pragma unroll
    for (int rest = 32 / NV; rest >= 1; rest /= 2) v[0] += __shfl_xor(v[0], rest, SPLATAD_WAVE);
}

template <int NV>
__device__ __forceinline__ int wave_reduce_slot(int lane) {
    return NV == 64 ? lane : lane / (64 / NV);
}

__device__ __forceinline__ int wave_max_i32(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        int o = __shfl_xor(v, off, SPLATAD_WAVE);
        v = o > v ? o : v;
    }
    return v;
}

#endif // __HIPCC__
