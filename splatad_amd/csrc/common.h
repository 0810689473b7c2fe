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

// The reverse: a per-lane predicate from a lane mask held in scalar registers (free: the
// hardware keeps predicates as such masks).  Predicates that are combined with scalar logic on
// their masks cost no vector instructions, and "no lane left" is a scalar compare.
__device__ __forceinline__ bool wave_lanes(uint64_t mask) {
    return __builtin_amdgcn_inverse_ballot_w64(mask);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, SPLATAD_WAVE);
    return v;
}

// Lane permutations inside the vector ALU (no LDS round trip): `pattern` is a DPP control --
// 0x140 mirrors each row of 16 lanes, 0x141 each half row of 8, 0x4E swaps the pairs of a quad
// (lane ^ 2), 0xB1 the neighbours (lane ^ 1).  All lanes of the wavefront must be active.
template <int pattern>
__device__ __forceinline__ float wave_dpp(float v) {
    return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), pattern, 0xF, 0xF, false));
}

// One step of a reduce-scatter between lanes that differ in bit `BIT` (5..0) of the lane
// index: afterwards the lanes whose bit is clear hold, in `a`, the pair's sum of `a`, the
// others the pair's sum of `b`.  Bits 5 and 4 use the gfx950 half-swaps (the upper 32 or the
// odd 16 lanes of one register change places with the lower 32 or even 16 of the other, so a
// single add finishes the step); bits 3 and 2 pair lanes by mirroring a row or a half row,
// which also flips lower bits -- harmless, those have not been used yet.
template <int BIT>
__device__ __forceinline__ float wave_pair_step(float a, float b, int lane) {
    if constexpr (BIT == 5) {
        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
        return __uint_as_float(r[0]) + __uint_as_float(r[1]);
    } else if constexpr (BIT == 4) {
        const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
        return __uint_as_float(r[0]) + __uint_as_float(r[1]);
    } else {
        constexpr int pattern = BIT == 3 ? 0x140 : (BIT == 2 ? 0x141 : (BIT == 1 ? 0x4E : 0xB1));
        const float sa = a + wave_dpp<pattern>(a), sb = b + wave_dpp<pattern>(b);
        return (lane & (1 << BIT)) == 0 ? sa : sb;
    }
}

template <int NV, int BIT>
__device__ __forceinline__ void wave_reduce_scatter_from(float (&v)[NV], int lane) {
    constexpr int half = NV >> (6 - BIT); // values still held per lane, halved by this step
    if constexpr (half >= 1) {
#pragma unroll
        for (int k = 0; k < half; ++k) v[k] = wave_pair_step<BIT>(v[k], v[k + half], lane);
        if constexpr (BIT > 0) wave_reduce_scatter_from<NV, BIT - 1>(v, lane);
    } else {
        // one value left per lane: the lanes that share it add up their parts
        constexpr int pattern = BIT == 3 ? 0x140 : (BIT == 2 ? 0x141 : (BIT == 1 ? 0x4E : 0xB1));
        static_assert(BIT <= 3, "at least four values per lane");
        v[0] += wave_dpp<pattern>(v[0]);
        if constexpr (BIT > 0) wave_reduce_scatter_from<NV, BIT - 1>(v, lane);
    }
}

// Sums NV (a power of two, 4..64) per-lane values over the 64 lanes of a wavefront: at every
// step a lane hands half of its values to a partner that keeps accumulating them, so the
// work halves from step to step (NV - 1 exchanges instead of 6 NV).  Afterwards every lane
// holds, in v[0], the wavefront total of value `wave_reduce_slot<NV>(lane)`; 64 / NV lanes
// hold each.  All 64 lanes must be active.
template <int NV>
__device__ __forceinline__ void wave_reduce_scatter(float (&v)[NV], int lane) {
    static_assert(NV >= 4 && NV <= 64 && (NV & (NV - 1)) == 0, "NV must be a power of two in 4..64");
    wave_reduce_scatter_from<NV, 5>(v, lane);
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
