// Real spherical-harmonic colour evaluation (degree 0..4) and its VJP for gfx950.
//
// One lane per direction: the basis values are computed once and contracted with the three
// colour channels.  The basis follows Sloan's "Efficient Spherical Harmonic Evaluation"
// (JCGT 2013) with the Condon-Shortley phase kept, the convention of
// gsplat/cuda/csrc/sh.cu:13-93 of the reference.  The azimuthal factors are
// C_m + i S_m = (x + i y)^m, so their derivatives are m (C_{m-1}, S_{m-1}) in x and
// m (-S_{m-1}, C_{m-1}) in y; the backward pass uses those closed forms.
#include "common.h"

namespace {

// Calls f(k, b, db/dx, db/dy, db/dz) for every active basis function k at the unit vector
// (x, y, z).  The derivatives treat x, y, z as independent variables.
template <typename F>
__device__ __forceinline__ void sh_for_each_basis(uint32_t degree, float x, float y, float z, F &&f) {
    f(0, 0.2820947917738781f, 0.f, 0.f, 0.f);
    if (degree < 1) return;
    const float k1 = 0.48860251190292f;
    f(1, -k1 * y, 0.f, -k1, 0.f);
    f(2, k1 * z, 0.f, 0.f, k1);
    f(3, -k1 * x, -k1, 0.f, 0.f);
    if (degree < 2) return;
    const float z2 = z * z;
    const float c1 = x * x - y * y, s1 = 2.f * x * y; // (x+iy)^2
    const float k2 = 0.5462742152960395f, k2z = -1.092548430592079f;
    f(4, k2 * s1, k2 * 2.f * y, k2 * 2.f * x, 0.f);
    f(5, k2z * z * y, 0.f, k2z * z, k2z * y);
    f(6, 0.9461746957575601f * z2 - 0.3153915652525201f, 0.f, 0.f, 2.f * 0.9461746957575601f * z);
    f(7, k2z * z * x, k2z * z, 0.f, k2z * x);
    f(8, k2 * c1, k2 * 2.f * x, -k2 * 2.f * y, 0.f);
    if (degree < 3) return;
    const float c2 = x * c1 - y * s1, s2 = x * s1 + y * c1; // (x+iy)^3
    const float k3 = -0.5900435899266435f, k3z = 1.445305721320277f;
    const float p3 = -2.285228997322329f * z2 + 0.4570457994644658f; // factor of m = +-1
    const float dp3 = -2.285228997322329f * 2.f * z;
    f(9, k3 * s2, k3 * 3.f * s1, k3 * 3.f * c1, 0.f);
    f(10, k3z * z * s1, k3z * z * 2.f * y, k3z * z * 2.f * x, k3z * s1);
    f(11, p3 * y, 0.f, p3, dp3 * y);
    f(12, z * (1.865881662950577f * z2 - 1.119528997770346f), 0.f, 0.f,
      3.f * 1.865881662950577f * z2 - 1.119528997770346f);
    f(13, p3 * x, p3, 0.f, dp3 * x);
    f(14, k3z * z * c1, k3z * z * 2.f * x, -k3z * z * 2.f * y, k3z * c1);
    f(15, k3 * c2, k3 * 3.f * c1, -k3 * 3.f * s1, 0.f);
    if (degree < 4) return;
    const float c3 = x * c2 - y * s2, s3 = x * s2 + y * c2; // (x+iy)^4
    const float k4 = 0.6258357354491763f, k4z = -1.770130769779931f;
    const float q4 = z * (-4.683325804901025f * z2 + 2.007139630671868f); // m = +-1
    const float dq4 = 3.f * -4.683325804901025f * z2 + 2.007139630671868f;
    const float r4 = 3.31161143515146f * z2 - 0.47308734787878f; // m = +-2
    const float dr4 = 2.f * 3.31161143515146f * z;
    const float b12 = z * (1.865881662950577f * z2 - 1.119528997770346f);
    const float db12 = 3.f * 1.865881662950577f * z2 - 1.119528997770346f;
    const float b6 = 0.9461746957575601f * z2 - 0.3153915652525201f;
    const float db6 = 2.f * 0.9461746957575601f * z;
    f(16, k4 * s3, k4 * 4.f * s2, k4 * 4.f * c2, 0.f);
    f(17, k4z * z * s2, k4z * z * 3.f * s1, k4z * z * 3.f * c1, k4z * s2);
    f(18, r4 * s1, r4 * 2.f * y, r4 * 2.f * x, dr4 * s1);
    f(19, q4 * y, 0.f, q4, dq4 * y);
    f(20, 1.984313483298443f * z * b12 - 1.006230589874905f * b6, 0.f, 0.f,
      1.984313483298443f * (b12 + z * db12) - 1.006230589874905f * db6);
    f(21, q4 * x, q4, 0.f, dq4 * x);
    f(22, r4 * c1, r4 * 2.f * x, -r4 * 2.f * y, dr4 * c1);
    f(23, k4z * z * c2, k4z * z * 3.f * c1, -k4z * z * 3.f * s1, k4z * c2);
    f(24, k4 * c3, k4 * 4.f * c2, -k4 * 4.f * s2, 0.f);
}

// Coefficient rows ([K][3] floats per direction) are 12 K bytes apart, so a lane-per-row
// store writes 4 bytes into each of 64 cache lines per instruction.  The backward kernel
// therefore collects a workgroup's gradient rows in LDS (rows padded by one float so that
// the lanes of a wavefront hit different banks) and stores them with coalesced accesses
// (consecutive lanes, consecutive floats).  Only the first `used` floats of a row
// (3 (degree + 1)^2) are moved.
struct ShRows {
    uint32_t K3;     // floats per row in global memory
    uint32_t used;   // floats per row that the degree needs
    uint32_t dq, dr; // blockDim.x / K3 and blockDim.x % K3
};

// f(lds_index, global_index) for every used float of the workgroup's `rows` rows
template <typename F>
__device__ __forceinline__ void sh_for_each_float(const ShRows &r, uint32_t rows, F &&f) {
    uint32_t row = threadIdx.x / r.K3, col = threadIdx.x % r.K3;
    const uint32_t total = rows * r.K3;
    for (uint32_t e = threadIdx.x; e < total; e += blockDim.x) {
        if (col < r.used) f(row * (r.used + 1) + col, e);
        row += r.dq;
        col += r.dr;
        if (col >= r.K3) { col -= r.K3; ++row; }
    }
}

// Forward: every lane reads its own row; the rows are read completely, so the cache lines a
// wavefront touches are all used (measured faster than staging through LDS).
__global__ void __launch_bounds__(SPLATAD_THREADS)
sh_fwd_kernel(uint32_t n, uint32_t K, uint32_t degree, const float *__restrict__ dirs,
              const float *__restrict__ coeffs, const uint8_t *__restrict__ masks,
              float *__restrict__ colors) {
    const uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    float r = 0.f, g = 0.f, b = 0.f;
    if (masks == nullptr || masks[e]) {
        const float dx = dirs[(size_t)e * 3], dy = dirs[(size_t)e * 3 + 1], dz = dirs[(size_t)e * 3 + 2];
        const float inorm = rsqrtf(dx * dx + dy * dy + dz * dz);
        const float *cf = coeffs + (size_t)e * K * 3;
        sh_for_each_basis(degree, dx * inorm, dy * inorm, dz * inorm,
                          [&](int k, float v, float, float, float) {
                              r += v * cf[k * 3];
                              g += v * cf[k * 3 + 1];
                              b += v * cf[k * 3 + 2];
                          });
    }
    colors[(size_t)e * 3] = r;
    colors[(size_t)e * 3 + 1] = g;
    colors[(size_t)e * 3 + 2] = b;
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
sh_bwd_kernel(uint32_t n, ShRows rows, uint32_t degree, const float *__restrict__ dirs,
              const float *__restrict__ coeffs, const uint8_t *__restrict__ masks,
              const float *__restrict__ v_colors, float *__restrict__ v_coeffs,
              float *__restrict__ v_dirs) {
    extern __shared__ float s_rows[];
    const uint32_t first = blockIdx.x * blockDim.x;
    const uint32_t here = min(blockDim.x, n - first);
    const bool want_dirs = v_dirs != nullptr;
    const uint32_t e = first + threadIdx.x;
    // every lane writes its row of coefficient gradients to LDS, from where the workgroup
    // stores them coalesced; rows of masked directions are zeros (their gradients are zero)
    float *row = s_rows + (size_t)threadIdx.x * (rows.used + 1);
    const float *cf = coeffs + (size_t)min(e, n - 1) * rows.K3;
    if (e < n) {
        const bool active = masks == nullptr || masks[e];
        const float dx = active ? dirs[(size_t)e * 3] : 0.f, dy = active ? dirs[(size_t)e * 3 + 1] : 0.f;
        const float dz = active ? dirs[(size_t)e * 3 + 2] : 0.f;
        const float inorm = active ? rsqrtf(dx * dx + dy * dy + dz * dz) : 0.f;
        const float x = dx * inorm, y = dy * inorm, z = active ? dz * inorm : 1.f;
        const float vr = active ? v_colors[(size_t)e * 3] : 0.f;
        const float vg = active ? v_colors[(size_t)e * 3 + 1] : 0.f;
        const float vb = active ? v_colors[(size_t)e * 3 + 2] : 0.f;
        float gx = 0.f, gy = 0.f, gz = 0.f;
        sh_for_each_basis(degree, x, y, z, [&](int k, float v, float bx, float by, float bz) {
            if (want_dirs) {
                const float w = cf[k * 3] * vr + cf[k * 3 + 1] * vg + cf[k * 3 + 2] * vb;
                gx += w * bx; gy += w * by; gz += w * bz;
            }
            row[k * 3] = v * vr;
            row[k * 3 + 1] = v * vg;
            row[k * 3 + 2] = v * vb;
        });
        if (want_dirs && active) {
            // through the normalisation: (I - n n^T) g / |d|
            const float dot = gx * x + gy * y + gz * z;
            v_dirs[(size_t)e * 3] = (gx - dot * x) * inorm;
            v_dirs[(size_t)e * 3 + 1] = (gy - dot * y) * inorm;
            v_dirs[(size_t)e * 3 + 2] = (gz - dot * z) * inorm;
        }
    }
    __syncthreads();
    float *gout = v_coeffs + (size_t)first * rows.K3;
    sh_for_each_float(rows, here, [&](uint32_t l, uint32_t f) { gout[f] = s_rows[l]; });
}

static ShRows sh_rows(uint32_t K, uint32_t degree) {
    ShRows r;
    r.K3 = K * 3;
    r.used = (degree + 1) * (degree + 1) * 3;
    r.dq = SPLATAD_THREADS / r.K3;
    r.dr = SPLATAD_THREADS % r.K3;
    return r;
}

template <typename Kernel>
static int sh_lds(Kernel kernel, const ShRows &r, size_t *bytes) {
    *bytes = (size_t)SPLATAD_THREADS * (r.used + 1) * sizeof(float);
    if (*bytes > 64 * 1024)
        SPLATAD_CHECK_HIP(hipFuncSetAttribute((const void *)kernel,
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)*bytes));
    return 0;
}

} // namespace

extern "C" int splatad_sh_fwd(uint32_t n, uint32_t K, uint32_t degree, const float *dirs,
                              const float *coeffs, const uint8_t *masks, float *colors,
                              splatad_stream_t stream) {
    SPLATAD_REQUIRE(degree <= 4, "spherical harmonics: degree %u is above 4", degree);
    SPLATAD_REQUIRE((degree + 1) * (degree + 1) <= K, "spherical harmonics: %u bases for degree %u", K, degree);
    if (n == 0) return 0;
    SPLATAD_REQUIRE(dirs && coeffs && colors, "spherical harmonics: null pointer argument");
    hipLaunchKernelGGL(sh_fwd_kernel, dim3((n + SPLATAD_THREADS - 1) / SPLATAD_THREADS),
                       dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, n, K, degree, dirs, coeffs,
                       masks, colors);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

extern "C" int splatad_sh_bwd(uint32_t n, uint32_t K, uint32_t degree, const float *dirs,
                              const float *coeffs, const uint8_t *masks, const float *v_colors,
                              float *v_coeffs, float *v_dirs, splatad_stream_t stream) {
    SPLATAD_REQUIRE(degree <= 4, "spherical harmonics: degree %u is above 4", degree);
    SPLATAD_REQUIRE((degree + 1) * (degree + 1) <= K, "spherical harmonics: %u bases for degree %u", K, degree);
    if (n == 0) return 0;
    SPLATAD_REQUIRE(dirs && coeffs && v_colors && v_coeffs, "spherical harmonics: null pointer argument");
    const ShRows r = sh_rows(K, degree);
    size_t lds = 0;
    if (int rc = sh_lds(sh_bwd_kernel, r, &lds)) return rc;
    hipLaunchKernelGGL(sh_bwd_kernel, dim3((n + SPLATAD_THREADS - 1) / SPLATAD_THREADS),
                       dim3(SPLATAD_THREADS), lds, (hipStream_t)stream, n, r, degree, dirs, coeffs,
                       masks, v_colors, v_coeffs, v_dirs);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}
