// Spherical-harmonic colour of one direction, shared by the colour kernels (sh.hip) and the
// compositing kernel that evaluates the colours of the Gaussians it stages (rasterize_fwd.hip):
// both run the same instructions, so their colours are equal bit for bit.
#pragma once

#include "common.h"

#ifdef __HIPCC__

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

// Position of the sensor in the world: the translation column of the inverse of [A | t], -A^-1 t.
__device__ __forceinline__ void sensor_position(const float *vm, float &px, float &py, float &pz) {
    const float a = vm[0], b = vm[1], c = vm[2], d = vm[4], e = vm[5], f = vm[6], g = vm[8], h = vm[9], i = vm[10];
    const float tx = vm[3], ty = vm[7], tz = vm[11];
    const float c00 = e * i - f * h, c01 = c * h - b * i, c02 = b * f - c * e;
    const float c10 = f * g - d * i, c11 = a * i - c * g, c12 = c * d - a * f;
    const float c20 = d * h - e * g, c21 = b * g - a * h, c22 = a * e - b * d;
    const float inv_det = 1.f / (a * c00 + b * c10 + c * c20);
    px = -(c00 * tx + c01 * ty + c02 * tz) * inv_det;
    py = -(c10 * tx + c11 * ty + c12 * tz) * inv_det;
    pz = -(c20 * tx + c21 * ty + c22 * tz) * inv_det;
}

// The coefficients of band L (bases L^2 .. (L+1)^2 - 1) of one row
template <int L>
__device__ __forceinline__ void sh_load_band(float *c, const float *__restrict__ cf) {
#pragma unroll
    for (int f = 3 * L * L; f < 3 * (L + 1) * (L + 1); ++f) c[f] = cf[f];
}

// r, g, b += the colour of coefficient row cf ([K][3] floats) in the direction (dx, dy, dz), which
// need not be normalised.  The whole row is requested before the first use: one memory round
// trip.
__device__ __forceinline__ void sh_color(uint32_t degree, const float *__restrict__ cf, float dx, float dy,
                                         float dz, float &r, float &g, float &b) {
    const float inorm = rsqrtf(dx * dx + dy * dy + dz * dz);
    float c[75];
    sh_load_band<0>(c, cf);
    if (degree >= 1) sh_load_band<1>(c, cf); // uniform
    if (degree >= 2) sh_load_band<2>(c, cf);
    if (degree >= 3) sh_load_band<3>(c, cf);
    if (degree >= 4) sh_load_band<4>(c, cf);
    sh_for_each_basis(degree, dx * inorm, dy * inorm, dz * inorm,
                      [&](int k, float v, float, float, float) {
                          r += v * c[k * 3];
                          g += v * c[k * 3 + 1];
                          b += v * c[k * 3 + 2];
                      });
}

// The same sum with every band's coefficients requested when the band is reached (a memory round
// trip per band, and no more than a band's 3 (2 L + 1) values in registers), for a kernel that
// has few registers to spare.  Same products in the same order: the same colour bit for bit.
__device__ __forceinline__ void sh_color_by_band(uint32_t degree, const float *__restrict__ cf, float dx,
                                                 float dy, float dz, float &r, float &g, float &b) {
    const float inorm = rsqrtf(dx * dx + dy * dy + dz * dz);
    sh_for_each_basis(degree, dx * inorm, dy * inorm, dz * inorm,
                      [&](int k, float v, float, float, float) {
                          // the wide bands in two halves: the scheduler does not move the second
                          // half's loads up to the first's
                          if (k == 12 || k == 20) __builtin_amdgcn_sched_barrier(0);
                          r += v * cf[k * 3];
                          g += v * cf[k * 3 + 1];
                          b += v * cf[k * 3 + 2];
                      });
}

} // namespace

#endif // __HIPCC__
