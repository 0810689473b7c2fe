// Pieces shared by the forward and backward compositing kernels: the staged form of a
// Gaussian's exponent, the folded angle difference of the lidar path and the per-wavefront
// footprint tests that let a wavefront skip Gaussians none of its 64 lanes can see.
#pragma once

#include "common.h"

#ifdef __HIPCC__
namespace {

constexpr float kLog2e = 1.44269504088896341f;
constexpr float kLn2 = 0.693147180559945309f;
constexpr float kLog2Of255 = 7.99435343685886f;

// Staged exponent of a Gaussian: alpha = exp2(L - (A dx^2 + B dx dy + C dy^2)), i.e.
// A = a log2(e) / 2, B = b log2(e), C = c log2(e) / 2 for the conic (a, b, c) and
// L = log2(opacity) (-inf for opacity <= 0, which can then never reach alpha >= 1/255).
__device__ __forceinline__ float4 staged_exponent(float a, float b, float c, float opacity) {
#pragma clang fp contract(off)
    return make_float4(0.5f * kLog2e * a, kLog2e * b, 0.5f * kLog2e * c,
                       opacity > 0.f ? __log2f(opacity) : -INFINITY);
}

// The arithmetic behind the two discontinuous decisions of the compositing rule (alpha >=
// 1/255, transmittance <= 1e-4), with every rounding spelled out.  All compositing kernels
// (forward, backward, index lists, every channel width) go through these, so that they take
// the same decisions for the same inputs; left to the compiler, the fusing of multiplies and
// adds differs from one instantiation to the next and with it the last bit of alpha.
__device__ __forceinline__ float gaussian_offset(float mean, float velocity, float roll, float at) {
    return fmaf(roll, velocity, mean) - at;
}
__device__ __forceinline__ float gaussian_power(const float4 e, float dx, float dy) {
    const float cross = fmaf(e.x, dx, e.y * dy);
    const float along = dx * cross;
    return fmaf(dy, e.z * dy, along);
}
__device__ __forceinline__ float transmittance_behind(float T, float alpha) {
    return fmaf(-alpha, T, T); // T (1 - alpha)
}

// Difference of two angles in degrees folded into [-180, 180), as the reference's
// fmodf(a - b + 180, 360) - 180 with negative results raised by 360
// (gsplat/cuda/csrc/utils.cuh:552-555).  Without the detour through +180 / -180 the difference of two
// nearby angles is exact in float32.
__device__ __forceinline__ float angle_difference(float a, float b) {
    const float d = a - b;
    if (d >= -180.f && d < 180.f) return d;
    float m = fmodf(d + 180.f, 360.f);
    if (m < 0.f) m += 360.f;
    return m - 180.f;
}

// Smallest value of p(d) = A dx^2 + B dx dy + C dy^2 over the box [x0, x1] x [y0, y1] of
// offsets, compared with the largest p that still passes alpha >= 1/255, L + log2(255).
// p is convex for a positive definite conic, so off the centre its minimum over the box lies
// on one of the four edges.  A margin covers the rounding of the test itself; Gaussians with
// a degenerate conic are never rejected.  Returns false when no offset in the box can pass.
// half_inv_free = 1 / (2 free_coef): the minimiser along the edge is -cross * fixed / (2 free_coef),
// clamped to the edge; an error of a few ulp in it moves the minimum in second order only.
__device__ __forceinline__ float edge_min(float fixed_coef, float free_coef, float cross,
                                          float half_inv_free, float fixed, float lo, float hi) {
    const float free_c = fminf(fmaxf(-cross * fixed * half_inv_free, lo), hi);
    return fixed_coef * fixed * fixed + free_c * (free_coef * free_c + cross * fixed);
}

__device__ __forceinline__ bool box_may_pass(const float4 e, float x0, float x1, float y0, float y1) {
    const float A = e.x, B = e.y, C = e.z;
    const bool definite = A > 0.f && C > 0.f && 4.f * A * C - B * B > 0.f;
    const bool centre_in = x0 <= 0.f && x1 >= 0.f && y0 <= 0.f && y1 >= 0.f;
    const float hA = 0.5f * __builtin_amdgcn_rcpf(A), hC = 0.5f * __builtin_amdgcn_rcpf(C);
    const float q = fminf(fminf(edge_min(A, C, B, hC, x0, y0, y1), edge_min(A, C, B, hC, x1, y0, y1)),
                          fminf(edge_min(C, A, B, hA, y0, x0, x1), edge_min(C, A, B, hA, y1, x0, x1)));
    const float limit = e.w + kLog2Of255;
    return !(definite && !centre_in && q > limit + 1e-3f * fabsf(limit) + 0.02f);
}

// Footprint of a wavefront of camera pixels: bounding box of the pixel centres and range of
// the rolling-shutter factor over its lanes (all 64 lanes must exist).
struct WaveCull {
    bool enabled;
    float cx, cy, hx, hy;
    float roll_mid, roll_half;

    __device__ __forceinline__ void init(float px, float py, float roll, bool full_wavefront) {
        init(px, py, py, roll, roll, full_wavefront);
    }
    // a lane with several pixels in one column: rows py_a .. py_b, factors roll_a .. roll_b
    __device__ __forceinline__ void init(float px, float py_a, float py_b, float roll_a, float roll_b,
                                         bool full_wavefront) {
        enabled = full_wavefront;
        float x_lo = px, x_hi = px, y_lo = fminf(py_a, py_b), y_hi = fmaxf(py_a, py_b);
        float r_lo = fminf(roll_a, roll_b), r_hi = fmaxf(roll_a, roll_b);
        if (enabled) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                x_lo = fminf(x_lo, __shfl_xor(x_lo, off, SPLATAD_WAVE));
                x_hi = fmaxf(x_hi, __shfl_xor(x_hi, off, SPLATAD_WAVE));
                y_lo = fminf(y_lo, __shfl_xor(y_lo, off, SPLATAD_WAVE));
                y_hi = fmaxf(y_hi, __shfl_xor(y_hi, off, SPLATAD_WAVE));
                r_lo = fminf(r_lo, __shfl_xor(r_lo, off, SPLATAD_WAVE));
                r_hi = fmaxf(r_hi, __shfl_xor(r_hi, off, SPLATAD_WAVE));
            }
        }
        cx = 0.5f * (x_lo + x_hi); hx = 0.5f * (x_hi - x_lo);
        cy = 0.5f * (y_lo + y_hi); hy = 0.5f * (y_hi - y_lo);
        roll_mid = 0.5f * (r_lo + r_hi);
        roll_half = 0.5f * (r_hi - r_lo) * 1.0001f + 1e-12f;
    }

    // xyv = {mean x, mean y, pixel velocity x, y}: the offsets mean + roll * velocity -
    // pixel of the wavefront lie in a box around (mean + roll_mid * velocity - centre)
    __device__ __forceinline__ bool may_touch(const float4 xyv, const float4 e) const {
        if (!enabled) return true;
        const float mx = xyv.x + roll_mid * xyv.z - cx, my = xyv.y + roll_mid * xyv.w - cy;
        const float ex = hx + fabsf(xyv.z) * roll_half, ey = hy + fabsf(xyv.w) * roll_half;
        return box_may_pass(e, mx - ex, mx + ex, my - ey, my + ey);
    }
};

// Footprint of a wavefront of lidar points.  All angles are taken relative to a reference
// point of the tile, so that neither the +-180 degree seam nor the size of the absolute
// angles matters: the staged record holds u = (mean - reference) and the lane r = (point -
// reference), both folded, and the offset of a pair is u + roll * velocity - r as long as
// that cannot leave (-180, 180).  The test decides for every Gaussian whether any lane can
// reach alpha >= 1/255 and whether the unfolded difference is safe (it is unless the
// Gaussian sits half a turn away from the tile).
struct WavePointCull {
    bool enabled;
    float x_lo, x_hi, y_lo, y_hi; // box of the lanes' r
    float roll_mid, roll_half;

    __device__ __forceinline__ void init(bool alive, float rx, float ry, float roll,
                                         bool full_wavefront) {
        enabled = full_wavefront;
        const float inf = INFINITY;
        float xl = alive ? rx : inf, xh = alive ? rx : -inf;
        float yl = alive ? ry : inf, yh = alive ? ry : -inf;
        float rl = alive ? roll : inf, rh = alive ? roll : -inf;
        if (enabled) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                xl = fminf(xl, __shfl_xor(xl, off, SPLATAD_WAVE));
                xh = fmaxf(xh, __shfl_xor(xh, off, SPLATAD_WAVE));
                yl = fminf(yl, __shfl_xor(yl, off, SPLATAD_WAVE));
                yh = fmaxf(yh, __shfl_xor(yh, off, SPLATAD_WAVE));
                rl = fminf(rl, __shfl_xor(rl, off, SPLATAD_WAVE));
                rh = fmaxf(rh, __shfl_xor(rh, off, SPLATAD_WAVE));
            }
        } else { // partial wavefront: no culling, bounds of the whole folded range
            xl = yl = -180.f; xh = yh = 180.f;
            rl = rh = roll;
        }
        // slightly widened against the rounding of the test itself
        x_lo = xl - 1e-4f; x_hi = xh + 1e-4f;
        y_lo = yl - 1e-4f; y_hi = yh + 1e-4f;
        roll_mid = 0.5f * (rl + rh);
        roll_half = 0.5f * (rh - rl) * 1.0001f + 1e-12f;
    }

    __device__ __forceinline__ bool may_touch(const float4 uv, const float4 e, bool &unfolded_ok) const {
        const float cx = uv.x + roll_mid * uv.z, cy = uv.y + roll_mid * uv.w;
        const float ex = fabsf(uv.z) * roll_half, ey = fabsf(uv.w) * roll_half;
        const float x0 = cx - x_hi - ex, x1 = cx - x_lo + ex;
        const float y0 = cy - y_hi - ey, y1 = cy - y_lo + ey;
        unfolded_ok = fmaxf(fmaxf(fabsf(x0), fabsf(x1)), fmaxf(fabsf(y0), fabsf(y1))) < 179.f;
        if (!unfolded_ok || !enabled) return true;
        return box_may_pass(e, x0, x1, y0, y1);
    }
};

// ---------------------------------------------------------------------------------------------
// The exponent of a camera pixel as a polynomial in tile-centred pixel coordinates.
//
// With the rolling-shutter factor linear in the pixel row, roll = roll_c + roll_s Y, the offset
// of pixel (X, Y) (relative to the tile centre) from a Gaussian is dx = dx0 - X + sx Y, dy = dy0 +
// sy Y, and log2(alpha) = L - (A dx^2 + B dx dy + C dy^2) is a quadratic polynomial in (X, Y)
// whose six coefficients depend on the Gaussian and the tile only.  They are computed once per
// (tile, Gaussian) when the Gaussian is staged; a pixel then needs five fused multiply-adds
// with its own constants (X, Y, X^2, Y^2; exact in float32 for half-integers) instead of
// the ten operations of the offset form, and every kernel that evaluates a pixel through
// pixel_exponent() gets the same bits, whatever its lane layout.  Inside a 16 x 16 tile |X|, |Y|
// <= 7.5, and the cancellation between the terms costs at most a few 1e-5 of absolute accuracy
// in the exponent for the sharpest Gaussians the projection can produce (conic 1 / eps2d).
struct TileFrame {
    float cx, cy;         // tile centre in pixel coordinates
    float roll_c, roll_s; // rolling-shutter factor at the centre row, and per row
};

__device__ __forceinline__ TileFrame tile_frame(uint32_t tile_x, uint32_t tile_y, uint32_t tile_size,
                                                float rs_time, uint32_t H) {
#pragma clang fp contract(off)
    TileFrame f;
    f.cx = (float)(tile_x * tile_size) + 0.5f * (float)tile_size;
    f.cy = (float)(tile_y * tile_size) + 0.5f * (float)tile_size;
    // rasterization.cu:1401: roll = rs_time * (row / (H - 1) - 0.5), row = pixel centre - 0.5
    f.roll_s = rs_time / (float)(H - 1);
    f.roll_c = rs_time * ((f.cy - 0.5f) / (float)(H - 1) - 0.5f);
    return f;
}

// a = {c0, cX, cY, cXX}, b = {cXY, cYY, X*, Y* or L}: exponent(X, Y) = c0 + cX X + cY Y + cXX X^2
// + cXY X Y + cYY Y^2.  For a positive definite conic with opacity <= 0.999 (alpha then never
// reaches the 0.999 clamp and sigma is never negative) b.z, b.w hold the pixel offset (X*, Y*) at
// which the exponent peaks, which the footprint test uses.  Otherwise b.z is NaN ("general": the
// compositing loop applies the clamp and the sigma < 0 rule, the footprint test keeps the
// Gaussian) and b.w holds L for an indefinite conic, +inf for a definite one (sigma < 0 <=>
// exponent > L can then never hold).
//
// No implicit contraction in here: every kernel that stages a Gaussian has to arrive at the same
// bits (they take the alpha >= 1/255 decisions from them), and left to itself the compiler fuses
// multiplies and adds differently from one template instantiation to the next.
__device__ __forceinline__ void pixel_polynomial(const TileFrame &f, float2 xy, float2 v, float ca,
                                                 float cb, float cc, float opacity, float4 &a, float4 &b) {
#pragma clang fp contract(off)
    const float4 e = staged_exponent(ca, cb, cc, opacity);
    const float A = e.x, B = e.y, C = e.z, L = e.w;
    const float dx0 = fmaf(f.roll_c, v.x, xy.x - f.cx), dy0 = fmaf(f.roll_c, v.y, xy.y - f.cy);
    const float sx = f.roll_s * v.x, sy = fmaf(f.roll_s, v.y, -1.f);
    const float Adx = A * dx0, Cdy = C * dy0;
    a.x = L - (dx0 * fmaf(B, dy0, Adx) + Cdy * dy0);
    a.y = fmaf(2.f, Adx, B * dy0);
    a.z = -(2.f * Adx * sx + B * fmaf(dx0, sy, sx * dy0) + 2.f * Cdy * sy);
    a.w = -A;
    b.x = fmaf(2.f * A, sx, B * sy);
    b.y = -(sx * fmaf(A, sx, B * sy) + C * sy * sy);
    const bool definite = A > 0.f && C > 0.f && 4.f * A * C - B * B > 0.f;
    const bool plain = definite && opacity <= 0.999f && fabsf(sy) > 1e-3f && b.y < 0.f;
    if (plain) {
        const float ys = -dy0 * __builtin_amdgcn_rcpf(sy); // dy = 0
        b.w = ys;
        b.z = fmaf(sx, ys, dx0);                           // dx = 0
    } else {
        b.z = NAN;
        b.w = definite ? INFINITY : L;
    }
}

struct PixelConstants {
    float X, Y, XX, YY;
    __device__ __forceinline__ void init(float px, float py, const TileFrame &f) {
#pragma clang fp contract(off)
        X = px - f.cx; Y = py - f.cy;
        XX = X * X; YY = Y * Y;
    }
};

// Evaluated as (c0 + cX X + cXX X^2) + (cY + cXY X) Y + cYY Y^2: the two brackets depend on the
// pixel's column only, so a lane whose pixels share a column (rows y and y + 8 in the kernels with
// two pixels per lane) computes them once, seven fused multiply-adds for two pixels instead of ten.
// Every kernel evaluates in this order, one pixel per lane or two.
__device__ __forceinline__ float pixel_exponent(const float4 a, float cXY, float cYY, const PixelConstants &p) {
    const float column = fmaf(a.w, p.XX, fmaf(a.y, p.X, a.x));
    const float slope = fmaf(cXY, p.X, a.z);
    return fmaf(cYY, p.YY, fmaf(slope, p.Y, column));
}

// Footprint of a wavefront of camera pixels in tile-centred coordinates, and the test whether
// any pixel in it can reach alpha >= 1/255 for a staged polynomial: the exponent is concave for
// a definite conic, so over a box that does not contain its peak it is largest on one of the
// four edges, where it is a parabola.  A margin covers the rounding of the test itself.
struct WaveBox {
    bool enabled;
    float x0, x1, y0, y1;

    __device__ __forceinline__ void init(float x_lo, float x_hi, float y_lo, float y_hi, bool full_wavefront) {
        enabled = full_wavefront;
        if (enabled) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                x_lo = fminf(x_lo, __shfl_xor(x_lo, off, SPLATAD_WAVE));
                x_hi = fmaxf(x_hi, __shfl_xor(x_hi, off, SPLATAD_WAVE));
                y_lo = fminf(y_lo, __shfl_xor(y_lo, off, SPLATAD_WAVE));
                y_hi = fmaxf(y_hi, __shfl_xor(y_hi, off, SPLATAD_WAVE));
            }
        }
        x0 = x_lo; x1 = x_hi; y0 = y_lo; y1 = y_hi;
    }

    __device__ __forceinline__ float edge_x(const float4 a, float cXY, float cYY, float hYY, float xe) const {
        const float a0 = fmaf(xe, fmaf(a.w, xe, a.y), a.x), a1 = fmaf(cXY, xe, a.z);
        const float yc = __builtin_amdgcn_fmed3f(a1 * hYY, y0, y1);
        return fmaf(yc, fmaf(cYY, yc, a1), a0);
    }
    __device__ __forceinline__ float edge_y(const float4 a, float cXY, float cYY, float hXX, float ye) const {
        const float b0 = fmaf(ye, fmaf(cYY, ye, a.z), a.x), b1 = fmaf(cXY, ye, a.y);
        const float xc = __builtin_amdgcn_fmed3f(b1 * hXX, x0, x1);
        return fmaf(xc, fmaf(a.w, xc, b1), b0);
    }

    __device__ __forceinline__ bool may_touch(const float4 a, const float4 b) const {
        if (!enabled || !(b.z == b.z)) return true;
        if (b.z >= x0 && b.z <= x1 && b.w >= y0 && b.w <= y1) return true;
        const float hYY = -0.5f * __builtin_amdgcn_rcpf(b.y), hXX = -0.5f * __builtin_amdgcn_rcpf(a.w);
        const float m = fmaxf(fmaxf(edge_x(a, b.x, b.y, hYY, x0), edge_x(a, b.x, b.y, hYY, x1)),
                              fmaxf(edge_y(a, b.x, b.y, hXX, y0), edge_y(a, b.x, b.y, hXX, y1)));
        return !(m < -kLog2Of255 - 0.05f - 4e-6f * fabsf(a.x));
    }
};

// Lane -> pixel inside a camera tile: wavefronts cover 8x8 squares when the tile allows it
// (a compact footprint is what makes the per-wavefront test effective), rows otherwise.
__device__ __forceinline__ void pixel_of_lane(uint32_t tile_size, uint32_t tr, uint32_t &lx, uint32_t &ly) {
    lx = tr % tile_size;
    ly = tr / tile_size;
    if (tile_size % 8 == 0) {
        const uint32_t squares_per_row = tile_size / 8, square = tr / SPLATAD_WAVE;
        const uint32_t lane = tr & (SPLATAD_WAVE - 1);
        lx = (square % squares_per_row) * 8 + (lane & 7);
        ly = (square / squares_per_row) * 8 + (lane >> 3);
    }
}

// Lane -> point inside a lidar tile: a wavefront covers 16 columns of all four rows when the
// tile allows it (more compact than one row of 64 columns).
__device__ __forceinline__ void point_of_lane(uint32_t tile_width, uint32_t tile_height, uint32_t tr,
                                              uint32_t &lx, uint32_t &ly) {
    lx = tr % tile_width;
    ly = tr / tile_width;
    if (tile_height == 4 && tile_width % 16 == 0) {
        const uint32_t lane = tr & (SPLATAD_WAVE - 1);
        lx = (tr / SPLATAD_WAVE) * 16 + (lane & 15);
        ly = lane >> 4;
    }
}

} // namespace
#endif // __HIPCC__
