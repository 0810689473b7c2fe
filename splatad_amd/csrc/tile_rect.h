// Tile rectangle of a projected Gaussian on a camera's tile grid: rasterization.cu:44-57 of the
// reference (floor / ceil of centre -+ radius in tile units, clamped to the grid).  Shared by the
// tile intersection and by the packed projection, which counts the intersections of the rows it
// keeps so that the caller learns both numbers with one wait.
#pragma once

#include "common.h"

#ifdef __HIPCC__

__device__ __forceinline__ uint32_t splatad_f2u_sat(float v) {
    if (!(v > 0.0f)) return 0u;
    if (v >= 4294967296.0f) return 0xFFFFFFFFu;
    return (uint32_t)v;
}

// x in [x0, x1), y in [y0, y1); false for a culled Gaussian (radius <= 0).  The bounds are
// float32 expressions whose rounding decides which tiles a Gaussian touches: no contraction.
__device__ __forceinline__ bool splatad_camera_tile_rect(uint32_t tile_size, uint32_t tile_w,
                                                         uint32_t tile_h, float2 mu, int2 r,
                                                         int32_t &x0, int32_t &y0, int32_t &x1,
                                                         int32_t &y1) {
#pragma clang fp contract(off)
    if (r.x <= 0) return false;
    const float ts = (float)tile_size;
    const float ex = (float)r.x / ts, ey = (float)r.y / ts;
    const float tx = mu.x / ts, ty = mu.y / ts;
    x0 = (int32_t)min(splatad_f2u_sat(floorf(tx - ex)), tile_w);
    y0 = (int32_t)min(splatad_f2u_sat(floorf(ty - ey)), tile_h);
    x1 = (int32_t)min(splatad_f2u_sat(ceilf(tx + ex)), tile_w);
    y1 = (int32_t)min(splatad_f2u_sat(ceilf(ty + ey)), tile_h);
    return true;
}

#endif // __HIPCC__
