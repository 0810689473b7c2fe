// Entry points declared in the header whose kernels are not written yet: they fail loudly.
#include "common.h"

#define PENDING(name)                                     \
    splatad_set_error(name ": not implemented yet");      \
    return -100;

extern "C" int splatad_projection_bwd(uint32_t, uint32_t, const float *, const float *, const float *, const float *, const float *, const float *, const float *, uint32_t, uint32_t, const float *, const float *, const float *, float, const int64_t *, const int64_t *, int64_t, const int32_t *, const float *, const float *, const float *, const float *, const float *, const float *, const float *, int, float *, float *, float *, float *, float *, float *, splatad_stream_t) { PENDING("splatad_projection_bwd") }
extern "C" int splatad_lidar_projection_bwd(uint32_t, uint32_t, const float *, const float *, const float *, const float *, const float *, const float *, const float *, const float *, const float *, float, const float *, const float *, const float *, const float *, const float *, const float *, const float *, const float *, const float *, float *, float *, float *, float *, float *, float *, splatad_stream_t) { PENDING("splatad_lidar_projection_bwd") }
extern "C" int splatad_rasterize_to_pixels_bwd(uint32_t, int64_t, uint32_t, const float *, const float *, const float *, const float *, const float *, const float *, const float *, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, const int32_t *, const int32_t *, const float *, const int32_t *, const float *, const float *, float *, float *, float *, float *, float *, float *, splatad_stream_t) { PENDING("splatad_rasterize_to_pixels_bwd") }
extern "C" int splatad_rasterize_to_points_bwd(uint32_t, int64_t, uint32_t, const float *, const float *, const float *, const float *, const float *, const float *, const float *, const float *, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, int, float, const int32_t *, const int32_t *, uint32_t, const float *, const int32_t *, const float *, const float *, const float *, float *, float *, float *, float *, float *, float *, float *, splatad_stream_t) { PENDING("splatad_rasterize_to_points_bwd") }
