// Backward of the alpha compositing for camera pixels and lidar points on gfx950.
//
// One workgroup per (sensor, tile), one lane per pixel / point.  Each pixel replays its
// tile's list back to front, starting at the last Gaussian it took in the forward pass,
// and recovers the transmittance by dividing (T_before = T_after / (1 - alpha)).  Batches of
// the list are staged in LDS together with the colours.  Per Gaussian, the pixel gradients
// are summed over the 64 lanes of each wavefront, accumulated across the wavefronts of the
// workgroup in LDS, and flushed with one global atomic per value and (tile, Gaussian) when
// the batch is finished.  Batches behind the deepest entry any pixel of the tile consumed
// are never loaded.
//
// Gradient rules follow gsplat/cuda/csrc/rasterization.cu:2833-3089 (pixels) and :3728-4054
// (points) of the reference.  Channels beyond 33 are handled in passes; the geometry
// gradients are linear in the per-channel terms, so the passes add up exactly (the absolute
// gradient v_means2d_abs then adds the per-pass magnitudes).
#include "common.h"

namespace {

// fmodf(a - b + 180, 360) - 180 folded into (-180, 180], see the forward kernel
__device__ __forceinline__ float angle_difference(float a, float b) {
    const float d = a - b + 180.f;
    const float m = (d >= 0.f && d < 360.f) ? d : fmodf(d, 360.f);
    const float r = m - 180.f;
    return r < -180.f ? r + 360.f : r;
}

struct BwdArgs {
    uint32_t C;
    int64_t n_isects;
    uint32_t color_stride, ch_offset, n_ch;
    const float *means2d, *conics, *colors, *opacities, *pix_vels, *depth_comps, *rs_time,
        *backgrounds, *raster_pts;
    uint32_t W, H, tile_w_px, tile_h_px, grid_w, grid_h;
    int compute_alpha_sum;
    float threshold;
    const int32_t *tile_offsets, *flatten_ids;
    uint32_t depth_idx;
    const float *render_alphas;
    const int32_t *last_ids;
    const float *v_render_colors, *v_render_alphas, *v_alpha_sum;
    float *v_means2d_abs, *v_means2d, *v_conics, *v_colors, *v_opacities, *v_pix_vels, *v_depth_comps;
    int first_pass; // adds the alpha / alpha-sum terms exactly once over the channel passes
};

// Geometry gradient slots per Gaussian in the LDS accumulator, after the CH colour slots.
enum { G_CONIC = 0, G_XY = 3, G_ABS = 5, G_VEL = 7, G_OPAC = 10, G_DC = 11, G_COUNT = 13 };

template <int CH, bool LIDAR>
__global__ void __launch_bounds__(256)
rasterize_bwd_kernel(BwdArgs a) {
    extern __shared__ float4 lds4[];
    const uint32_t block_size = blockDim.x * blockDim.y;
    float4 *s_xyv = lds4;                  // {x, y, vx, vy}
    float4 *s_con = lds4 + block_size;     // {conic a, b, c, opacity}
    float4 *s_ext = lds4 + 2 * block_size; // lidar: {v_range, depth comp 0, depth comp 1, depth}
    int32_t *s_id = reinterpret_cast<int32_t *>(lds4 + 3 * block_size);
    float *s_col = reinterpret_cast<float *>(s_id + block_size);        // [block_size][CH]
    float *s_acc = s_col + (size_t)block_size * CH;                     // [block_size][CH + G_COUNT]
    __shared__ int32_t s_block_final;
    constexpr int ACC = CH + G_COUNT;

    const uint32_t tiles_per_cam = a.grid_w * a.grid_h;
    const uint32_t cam = blockIdx.x / tiles_per_cam;
    const uint32_t tile_id = blockIdx.x % tiles_per_cam;
    const uint32_t i = (tile_id / a.grid_w) * a.tile_h_px + threadIdx.y;
    const uint32_t j = (tile_id % a.grid_w) * a.tile_w_px + threadIdx.x;
    const uint32_t tr = threadIdx.y * blockDim.x + threadIdx.x;
    const int lane = tr & (SPLATAD_WAVE - 1);

    const bool in_image = (i < a.H && j < a.W);
    const size_t pix = in_image ? ((size_t)cam * a.H + i) * a.W + j : 0;
    float px, py, pz = 1.f, roll;
    if (LIDAR) {
        px = py = roll = 0.f;
        pz = 0.f;
        if (in_image) {
            const float4 p = reinterpret_cast<const float4 *>(a.raster_pts)[pix];
            px = p.x; py = p.y; pz = p.z; roll = p.w;
        }
    } else {
        px = (float)j + 0.5f;
        py = (float)i + 0.5f;
        roll = a.rs_time[cam] * ((py - 0.5f) / (float)(a.H - 1) - 0.5f);
    }
    const bool inside = in_image && pz > 0.f;

    const int32_t *offs = a.tile_offsets + (size_t)cam * tiles_per_cam;
    const int32_t range_start = offs[tile_id];
    const int32_t range_end = (cam == a.C - 1 && tile_id == tiles_per_cam - 1)
                                  ? (int32_t)a.n_isects
                                  : offs[tile_id + 1];

    const float T_final = inside ? 1.0f - a.render_alphas[pix] : 1.0f;
    float T = T_final;
    const int32_t bin_final = inside ? a.last_ids[pix] : -1;
    float buffer[CH], v_out[CH];
#pragma unroll
    for (int k = 0; k < CH; ++k) {
        buffer[k] = 0.f;
        v_out[k] = (inside && (uint32_t)k < a.n_ch) ? a.v_render_colors[pix * a.color_stride + a.ch_offset + k] : 0.f;
    }
    const float v_render_a = (inside && a.first_pass) ? a.v_render_alphas[pix] : 0.f;
    const float v_asum = (LIDAR && inside && a.first_pass && a.compute_alpha_sum && a.v_alpha_sum) ? a.v_alpha_sum[pix] : 0.f;
    float bg_dot = 0.f; // sum_k background_k v_out_k
    if (a.backgrounds != nullptr) {
        const float *bg = a.backgrounds + (size_t)cam * a.color_stride + a.ch_offset;
#pragma unroll
        for (int k = 0; k < CH; ++k)
            if ((uint32_t)k < a.n_ch) bg_dot += bg[k] * v_out[k];
    }
    const bool has_depth = LIDAR && a.depth_idx >= a.ch_offset && a.depth_idx < a.ch_offset + a.n_ch;
    const int depth_local = has_depth ? (int)(a.depth_idx - a.ch_offset) : -1;
    float v_out_depth = 0.f; // v_out of the depth channel, valid in the pass that owns it
    float buffer_extra = 0.f; // depth-channel part of `buffer` coming from the extra terms
#pragma unroll
    for (int k = 0; k < CH; ++k)
        if (k == depth_local) v_out_depth = v_out[k];

    // deepest entry any pixel of the tile consumed
    if (tr == 0) s_block_final = -1;
    __syncthreads();
    const int32_t wave_final = wave_max_i32(bin_final);
    if (lane == 0 && wave_final >= 0) atomicMax(&s_block_final, wave_final);
    __syncthreads();
    const int32_t list_end = min(range_end, s_block_final + 1); // exclusive
    if (list_end <= range_start) return;
    const uint32_t num_batches = (uint32_t)(list_end - range_start + block_size - 1) / block_size;

    for (uint32_t b = 0; b < num_batches; ++b) {
        __syncthreads(); // previous batch fully flushed
        const int32_t batch_end = list_end - 1 - (int32_t)(block_size * b);
        const int32_t batch_size = min((int32_t)block_size, batch_end + 1 - range_start);
        const int32_t idx = batch_end - (int32_t)tr;
        if (idx >= range_start) {
            const int32_t g = a.flatten_ids[idx];
            s_id[tr] = g;
            const float2 xy = reinterpret_cast<const float2 *>(a.means2d)[g];
            const float *cn = a.conics + (size_t)g * 3;
            s_con[tr] = make_float4(cn[0], cn[1], cn[2], a.opacities[g]);
            const float *crow = a.colors + (size_t)g * a.color_stride;
            if (LIDAR) {
                const float *v = a.pix_vels + (size_t)g * 3;
                const float2 dc = reinterpret_cast<const float2 *>(a.depth_comps)[g];
                s_xyv[tr] = make_float4(xy.x, xy.y, v[0], v[1]);
                s_ext[tr] = make_float4(v[2], dc.x, dc.y, crow[a.depth_idx]);
            } else {
                const float2 v = reinterpret_cast<const float2 *>(a.pix_vels)[g];
                s_xyv[tr] = make_float4(xy.x, xy.y, v.x, v.y);
            }
#pragma unroll
            for (int k = 0; k < CH; ++k) s_col[tr * CH + k] = (uint32_t)k < a.n_ch ? crow[a.ch_offset + k] : 0.f;
        }
        for (uint32_t k = tr; k < (uint32_t)batch_size * ACC; k += block_size) s_acc[k] = 0.f;
        __syncthreads();

        // entry t of the batch sits at list position batch_end - t
        const int32_t t0 = max(0, batch_end - wave_final);
        for (int32_t t = t0; t < batch_size; ++t) {
            bool valid = inside && (batch_end - t <= bin_final);
            float alpha = 0.f, opac = 0.f, vis = 0.f, dx = 0.f, dy = 0.f;
            float4 con = make_float4(0.f, 0.f, 0.f, 0.f), ext = make_float4(0.f, 0.f, 0.f, 0.f);
            if (valid) {
                con = s_con[t];
                const float4 xyv = s_xyv[t];
                opac = con.w;
                if (LIDAR) {
                    ext = s_ext[t];
                    dx = angle_difference(xyv.x + roll * xyv.z, px);
                    dy = angle_difference(xyv.y + roll * xyv.w, py);
                } else {
                    dx = xyv.x + roll * xyv.z - px;
                    dy = xyv.y + roll * xyv.w - py;
                }
                const float sigma = 0.5f * (con.x * dx * dx + con.z * dy * dy) + con.y * dx * dy;
                vis = __expf(-sigma);
                alpha = fminf(0.999f, opac * vis);
                if (sigma < 0.f || alpha < 1.f / 255.f) valid = false;
            }
            if (__ballot(valid) == 0) continue;

            float g_col[CH];
            float g_conic0 = 0.f, g_conic1 = 0.f, g_conic2 = 0.f, g_x = 0.f, g_y = 0.f, g_ax = 0.f,
                  g_ay = 0.f, g_vx = 0.f, g_vy = 0.f, g_vz = 0.f, g_op = 0.f, g_dc0 = 0.f, g_dc1 = 0.f;
#pragma unroll
            for (int k = 0; k < CH; ++k) g_col[k] = 0.f;
            if (valid) {
                const float ra = 1.0f / (1.0f - alpha);
                T *= ra; // transmittance in front of this Gaussian
                const float fac = alpha * T;
                float v_alpha = 0.f;
#pragma unroll
                for (int k = 0; k < CH; ++k) {
                    g_col[k] = fac * v_out[k];
                    v_alpha += (s_col[t * CH + k] * T - buffer[k] * ra) * v_out[k];
                }
                float extra = 0.f;
                if (LIDAR) {
                    extra = ext.y * dx + ext.z * dy + ext.x * roll;
                    // depth channel = colour + extra: both enter c*T and the buffer
                    v_alpha += (extra * T - buffer_extra * ra) * v_out_depth;
                }
                v_alpha += T_final * ra * v_render_a;
                v_alpha += -T_final * ra * bg_dot;
                const float g_depth = fac * v_out_depth; // gradient of the depth channel value
                if (opac * vis <= 0.999f) {
                    const float v_sigma = -opac * vis * v_alpha;
                    g_conic0 = 0.5f * v_sigma * dx * dx;
                    g_conic1 = v_sigma * dx * dy;
                    g_conic2 = 0.5f * v_sigma * dy * dy;
                    g_x = v_sigma * (con.x * dx + con.y * dy);
                    g_y = v_sigma * (con.y * dx + con.z * dy);
                    if (LIDAR) {
                        g_dc0 = g_depth * dx;
                        g_dc1 = g_depth * dy;
                        g_vz = g_depth * roll;
                        g_x += g_depth * ext.y;
                        g_y += g_depth * ext.z;
                    }
                    g_vx = g_x * roll;
                    g_vy = g_y * roll;
                    g_ax = fabsf(g_x);
                    g_ay = fabsf(g_y);
                    g_op = vis * v_alpha;
                }
#pragma unroll
                for (int k = 0; k < CH; ++k) buffer[k] += s_col[t * CH + k] * fac;
                if (LIDAR) {
                    buffer_extra += extra * fac;
                    if (a.compute_alpha_sum && ext.w < pz - a.threshold) {
                        const float v_sig2 = v_asum * -opac * vis;
                        const float ex = v_sig2 * (con.x * dx + con.y * dy);
                        const float ey = v_sig2 * (con.y * dx + con.z * dy);
                        g_x += ex; g_y += ey;
                        g_vx += ex * roll; g_vy += ey * roll;
                        g_ax += fabsf(ex); g_ay += fabsf(ey);
                        g_conic0 += v_sig2 * 0.5f * dx * dx;
                        g_conic1 += v_sig2 * dx * dy;
                        g_conic2 += v_sig2 * 0.5f * dy * dy;
                        g_op += v_asum * vis;
                    }
                }
            }
            // sum over the wavefront, then one LDS atomic per value and wavefront
            float *acc = s_acc + (size_t)t * ACC;
#pragma unroll
            for (int k = 0; k < CH; ++k) {
                const float s = wave_sum(g_col[k]);
                if (lane == 0 && (uint32_t)k < a.n_ch) atomicAdd(acc + k, s);
            }
            float geo[G_COUNT] = {g_conic0, g_conic1, g_conic2, g_x, g_y, g_ax, g_ay,
                                  g_vx, g_vy, g_vz, g_op, g_dc0, g_dc1};
#pragma unroll
            for (int q = 0; q < G_COUNT; ++q) {
                if (!LIDAR && (q == G_VEL + 2 || q >= G_DC)) continue;
                const float s = wave_sum(geo[q]);
                if (lane == 0) atomicAdd(acc + CH + q, s);
            }
        }
        __syncthreads();

        // flush the batch: lane tr owns Gaussian tr of the batch
        if ((int32_t)tr < batch_size) {
            const int32_t g = s_id[tr];
            const float *acc = s_acc + (size_t)tr * ACC;
            float *vc = a.v_colors + (size_t)g * a.color_stride + a.ch_offset;
#pragma unroll
            for (int k = 0; k < CH; ++k)
                if ((uint32_t)k < a.n_ch && acc[k] != 0.f) atomicAdd(vc + k, acc[k]);
            const float *geo = acc + CH;
            if (geo[G_OPAC] != 0.f || geo[G_XY] != 0.f || geo[G_XY + 1] != 0.f || geo[G_CONIC] != 0.f ||
                geo[G_CONIC + 1] != 0.f || geo[G_CONIC + 2] != 0.f || geo[G_ABS] != 0.f || geo[G_ABS + 1] != 0.f) {
                atomicAdd(a.v_conics + (size_t)g * 3, geo[G_CONIC]);
                atomicAdd(a.v_conics + (size_t)g * 3 + 1, geo[G_CONIC + 1]);
                atomicAdd(a.v_conics + (size_t)g * 3 + 2, geo[G_CONIC + 2]);
                atomicAdd(a.v_means2d + (size_t)g * 2, geo[G_XY]);
                atomicAdd(a.v_means2d + (size_t)g * 2 + 1, geo[G_XY + 1]);
                if (a.v_means2d_abs != nullptr) {
                    atomicAdd(a.v_means2d_abs + (size_t)g * 2, geo[G_ABS]);
                    atomicAdd(a.v_means2d_abs + (size_t)g * 2 + 1, geo[G_ABS + 1]);
                }
                const int nv = LIDAR ? 3 : 2;
                atomicAdd(a.v_pix_vels + (size_t)g * nv, geo[G_VEL]);
                atomicAdd(a.v_pix_vels + (size_t)g * nv + 1, geo[G_VEL + 1]);
                atomicAdd(a.v_opacities + g, geo[G_OPAC]);
            }
            if (LIDAR && (geo[G_VEL + 2] != 0.f || geo[G_DC] != 0.f || geo[G_DC + 1] != 0.f)) {
                atomicAdd(a.v_pix_vels + (size_t)g * 3 + 2, geo[G_VEL + 2]);
                atomicAdd(a.v_depth_comps + (size_t)g * 2, geo[G_DC]);
                atomicAdd(a.v_depth_comps + (size_t)g * 2 + 1, geo[G_DC + 1]);
            }
        }
    }
}

constexpr int kWidths[] = {1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33};
constexpr int kMaxPass = 33;

static inline int pick_width(uint32_t n) {
    for (int w : kWidths)
        if ((uint32_t)w >= n) return w;
    return -1;
}

template <int CH, bool LIDAR>
static int launch_bwd(const BwdArgs &a, dim3 grid, dim3 block, hipStream_t stream) {
    const size_t bs = (size_t)block.x * block.y;
    const size_t lds = bs * (48 + 4) + bs * 4 * CH + bs * 4 * (CH + G_COUNT);
    if (lds > 64 * 1024)
        SPLATAD_CHECK_HIP(hipFuncSetAttribute((const void *)rasterize_bwd_kernel<CH, LIDAR>,
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL((rasterize_bwd_kernel<CH, LIDAR>), grid, block, lds, stream, a);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

template <bool LIDAR>
static int dispatch_bwd(int w, const BwdArgs &a, dim3 grid, dim3 block, hipStream_t s) {
    switch (w) {
    case 1: return launch_bwd<1, LIDAR>(a, grid, block, s);
    case 2: return launch_bwd<2, LIDAR>(a, grid, block, s);
    case 3: return launch_bwd<3, LIDAR>(a, grid, block, s);
    case 4: return launch_bwd<4, LIDAR>(a, grid, block, s);
    case 5: return launch_bwd<5, LIDAR>(a, grid, block, s);
    case 8: return launch_bwd<8, LIDAR>(a, grid, block, s);
    case 9: return launch_bwd<9, LIDAR>(a, grid, block, s);
    case 16: return launch_bwd<16, LIDAR>(a, grid, block, s);
    case 17: return launch_bwd<17, LIDAR>(a, grid, block, s);
    case 32: return launch_bwd<32, LIDAR>(a, grid, block, s);
    case 33: return launch_bwd<33, LIDAR>(a, grid, block, s);
    default: break;
    }
    splatad_set_error("rasterize backward: no kernel for %d channels per pass", w);
    return -1;
}

template <bool LIDAR>
static int run_passes(BwdArgs &a, uint32_t channels, dim3 grid, dim3 block, hipStream_t stream) {
    const uint32_t pass = channels <= (uint32_t)kMaxPass ? channels : 32u;
    for (uint32_t off = 0; off < channels; off += pass) {
        a.ch_offset = off;
        a.n_ch = min(pass, channels - off);
        a.first_pass = off == 0;
        int rc = dispatch_bwd<LIDAR>(pick_width(a.n_ch), a, grid, block, stream);
        if (rc) return rc;
    }
    return 0;
}

} // namespace

extern "C" int splatad_rasterize_to_pixels_bwd(
    uint32_t C, int64_t n_isects, uint32_t channels, const float *means2d, const float *conics,
    const float *colors, const float *opacities, const float *pix_vels, const float *rs_time,
    const float *backgrounds, uint32_t W, uint32_t H, uint32_t tile_size, uint32_t tile_w,
    uint32_t tile_h, const int32_t *tile_offsets, const int32_t *flatten_ids,
    const float *render_alphas, const int32_t *last_ids, const float *v_render_colors,
    const float *v_render_alphas, float *v_means2d_abs, float *v_means2d, float *v_conics,
    float *v_colors, float *v_opacities, float *v_pix_vels, splatad_stream_t stream) {
    SPLATAD_REQUIRE(channels >= 1, "rasterize_to_pixels bwd: zero channels");
    SPLATAD_REQUIRE(tile_size >= 1 && tile_size * tile_size <= 256,
                    "rasterize_to_pixels bwd: tile_size %u is outside 1..16", tile_size);
    if (C == 0 || W == 0 || H == 0 || n_isects == 0) return 0;
    SPLATAD_REQUIRE((uint64_t)tile_w * tile_size >= W && (uint64_t)tile_h * tile_size >= H,
                    "rasterize_to_pixels bwd: tile grid does not cover the image");
    SPLATAD_REQUIRE(n_isects > 0 && n_isects < (1ll << 31), "rasterize_to_pixels bwd: bad n_isects");
    SPLATAD_REQUIRE(means2d && conics && colors && opacities && pix_vels && rs_time && tile_offsets &&
                        flatten_ids && render_alphas && last_ids && v_render_colors && v_render_alphas &&
                        v_means2d && v_conics && v_colors && v_opacities && v_pix_vels,
                    "rasterize_to_pixels bwd: null pointer argument");
    BwdArgs a = {};
    a.C = C; a.n_isects = n_isects; a.color_stride = channels;
    a.means2d = means2d; a.conics = conics; a.colors = colors; a.opacities = opacities;
    a.pix_vels = pix_vels; a.rs_time = rs_time; a.backgrounds = backgrounds;
    a.W = W; a.H = H; a.tile_w_px = tile_size; a.tile_h_px = tile_size; a.grid_w = tile_w; a.grid_h = tile_h;
    a.tile_offsets = tile_offsets; a.flatten_ids = flatten_ids;
    a.render_alphas = render_alphas; a.last_ids = last_ids;
    a.v_render_colors = v_render_colors; a.v_render_alphas = v_render_alphas;
    a.v_means2d_abs = v_means2d_abs; a.v_means2d = v_means2d; a.v_conics = v_conics;
    a.v_colors = v_colors; a.v_opacities = v_opacities; a.v_pix_vels = v_pix_vels;
    return run_passes<false>(a, channels, dim3(C * tile_w * tile_h), dim3(tile_size, tile_size),
                             (hipStream_t)stream);
}

extern "C" int splatad_rasterize_to_points_bwd(
    uint32_t C, int64_t n_isects, uint32_t channels, const float *means2d, const float *conics,
    const float *colors, const float *opacities, const float *pix_vels, const float *depth_comps,
    const float *backgrounds, const float *raster_pts, uint32_t W, uint32_t H,
    uint32_t tile_width, uint32_t tile_height, uint32_t grid_w, uint32_t grid_h,
    int compute_alpha_sum, float threshold, const int32_t *tile_offsets,
    const int32_t *flatten_ids, uint32_t depth_idx, const float *render_alphas,
    const int32_t *last_ids, const float *v_render_colors, const float *v_render_alphas,
    const float *v_alpha_sum, float *v_means2d_abs, float *v_means2d, float *v_conics,
    float *v_colors, float *v_opacities, float *v_pix_vels, float *v_depth_comps,
    splatad_stream_t stream) {
    SPLATAD_REQUIRE(channels >= 1, "rasterize_to_points bwd: zero channels");
    SPLATAD_REQUIRE(depth_idx < channels, "rasterize_to_points bwd: depth channel %u of %u", depth_idx, channels);
    SPLATAD_REQUIRE(tile_width >= 1 && tile_height >= 1 && tile_width * tile_height <= 256,
                    "rasterize_to_points bwd: tile %ux%u exceeds 256 points", tile_width, tile_height);
    if (C == 0 || W == 0 || H == 0 || n_isects == 0) return 0;
    SPLATAD_REQUIRE((uint64_t)grid_w * tile_width >= W && (uint64_t)grid_h * tile_height >= H,
                    "rasterize_to_points bwd: tile grid does not cover the point image");
    SPLATAD_REQUIRE(n_isects > 0 && n_isects < (1ll << 31), "rasterize_to_points bwd: bad n_isects");
    SPLATAD_REQUIRE(means2d && conics && colors && opacities && pix_vels && depth_comps && raster_pts &&
                        tile_offsets && flatten_ids && render_alphas && last_ids && v_render_colors &&
                        v_render_alphas && v_means2d && v_conics && v_colors && v_opacities &&
                        v_pix_vels && v_depth_comps,
                    "rasterize_to_points bwd: null pointer argument");
    BwdArgs a = {};
    a.C = C; a.n_isects = n_isects; a.color_stride = channels;
    a.means2d = means2d; a.conics = conics; a.colors = colors; a.opacities = opacities;
    a.pix_vels = pix_vels; a.depth_comps = depth_comps; a.backgrounds = backgrounds;
    a.raster_pts = raster_pts; a.W = W; a.H = H; a.tile_w_px = tile_width; a.tile_h_px = tile_height;
    a.grid_w = grid_w; a.grid_h = grid_h; a.compute_alpha_sum = compute_alpha_sum;
    a.threshold = threshold; a.tile_offsets = tile_offsets; a.flatten_ids = flatten_ids;
    a.depth_idx = depth_idx; a.render_alphas = render_alphas; a.last_ids = last_ids;
    a.v_render_colors = v_render_colors; a.v_render_alphas = v_render_alphas; a.v_alpha_sum = v_alpha_sum;
    a.v_means2d_abs = v_means2d_abs; a.v_means2d = v_means2d; a.v_conics = v_conics;
    a.v_colors = v_colors; a.v_opacities = v_opacities; a.v_pix_vels = v_pix_vels;
    a.v_depth_comps = v_depth_comps;
    return run_passes<true>(a, channels, dim3(C * grid_w * grid_h), dim3(tile_width, tile_height),
                            (hipStream_t)stream);
}
