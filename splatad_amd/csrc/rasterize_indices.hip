// Lists the (Gaussian, pixel) pairs that take part in compositing, for camera pixels and
// lidar points, over a range of batches of each tile's depth-sorted list.
//
// The lists feed compositing written in plain tensor operations (autograd instead of the
// hand-written backward pass).  A call covers batches [range_start, range_end) of every tile,
// a batch being as many Gaussians as the tile has pixels, and starts from the transmittance
// the caller has reached so far, so that a long list can be walked in several calls.
//
// Two passes of the same kernel make the output dense without atomics: the first counts the
// pairs of every pixel, an exclusive scan of the counts gives every pixel its place in the
// output, the second pass writes.  Both passes take the same decisions because they run the
// same arithmetic on the same inputs.  Within a pixel the pairs are in front-to-back order;
// pixels follow each other in row-major order, sensor by sensor.
//
// The per-pair decisions follow gsplat/cuda/csrc/rasterization.cu:839-1001 (pixels) and
// :1100-1268 (points) of the reference: alpha = min(0.999, o * exp(-sigma)); a Gaussian is
// skipped when sigma < 0 or alpha < 1/255; a pixel stops, without taking the Gaussian, when
// its transmittance would fall to 1e-4 or below; points with range <= 0 take nothing.
//
// The workgroup layout, the staged records and the per-wavefront footprint test are those of
// the compositing kernels.
#include "raster_common.h"
#include "scan.h"

namespace {

struct IndexArgs {
    uint32_t range_start, range_end; // batches
    uint32_t C, N;
    int64_t n_isects;
    const float *transmittances, *means2d, *conics, *opacities, *pix_vels;
    const float *rs_time;    // cameras
    const float *raster_pts; // lidars
    uint32_t W, H, tile_width, tile_height, grid_w, grid_h;
    const int32_t *tile_offsets, *flatten_ids;
    int32_t *counts;             // counting pass
    const int64_t *chunk_starts; // writing pass
    int64_t *gaussian_ids, *indices;
};

template <bool LIDAR, bool WRITE>
__global__ void __launch_bounds__(1024)
rasterize_to_indices_kernel(IndexArgs a) {
    extern __shared__ float4 lds4[];
    __shared__ uint32_t s_ref_thread;
    __shared__ float s_ref[2];
    const uint32_t block_size = blockDim.x * blockDim.y;
    // per Gaussian: {x, y, vx, vy} (lidar: angles relative to the tile's reference point) and
    // {A, B, C, L} with alpha = exp2(L - (A dx^2 + B dx dy + C dy^2)); then the Gaussian ids
    float4 *s_rec = lds4;
    int32_t *s_id = reinterpret_cast<int32_t *>(lds4 + 2 * block_size);

    const uint32_t tiles_per_cam = a.grid_w * a.grid_h;
    const uint32_t cam = blockIdx.x / tiles_per_cam;
    const uint32_t tile_id = blockIdx.x % tiles_per_cam;
    const uint32_t tr = threadIdx.y * blockDim.x + threadIdx.x;
    const uint32_t lane = tr & (SPLATAD_WAVE - 1);
    uint32_t lx, ly;
    if (LIDAR) point_of_lane(a.tile_width, a.tile_height, tr, lx, ly);
    else pixel_of_lane(a.tile_width, tr, lx, ly);
    const uint32_t i = (tile_id / a.grid_w) * a.tile_height + ly;
    const uint32_t j = (tile_id % a.grid_w) * a.tile_width + lx;
    const bool in_image = (i < a.H && j < a.W);
    const size_t pix = ((size_t)cam * a.H + i) * a.W + j;

    float px = (float)j + 0.5f, py = (float)i + 0.5f, roll = 0.f;
    bool inside = in_image;
    float ref_x = 0.f, ref_y = 0.f;
    bool any_point = true;
    if (LIDAR) {
        float pz = 0.f;
        px = py = 0.f;
        if (in_image) {
            const float4 p = reinterpret_cast<const float4 *>(a.raster_pts)[pix];
            px = p.x; py = p.y; pz = p.z; roll = p.w;
        }
        inside = in_image && pz > 0.f;
        // reference point of the tile: its first valid point
        if (tr == 0) s_ref_thread = 0xFFFFFFFFu;
        __syncthreads();
        if (inside) atomicMin(&s_ref_thread, tr);
        __syncthreads();
        if (tr == s_ref_thread) { s_ref[0] = px; s_ref[1] = py; }
        __syncthreads();
        any_point = s_ref_thread != 0xFFFFFFFFu; // uniform
        ref_x = any_point ? s_ref[0] : 0.f;
        ref_y = any_point ? s_ref[1] : 0.f;
        px = angle_difference(px, ref_x);
        py = angle_difference(py, ref_y);
    } else {
        roll = a.rs_time[cam] * ((py - 0.5f) / (float)(a.H - 1) - 0.5f);
    }
    uint64_t alive_bits = wave_ballot(inside); // lanes still compositing, as in the compositing kernels

    const int32_t *offs = a.tile_offsets + (size_t)cam * tiles_per_cam;
    const int32_t list_start = offs[tile_id];
    const int32_t list_end = (cam == a.C - 1 && tile_id == tiles_per_cam - 1)
                                 ? (int32_t)a.n_isects
                                 : offs[tile_id + 1];
    const uint32_t num_batches =
        any_point ? (uint32_t)(list_end - list_start + block_size - 1) / block_size : 0u;
    const uint32_t batch_end = min(a.range_end, num_batches);

    // Cameras: the exponent is the polynomial in tile-centred pixel coordinates that the
    // compositing kernels stage and evaluate (same functions, same bits, hence the same alpha >=
    // 1/255 and sigma < 0 decisions); the footprint test works on the polynomial too.
    WaveBox box;
    WavePointCull pcull;
    TileFrame frame = {};
    PixelConstants pc = {};
    const bool full = block_size % SPLATAD_WAVE == 0;
    if (LIDAR) {
        pcull.init(inside, px, py, roll, full);
    } else {
        frame = tile_frame(tile_id % a.grid_w, tile_id / a.grid_w, a.tile_width, a.rs_time[cam], a.H);
        pc.init(px, py, frame);
        box.init(pc.X, pc.X, pc.Y, pc.Y, full);
    }

    float T = inside ? a.transmittances[pix] : 0.f;
    int64_t *out_g = nullptr, *out_i = nullptr;
    if (WRITE && inside) {
        const int64_t base = a.chunk_starts[pix];
        out_g = a.gaussian_ids + base;
        out_i = a.indices + base;
    }
    int32_t cnt = 0;

    for (uint32_t b = a.range_start; b < batch_end; ++b) {
        // also orders the previous batch's LDS reads before this batch's writes
        if (__syncthreads_count(!wave_lanes(alive_bits)) >= (int)block_size) break;
        const uint32_t batch_start = (uint32_t)list_start + block_size * b;
        const uint32_t idx = batch_start + tr;
        if (idx < (uint32_t)list_end) {
            const int32_t g = a.flatten_ids[idx];
            const float2 xy = reinterpret_cast<const float2 *>(a.means2d)[g];
            const float *v = a.pix_vels + (size_t)g * (LIDAR ? 3 : 2);
            const float *cn = a.conics + (size_t)g * 3;
            if (LIDAR) {
                s_rec[2 * tr] = make_float4(angle_difference(xy.x, ref_x), angle_difference(xy.y, ref_y), v[0], v[1]);
                s_rec[2 * tr + 1] = staged_exponent(cn[0], cn[1], cn[2], a.opacities[g]);
            } else {
                float4 pa, pb;
                pixel_polynomial(frame, xy, make_float2(v[0], v[1]), cn[0], cn[1], cn[2], a.opacities[g], pa, pb);
                s_rec[2 * tr] = pa;
                s_rec[2 * tr + 1] = pb;
            }
            s_id[tr] = (int32_t)((uint32_t)g % a.N);
        }
        __syncthreads();

        const uint32_t batch_size = min(block_size, (uint32_t)list_end - batch_start);
        for (uint32_t base = 0; base < batch_size && alive_bits != 0; base += SPLATAD_WAVE) {
            bool keep = base + lane < batch_size, unfolded_ok = true;
            if (keep) {
                const float4 r0 = s_rec[2 * (base + lane)], r1 = s_rec[2 * (base + lane) + 1];
                keep = LIDAR ? pcull.may_touch(r0, r1, unfolded_ok) : box.may_touch(r0, r1);
            }
            uint64_t todo = wave_ballot(keep);
            const uint64_t folded = LIDAR ? wave_ballot(keep && !unfolded_ok) : 0ull;
            while (todo) {
                const uint32_t bit = (uint32_t)__ffsll((unsigned long long)todo) - 1u;
                const uint32_t t = base + bit;
                todo &= todo - 1;
                const float4 xyv = s_rec[2 * t];
                const float4 con = s_rec[2 * t + 1];
                float alpha;
                bool sigma_ok;
                if constexpr (LIDAR) {
                    float dx = gaussian_offset(xyv.x, xyv.z, roll, px);
                    float dy = gaussian_offset(xyv.y, xyv.w, roll, py);
                    if ((folded >> bit) & 1ull) { // uniform, rare: half a turn away
                        dx = angle_difference(fmaf(roll, xyv.z, xyv.x), px);
                        dy = angle_difference(fmaf(roll, xyv.w, xyv.y), py);
                    }
                    const float power = gaussian_power(con, dx, dy);
                    alpha = fminf(0.999f, __builtin_amdgcn_exp2f(con.w - power));
                    sigma_ok = !(power < 0.f);
                } else { // xyv, con hold the polynomial {c0, cX, cY, cXX}, {cXY, cYY, X* or NaN, Y* or L}
                    const float ex = pixel_exponent(xyv, con.x, con.y, pc);
                    alpha = fminf(0.999f, __builtin_amdgcn_exp2f(ex));
                    sigma_ok = !(ex > (con.z == con.z ? INFINITY : con.w));
                }
                const float next_T = transmittance_behind(T, alpha); // as in the compositing kernels
                const uint64_t valid_bits = alive_bits & wave_ballot(sigma_ok) &
                                            wave_ballot(!(alpha < 1.f / 255.f));
                const uint64_t stop_bits = valid_bits & wave_ballot(next_T <= 1e-4f);
                alive_bits &= ~stop_bits;
                if (wave_lanes(valid_bits & ~stop_bits)) {
                    if (WRITE) {
                        out_g[cnt] = (int64_t)s_id[t];
                        out_i[cnt] = (int64_t)pix;
                    }
                    ++cnt;
                    T = next_T;
                }
                if (alive_bits == 0) break;
            }
        }
    }

    if (!WRITE && in_image) a.counts[pix] = cnt;
}

struct IndexWorkspace {
    int32_t *counts;
    int64_t *block_sums;
};

static size_t index_ws_bytes(int64_t n_pixels) {
    return splatad_align256((size_t)(n_pixels > 0 ? n_pixels : 1) * sizeof(int32_t)) +
           scan_workspace_bytes(n_pixels);
}

static IndexWorkspace carve_index_ws(void *ws, int64_t n_pixels) {
    IndexWorkspace w;
    w.counts = reinterpret_cast<int32_t *>(ws);
    w.block_sums = reinterpret_cast<int64_t *>(
        reinterpret_cast<char *>(ws) +
        splatad_align256((size_t)(n_pixels > 0 ? n_pixels : 1) * sizeof(int32_t)));
    return w;
}

static uint32_t clamp_batches(int64_t v) {
    return v < 0 ? 0u : (v > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)v);
}

template <bool LIDAR>
static int check_args(const char *what, const IndexArgs &a, int64_t range_start, int64_t range_end) {
    SPLATAD_REQUIRE(range_start >= 0 && range_end >= range_start,
                    "%s: batch range [%lld, %lld) is not ordered", what, (long long)range_start,
                    (long long)range_end);
    SPLATAD_REQUIRE(a.tile_width >= 1 && a.tile_height >= 1 &&
                        a.tile_width * a.tile_height <= (LIDAR ? 256u : 1024u),
                    "%s: tile %ux%u has too many pixels", what, a.tile_width, a.tile_height);
    SPLATAD_REQUIRE((uint64_t)a.grid_w * a.tile_width >= a.W && (uint64_t)a.grid_h * a.tile_height >= a.H,
                    "%s: tile grid %ux%u does not cover the %ux%u image", what, a.grid_w, a.grid_h,
                    a.W, a.H);
    SPLATAD_REQUIRE(a.n_isects >= 0 && a.n_isects < (1ll << 31), "%s: bad n_isects", what);
    SPLATAD_REQUIRE(a.N >= 1 || a.n_isects == 0, "%s: intersections without Gaussians", what);
    SPLATAD_REQUIRE(a.transmittances && a.tile_offsets && (LIDAR ? a.raster_pts : a.rs_time),
                    "%s: null pointer argument", what);
    SPLATAD_REQUIRE(a.n_isects == 0 || (a.means2d && a.conics && a.opacities && a.pix_vels && a.flatten_ids),
                    "%s: null pointer argument", what);
    return 0;
}

template <bool LIDAR, bool WRITE>
static int launch_indices(const IndexArgs &a, hipStream_t stream) {
    const dim3 grid(a.C * a.grid_w * a.grid_h), block(a.tile_width, a.tile_height);
    const size_t lds = (size_t)block.x * block.y * (2 * sizeof(float4) + sizeof(int32_t));
    hipLaunchKernelGGL((rasterize_to_indices_kernel<LIDAR, WRITE>), grid, block, lds, stream, a);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

template <bool LIDAR>
static int indices_count(const char *what, IndexArgs a, int64_t range_start, int64_t range_end,
                         void *workspace, size_t workspace_bytes, int64_t *chunk_starts,
                         int64_t *n_elems, hipStream_t stream) {
    if (int rc = check_args<LIDAR>(what, a, range_start, range_end)) return rc;
    SPLATAD_REQUIRE(n_elems, "%s: n_elems is null", what);
    const int64_t n_pixels = (int64_t)a.C * a.H * a.W;
    SPLATAD_REQUIRE(n_pixels == 0 || (workspace && chunk_starts), "%s: null pointer argument", what);
    SPLATAD_REQUIRE(workspace_bytes >= index_ws_bytes(n_pixels), "%s: workspace of %zu bytes, %zu needed",
                    what, workspace_bytes, index_ws_bytes(n_pixels));
    a.range_start = clamp_batches(range_start);
    a.range_end = clamp_batches(range_end);
    IndexWorkspace w = carve_index_ws(workspace, n_pixels);
    a.counts = w.counts;
    if (n_pixels > 0)
        if (int rc = launch_indices<LIDAR, false>(a, stream)) return rc;
    return launch_exclusive_scan<int64_t>(w.counts, n_pixels, 1, 0, chunk_starts, n_elems,
                                          w.block_sums, stream);
}

template <bool LIDAR>
static int indices_fill(const char *what, IndexArgs a, int64_t range_start, int64_t range_end,
                        hipStream_t stream) {
    if (int rc = check_args<LIDAR>(what, a, range_start, range_end)) return rc;
    if ((int64_t)a.C * a.H * a.W == 0) return 0;
    SPLATAD_REQUIRE(a.chunk_starts && a.gaussian_ids && a.indices, "%s: null pointer argument", what);
    a.range_start = clamp_batches(range_start);
    a.range_end = clamp_batches(range_end);
    return launch_indices<LIDAR, true>(a, stream);
}

static IndexArgs pixel_args(uint32_t C, uint32_t N, int64_t n_isects, const float *transmittances,
                            const float *means2d, const float *conics, const float *opacities,
                            const float *pix_vels, const float *rs_time, uint32_t W, uint32_t H,
                            uint32_t tile_size, uint32_t tile_w, uint32_t tile_h,
                            const int32_t *tile_offsets, const int32_t *flatten_ids) {
    IndexArgs a = {};
    a.C = C; a.N = N; a.n_isects = n_isects; a.transmittances = transmittances;
    a.means2d = means2d; a.conics = conics; a.opacities = opacities; a.pix_vels = pix_vels;
    a.rs_time = rs_time; a.W = W; a.H = H; a.tile_width = tile_size; a.tile_height = tile_size;
    a.grid_w = tile_w; a.grid_h = tile_h; a.tile_offsets = tile_offsets; a.flatten_ids = flatten_ids;
    return a;
}

static IndexArgs point_args(uint32_t C, uint32_t N, int64_t n_isects, const float *transmittances,
                            const float *means2d, const float *conics, const float *opacities,
                            const float *pix_vels, const float *raster_pts, uint32_t W, uint32_t H,
                            uint32_t tile_width, uint32_t tile_height, uint32_t grid_w,
                            uint32_t grid_h, const int32_t *tile_offsets,
                            const int32_t *flatten_ids) {
    IndexArgs a = {};
    a.C = C; a.N = N; a.n_isects = n_isects; a.transmittances = transmittances;
    a.means2d = means2d; a.conics = conics; a.opacities = opacities; a.pix_vels = pix_vels;
    a.raster_pts = raster_pts; a.W = W; a.H = H; a.tile_width = tile_width;
    a.tile_height = tile_height; a.grid_w = grid_w; a.grid_h = grid_h;
    a.tile_offsets = tile_offsets; a.flatten_ids = flatten_ids;
    return a;
}

} // namespace

extern "C" size_t splatad_rasterize_to_indices_workspace_bytes(uint32_t C, uint32_t W, uint32_t H) {
    return index_ws_bytes((int64_t)C * H * W);
}

extern "C" int splatad_rasterize_to_indices_in_range_count(
    int64_t range_start, int64_t range_end, uint32_t C, uint32_t N, int64_t n_isects,
    const float *transmittances, const float *means2d, const float *conics,
    const float *opacities, const float *pix_vels, const float *rs_time, uint32_t W, uint32_t H,
    uint32_t tile_size, uint32_t tile_w, uint32_t tile_h, const int32_t *tile_offsets,
    const int32_t *flatten_ids, void *workspace, size_t workspace_bytes, int64_t *chunk_starts,
    int64_t *n_elems, splatad_stream_t stream) {
    return indices_count<false>("rasterize_to_indices_in_range",
                                pixel_args(C, N, n_isects, transmittances, means2d, conics, opacities,
                                           pix_vels, rs_time, W, H, tile_size, tile_w, tile_h,
                                           tile_offsets, flatten_ids),
                                range_start, range_end, workspace, workspace_bytes, chunk_starts,
                                n_elems, (hipStream_t)stream);
}

extern "C" int splatad_rasterize_to_indices_in_range_fill(
    int64_t range_start, int64_t range_end, uint32_t C, uint32_t N, int64_t n_isects,
    const float *transmittances, const float *means2d, const float *conics,
    const float *opacities, const float *pix_vels, const float *rs_time, uint32_t W, uint32_t H,
    uint32_t tile_size, uint32_t tile_w, uint32_t tile_h, const int32_t *tile_offsets,
    const int32_t *flatten_ids, const int64_t *chunk_starts, int64_t *gaussian_ids,
    int64_t *indices, splatad_stream_t stream) {
    IndexArgs a = pixel_args(C, N, n_isects, transmittances, means2d, conics, opacities, pix_vels,
                             rs_time, W, H, tile_size, tile_w, tile_h, tile_offsets, flatten_ids);
    a.chunk_starts = chunk_starts; a.gaussian_ids = gaussian_ids; a.indices = indices;
    return indices_fill<false>("rasterize_to_indices_in_range", a, range_start, range_end,
                               (hipStream_t)stream);
}

extern "C" int splatad_rasterize_to_indices_in_range_lidar_count(
    int64_t range_start, int64_t range_end, uint32_t C, uint32_t N, int64_t n_isects,
    const float *transmittances, const float *means2d, const float *conics,
    const float *opacities, const float *pix_vels, const float *raster_pts, uint32_t W,
    uint32_t H, uint32_t tile_width, uint32_t tile_height, uint32_t grid_w, uint32_t grid_h,
    const int32_t *tile_offsets, const int32_t *flatten_ids, void *workspace,
    size_t workspace_bytes, int64_t *chunk_starts, int64_t *n_elems, splatad_stream_t stream) {
    return indices_count<true>("rasterize_to_indices_in_range_lidar",
                               point_args(C, N, n_isects, transmittances, means2d, conics, opacities,
                                          pix_vels, raster_pts, W, H, tile_width, tile_height, grid_w,
                                          grid_h, tile_offsets, flatten_ids),
                               range_start, range_end, workspace, workspace_bytes, chunk_starts,
                               n_elems, (hipStream_t)stream);
}

extern "C" int splatad_rasterize_to_indices_in_range_lidar_fill(
    int64_t range_start, int64_t range_end, uint32_t C, uint32_t N, int64_t n_isects,
    const float *transmittances, const float *means2d, const float *conics,
    const float *opacities, const float *pix_vels, const float *raster_pts, uint32_t W,
    uint32_t H, uint32_t tile_width, uint32_t tile_height, uint32_t grid_w, uint32_t grid_h,
    const int32_t *tile_offsets, const int32_t *flatten_ids, const int64_t *chunk_starts,
    int64_t *gaussian_ids, int64_t *indices, splatad_stream_t stream) {
    IndexArgs a = point_args(C, N, n_isects, transmittances, means2d, conics, opacities, pix_vels,
                             raster_pts, W, H, tile_width, tile_height, grid_w, grid_h, tile_offsets,
                             flatten_ids);
    a.chunk_starts = chunk_starts; a.gaussian_ids = gaussian_ids; a.indices = indices;
    return indices_fill<true>("rasterize_to_indices_in_range_lidar", a, range_start, range_end,
                              (hipStream_t)stream);
}
