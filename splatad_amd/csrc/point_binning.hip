// Lidar point binning for gfx950: which tile a (azimuth, elevation) point falls into, the
// points of every tile as a contiguous run, the per-tile offsets, and an image filled from
// those runs.  Results are identical to gsplat/cuda/csrc/rasterization.cu:531-833 of the
// reference (one key per point, cub::DeviceRadixSort::SortPairs on the 64-bit keys).
//
// The keys take few distinct values (camera << 32 | tile) and a stable sort keeps equal keys
// in point order, so the sort is a stable counting sort: every workgroup (one wavefront) owns
// a contiguous range of points, counts them per tile in LDS and writes its counts to its row
// of a [workgroup][tile] table; the table is scanned tile-major; the same workgroup then walks
// its range again, 64 points at a time, and places every point at its tile's cursor plus its
// rank among the equal keys of the wavefront (ballots).  No atomics between workgroups, and
// the order inside a tile is the point order by construction.
#include "common.h"
#include "scan.h"

#include <mutex>

namespace {

struct PointGrid {
    uint32_t n_tiles_azim, n_tiles_elev;
    float azim_res, min_azim;
    const float *elev_boundaries;
};

// rasterization.cu:617-634
__device__ __forceinline__ uint32_t point_tile(const PointGrid &g, float2 p) {
    const float azim = p.x - g.min_azim;
    float tile_azim;
    if (azim >= 0.f && azim < 360.f) tile_azim = azim / g.azim_res;
    else tile_azim = fmodf(azim + 360.f, 360.f) / g.azim_res;
    const int32_t x = (int32_t)tile_azim;
    // first of the leading n_tiles_elev boundaries that is not below the point (the
    // reference walks them upwards; they ascend)
    int32_t lo = 0, hi = (int32_t)g.n_tiles_elev;
    while (lo < hi) {
        const int32_t mid = (lo + hi) >> 1;
        if (g.elev_boundaries[mid] < p.y) lo = mid + 1; else hi = mid;
    }
    const int32_t y = max(lo - 1, 0);
    return (uint32_t)(y * (int32_t)g.n_tiles_azim + x);
}

__device__ __forceinline__ int64_t point_camera(uint64_t idx, uint32_t N, const int64_t *camera_ids) {
    return camera_ids ? camera_ids[idx] : (int64_t)(idx / N);
}

// sort == false: keys in point order
__global__ void __launch_bounds__(SPLATAD_THREADS)
points_keys_kernel(PointGrid g, uint64_t total, uint32_t N, const int64_t *__restrict__ camera_ids,
                   const float *__restrict__ points2d, int64_t *__restrict__ tile_ids,
                   int32_t *__restrict__ flatten_ids) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const uint32_t tile = point_tile(g, reinterpret_cast<const float2 *>(points2d)[idx]);
    tile_ids[idx] = (point_camera(idx, N, camera_ids) << 32) | (int64_t)tile;
    flatten_ids[idx] = (int32_t)idx;
}

// One wavefront per workgroup.  FILL == false: counts per (camera, tile) of the range
// [blockIdx.x * span, +span) into row blockIdx.x of the table.  FILL == true: the row holds the
// start of this workgroup's run in every tile's segment; points are placed in point order.
template <bool FILL>
__global__ void __launch_bounds__(SPLATAD_WAVE)
points_bin_kernel(PointGrid g, uint64_t total, uint64_t span, uint32_t N,
                  const int64_t *__restrict__ camera_ids, const float *__restrict__ points2d,
                  uint32_t n_slots, int32_t *table, int64_t *__restrict__ tile_ids,
                  int32_t *__restrict__ flatten_ids) {
    extern __shared__ int32_t s_slots[];
    const uint32_t lane = threadIdx.x;
    const uint32_t tiles_per_cam = g.n_tiles_azim * g.n_tiles_elev;
    int32_t *row = table + (size_t)blockIdx.x * n_slots;
    for (uint32_t s = lane; s < n_slots; s += SPLATAD_WAVE) s_slots[s] = FILL ? row[s] : 0;
    __syncthreads();
    const uint64_t first = (uint64_t)blockIdx.x * span;
    const uint64_t last = min(total, first + span);
    const uint64_t below = (1ull << lane) - 1ull;
    for (uint64_t base = first; base < last; base += SPLATAD_WAVE) { // uniform
        const uint64_t idx = base + lane;
        const bool has = idx < last;
        uint32_t tile = 0, slot = 0xFFFFFFFFu;
        int64_t cam = 0;
        if (has) {
            tile = point_tile(g, reinterpret_cast<const float2 *>(points2d)[idx]);
            cam = point_camera(idx, N, camera_ids);
            // keys outside the grid (a point beyond the last column) share the last slot;
            // they are rare and only their relative order matters here
            const uint64_t s = (uint64_t)cam * tiles_per_cam + tile;
            slot = (uint32_t)min(s, (uint64_t)n_slots - 1);
        }
        uint64_t todo = wave_ballot(has);
        while (todo) { // the lanes of one slot at a time, lowest lane first
            const int leader = __ffsll((unsigned long long)todo) - 1;
            const uint32_t cur = (uint32_t)__shfl((int)slot, leader, SPLATAD_WAVE);
            const bool in = has && slot == cur;
            const uint64_t group = wave_ballot(in);
            todo &= ~group;
            if (in) {
                const int32_t at = s_slots[cur] + (int32_t)__popcll(group & below);
                if (FILL) {
                    tile_ids[at] = (cam << 32) | (int64_t)tile;
                    flatten_ids[at] = (int32_t)idx;
                }
            }
            if ((int)lane == leader) s_slots[cur] += (int32_t)__popcll(group);
        }
    }
    if (!FILL) {
        __syncthreads();
        for (uint32_t s = lane; s < n_slots; s += SPLATAD_WAVE) row[s] = s_slots[s];
    }
}

// rasterization.cu:531-574
__global__ void __launch_bounds__(SPLATAD_THREADS)
points_offset_encode_kernel(int64_t n_points, const int64_t *__restrict__ point_ids,
                            uint32_t n_tiles, int64_t total_tiles, int32_t *__restrict__ offsets) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_points) return;
    const int64_t id = point_ids[idx];
    const int64_t id_curr = (id >> 32) * n_tiles + (id & 0xFFFFFFFFll);
    int64_t first;
    if (idx == 0) {
        first = 0;
    } else {
        const int64_t prev = point_ids[idx - 1];
        first = prev == id ? id_curr + 1 : (prev >> 32) * n_tiles + (prev & 0xFFFFFFFFll) + 1;
    }
    for (int64_t i = first; i <= id_curr && i < total_tiles; ++i) offsets[i] = (int32_t)idx;
    if (idx == n_points - 1)
        for (int64_t i = id_curr + 1; i < total_tiles; ++i) offsets[i] = (int32_t)n_points;
}

__global__ void points_fill_zero_kernel(float *p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.f;
}

__global__ void points_fill_zero_i32_kernel(int32_t *p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

// rasterization.cu:772-805: workgroup per (camera, tile); thread k of the tile takes the
// k-th point of the tile's run
__global__ void populate_image_kernel(uint32_t C, int64_t n_points, const float *__restrict__ points,
                                      uint32_t W, uint32_t H, uint32_t tile_width,
                                      uint32_t tile_height, uint32_t grid_w, uint32_t grid_h,
                                      const int32_t *__restrict__ tile_offsets,
                                      const int32_t *__restrict__ flatten_ids,
                                      float *__restrict__ image) {
    const uint32_t tiles_per_cam = grid_w * grid_h;
    const uint32_t cam = blockIdx.x / tiles_per_cam, tile = blockIdx.x % tiles_per_cam;
    const uint32_t tr = threadIdx.x;
    if (tr >= tile_width * tile_height) return;
    const uint32_t i = (tile / grid_w) * tile_height + tr / tile_width;
    const uint32_t j = (tile % grid_w) * tile_width + tr % tile_width;
    if (i >= H || j >= W) return;
    const int32_t *offs = tile_offsets + (size_t)cam * tiles_per_cam;
    const int64_t start = offs[tile];
    const int64_t end = (cam == C - 1 && tile == tiles_per_cam - 1) ? n_points : (int64_t)offs[tile + 1];
    const int64_t k = start + tr;
    if (k >= end) return;
    const float *src = points + (size_t)flatten_ids[k] * 5;
    float *dst = image + (((size_t)cam * H + i) * W + j) * 5;
#pragma unroll
    for (int q = 0; q < 5; ++q) dst[q] = src[q];
}

constexpr uint32_t kMaxSlots = 36864; // LDS counters of one workgroup, 144 KB

static uint32_t bin_workgroups(uint64_t total, uint64_t n_slots) {
    uint64_t wgs = (1ull << 20) / (n_slots ? n_slots : 1); // table of about a million entries
    if (wgs > 1024) wgs = 1024;
    if (wgs < 16) wgs = 16;
    const uint64_t needed = (total + SPLATAD_WAVE - 1) / SPLATAD_WAVE;
    if (wgs > needed) wgs = needed ? needed : 1;
    return (uint32_t)wgs;
}

struct BinWorkspace {
    int32_t *counts, *starts;
    int64_t *scan_total, *block_sums;
};

static size_t carve_bin(void *ws, uint64_t table, BinWorkspace *out) {
    char *p = (char *)ws;
    BinWorkspace w;
    w.scan_total = (int64_t *)p;  p += 256;
    w.counts = (int32_t *)p;      p += splatad_align256(table * 4);
    w.starts = (int32_t *)p;      p += splatad_align256(table * 4);
    w.block_sums = (int64_t *)p;  p += scan_workspace_bytes((int64_t)table);
    if (out) *out = w;
    return (size_t)(p - (char *)ws);
}

} // namespace

extern "C" size_t splatad_map_points_to_lidar_tiles_workspace_bytes(uint64_t total, uint32_t C,
                                                                    uint32_t n_tiles) {
    const uint64_t n_slots = (uint64_t)C * n_tiles;
    return carve_bin(nullptr, n_slots * bin_workgroups(total, n_slots), nullptr);
}

namespace {

// The sorted binning behind both entry points.  `max_table` bounds the [workgroup][slot] counter
// table (and with it the scratch the caller has to provide): fewer workgroups are used when
// the plain choice would exceed it.
static int map_points_sorted(const PointGrid &g, uint64_t total, uint32_t N, const int64_t *camera_ids,
                             const float *points2d, uint32_t C, void *workspace, uint64_t max_table,
                             int64_t *tile_ids, int32_t *flatten_ids, hipStream_t stream) {
    const uint64_t n_slots64 = (uint64_t)C * g.n_tiles_azim * g.n_tiles_elev;
    SPLATAD_REQUIRE(n_slots64 <= kMaxSlots, "map_points_to_lidar_tiles: %llu (sensor, tile) pairs exceed "
                    "the binning capacity of %u", (unsigned long long)n_slots64, kMaxSlots);
    const uint32_t n_slots = (uint32_t)n_slots64;
    uint32_t wgs = bin_workgroups(total, n_slots);
    if ((uint64_t)wgs * n_slots > max_table) wgs = (uint32_t)(max_table / n_slots);
    SPLATAD_REQUIRE(wgs >= 1, "map_points_to_lidar_tiles: %u (sensor, tile) pairs exceed the counter table "
                    "of %llu entries", n_slots, (unsigned long long)max_table);
    const uint64_t span = ((total + wgs - 1) / wgs + SPLATAD_WAVE - 1) / SPLATAD_WAVE * SPLATAD_WAVE;
    BinWorkspace w;
    carve_bin(workspace, (uint64_t)n_slots * wgs, &w);
    const size_t lds = (size_t)n_slots * 4;
    {   // once per device, at the first sorted call on it (which therefore cannot be a captured one)
        static std::mutex guard;
        static bool raised[64] = {};
        int dev = 0;
        SPLATAD_CHECK_HIP(hipGetDevice(&dev));
        SPLATAD_REQUIRE(dev >= 0 && dev < 64, "map_points_to_lidar_tiles: device index %d out of range", dev);
        std::lock_guard<std::mutex> lock(guard);
        if (!raised[dev]) {
            SPLATAD_CHECK_HIP(hipFuncSetAttribute((const void *)points_bin_kernel<false>,
                                                  hipFuncAttributeMaxDynamicSharedMemorySize,
                                                  (int)(kMaxSlots * 4)));
            SPLATAD_CHECK_HIP(hipFuncSetAttribute((const void *)points_bin_kernel<true>,
                                                  hipFuncAttributeMaxDynamicSharedMemorySize,
                                                  (int)(kMaxSlots * 4)));
            raised[dev] = true;
        }
    }
    hipLaunchKernelGGL(points_bin_kernel<false>, dim3(wgs), dim3(SPLATAD_WAVE), lds, stream, g, total,
                       span, N, camera_ids, points2d, n_slots, w.counts, (int64_t *)nullptr,
                       (int32_t *)nullptr);
    SPLATAD_LAUNCH_CHECK();
    int rc = launch_exclusive_scan<int32_t>(w.counts, (int64_t)n_slots * wgs, wgs > 1 ? -(int)wgs : 1,
                                            0, w.starts, w.scan_total, w.block_sums, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(points_bin_kernel<true>, dim3(wgs), dim3(SPLATAD_WAVE), lds, stream, g, total,
                       span, N, camera_ids, points2d, n_slots, w.starts, tile_ids, flatten_ids);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

static int map_points_check(uint64_t total, uint32_t N, const int64_t *camera_ids, const float *points2d,
                            uint32_t C, const float *elev_boundaries, uint32_t n_tiles_azim,
                            uint32_t n_tiles_elev, const int64_t *tile_ids, const int32_t *flatten_ids) {
    SPLATAD_REQUIRE(total < (1ull << 31), "map_points_to_lidar_tiles: number of points must be below 2^31");
    SPLATAD_REQUIRE(points2d && elev_boundaries && tile_ids && flatten_ids,
                    "map_points_to_lidar_tiles: null pointer argument");
    SPLATAD_REQUIRE(camera_ids != nullptr || N > 0, "map_points_to_lidar_tiles: N is zero for unpacked input");
    SPLATAD_REQUIRE(C > 0 && n_tiles_azim > 0 && n_tiles_elev > 0, "map_points_to_lidar_tiles: empty tile grid");
    return 0;
}

static int map_points_unsorted(const PointGrid &g, uint64_t total, uint32_t N, const int64_t *camera_ids,
                               const float *points2d, int64_t *tile_ids, int32_t *flatten_ids,
                               hipStream_t stream) {
    hipLaunchKernelGGL(points_keys_kernel, dim3((uint32_t)((total + SPLATAD_THREADS - 1) / SPLATAD_THREADS)),
                       dim3(SPLATAD_THREADS), 0, stream, g, total, N, camera_ids, points2d, tile_ids,
                       flatten_ids);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

// Scratch of the entry point that allocates nothing: a counter table of at most kStaticTable
// entries, its scan, the scan's block sums and total, laid out by carve_bin().  Every GPU the
// library runs on holds its own copy of this array from the moment the library is loaded until
// the process ends (about 2 MiB).
constexpr uint64_t kStaticTable = 1ull << 18;
constexpr size_t kStaticScratchBytes =
    256 + 2 * (size_t)kStaticTable * 4 + ((kStaticTable + SCAN_TILE - 1) / SCAN_TILE) * 8 + 256;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Address of the current device's copy of `scratch`, looked up once per device.  In host code
// the array's name is only a handle for this lookup, never an address a kernel could use.
static int static_scratch(void **out) {
    static std::mutex guard;
    static void *table[64] = {};
    int dev = 0;
    SPLATAD_CHECK_HIP(hipGetDevice(&dev));
    SPLATAD_REQUIRE(dev >= 0 && dev < 64, "map_points_to_lidar_tiles: device index %d out of range", dev);
    SPLATAD_REQUIRE(carve_bin(nullptr, kStaticTable, nullptr) <= kStaticScratchBytes,
                    "map_points_to_lidar_tiles: the static scratch is smaller than its layout");
    std::lock_guard<std::mutex> lock(guard);
    if (table[dev] == nullptr) {
        void *ptr = nullptr;
        SPLATAD_CHECK_HIP(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
        SPLATAD_REQUIRE(ptr != nullptr, "map_points_to_lidar_tiles: the static scratch has no device address");
        table[dev] = ptr;
    }
    *out = table[dev];
    return 0;
}

} // namespace

extern "C" int splatad_map_points_to_lidar_tiles(
    uint64_t total, uint32_t N, const int64_t *camera_ids, const float *points2d, uint32_t C,
    const float *elev_boundaries, float tile_azim_resolution, float min_azim,
    uint32_t n_tiles_azim, uint32_t n_tiles_elev, int sort, void *workspace, int64_t *tile_ids,
    int32_t *flatten_ids, splatad_stream_t stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (total == 0) return 0;
    if (int rc = map_points_check(total, N, camera_ids, points2d, C, elev_boundaries, n_tiles_azim,
                                  n_tiles_elev, tile_ids, flatten_ids))
        return rc;
    PointGrid g{n_tiles_azim, n_tiles_elev, tile_azim_resolution, min_azim, elev_boundaries};
    if (!sort) return map_points_unsorted(g, total, N, camera_ids, points2d, tile_ids, flatten_ids, stream);
    SPLATAD_REQUIRE(workspace != nullptr, "map_points_to_lidar_tiles: workspace is null");
    return map_points_sorted(g, total, N, camera_ids, points2d, C, workspace, ~0ull, tile_ids, flatten_ids,
                             stream);
}

extern "C" uint64_t splatad_map_points_to_lidar_tiles_noalloc_max_points(void) { return 1ull << 22; }
extern "C" uint32_t splatad_map_points_to_lidar_tiles_noalloc_max_tiles(void) { return 16384u; }

extern "C" int splatad_map_points_to_lidar_tiles_noalloc(
    uint64_t total, uint32_t N, const int64_t *camera_ids, const float *points2d, uint32_t C,
    const float *elev_boundaries, float tile_azim_resolution, float min_azim,
    uint32_t n_tiles_azim, uint32_t n_tiles_elev, int sort, int64_t *tile_ids,
    int32_t *flatten_ids, splatad_stream_t stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (total == 0) return 0;
    if (int rc = map_points_check(total, N, camera_ids, points2d, C, elev_boundaries, n_tiles_azim,
                                  n_tiles_elev, tile_ids, flatten_ids))
        return rc;
    SPLATAD_REQUIRE(total <= splatad_map_points_to_lidar_tiles_noalloc_max_points(),
                    "map_points_to_lidar_tiles_noalloc: %llu points exceed the limit of %llu of the entry "
                    "point that allocates nothing; use splatad_map_points_to_lidar_tiles with a workspace",
                    (unsigned long long)total,
                    (unsigned long long)splatad_map_points_to_lidar_tiles_noalloc_max_points());
    const uint64_t n_slots = (uint64_t)C * n_tiles_azim * n_tiles_elev;
    SPLATAD_REQUIRE(n_slots <= splatad_map_points_to_lidar_tiles_noalloc_max_tiles(),
                    "map_points_to_lidar_tiles_noalloc: %llu (sensor, tile) pairs exceed the limit of %u of "
                    "the entry point that allocates nothing; use splatad_map_points_to_lidar_tiles with a "
                    "workspace", (unsigned long long)n_slots, splatad_map_points_to_lidar_tiles_noalloc_max_tiles());
    PointGrid g{n_tiles_azim, n_tiles_elev, tile_azim_resolution, min_azim, elev_boundaries};
    if (!sort) return map_points_unsorted(g, total, N, camera_ids, points2d, tile_ids, flatten_ids, stream);
    void *ptr = nullptr;
    if (int rc = static_scratch(&ptr)) return rc;
    // Every word of the scratch that a kernel reads is written by an earlier kernel of the same
    // call (the counting pass stores whole rows of the table, the scan its block sums, its
    // output and its total), so nothing has to be cleared between calls.
    return map_points_sorted(g, total, N, camera_ids, points2d, C, ptr, kStaticTable, tile_ids, flatten_ids,
                             stream);
}

extern "C" int splatad_points_mapping_offset_encode(int64_t n_points, const int64_t *point_ids,
                                                    uint32_t C, uint32_t n_tiles, int32_t *offsets,
                                                    splatad_stream_t stream) {
    const int64_t total_tiles = (int64_t)C * n_tiles;
    if (total_tiles == 0) return 0;
    SPLATAD_REQUIRE(offsets != nullptr, "points_mapping_offset_encode: offsets is null");
    if (n_points == 0) {
        hipLaunchKernelGGL(points_fill_zero_i32_kernel, dim3((uint32_t)((total_tiles + 255) / 256)),
                           dim3(256), 0, (hipStream_t)stream, offsets, total_tiles);
        SPLATAD_LAUNCH_CHECK();
        return 0;
    }
    SPLATAD_REQUIRE(point_ids != nullptr, "points_mapping_offset_encode: point_ids is null");
    hipLaunchKernelGGL(points_offset_encode_kernel, dim3((uint32_t)((n_points + 255) / 256)), dim3(256),
                       0, (hipStream_t)stream, n_points, point_ids, n_tiles, total_tiles, offsets);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

extern "C" int splatad_populate_image_from_points(
    uint32_t C, int64_t n_points, const float *points, uint32_t image_width, uint32_t image_height,
    uint32_t tile_width, uint32_t tile_height, uint32_t grid_w, uint32_t grid_h,
    const int32_t *tile_offsets, const int32_t *flatten_ids, float *image, splatad_stream_t stream) {
    const int64_t n_out = (int64_t)C * image_height * image_width * 5;
    if (n_out == 0) return 0;
    SPLATAD_REQUIRE(image != nullptr, "populate_image_from_points: image is null");
    SPLATAD_REQUIRE(tile_width >= 1 && tile_height >= 1 && tile_width * tile_height <= 1024,
                    "populate_image_from_points: tile %ux%u exceeds 1024 points", tile_width, tile_height);
    hipLaunchKernelGGL(points_fill_zero_kernel, dim3((uint32_t)((n_out + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, image, n_out);
    SPLATAD_LAUNCH_CHECK();
    if (n_points == 0 || grid_w * grid_h == 0) return 0;
    SPLATAD_REQUIRE(points && tile_offsets && flatten_ids, "populate_image_from_points: null pointer argument");
    const uint32_t threads = (tile_width * tile_height + 63) / 64 * 64;
    hipLaunchKernelGGL(populate_image_kernel, dim3(C * grid_w * grid_h), dim3(threads), 0,
                       (hipStream_t)stream, C, n_points, points, image_width, image_height, tile_width,
                       tile_height, grid_w, grid_h, tile_offsets, flatten_ids, image);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}
