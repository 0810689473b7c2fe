// Tile intersection, segmented sort and tile-offset encoding for gfx950.
//
// Results are bit-identical to gsplat/cuda/csrc/rasterization.cu:15-529 of the reference
// (two-pass emit + cub::DeviceRadixSort on (camera | tile | depth) keys) but are produced
// differently, by binning instead of a global sort:
//   1. coarse binning: every Gaussian is entered, with one global atomic each in a counting
//      and a filling pass, into the lists of the coarse blocks (4 x 4 tiles) it touches,
//      together with the 16-bit mask of the block's tiles it covers;
//   2. tile binning: wavefronts walk the coarse lists, 64 entries of one block at a time,
//      and turn the masks into per-tile counts and ranks with ballots, so that a tile
//      counter sees one atomic per wavefront instead of one per intersection; an exclusive
//      scan of the tile counts in between gives every tile's segment in the output;
//   3. one workgroup per tile sorts its segment of (depth bits, flatten id) pairs in LDS and
//      writes the final 64-bit keys and the ids.
// Camera frames replace steps 2 and 3 by a sort of the coarse lists themselves (cut into depth
// slabs), from which the tile lists are written in order ("Cameras: the coarse lists are
// sorted" below); lidar sweeps, and frames with a coarse list too long for that, keep them.
// A stable sort by (camera, tile, depth) with ties kept in emission order equals a sort
// by (camera, tile, depth, flatten id), because the emission loop visits flatten ids in
// ascending order; that is what makes the unordered binning legal.  Depths must have a
// clear sign bit.
//
// Built with -ffp-contract=off: the tile bounds are float32 expressions whose rounding
// decides which tiles a Gaussian touches.
#include "common.h"
#include "host_word.h"
#include "scan.h"
#include "tile_rect.h"

#include <mutex>

namespace {

struct TileGrid {
    uint32_t tile_size;   // camera only
    uint32_t tile_w, tile_h;
    float azim_res, min_azim; // lidar only
    const float *elev_boundaries;
};

// Number of leading boundaries below v (boundaries ascending).
__device__ __forceinline__ int32_t elev_lower_bound(const float *b, int32_t count, float v) {
    int32_t lo = 0, hi = count;
    while (lo < hi) {
        const int32_t mid = (lo + hi) >> 1;
        if (b[mid] < v) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// Lidar kernels read the elevation boundaries from LDS when they fit.
constexpr uint32_t kElevLds = 1025;
#define SPLATAD_STAGE_ELEVATIONS(g)                                                          \
    __shared__ float s_elev[kElevLds];                                                       \
    if (LIDAR && (g).tile_h + 1 <= kElevLds) {                                               \
        for (uint32_t e = threadIdx.x; e <= (g).tile_h; e += blockDim.x)                     \
            s_elev[e] = (g).elev_boundaries[e];                                              \
        __syncthreads();                                                                     \
        (g).elev_boundaries = s_elev;                                                        \
    }

// Tile rectangle of one projected Gaussian: x in [x0, x1), y in [y0, y1).  For lidars x
// may be negative or exceed tile_w (wrapped at emission).
// `radii` holds the two words of the Gaussian's radii: int32 for cameras, float for lidars.
template <bool LIDAR>
__device__ __forceinline__ bool tile_rect_of(const TileGrid &g, float2 mu, uint2 radii,
                                             int32_t &x0, int32_t &y0, int32_t &x1, int32_t &y1) {
    if (!LIDAR) {
        return splatad_camera_tile_rect(g.tile_size, g.tile_w, g.tile_h, mu,
                                        make_int2((int32_t)radii.x, (int32_t)radii.y), x0, y0, x1, y1);
    } else {
        const float2 r = make_float2(__uint_as_float(radii.x), __uint_as_float(radii.y));
        if (r.x <= 0.f) return false;
        const float elev_low = mu.y - r.y, elev_high = mu.y + r.y;
        const float azim = mu.x - g.min_azim;
        const float azim_low = azim - r.x, azim_high = azim + r.x;
        const float azim_max = (float)g.tile_w * g.azim_res;
        float t_low, t_high;
        if (azim_low >= 0.f)
            t_low = azim_low / g.azim_res;
        else
            t_low = (fmodf(azim_low + 360.f, 360.f) - azim_max) / g.azim_res;
        if (azim_high <= 360.f)
            t_high = azim_high / g.azim_res;
        else
            t_high = (float)g.tile_w + fmodf(azim_high + 360.f, 360.f) / g.azim_res;
        x0 = (int32_t)floorf(t_low);
        x1 = (int32_t)ceilf(t_high);
        // The reference walks the boundaries upwards (rasterization.cu:346-356): i = first
        // boundary >= elev_low, then on to the first >= elev_high.  For ascending boundaries
        // these are two lower bounds, found here by bisection.
        const int32_t n = (int32_t)g.tile_h;
        const int32_t i_low = elev_lower_bound(g.elev_boundaries, n + 1, elev_low);
        const int32_t i_high = max(i_low, elev_lower_bound(g.elev_boundaries, n + 1, elev_high));
        y0 = max(i_low - 1, 0);
        y1 = min(i_high, n);
    }
    return true;
}

template <bool LIDAR>
__device__ __forceinline__ bool tile_rect(const TileGrid &g, const float *__restrict__ means2d,
                                          const void *__restrict__ radii_v, uint64_t idx,
                                          int32_t &x0, int32_t &y0, int32_t &x1, int32_t &y1) {
    return tile_rect_of<LIDAR>(g, reinterpret_cast<const float2 *>(means2d)[idx],
                               reinterpret_cast<const uint2 *>(radii_v)[idx], x0, y0, x1, y1);
}

// Keeps the compiler from moving the loads of x and y down to their first use behind a
// branch: both values have to be in registers here.  Emits no instruction.
__device__ __forceinline__ void loaded_here(float2 &mu, uint2 &r) {
    asm volatile("" : "+v"(mu.x), "+v"(mu.y), "+v"(r.x), "+v"(r.y));
}

// Mathematical x mod n; columns within one turn of the grid (nearly all) need no division.
__device__ __forceinline__ int32_t wrap_column(int32_t x, int32_t n) {
    if (x >= 0 && x < n) return x;
    if (x < 0 && x >= -n) return x + n;
    if (x >= n && x < 2 * n) return x - n;
    return ((x % n) + n) % n;
}

template <bool LIDAR>
__device__ __forceinline__ uint32_t tile_index(const TileGrid &g, int32_t y, int32_t x) {
    if (LIDAR) {
        // Mathematical modulo.  For x >= -tile_w this equals (x + tile_w) % tile_w of the
        // reference (rasterization.cu:384).  That sum is unsigned there, so for x < -tile_w (an
        // azimuth extent reaching below -360 degrees) it wraps modulo 2^32 first: the same
        // column as here when tile_w is a power of two, a column shifted by 2^32 mod tile_w
        // otherwise.
        x = wrap_column(x, (int32_t)g.tile_w);
    }
    return (uint32_t)y * g.tile_w + (uint32_t)x;
}

// Grid-stride over the Gaussians.  `counters` (kCountWords words, zero when the kernel starts
// and zero again when it ends) takes the partial sums; the total goes to the host's pinned
// slot.  On its way the kernel clears `clear_words` words from `clear` on: the counters of the
// binning kernels behind it, which spares the launch of a clearing kernel.
constexpr uint32_t kSlabShiftMax = 6;          // 64 slabs at most (the block sort's lists)
constexpr uint32_t kSegmentSlabShiftMax = 4;   // the segment sort cuts its tile segments into 16 at most
constexpr uint32_t kSlabSamples = 256;
constexpr uint32_t kSlabEstimates = 4; // independent sets of samples, a workgroup each

template <typename Load, typename Store>
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t L, uint32_t tid, uint32_t nt,
                                                         uint32_t *s_wave, Load &&load, Store &&store) {
    const uint32_t lane = tid & (SPLATAD_WAVE - 1), wave = tid / SPLATAD_WAVE;
    const uint32_t per = (L + nt - 1) / nt;
    const uint32_t b0 = min(L, tid * per), b1 = min(L, b0 + per);
    uint32_t sum = 0;
    for (uint32_t b = b0; b < b1; ++b) sum += load(b);
    uint32_t incl = sum;
#pragma unroll
    for (int off = 1; off < SPLATAD_WAVE; off <<= 1) {
        const uint32_t o = (uint32_t)__shfl_up((int)incl, off, SPLATAD_WAVE);
        if ((int)lane >= off) incl += o;
    }
    if (lane == SPLATAD_WAVE - 1) s_wave[wave] = incl;
    __syncthreads();
    uint32_t run = incl - sum, total = 0;
    for (uint32_t w = 0; w < nt / SPLATAD_WAVE; ++w) {
        const uint32_t v = s_wave[w];
        if (w < wave) run += v;
        total += v;
    }
    for (uint32_t b = b0; b < b1; ++b) {
        const uint32_t v = load(b);
        store(b, run, v);
        run += v;
    }
    __syncthreads();
    return total;
}

// All comparators of this bitonic network point the same way (the first stage of every
// merge is a "flip"), so a virtual +inf tail needs no storage: pairs whose upper index is
// >= n are skipped.
template <typename Ptr>
__device__ __forceinline__ void bitonic_sort_ascending(Ptr a, uint32_t n, uint32_t tid,
                                                       uint32_t nthreads) {
    uint32_t m = 1;
    while (m < n) m <<= 1;
    for (uint32_t k = 2; k <= m; k <<= 1) {
        for (uint32_t i = tid; i < m / 2; i += nthreads) {
            const uint32_t lo = ((i / (k / 2)) * k) + (i % (k / 2));
            const uint32_t hi = lo ^ (k - 1);
            if (hi < n) {
                const uint64_t x = a[lo], y = a[hi];
                if (y < x) { a[lo] = y; a[hi] = x; }
            }
        }
        __syncthreads();
        for (uint32_t j = k / 4; j > 0; j >>= 1) {
            for (uint32_t i = tid; i < m / 2; i += nthreads) {
                const uint32_t lo = ((i / j) * (2 * j)) + (i % j);
                const uint32_t hi = lo + j;
                if (hi < n) {
                    const uint64_t x = a[lo], y = a[hi];
                    if (y < x) { a[lo] = y; a[hi] = x; }
                }
            }
            __syncthreads();
        }
    }
}

// One workgroup, one sample per lane: kSlabSamples Gaussians at a fixed stride, ordered by
// depth (every lane counts the smaller keys; all lanes read the same LDS words, which are
// broadcasts).  A key is the depth bits with the sample's index in the low bits, which makes
// the keys distinct at a depth resolution of 2^-14, plenty for a bound.  Bound k is the key at
// which the running sum of the samples' tile counts passes k / n_slabs of the total.
// weight_of(i): the tiles Gaussian i meets.  Run by one workgroup of the counting kernel, beside
// the workgroups that count (as a launch of its own it stood in the chain of dependent kernels:
// 6 us and a launch gap per lidar call).
template <typename Weight>
__device__ __forceinline__ void slab_bounds_workgroup(uint64_t total, const float *__restrict__ depths,
                                                      Weight &&weight_of, uint32_t n_slabs, uint32_t estimate,
                                                      uint32_t *__restrict__ bounds) {
    static_assert((kSlabSamples & (kSlabSamples - 1)) == 0 && kSlabSamples % 4 == 0, "power of two");
    static_assert(kSlabSamples == SPLATAD_THREADS, "one sample per lane of a counting workgroup");
    __shared__ __align__(16) uint32_t s_key[kSlabSamples];
    __shared__ uint32_t s_sorted[kSlabSamples];
    __shared__ uint32_t s_weight[kSlabSamples];
    __shared__ uint32_t s_before[kSlabSamples];
    __shared__ uint32_t s_wave[2 * (kSlabSamples / SPLATAD_WAVE)];
    const uint32_t tid = threadIdx.x;
    // (estimate e of kSlabEstimates takes every kSlabEstimates-th of the samples, from the e-th on)
    const uint64_t n_all = total < kSlabSamples * kSlabEstimates ? total : kSlabSamples * kSlabEstimates;
    const uint64_t stride = n_all ? total / n_all : 1;
    const uint64_t at = ((uint64_t)tid * kSlabEstimates + estimate) * stride;
    uint32_t key = ~(kSlabSamples - 1u) | tid, weight = 0; // no tiles: behind every depth
    bounds += (size_t)estimate << kSlabShiftMax;
    if (at < total) {
        const int32_t w = weight_of(at);
        if (w > 0) {
            key = (__float_as_uint(depths[at]) & ~(kSlabSamples - 1u)) | tid;
            weight = (uint32_t)min(w, 1 << 20); // capped: the sum stays below 2^32
        }
    }
    s_key[tid] = key;
    if (tid < n_slabs) bounds[tid] = 0xFFFFFFFFu;
    __syncthreads();
    uint32_t rank = 0;
    for (uint32_t j = 0; j < kSlabSamples; j += 4) {
        const uint4 q = *reinterpret_cast<const uint4 *>(&s_key[j]);
        rank += (q.x < key ? 1u : 0u) + (q.y < key ? 1u : 0u) + (q.z < key ? 1u : 0u) + (q.w < key ? 1u : 0u);
    }
    s_sorted[rank] = key;
    s_weight[rank] = weight;
    __syncthreads();
    const uint32_t sum = block_exclusive_scan(
        kSlabSamples, tid, kSlabSamples, s_wave, [&](uint32_t i) { return s_weight[i]; },
        [&](uint32_t i, uint32_t before, uint32_t) { s_before[i] = before; });
    const uint32_t w = s_weight[tid], before = s_before[tid];
    if (w == 0) return;
    const uint32_t shift = 31u - (uint32_t)__clz((int)n_slabs); // the slabs are a power of two: no division per bound
    for (uint32_t k = 1; k < n_slabs; ++k) {
        const uint32_t target = (uint32_t)(((uint64_t)sum * k) >> shift);
        if (before < target && target <= before + w) bounds[k - 1] = s_sorted[tid];
    }
}

constexpr uint32_t kCountGroups = 32;
constexpr uint32_t kCountWords = 8 + 8 * kCountGroups;
template <bool LIDAR, bool SLABS>
__global__ void __launch_bounds__(SPLATAD_THREADS)
isect_count_kernel(TileGrid g, uint64_t total, const float *__restrict__ means2d,
                   const void *__restrict__ radii, int32_t *__restrict__ tiles_per_gauss,
                   unsigned long long *__restrict__ counters,
                   unsigned long long *__restrict__ n_isects_host, int32_t *__restrict__ clear,
                   uint64_t clear_words, const float *__restrict__ depths, uint32_t n_slabs,
                   uint32_t *__restrict__ slab_bounds, int unit_weights, int count_rows) {
    SPLATAD_STAGE_ELEVATIONS(g)
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < clear_words;
         i += (uint64_t)gridDim.x * blockDim.x)
        clear[i] = 0;
    // SLABS: the launch has kSlabEstimates workgroups more than count, and those find the depth
    // slabs' bounds meanwhile, each from samples of its own (they count their samples' tiles
    // themselves); the bounds used are the means of the estimates.  They are the launch's first
    // workgroups: theirs is the longest chain of dependent steps in the kernel, so they start first.
    const uint32_t n_wgs = gridDim.x - (SLABS ? kSlabEstimates : 0u);
    const uint32_t slab_wgs = SLABS ? kSlabEstimates : 0u;
    if (SLABS && blockIdx.x < slab_wgs) { // uniform across the workgroup
        slab_bounds_workgroup(total, depths, [&](uint64_t i) -> int32_t {
            float2 mu = reinterpret_cast<const float2 *>(means2d)[i];
            uint2 rad = reinterpret_cast<const uint2 *>(radii)[i];
            int32_t x0, y0, x1, y1;
            if (!tile_rect_of<LIDAR>(g, mu, rad, x0, y0, x1, y1)) return 0;
            const int32_t tiles = max(y1 - y0, 0) * max(x1 - x0, 0);
            return unit_weights ? min(tiles, 1) : tiles;
        }, n_slabs, blockIdx.x, slab_bounds);
        return;
    }
    if (!count_rows) return; // uniform: a caller that knows the count wants the clearing and the slabs only
    long long s = 0;
    // four Gaussians per lane and step, so that their loads are in flight together (the
    // kernel is bound by memory latency otherwise)
    const uint64_t stride = (uint64_t)n_wgs * blockDim.x;
    const uint32_t wg = blockIdx.x - slab_wgs;
    for (uint64_t i0 = (uint64_t)wg * blockDim.x + threadIdx.x; i0 < total; i0 += 4 * stride) {
        float2 mu[4];
        uint2 rad[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint64_t idx = min(i0 + k * stride, total - 1); // in range; unused if clamped
            mu[k] = reinterpret_cast<const float2 *>(means2d)[idx];
            rad[k] = reinterpret_cast<const uint2 *>(radii)[idx];
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) loaded_here(mu[k], rad[k]);
        int32_t cnt[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            int32_t x0, y0, x1, y1;
            cnt[k] = 0;
            // An empty rectangle counts as zero tiles, as in make_work(): a lidar whose tile
            // columns span less than a full turn gives x1 < x0 for a Gaussian that straddles
            // min_azim (the reference's product goes negative there, rasterization.cu:359-361,
            // and its lists are corrupt from that Gaussian on).
            if (i0 + k * stride < total && tile_rect_of<LIDAR>(g, mu[k], rad[k], x0, y0, x1, y1))
                cnt[k] = max(y1 - y0, 0) * max(x1 - x0, 0);
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint64_t idx = i0 + k * stride;
            if (idx < total) tiles_per_gauss[idx] = cnt[k];
            s += cnt[k];
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, SPLATAD_WAVE);
    __shared__ long long wsum[SPLATAD_THREADS / SPLATAD_WAVE];
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0 && counters != nullptr) { // null: the caller knows the total already
        long long t = 0;
        for (int w = 0; w < SPLATAD_THREADS / SPLATAD_WAVE; ++w) t += wsum[w];
        // A workgroup reports with one atomic that carries both its sum (low 48 bits) and a
        // count of one (the bits above), so the workgroup that finds everybody else counted
        // also holds the total and no fence has to order a sum before a counter (a device-scope
        // release writes back the L2 cache of a multi-die GPU; one per workgroup was most of this
        // kernel's time).  Atomics of different workgroups on one address are served one after
        // the other, so the workgroups report in groups (a 64-byte line each, counters + 8 + 8
        // group) and the last of a group reports the group's sum to the root, counters[0].
        // The workgroup that finishes last of all hands the total to the host, which spins on
        // the pinned slot: no copy command, no event and no system-scope fence stand between
        // this kernel and the host or the work enqueued behind it.
        const unsigned long long one = 1ull << 48, low = one - 1ull;
        const uint32_t groups = min(n_wgs, kCountGroups);
        const uint32_t group = wg % groups;
        const uint32_t members = n_wgs / groups + (group < n_wgs % groups ? 1u : 0u);
        // The counters are put back to zero on the way, each by the last workgroup that touches
        // it, with an exchange whose result the next step needs: the exchange has been performed
        // before the report that depends on it is issued, so by the time the host sees the total
        // (and may start the next counting kernel on these counters, on any stream) they are zero.
        unsigned long long *mine = counters + 8 + 8 * group;
        const unsigned long long before = atomicAdd(mine, one | (unsigned long long)t);
        if ((before >> 48) == members - 1) {
            const unsigned long long group_sum = atomicExch(mine, 0ull) & low; // (before & low) + t
            const unsigned long long root = atomicAdd(counters, one | group_sum);
            if ((root >> 48) == groups - 1) {
                const unsigned long long sum = atomicExch(counters, 0ull) & low; // (root & low) + group_sum
                __hip_atomic_store(n_isects_host, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
        }
    }
}

__device__ __forceinline__ uint32_t camera_of(uint64_t idx, uint32_t N,
                                              const int64_t *__restrict__ camera_ids) {
    if (camera_ids) return (uint32_t)camera_ids[idx];
    // idx < 2^31 (checked by the callers): a 32-bit division, and none at all for one sensor
    return (uint32_t)idx < N ? 0u : (uint32_t)idx / N;
}

// n / d for a divisor whose reciprocal (1.0f / (float)d, correctly rounded) is at hand: below
// 2^20, (n + 0.5) / d stays at least 0.5 / d away from an integer, several times the rounding
// error of the product, so truncation gives the quotient; above, the integer division.
constexpr uint32_t kFloatDivLimit = 1u << 20;
__device__ __forceinline__ uint32_t div_by(uint32_t n, uint32_t d, float inv_d) {
    return n < kFloatDivLimit ? (uint32_t)(((float)n + 0.5f) * inv_d) : n / d;
}

// Work item of one lane: the tile rectangle of its Gaussian plus what the emitters need.
struct LaneWork {
    int32_t x0, y0, w, cnt; // rectangle origin, width and number of tiles (0 = nothing)
    uint32_t base;          // camera * tiles per camera
    uint32_t idx;           // flatten id
    uint32_t depth_bits;
    uint32_t slab;          // depth slab (binning with depth slabs only)
    int64_t cum;            // emission position of the first tile (unsorted output only)
    int32_t tx0, ty0, tx1, ty1; // tile rectangle, when x0.. describe coarse blocks instead
};

__device__ __forceinline__ LaneWork broadcast_work(const LaneWork &w, int leader) {
    LaneWork o;
    o.x0 = __shfl(w.x0, leader, SPLATAD_WAVE);
    o.y0 = __shfl(w.y0, leader, SPLATAD_WAVE);
    o.w = __shfl(w.w, leader, SPLATAD_WAVE);
    o.cnt = __shfl(w.cnt, leader, SPLATAD_WAVE);
    o.base = __shfl(w.base, leader, SPLATAD_WAVE);
    o.idx = __shfl(w.idx, leader, SPLATAD_WAVE);
    o.depth_bits = __shfl(w.depth_bits, leader, SPLATAD_WAVE);
    o.slab = __shfl(w.slab, leader, SPLATAD_WAVE);
    o.cum = __shfl(w.cum, leader, SPLATAD_WAVE);
    o.tx0 = __shfl(w.tx0, leader, SPLATAD_WAVE);
    o.ty0 = __shfl(w.ty0, leader, SPLATAD_WAVE);
    o.tx1 = __shfl(w.tx1, leader, SPLATAD_WAVE);
    o.ty1 = __shfl(w.ty1, leader, SPLATAD_WAVE);
    return o;
}

// Tile counts per Gaussian span four orders of magnitude (a Gaussian next to the sensor
// covers thousands of tiles, a distant one a single tile), so a lane-per-Gaussian loop
// leaves 63 lanes idle behind one busy lane.  Rectangles above kCoopTiles are therefore
// expanded by the whole wavefront, 64 tiles per step; the rest stay lane-private.
constexpr int32_t kCoopTiles = 16;

template <typename Emit>
__device__ __forceinline__ void for_each_tile_balanced(const LaneWork &mine, Emit &&emit) {
    const int lane = threadIdx.x & (SPLATAD_WAVE - 1);
    uint64_t big = __ballot(mine.cnt > kCoopTiles);
    while (big) {
        const int leader = __ffsll((unsigned long long)big) - 1;
        big &= big - 1;
        const LaneWork w = broadcast_work(mine, leader);
        const float inv_w = 1.0f / (float)w.w;
        for (int32_t t = lane; t < w.cnt; t += SPLATAD_WAVE) {
            const int32_t row = (int32_t)div_by((uint32_t)t, (uint32_t)w.w, inv_w);
            emit(w, w.y0 + row, w.x0 + (t - row * w.w), t);
        }
    }
    if (mine.cnt <= kCoopTiles) { // row by row, no division
        int32_t x = mine.x0, y = mine.y0;
        const int32_t x_end = mine.x0 + mine.w;
        for (int32_t t = 0; t < mine.cnt; ++t) {
            emit(mine, y, x, t);
            if (++x == x_end) { x = mine.x0; ++y; }
        }
    }
}

// What a lane reads for its work item, and the work item made from it.  Reading and making
// are separate so that a loop can request the next round's inputs before it works on this
// round's.
struct WorkInputs {
    float2 mu;
    uint2 radii;
    uint32_t cam, depth_bits;
    int64_t cum;
    uint64_t idx;
    bool in_range;
};

__device__ __forceinline__ WorkInputs fetch_work(uint64_t idx, uint64_t total, uint32_t N,
                                                 const int64_t *__restrict__ camera_ids,
                                                 const float *__restrict__ means2d,
                                                 const void *__restrict__ radii,
                                                 const float *__restrict__ depths,
                                                 const int64_t *__restrict__ cum_before) {
    WorkInputs in;
    in.idx = idx;
    in.in_range = idx < total;
    const uint64_t j = in.in_range ? idx : 0; // everything is read, whatever the radius says
    in.mu = reinterpret_cast<const float2 *>(means2d)[j];
    in.radii = reinterpret_cast<const uint2 *>(radii)[j];
    in.cam = camera_of(j, N, camera_ids);
    in.depth_bits = depths ? __float_as_uint(depths[j]) : 0u;
    in.cum = cum_before ? cum_before[j] : 0;
    return in;
}

template <bool LIDAR>
__device__ __forceinline__ LaneWork make_work(const TileGrid &g, WorkInputs in) {
    loaded_here(in.mu, in.radii);
    LaneWork w;
    w.x0 = w.y0 = w.cnt = 0;
    w.w = 1;
    w.base = 0;
    w.idx = (uint32_t)in.idx;
    w.depth_bits = 0;
    w.slab = 0;
    w.cum = 0;
    w.tx0 = w.ty0 = w.tx1 = w.ty1 = 0;
    int32_t x0, y0, x1, y1;
    if (in.in_range && tile_rect_of<LIDAR>(g, in.mu, in.radii, x0, y0, x1, y1)) {
        w.tx0 = x0; w.ty0 = y0; w.tx1 = x1; w.ty1 = y1;
        w.x0 = x0; w.y0 = y0;
        w.w = max(x1 - x0, 1);
        w.cnt = max(x1 - x0, 0) * max(y1 - y0, 0);
        w.base = in.cam * g.tile_w * g.tile_h;
        w.depth_bits = in.depth_bits;
        w.cum = in.cum;
    }
    return w;
}

// Coarse blocks of (1 << bshift) x 4 tiles.  The width is 4 tiles for cameras; for lidars,
// whose tile columns wrap around, it is the largest of 4, 2, 1 that divides the number of
// columns, so that an unwrapped block column maps onto one wrapped block column.
struct CoarseGrid {
    uint32_t bshift;
    uint32_t cw, ch; // blocks per row and per column
};
constexpr uint32_t kCoarseRowShift = 2;

// Turns the tile rectangle of a lane's work into the rectangle of coarse blocks to visit.
__device__ __forceinline__ void to_coarse(LaneWork &w, const CoarseGrid &cg) {
    if (w.cnt <= 0) return;
    const int32_t cx0 = w.tx0 >> cg.bshift, cx1 = ((w.tx1 - 1) >> cg.bshift) + 1;
    const int32_t cy0 = w.ty0 >> kCoarseRowShift, cy1 = ((w.ty1 - 1) >> kCoarseRowShift) + 1;
    w.x0 = cx0; w.y0 = cy0;
    w.w = cx1 - cx0;
    w.cnt = (cx1 - cx0) * (cy1 - cy0);
}

template <bool LIDAR>
__device__ __forceinline__ uint32_t coarse_index(const CoarseGrid &cg, int32_t cy, int32_t cx) {
    if (LIDAR) cx = wrap_column(cx, (int32_t)cg.cw);
    return (uint32_t)cy * cg.cw + (uint32_t)cx;
}

// Bit (ly << bshift | lx) is set when tile (lx, ly) of block (cx, cy) lies in the rectangle.
__device__ __forceinline__ uint32_t coarse_mask(const LaneWork &w, const CoarseGrid &cg,
                                                int32_t cy, int32_t cx) {
    const int32_t bx = 1 << cg.bshift;
    const int32_t by = 1 << kCoarseRowShift;
    const int32_t xa = max(w.tx0 - cx * bx, 0), xb = min(w.tx1 - cx * bx, bx);
    const int32_t ya = max(w.ty0 - cy * by, 0), yb = min(w.ty1 - cy * by, by);
    if (xb <= xa || yb <= ya) return 0u;
    const uint32_t row = ((1u << xb) - 1u) & ~((1u << xa) - 1u);
    // the row repeated in the block rows ya .. yb - 1: a product with one bit per block row
    // (the rows do not overlap, so nothing carries)
    const uint32_t every = cg.bshift == 2 ? 0x1111u : (cg.bshift == 1 ? 0x55u : 0xFu);
    const uint32_t rows = every & ((1u << (yb << cg.bshift)) - 1u) & ~((1u << (ya << cg.bshift)) - 1u);
    return __umul24(row, rows);
}

// Depth slabs.  Where a tile meets thousands of Gaussians (a lidar sweep's wide tiles), one
// workgroup per tile segment sorts too few, too long segments to keep the GPU busy.  The
// binning then cuts the depth axis into 1 << sshift slabs at bounds that are the same for all
// tiles, and bins into (tile, slab) pairs: a tile's segment becomes consecutive sub-segments
// in slab order, each sorted on its own, and since the slab is a non-decreasing function of
// the depth bits the result is the same list.  The bounds are weighted quantiles of a sample
// of the depths (weight = tiles met), so the sub-segments of an average tile are about equal;
// any bounds whatsoever give the same output, balance is all they decide.
// Slabs pay once a tile's segment outgrows the sort's short classes (beyond about 8000 entries,
// i.e. several hundred Gaussians per tile); below that they only lengthen the binning.  Measured
// on lidar sweeps of 0.25-4M Gaussians on 1024 tiles (whole call in ms with 0 / 4 / 8 / 16 slabs:
// 488 Gaussians per tile 0.255 / 0.267 / 0.266 / 0.281, 732: 0.320 / 0.296 / 0.297 / 0.311,
// 977: 0.516 / 0.397 / 0.382 / 0.396, 1953: 0.582 / 0.445 / 0.428 / 0.448, 3906: 1.59 / 1.11 /
// 0.96 / 0.90) and on camera frames: one camera with 1M Gaussians on 8160 tiles (123 per tile)
// and a rig of six with 2M (245) are fastest without slabs, single frames with 2M and 4M
// Gaussians would gain 7 % from 4 slabs, which the number of Gaussians per tile does not tell
// from the rig.
constexpr uint64_t kSlabMinPerTile = 704;

// Slabs for `total` projected Gaussians on `segs` tiles, from the sizes alone.
static uint32_t slab_shift_for(uint64_t total, uint64_t segs) {
    const uint64_t per_tile = segs ? total / segs : 0;
    if (per_tile < kSlabMinPerTile) return 0;
    if (per_tile < 896) return 2;
    if (per_tile < 2816) return 3;
    return kSegmentSlabShiftMax;
}

// Bound k from the kSlabEstimates estimates of it ([estimate][1 << kSlabShiftMax]): the mean of
// those that found one (an estimate whose samples met no tile has none).
__device__ __forceinline__ uint32_t slab_bound(const uint32_t *__restrict__ estimates, uint32_t k) {
    uint64_t sum = 0;
    uint32_t found = 0;
    for (uint32_t e = 0; e < kSlabEstimates; ++e) {
        const uint32_t b = estimates[(e << kSlabShiftMax) + k];
        if (b != 0xFFFFFFFFu) { sum += b; ++found; }
    }
    return found ? (uint32_t)(sum / found) : 0xFFFFFFFFu;
}

// Number of bounds at or below the depth bits: non-decreasing in d whatever the bounds hold.
__device__ __forceinline__ uint32_t slab_of(uint32_t d, const uint32_t *bounds, uint32_t n_bounds) {
    uint32_t s = 0;
    for (uint32_t k = 0; k < n_bounds; ++k) s += bounds[k] <= d ? 1u : 0u;
    return s;
}

// Exclusive scan over L values held in LDS by a workgroup of nt threads (a multiple of 64):
// thread t owns ceil(L / nt) consecutive values; load(i) gives value i, store(i, before, v)
// receives the sum of the values before i.  Returns the total.  Ends with a barrier.
// Coarse binning with one global atomic per (workgroup, block).  A fixed grid of workgroups
// strides over the Gaussians; each keeps the counters of all coarse blocks in LDS.  COUNT pass:
// at its end the workgroup adds its count of every block to the block's total (`totals`, zero
// before the pass) and keeps what the addition returns, the start of its run inside the block's
// list, in its own row of a [workgroup][block] table; the order of the runs inside a list is
// whatever the atomics give, and no later stage depends on it.  FILL pass: the same workgroup
// meets the same Gaussians; it scans the totals (a few hundred to a few thousand values, by
// every workgroup for itself: no scan kernels between the passes), starts its LDS cursors at
// block start + run start and writes the entries {flatten id, depth bits, block, tile mask}.
// One launch covers the cameras [cam_lo, cam_hi) (as many as the LDS holds counters for).
constexpr uint32_t kCoarseThreads = 1024;
constexpr uint32_t kCoarseLdsBlocks = 36864; // counters per workgroup, 144 KB

template <bool LIDAR, bool FILL>
__global__ void __launch_bounds__(kCoarseThreads)
isect_coarse_kernel(TileGrid g, CoarseGrid cg, uint64_t total, uint32_t N,
                    const int64_t *__restrict__ camera_ids, const float *__restrict__ means2d,
                    const void *__restrict__ radii, const float *__restrict__ depths,
                    uint32_t cam_lo, uint32_t cam_hi, uint32_t n_blocks, int32_t *table,
                    uint4 *__restrict__ entries, uint32_t sshift,
                    const uint32_t *__restrict__ slab_bounds, const int32_t *__restrict__ remap,
                    const int32_t *__restrict__ remap_offsets,
                    int32_t *__restrict__ tiles_out, int32_t *__restrict__ totals,
                    int64_t *__restrict__ n_entries, uint32_t entries_cap,
                    uint32_t *__restrict__ list_starts, unsigned long long *__restrict__ longest_host) {
    extern __shared__ int32_t s_blocks[];
    __shared__ uint32_t s_bounds[1u << kSlabShiftMax];
    __shared__ uint32_t s_scan[kCoarseThreads / SPLATAD_WAVE];
    __shared__ uint32_t s_longest;
    SPLATAD_STAGE_ELEVATIONS(g)
    // blocks and block counters below are (coarse block, slab) pairs, the slab in the low bits
    const uint32_t per_cam = (cg.cw * cg.ch) << sshift;
    const uint32_t first = cam_lo * per_cam, count = (cam_hi - cam_lo) * per_cam;
    const uint32_t n_bounds = (1u << sshift) - 1u;
    int32_t *row = table + (size_t)blockIdx.x * n_blocks + first;
    if (FILL) {
        // Cursor of list j: the lists before it (of all launches) plus this workgroup's run start.
        // The totals pass through LDS and the table rows are read lane by lane (a lane that walked
        // its own consecutive lists in global memory waited for every load in turn: 25 us on a frame
        // with 8160 lists).  list_starts: the first workgroup also leaves the lists' starts, and the
        // end behind them, for the kernels that walk the lists; longest_host: and tells the host the
        // longest list, a word in pinned memory like the number of intersections.
        const bool tells = blockIdx.x == 0 && list_starts != nullptr;
        uint32_t longest = 0, head = 0; // head: the entries of the launches before this one
        if (threadIdx.x == 0) s_longest = 0;
        for (uint32_t j = threadIdx.x; j < first; j += blockDim.x) {
            const uint32_t v = (uint32_t)totals[j];
            head += v;
            longest = max(longest, v);
        }
        for (uint32_t j = threadIdx.x; j < count; j += blockDim.x) s_blocks[j] = totals[first + j];
        if (first != 0) { // uniform
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) head += (uint32_t)__shfl_xor((int)head, off, SPLATAD_WAVE);
            if ((threadIdx.x & (SPLATAD_WAVE - 1)) == 0) s_scan[threadIdx.x / SPLATAD_WAVE] = head;
            __syncthreads();
            head = 0;
            for (uint32_t w = 0; w < blockDim.x / SPLATAD_WAVE; ++w) head += s_scan[w];
        }
        __syncthreads();
        const uint32_t all = head + block_exclusive_scan(
            count, threadIdx.x, blockDim.x, s_scan, [&](uint32_t j) { return (uint32_t)s_blocks[j]; },
            [&](uint32_t j, uint32_t before, uint32_t v) {
                s_blocks[j] = (int32_t)(head + before);
                longest = max(longest, v);
            });
        // (entries_cap, the caller's number of intersections, bounds the list: it holds whenever the
        // lists were sized for these very rows, and keeps a caller's mismatch inside the lists)
        for (uint32_t j = threadIdx.x; j < count; j += blockDim.x) {
            const int32_t start = s_blocks[j];
            if (tells) list_starts[first + j] = min((uint32_t)start, entries_cap);
            s_blocks[j] = start + row[j];
        }
        const bool last_launch = first + count == n_blocks;
        if (blockIdx.x == 0 && threadIdx.x == 0 && last_launch) {
            *n_entries = (int64_t)min(all, entries_cap);
            if (list_starts != nullptr) list_starts[n_blocks] = min(all, entries_cap);
        }
        if (blockIdx.x == 0 && last_launch && longest_host != nullptr) { // uniform
            if (longest) atomicMax(&s_longest, longest);
            __syncthreads();
            // a list that would not fit the caller's memory counts as too long for everything
            if (threadIdx.x == 0)
                __hip_atomic_store(longest_host, (unsigned long long)(all > entries_cap ? 0xFFFFFFFFu : s_longest),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    } else {
        for (uint32_t b = threadIdx.x; b < count; b += blockDim.x) s_blocks[b] = 0;
    }
    if (threadIdx.x < n_bounds) s_bounds[threadIdx.x] = slab_bound(slab_bounds, threadIdx.x);
    __syncthreads();
    const float *depths_needed = FILL || sshift ? depths : nullptr;
    const uint64_t round = (uint64_t)gridDim.x * blockDim.x;
    WorkInputs ahead = fetch_work((uint64_t)blockIdx.x * blockDim.x + threadIdx.x, total, N, camera_ids,
                                  means2d, radii, depths_needed, nullptr);
    for (uint64_t base = (uint64_t)blockIdx.x * blockDim.x; base < total; base += round) { // uniform
        const bool was_kept = ahead.in_range && (LIDAR ? __uint_as_float(ahead.radii.x) > 0.f
                                                       : (int32_t)ahead.radii.x > 0);
        const uint32_t cam = ahead.cam;
        LaneWork mine = make_work<LIDAR>(g, ahead);
        // the inputs of the next round are requested before this round's emission
        ahead = fetch_work(base + round + threadIdx.x, total, N, camera_ids, means2d, radii,
                           depths_needed, nullptr);
        if (cam < cam_lo || cam >= cam_hi) mine.cnt = 0;
        // Rows of a dense [C, N] projection standing in for its packed rows: the entries carry
        // the row's position among the kept rows (an increasing function of the dense index, so
        // ties keep their order), and the kept rows' tile counts are gathered on the way.
        if (FILL && remap != nullptr && was_kept) {
            // (a row's place: remap, plus, where given, that of its group of SPLATAD_THREADS rows)
            const uint32_t at = (uint32_t)(remap[mine.idx] +
                                           (remap_offsets != nullptr ? remap_offsets[mine.idx / SPLATAD_THREADS] : 0));
            if (tiles_out != nullptr && cam >= cam_lo && cam < cam_hi) tiles_out[at] = mine.cnt;
            mine.idx = at;
        }
        mine.base = (cam - cam_lo) * per_cam;
        mine.slab = slab_of(mine.depth_bits, s_bounds, n_bounds);
        to_coarse(mine, cg);
        for_each_tile_balanced(mine, [&](const LaneWork &w, int32_t y, int32_t x, int32_t) {
            const uint32_t local = w.base + ((coarse_index<LIDAR>(cg, y, x) << sshift) | w.slab);
            const int32_t slot = atomicAdd(&s_blocks[local], 1);
            if (FILL && (uint32_t)slot < entries_cap)
                entries[slot] = make_uint4(w.idx, w.depth_bits, first + local, coarse_mask(w, cg, y, x));
        });
    }
    if (!FILL) {
        __syncthreads();
        // (eight lists per lane and step, so that their atomics are in flight together)
        for (uint32_t b0 = threadIdx.x; b0 < count; b0 += 8 * blockDim.x) {
            int32_t c[8], start[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t b = b0 + k * blockDim.x;
                c[k] = b < count ? s_blocks[b] : 0;
            }
#pragma unroll
            for (int k = 0; k < 8; ++k)
                start[k] = c[k] ? atomicAdd(&totals[first + b0 + k * blockDim.x], c[k]) : 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t b = b0 + k * blockDim.x;
                if (b < count) row[b] = start[k];
            }
        }
    }
}

// Size classes of the segment sort: class c holds the segments with kSortClassMin[c] < n <=
// kSortClassMin[c + 1]; the host launches one kernel configuration per class.
constexpr int kSortClasses = 7;
__constant__ const uint32_t kSortClassMin[kSortClasses + 1] = {0u,    512u,   2048u,  4096u,
                                                               8192u, 12288u, 32768u, 0x7FFFFFFFu};

// A table scanned by scan_local_kernel holds prefixes inside scan blocks; what has to be added is
// the sum of the blocks before an element's.  Every wavefront that needs it keeps those sums for
// the (at most 128) blocks, two per lane.  before() is called by all lanes of the wavefront
// together (it shuffles).
struct ScanBlocks {
    int32_t even, odd; // sums of the totals of the blocks before block 2 * lane and 2 * lane + 1
    bool local;        // false: the table holds complete prefixes
    bool summed;
    // request() only issues the loads of the totals, so that a caller can issue other loads
    // behind them before sum() waits for them.
    __device__ __forceinline__ void request(const int64_t *__restrict__ totals, uint32_t n_blocks, uint32_t lane) {
        local = totals != nullptr;
        summed = !local;
        even = odd = 0;
        if (!local) return; // uniform
        even = 2 * lane < n_blocks ? (int32_t)totals[2 * lane] : 0;
        odd = 2 * lane + 1 < n_blocks ? (int32_t)totals[2 * lane + 1] : 0;
    }
    __device__ __forceinline__ void sum(uint32_t lane) {
        if (summed) return; // uniform
        summed = true;
        const int32_t v0 = even, v1 = odd;
        int32_t incl = v0 + v1;
#pragma unroll
        for (int off = 1; off < SPLATAD_WAVE; off <<= 1) {
            const int32_t o = __shfl_up(incl, off, SPLATAD_WAVE);
            if ((int)lane >= off) incl += o;
        }
        even = incl - v0 - v1;
        odd = even + v0;
    }
    __device__ __forceinline__ int32_t before(uint32_t logical) const {
        if (!local) return 0; // uniform
        const uint32_t b = logical / SCAN_TILE;
        const int32_t e = __shfl(even, (int)(b >> 1), SPLATAD_WAVE);
        const int32_t o = __shfl(odd, (int)(b >> 1), SPLATAD_WAVE);
        return (b & 1u) ? o : e;
    }
};

// Enters segment `seg` (one per lane; lanes beyond n_segments idle) into the list of its size
// class: seg_lists[c * n_segments + k], k < seg_counts[c] (zeroed beforehand).  The order inside
// a class is whatever the atomics give; every segment is sorted on its own, so the result does
// not depend on it.  Also writes the tile offsets: a tile's offset is the start of its segment
// (with depth slabs: of its first slab's), the first row of the scanned table.
__device__ __forceinline__ void classify_segment(uint32_t seg, uint32_t lane, uint32_t n_segments,
                                                 uint32_t sshift, int64_t n_isects,
                                                 const int32_t *__restrict__ tile_starts,
                                                 const ScanBlocks &scan, uint32_t copies,
                                                 int32_t *__restrict__ seg_starts,
                                                 uint32_t *__restrict__ seg_counts,
                                                 uint32_t *__restrict__ seg_lists,
                                                 int32_t *__restrict__ tile_offsets) {
    uint32_t n = 0;
    // the first copy of segment s is logical element s * copies of the scanned table
    const int32_t before_here = scan.before(min(seg, n_segments - 1u) * copies);
    const int32_t before_next = scan.before(min(seg + 1u, n_segments - 1u) * copies);
    if (seg < n_segments) {
        const int64_t start = (int64_t)tile_starts[seg] + before_here;
        const int64_t stop = min(seg + 1 == n_segments ? n_isects : (int64_t)tile_starts[seg + 1] + before_next,
                                 n_isects);
        seg_starts[seg] = (int32_t)start; // what the sort kernels read
        n = stop > start ? (uint32_t)(stop - start) : 0u;
        if (tile_offsets != nullptr && (seg & ((1u << sshift) - 1u)) == 0)
            tile_offsets[seg >> sshift] = (int32_t)start;
    }
    int c = n == 0 ? -1 : 0;
    while (c >= 0 && c + 1 < kSortClasses && n > kSortClassMin[c + 1]) ++c;
    // one atomic per wavefront and class: thousands of segments share a class, and atomics on
    // one address are served one after the other
    for (int k = 0; k < kSortClasses; ++k) {
        const uint64_t members = wave_ballot(c == k);
        if (members == 0) continue; // uniform
        const int leader = __ffsll((unsigned long long)members) - 1;
        uint32_t base = 0;
        if ((int)lane == leader) base = atomicAdd(&seg_counts[k], (uint32_t)__popcll(members));
        base = (uint32_t)__shfl((int)base, leader, SPLATAD_WAVE);
        if (c == k)
            seg_lists[(size_t)k * n_segments + base + (uint32_t)__popcll(members & ((1ull << lane) - 1ull))] = seg;
    }
}

// Tile binning.  A wavefront takes 64 consecutive coarse entries, a workgroup 256; those of one
// block (nearly always all of them, the lists being contiguous) are handled together: for each
// tile of the block a ballot over the mask bit gives the number of entries and every entry's
// rank inside the wavefront, the wavefronts' counts are added up in LDS, and the lane that owns
// the tile issues one atomic for the workgroup.  FILL == false adds to the tile counts,
// FILL == true reserves the run in the tile's segment and writes the pairs.
// BITS == 16: blocks of 4 x 4 tiles (every camera grid, lidar grids whose columns divide by 4),
// the loops over the tiles unrolled with the ballots kept in scalar registers; BITS == 0: any
// block width.
template <bool FILL, int BITS>
__global__ void __launch_bounds__(SPLATAD_THREADS)
isect_tile_bin_kernel(CoarseGrid cg, uint32_t tile_w, uint32_t tile_h, uint32_t sshift,
                      uint32_t copies, uint32_t n_segments, const int64_t *__restrict__ n_entries_ptr,
                      const uint4 *__restrict__ entries, int32_t *__restrict__ tile_counts,
                      const int32_t *__restrict__ tile_starts, int32_t *__restrict__ tile_fill,
                      uint64_t *__restrict__ pairs, int64_t n_isects,
                      uint32_t *__restrict__ seg_counts, uint32_t *__restrict__ seg_lists,
                      int32_t *__restrict__ tile_offsets, const int64_t *__restrict__ scan_totals,
                      uint32_t n_scan_blocks, int32_t *__restrict__ seg_starts, uint32_t kshift) {
    // kshift: the coarse lists are cut into 1 << (sshift + kshift) depth slabs, the tile
    // segments into 1 << sshift
    const int64_t n_entries = *n_entries_ptr;
    const uint32_t lane = threadIdx.x & (SPLATAD_WAVE - 1);
    const int64_t wave_id = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / SPLATAD_WAVE;
    const int64_t n_waves = (int64_t)gridDim.x * blockDim.x / SPLATAD_WAVE;
    // scan_totals: tile_starts holds prefixes inside scan blocks, and this kernel adds the
    // blocks before (one scan launch instead of two)
    ScanBlocks scan;
    scan.request(FILL ? scan_totals : nullptr, n_scan_blocks, lane);
    // the filling pass also lists the segments by size class for the sort that follows (the
    // scanned starts are complete before this kernel begins): a lane per segment
    if (FILL && seg_lists != nullptr)
        for (int64_t s0 = wave_id * SPLATAD_WAVE; s0 < (int64_t)n_segments; s0 += n_waves * SPLATAD_WAVE) {
            scan.sum(lane);
            classify_segment((uint32_t)s0 + lane, lane, n_segments, sshift, n_isects, tile_starts, scan,
                             copies, seg_starts, seg_counts, seg_lists, tile_offsets);
        }
    const uint32_t bits = 4u << cg.bshift, per_cam = cg.cw * cg.ch;
    const float inv_cw = 1.0f / (float)cg.cw;
    const uint32_t cap = (uint32_t)n_isects; // below 2^31
    const uint64_t below = (1ull << lane) - 1ull;
    constexpr uint32_t kWaves = SPLATAD_THREADS / SPLATAD_WAVE;
    constexpr uint32_t kNone = 0xFFFFFFFFu, kMixed = 0xFFFFFFFEu; // no (block, slab) pair reaches 2^31
    __shared__ uint32_t s_block[kWaves];   // the one block of a wavefront's entries, or kNone / kMixed
    __shared__ uint32_t s_cnt[kWaves][16]; // entries per tile of that block, per wavefront
    __shared__ int32_t s_base[16];         // where the workgroup's run starts in each tile's segment
    const uint32_t wave = threadIdx.x / SPLATAD_WAVE;
    // the tile counters are replicated like the coarse ones; both passes run on the same
    // grid, so an entry meets the same copy in both
    const int64_t copy_base = (int64_t)(blockIdx.x & (copies - 1)) * n_segments;

    // counts the entries of the group `in` per tile (lane t < bits gets tile t's) and keeps the ballots
    uint64_t hits[BITS > 0 ? BITS : 1];
    auto count_group = [&](uint32_t mask) -> uint32_t {
        uint32_t my_cnt = 0;
        if (BITS > 0) {
#pragma unroll
            for (int t = 0; t < BITS; ++t) {
                hits[t] = __ballot((mask >> t) & 1u);
                const uint32_t n_hits = (uint32_t)__popcll(hits[t]); // uniform
                asm("v_writelane_b32 %0, %1, %2" : "+v"(my_cnt) : "s"(n_hits), "n"(t));
            }
        } else {
            for (uint32_t t = 0; t < bits; ++t) {
                const uint64_t b = __ballot((mask >> t) & 1u);
                if (lane == t) my_cnt = (uint32_t)__popcll(b);
            }
        }
        return my_cnt;
    };
    // counter of the tile that lane t < bits owns in the block
    auto tile_of = [&](uint32_t block_slab) -> int64_t {
        const uint32_t block = block_slab >> sshift, slab = block_slab & ((1u << sshift) - 1u);
        int64_t tile = copy_base;
        if (lane < bits) {
            const uint32_t cam = block < per_cam ? 0u : block / per_cam, r = block - cam * per_cam;
            const uint32_t by = div_by(r, cg.cw, inv_cw), bx = r - by * cg.cw;
            const uint32_t x = (bx << cg.bshift) + (lane & ((1u << cg.bshift) - 1u));
            const uint32_t y = (by << kCoarseRowShift) + (lane >> cg.bshift);
            tile += (((int64_t)cam * tile_w * tile_h + (int64_t)y * tile_w + x) << sshift) | slab;
        }
        return tile;
    };
    // writes the group's pairs: tile t's run of this wavefront starts at dst of lane t
    // (the bound `cap` holds whenever n_isects is the count of these very rows; it keeps a
    // caller's mismatch from writing outside the lists)
    auto write_group = [&](uint32_t mask, int32_t dst, uint64_t pair) {
        if (BITS > 0) {
#pragma unroll
            for (int t = 0; t < BITS; ++t) {
                if (hits[t] == 0) continue; // uniform
                const uint32_t first = (uint32_t)__builtin_amdgcn_readlane(dst, t);
                const uint32_t at = __builtin_amdgcn_mbcnt_hi(
                    (uint32_t)(hits[t] >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)hits[t], first));
                if (((mask >> t) & 1u) && at < cap) pairs[at] = pair;
            }
        } else {
            for (uint32_t t = 0; t < bits; ++t) {
                const bool hit = (mask >> t) & 1u;
                const uint64_t b = __ballot(hit);
                const int32_t first = __shfl(dst, (int)t, SPLATAD_WAVE);
                const uint32_t at = (uint32_t)first + (uint32_t)__popcll(b & below);
                if (hit && at < cap) pairs[at] = pair;
            }
        }
    };

    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t first_entry = (int64_t)blockIdx.x * blockDim.x; first_entry < n_entries;
         first_entry += stride) { // uniform across the workgroup
        const int64_t e0 = first_entry + (int64_t)wave * SPLATAD_WAVE;
        const bool has = e0 + lane < n_entries;
        uint4 rec = has ? entries[e0 + lane] : make_uint4(0, 0, kNone, 0);
        if (has) rec.z >>= kshift; // (coarse block, slab of the tile segments)
        const uint64_t pair = ((uint64_t)rec.y << 32) | (uint64_t)rec.x;
        if (FILL) scan.sum(lane); // (the first round: behind the request for the entries)
        const uint64_t have = __ballot(has);
        // Nearly always the 256 entries of the workgroup belong to one block: then the four
        // wavefronts add up their counts in LDS and one of them issues the atomics, a quarter of
        // what the wavefronts would issue on their own (the kernel is bound by those atomics).
        const uint32_t lead = (uint32_t)__builtin_amdgcn_readfirstlane((int)rec.z);
        const bool one = __ballot(has && rec.z != lead) == 0;
        if (lane == 0) s_block[wave] = have == 0 ? kNone : (one ? lead : kMixed);
        __syncthreads();
        uint32_t common = kNone;
        bool together = true;
#pragma unroll
        for (uint32_t w = 0; w < kWaves; ++w) {
            const uint32_t b = s_block[w];
            if (b == kMixed) together = false;
            else if (b != kNone) {
                if (common == kNone) common = b;
                else if (common != b) together = false;
            }
        }
        if (together && common != kNone) { // uniform across the workgroup
            const uint32_t mask = has ? rec.w : 0u;
            const uint32_t my_cnt = count_group(mask);
            if (lane < 16) s_cnt[wave][lane] = lane < bits ? my_cnt : 0u;
            __syncthreads();
            const int64_t tile = tile_of(common);
            uint32_t before = 0, all = 0; // entries of the wavefronts before this one, and of all
            if (lane < 16) {
#pragma unroll
                for (uint32_t w = 0; w < kWaves; ++w) {
                    const uint32_t c = s_cnt[w][lane];
                    if (w < wave) before += c;
                    all += c;
                }
            }
            if (!FILL) {
                if (wave == 0 && all) atomicAdd(&tile_counts[tile], (int32_t)all);
            } else {
                // (tile - copy_base is the segment; its copy's logical element in the scanned table)
                const int32_t blocks_before =
                    scan.before((uint32_t)(tile - copy_base) * copies + (blockIdx.x & (copies - 1)));
                if (wave == 0 && lane < 16)
                    s_base[lane] = all ? tile_starts[tile] + blocks_before + atomicAdd(&tile_fill[tile], (int32_t)all) : 0;
                __syncthreads();
                const int32_t dst = lane < 16 ? s_base[lane] + (int32_t)before : 0;
                write_group(mask, dst, pair);
            }
        } else {
            uint64_t todo = have;
            while (todo) {
                const int leader = __ffsll((unsigned long long)todo) - 1;
                // (coarse block, slab) of the leader; n_segments counts (tile, slab) pairs
                const uint32_t block_slab = (uint32_t)__shfl((int)rec.z, leader, SPLATAD_WAVE);
                const bool in = has && rec.z == block_slab;
                todo &= ~__ballot(in);
                const uint32_t mask = in ? rec.w : 0u;
                const uint32_t my_cnt = count_group(mask);
                const int64_t tile = tile_of(block_slab);
                if (!FILL) {
                    if (my_cnt) atomicAdd(&tile_counts[tile], (int32_t)my_cnt);
                } else {
                    int32_t dst = 0;
                    const int32_t blocks_before =
                        scan.before((uint32_t)(tile - copy_base) * copies + (blockIdx.x & (copies - 1)));
                    if (my_cnt) dst = tile_starts[tile] + blocks_before + atomicAdd(&tile_fill[tile], (int32_t)my_cnt);
                    write_group(mask, dst, pair);
                }
            }
        }
        __syncthreads(); // the next round reuses the LDS
    }
}

// Emission order without sorting (sort == false): rasterization.cu:65-89 / :366-394.
template <bool LIDAR>
__global__ void __launch_bounds__(SPLATAD_THREADS)
isect_emit_kernel(TileGrid g, uint64_t total, uint32_t N, const int64_t *__restrict__ camera_ids,
                  const float *__restrict__ means2d, const void *__restrict__ radii,
                  const float *__restrict__ depths, const int64_t *__restrict__ cum_before,
                  uint32_t tile_n_bits, int64_t *__restrict__ isect_ids,
                  int32_t *__restrict__ flatten_ids) {
    SPLATAD_STAGE_ELEVATIONS(g)
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const WorkInputs in = fetch_work(idx, total, N, camera_ids, means2d, radii, depths, cum_before);
    LaneWork mine = make_work<LIDAR>(g, in);
    mine.base = in.cam; // here the camera itself, not its first tile
    for_each_tile_balanced(mine, [&](const LaneWork &w, int32_t y, int32_t x, int32_t t) {
        const int64_t cid_enc = (int64_t)w.base << (32 + tile_n_bits);
        const int64_t depth_enc = (int64_t)(int32_t)w.depth_bits;
        const int64_t tile_id = tile_index<LIDAR>(g, y, x);
        isect_ids[w.cum + t] = cid_enc | (tile_id << 32) | depth_enc;
        flatten_ids[w.cum + t] = (int32_t)w.idx;
    });
}

constexpr uint32_t kSortFineBins = 512;     // first-level depth bins per segment
constexpr uint32_t kSortBucketMean = 8;     // aimed-at entries per bucket
constexpr uint32_t kSortSplit = 4096;       // buckets at most, beyond the fine bins
constexpr uint32_t kSortRankMax = 1024;     // largest bucket ordered by rank counting
constexpr uint32_t kSortWindow = 15360;     // LDS window (entries) when staging is global
constexpr uint32_t kSortDirectBins = 2048;  // short segments: bins of the direct path at most
constexpr uint32_t kSortDirectMean = 2;     // entries per bin it aims at
constexpr uint32_t kSortDirectMax = 64;     // fullest bin it accepts

// Bucket counters a segment of up to max_n entries can need.
__host__ __device__ inline uint32_t sort_bucket_capacity(uint32_t max_n) {
    const uint32_t split = max_n / kSortBucketMean < kSortSplit ? max_n / kSortBucketMean : kSortSplit;
    return split + kSortFineBins + 1;
}

// One workgroup per (camera, tile) segment: a bucket sort on the depth in three steps.
//  1. The segment's range of depth bits (for positive floats a piecewise-linear logarithm
//     of the depth) is cut into up to 512 equal fine bins and the entries are counted per
//     bin (LDS atomics).
//  2. Every fine bin is given ceil(count / 8) buckets that divide it evenly, so that the
//     buckets hold about eight entries whatever the distribution of the depths is; the
//     entries are counted per bucket, the counts scanned, and the entries scattered bucket
//     by bucket into a staging array.
//  3. Every entry finds its place inside its bucket by counting the bucket's smaller
//     (depth bits, flatten id) keys; equal keys (a lidar Gaussian wider than a full turn
//     meets a tile twice) are ordered by staging position.  Lanes of one bucket read the
//     same staging words, so those reads are LDS broadcasts.
//   ER     > 0: the segment (n <= ER * blockDim.x) is held in registers between the passes;
//          = 0: it is read from global memory once per pass.
//   IN_LDS: the staging array is LDS (lds_words entries).  Otherwise the isect_ids output
//          is the staging array and passes through LDS in windows of whole buckets.
// Buckets above 1024 entries (many equal depths) are ordered by a workgroup-wide bitonic
// network instead.  Segments with min_n < n <= max_n are handled, the others skipped.
// Dynamic LDS: lds_words * 8 bytes of staging, the fine bins, 2 * bucket_cap counters.
template <int ER, bool IN_LDS>
__device__ __forceinline__ void sort_segment(uint32_t seg, uint32_t n_segments, uint32_t n_tiles,
                                             uint32_t sshift, uint32_t tile_n_bits, uint32_t lds_words,
                                             uint32_t bucket_cap, int64_t n_isects,
                                             const int32_t *__restrict__ tile_starts,
                                             const uint64_t *__restrict__ pairs, int64_t *isect_ids,
                                             int32_t *__restrict__ flatten_ids,
                                             uint64_t *lds_staged, uint32_t *s_wave, uint32_t &s_big) {
    const int64_t start = tile_starts[seg];
    const int64_t stop = min(seg + 1 == n_segments ? n_isects : (int64_t)tile_starts[seg + 1], n_isects);
    const uint32_t n = stop > start ? (uint32_t)(stop - start) : 0u; // as classified
    uint32_t *s_fine = reinterpret_cast<uint32_t *>(lds_staged + lds_words);
    uint32_t *s_cursor = s_fine + kSortFineBins;
    uint32_t *s_first = s_cursor + bucket_cap;
    const uint64_t *g = pairs + start;
    int64_t *ids_out = isect_ids + start;
    int32_t *flat_out = flatten_ids + start;
    uint64_t *staged = IN_LDS ? lds_staged : reinterpret_cast<uint64_t *>(ids_out);
    const uint32_t tid = threadIdx.x, nt = blockDim.x;
    const uint32_t lane = tid & (SPLATAD_WAVE - 1), wave = tid / SPLATAD_WAVE;
    const uint32_t n_waves = nt / SPLATAD_WAVE;
    const uint64_t cam = (seg >> sshift) / n_tiles, tile = (seg >> sshift) % n_tiles;
    const uint64_t key_hi = ((cam << tile_n_bits) | tile) << 32;

    constexpr int NR = ER > 0 ? ER : 1;
    uint64_t held[NR];
    if (ER > 0) {
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            const uint32_t i = tid + k * nt;
            held[k] = i < n ? g[i] : ~0ull;
        }
    }
    // for_each_entry(f): f(entry) for the entries this thread owns
    auto for_each_entry = [&](auto &&f) {
        if (ER > 0) {
#pragma unroll
            for (int k = 0; k < NR; ++k)
                if (tid + k * nt < n) f(held[k]);
        } else {
            uint32_t i = tid;
            for (; i + 3 * nt < n; i += 4 * nt) { // independent loads in flight together
                const uint64_t p0 = g[i], p1 = g[i + nt], p2 = g[i + 2 * nt], p3 = g[i + 3 * nt];
                f(p0); f(p1); f(p2); f(p3);
            }
            for (; i < n; i += nt) f(g[i]);
        }
    };

    // range of the depth bits
    uint32_t lo = 0xFFFFFFFFu, hi = 0u;
    for_each_entry([&](uint64_t p) {
        const uint32_t d = (uint32_t)(p >> 32);
        lo = min(lo, d);
        hi = max(hi, d);
    });
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        lo = min(lo, (uint32_t)__shfl_xor((int)lo, off, SPLATAD_WAVE));
        hi = max(hi, (uint32_t)__shfl_xor((int)hi, off, SPLATAD_WAVE));
    }
    if (lane == 0) { s_wave[2 * wave] = lo; s_wave[2 * wave + 1] = hi; }
    if (tid == 0) s_big = 0;
    uint32_t n_fine = 1;
    while (n_fine < kSortFineBins && n_fine * 16 < n) n_fine <<= 1;
    for (uint32_t f = tid; f < n_fine; f += nt) s_fine[f] = 0;
    __syncthreads();
    for (uint32_t w = 0; w < n_waves; ++w) {
        lo = min(lo, s_wave[2 * w]);
        hi = max(hi, s_wave[2 * w + 1]);
    }
    const float scale = (float)n_fine / ((float)(hi - lo) + 1.f);
    // position on the fine-bin axis, non-decreasing in the depth bits
    auto fine_pos = [&](uint64_t p, uint32_t &f) -> float {
        const float x = (float)((uint32_t)(p >> 32) - lo) * scale;
        f = min(n_fine - 1, (uint32_t)x);
        return x;
    };
    __syncthreads(); // s_wave is reused by the scans

    // 1. entries per fine bin
    for_each_entry([&](uint64_t p) {
        uint32_t f;
        fine_pos(p, f);
        atomicAdd(&s_fine[f], 1u);
    });
    __syncthreads();

    // 2. buckets per fine bin; s_fine[f] becomes (first bucket | buckets << 16)
    const uint32_t mean = max(kSortBucketMean, (n + kSortSplit - 1) / kSortSplit);
    const uint32_t nb = block_exclusive_scan(
        n_fine, tid, nt, s_wave,
        [&](uint32_t f) { return (s_fine[f] + mean - 1) / mean; },
        [&](uint32_t f, uint32_t before, uint32_t v) { s_fine[f] = before | (v << 16); });
    auto bucket_of = [&](uint64_t p) -> uint32_t {
        uint32_t f;
        const float x = fine_pos(p, f);
        const uint32_t packed = s_fine[f];
        const uint32_t k = packed >> 16;
        const uint32_t sub = min(k - 1, (uint32_t)((x - (float)f) * (float)k));
        return (packed & 0xFFFFu) + sub;
    };
    for (uint32_t b = tid; b < nb; b += nt) s_cursor[b] = 0;
    __syncthreads();
    for_each_entry([&](uint64_t p) { atomicAdd(&s_cursor[bucket_of(p)], 1u); });
    __syncthreads();
    block_exclusive_scan(
        nb, tid, nt, s_wave, [&](uint32_t b) { return s_cursor[b]; },
        [&](uint32_t b, uint32_t before, uint32_t v) {
            s_cursor[b] = before;
            s_first[b] = before;
            if (v > kSortRankMax) s_big = 1;
        });

    // scatter into buckets
    for_each_entry([&](uint64_t p) { staged[atomicAdd(&s_cursor[bucket_of(p)], 1u)] = p; });
    __syncthreads(); // s_cursor[b] is now the end of bucket b

    if (s_big) { // uniform
        for (uint32_t b = 0; b < nb; ++b) {
            const uint32_t s0 = s_first[b], s = s_cursor[b] - s0;
            if (s > kSortRankMax) bitonic_sort_ascending(staged + s0, s, tid, nt); // uniform
        }
    }

    // 3. place = first of the bucket + number of smaller keys in the bucket; `view` is the
    // staging array seen through LDS, view[j - view_lo] == staged[j]
    auto place_of = [&](uint64_t p, uint32_t i, const uint64_t *view, uint32_t view_lo) -> uint32_t {
        const uint32_t b = bucket_of(p);
        const uint32_t s0 = s_first[b], s1 = s_cursor[b];
        if (s1 - s0 > kSortRankMax) return i; // ordered by the network above
        uint32_t place = s0;
        for (uint32_t j = s0; j < s1; ++j) {
            const uint64_t q = view[j - view_lo];
            place += (q < p || (q == p && j < i)) ? 1u : 0u;
        }
        return place;
    };
    auto emit = [&](uint32_t place, uint64_t p) {
        ids_out[place] = (int64_t)(key_hi | (uint64_t)(int64_t)(int32_t)(p >> 32));
        flat_out[place] = (int32_t)(uint32_t)p;
    };
    if (IN_LDS) {
        for (uint32_t i = tid; i < n; i += nt) {
            const uint64_t p = lds_staged[i];
            emit(place_of(p, i, lds_staged, 0), p);
        }
    } else {
        // windows of whole buckets, as many as fit the LDS: a window is loaded, then its
        // entries are ranked and written over the staging array they came from
        uint32_t b0 = 0;
        while (b0 < nb) { // uniform
            const uint32_t v0 = s_first[b0];
            uint32_t lo_b = b0, hi_b = nb; // largest b1 with end(b1 - 1) - v0 <= lds_words
            while (lo_b < hi_b) {
                const uint32_t mid = (lo_b + hi_b + 1) / 2;
                if (s_cursor[mid - 1] - v0 <= lds_words) lo_b = mid; else hi_b = mid - 1;
            }
            if (lo_b == b0) {
                // a single bucket beyond the window: ordered by the network already
                const uint32_t v1 = s_cursor[b0];
                for (uint32_t i = v0 + tid; i < v1; i += nt) emit(i, staged[i]);
                b0 = b0 + 1;
                continue;
            }
            const uint32_t count = s_cursor[lo_b - 1] - v0;
            uint32_t j = tid;
            for (; j + 3 * nt < count; j += 4 * nt) { // independent loads in flight together
                const uint64_t q0 = staged[v0 + j], q1 = staged[v0 + j + nt];
                const uint64_t q2 = staged[v0 + j + 2 * nt], q3 = staged[v0 + j + 3 * nt];
                lds_staged[j] = q0; lds_staged[j + nt] = q1;
                lds_staged[j + 2 * nt] = q2; lds_staged[j + 3 * nt] = q3;
            }
            for (; j < count; j += nt) lds_staged[j] = staged[v0 + j];
            __syncthreads();
            for (uint32_t i = v0 + tid; i < v0 + count; i += nt) {
                const uint64_t p = lds_staged[i - v0];
                emit(place_of(p, i, lds_staged, v0), p);
            }
            __syncthreads();
            b0 = lo_b;
        }
    }
}

// The sort for the short segments (n <= lds_words <= 12288, n <= ER * blockDim.x), shaped for the
// latency of its LDS accesses, which bounds the generic version above.  Where the depths of a
// segment are spread evenly enough, one histogram places the entries: bins that are linear in
// the depth, four entries each on average, and the atomic that counts an entry into its bin
// returns the entry's place inside the bin; after one scan of the bins every entry is written
// to its staging position and ranked among the entries of its bin.  A segment with a bin of
// more than kSortDirectMax entries (clustered depths, a range stretched by outliers), or with
// depths that are not positive finite floats, takes the equalised buckets of the generic sort
// instead (a second histogram, scan and scatter).  Both ways:
//  * an entry's bucket is computed once, kept in a register for the scatter, and written as
//    16 bits beside the entry's staging position for the rank step;
//  * the rank loop takes four staged entries per trip with no bounds test: what follows a
//    bucket in the staging array belongs to later buckets, whose depth bits are strictly larger
//    (the bucket is a non-decreasing function of the depth bits), and four words of all ones
//    follow the segment's last entry, so an entry read beyond the bucket never counts;
//  * without TIES the keys (depth bits, flatten id) of a segment are distinct and one 64-bit
//    comparison decides; TIES (lidar: a rectangle wider than the grid lists a tile twice) orders
//    equal keys by staging position.
// Dynamic LDS: (lds_words + 4) * 8 bytes of staging, the fine bins, 2 * bucket_cap + 1
// counters, lds_words * 2 bytes of bucket indices.
__host__ __device__ inline size_t sort_small_lds_bytes(uint32_t lds_words, uint32_t bucket_cap) {
    return ((size_t)lds_words + 4) * 8 + (kSortFineBins + 2 * (size_t)bucket_cap + 1) * 4 +
           (((size_t)lds_words * 2 + 7) & ~(size_t)7);
}

template <int ER, bool TIES>
__device__ __forceinline__ void sort_segment_small(uint32_t seg, uint32_t n_segments, uint32_t n_tiles,
                                                   uint32_t sshift, uint32_t tile_n_bits, uint32_t lds_words,
                                                   uint32_t bucket_cap, int64_t n_isects,
                                                   const int32_t *__restrict__ tile_starts,
                                                   const uint64_t *__restrict__ pairs,
                                                   int64_t *__restrict__ isect_ids,
                                                   int32_t *__restrict__ flatten_ids,
                                                   uint64_t *lds_staged, uint32_t *s_wave, uint32_t &s_big) {
    const int64_t start = tile_starts[seg];
    const int64_t stop = min(seg + 1 == n_segments ? n_isects : (int64_t)tile_starts[seg + 1], n_isects);
    const uint32_t n = stop > start ? (uint32_t)(stop - start) : 0u; // as classified
    // (the direct path's bins and the end marker behind them take the words from s_fine on,
    // across the bucket tables it does not use: see launch_small_segment_sort)
    uint32_t *s_fine = reinterpret_cast<uint32_t *>(lds_staged + lds_words + 4);
    uint32_t *s_first = s_fine + kSortFineBins;   // bucket_cap + 1 words: starts, then the end
    uint32_t *s_cursor = s_first + bucket_cap + 1;
    uint16_t *s_bucket = reinterpret_cast<uint16_t *>(s_cursor + bucket_cap);
    const uint64_t *g = pairs + start;
    int64_t *ids_out = isect_ids + start;
    int32_t *flat_out = flatten_ids + start;
    const uint32_t tid = threadIdx.x, nt = blockDim.x;
    const uint32_t lane = tid & (SPLATAD_WAVE - 1), wave = tid / SPLATAD_WAVE;
    const uint32_t n_waves = nt / SPLATAD_WAVE;
    const uint64_t cam = (seg >> sshift) / n_tiles, tile = (seg >> sshift) % n_tiles;
    const uint64_t key_hi = ((cam << tile_n_bits) | tile) << 32;

    uint64_t held[ER];
#pragma unroll
    for (int k = 0; k < ER; ++k) {
        const uint32_t i = tid + k * nt;
        held[k] = i < n ? g[i] : ~0ull;
    }
    uint32_t lo = 0xFFFFFFFFu, hi = 0u;
#pragma unroll
    for (int k = 0; k < ER; ++k)
        if (tid + k * nt < n) {
            const uint32_t d = (uint32_t)(held[k] >> 32);
            lo = min(lo, d);
            hi = max(hi, d);
        }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        lo = min(lo, (uint32_t)__shfl_xor((int)lo, off, SPLATAD_WAVE));
        hi = max(hi, (uint32_t)__shfl_xor((int)hi, off, SPLATAD_WAVE));
    }
    if (lane == 0) { s_wave[2 * wave] = lo; s_wave[2 * wave + 1] = hi; }
    if (tid == 0) s_big = 0;
    if (tid < 4) lds_staged[n + tid] = ~0ull;
    // Ranks the staged entries inside their buckets (first[b] .. first[b + 1]) and writes the lists.
    auto rank_and_write = [&](const uint32_t *first) {
        for (uint32_t i = tid; i < n; i += nt) {
            const uint64_t p = lds_staged[i];
            const uint32_t b = s_bucket[i];
            const uint32_t s0 = first[b], s1 = first[b + 1];
            uint32_t place = s0;
            if (s1 - s0 > kSortRankMax) {
                place = i; // ordered by the network
            } else {
                for (uint32_t j = s0; j < s1; j += 4) {
                    const uint64_t q0 = lds_staged[j], q1 = lds_staged[j + 1];
                    const uint64_t q2 = lds_staged[j + 2], q3 = lds_staged[j + 3];
                    if (TIES) {
                        place += (q0 < p || (q0 == p && j < i)) ? 1u : 0u;
                        place += (q1 < p || (q1 == p && j + 1 < i)) ? 1u : 0u;
                        place += (q2 < p || (q2 == p && j + 2 < i)) ? 1u : 0u;
                        place += (q3 < p || (q3 == p && j + 3 < i)) ? 1u : 0u;
                    } else {
                        place += (q0 < p ? 1u : 0u) + (q1 < p ? 1u : 0u) + (q2 < p ? 1u : 0u) + (q3 < p ? 1u : 0u);
                    }
                }
            }
            ids_out[place] = (int64_t)(key_hi | (uint64_t)(int64_t)(int32_t)(p >> 32));
            flat_out[place] = (int32_t)(uint32_t)p;
        }
    };

    // Direct path: bins of kSortDirectMean entries on average, linear in the depth; the atomic
    // that counts an entry into its bin also tells the entry's place inside the bin, so one
    // histogram and one scan place every entry.  Taken when no bin holds more than
    // kSortDirectMax entries; segments whose depths cluster take the equalised buckets below.
    uint32_t n_bins = 1;
    while (n_bins < kSortDirectBins && n_bins * kSortDirectMean < n) n_bins <<= 1;
    for (uint32_t f = tid; f < n_bins; f += nt) s_fine[f] = 0;
    __syncthreads();
    for (uint32_t w = 0; w < n_waves; ++w) {
        lo = min(lo, s_wave[2 * w]);
        hi = max(hi, s_wave[2 * w + 1]);
    }
    __syncthreads(); // s_wave is reused by the scans
    if (hi < 0x7F800000u) { // uniform; depths that are positive finite floats: bins linear in the depth
        const float lo_depth = __uint_as_float(lo), range = __uint_as_float(hi) - lo_depth;
        const float bin_scale = range > 0.f ? (float)n_bins / range : 0.f;
        uint32_t where[ER]; // bin, and above it the place inside the bin
#pragma unroll
        for (int k = 0; k < ER; ++k) {
            where[k] = 0;
            if (tid + k * nt < n) {
                const float x = (__uint_as_float((uint32_t)(held[k] >> 32)) - lo_depth) * bin_scale;
                const uint32_t f = min(n_bins - 1, (uint32_t)x);
                where[k] = f | (atomicAdd(&s_fine[f], 1u) << 16);
            }
        }
        __syncthreads();
        block_exclusive_scan(
            n_bins, tid, nt, s_wave, [&](uint32_t f) { return s_fine[f]; },
            [&](uint32_t f, uint32_t before, uint32_t v) {
                s_fine[f] = before;
                if (v > kSortDirectMax) s_big = 2;
            });
        if (s_big != 2) { // uniform
            if (tid == 0) s_fine[n_bins] = n;
#pragma unroll
            for (int k = 0; k < ER; ++k)
                if (tid + k * nt < n) {
                    const uint32_t f = where[k] & 0xFFFFu;
                    const uint32_t at = s_fine[f] + (where[k] >> 16);
                    lds_staged[at] = held[k];
                    s_bucket[at] = (uint16_t)f;
                }
            __syncthreads();
            rank_and_write(s_fine);
            return;
        }
        __syncthreads(); // every lane has read the flag
        if (tid == 0) s_big = 0;
    }

    uint32_t n_fine = 1;
    while (n_fine < kSortFineBins && n_fine * 16 < n) n_fine <<= 1;
    for (uint32_t f = tid; f < n_fine; f += nt) s_fine[f] = 0;
    const float scale = (float)n_fine / ((float)(hi - lo) + 1.f);
    auto fine_pos = [&](uint64_t p, uint32_t &f) -> float {
        const float x = (float)((uint32_t)(p >> 32) - lo) * scale;
        f = min(n_fine - 1, (uint32_t)x);
        return x;
    };
    __syncthreads();

#pragma unroll
    for (int k = 0; k < ER; ++k)
        if (tid + k * nt < n) {
            uint32_t f;
            fine_pos(held[k], f);
            atomicAdd(&s_fine[f], 1u);
        }
    __syncthreads();

    const uint32_t mean = kSortBucketMean;
    const uint32_t nb = block_exclusive_scan(
        n_fine, tid, nt, s_wave,
        [&](uint32_t f) { return (s_fine[f] + mean - 1) / mean; },
        [&](uint32_t f, uint32_t before, uint32_t v) { s_fine[f] = before | (v << 16); });
    for (uint32_t b = tid; b < nb; b += nt) s_cursor[b] = 0;
    __syncthreads();
    uint32_t bucket[ER];
#pragma unroll
    for (int k = 0; k < ER; ++k) {
        bucket[k] = 0;
        if (tid + k * nt < n) {
            uint32_t f;
            const float x = fine_pos(held[k], f);
            const uint32_t packed = s_fine[f];
            const uint32_t c = packed >> 16;
            bucket[k] = (packed & 0xFFFFu) + min(c - 1, (uint32_t)((x - (float)f) * (float)c));
            atomicAdd(&s_cursor[bucket[k]], 1u);
        }
    }
    __syncthreads();
    block_exclusive_scan(
        nb, tid, nt, s_wave, [&](uint32_t b) { return s_cursor[b]; },
        [&](uint32_t b, uint32_t before, uint32_t v) {
            s_cursor[b] = before;
            s_first[b] = before;
            if (v > kSortRankMax) s_big = 1;
        });
    if (tid == 0) s_first[nb] = n;
#pragma unroll
    for (int k = 0; k < ER; ++k)
        if (tid + k * nt < n) {
            const uint32_t at = atomicAdd(&s_cursor[bucket[k]], 1u);
            lds_staged[at] = held[k];
            s_bucket[at] = (uint16_t)bucket[k];
        }
    __syncthreads();

    if (s_big) { // uniform: more than 1024 entries in a bucket, i.e. that many equal depths
        for (uint32_t b = 0; b < nb; ++b) {
            const uint32_t s0 = s_first[b], c = s_first[b + 1] - s0;
            if (c > kSortRankMax) bitonic_sort_ascending(lds_staged + s0, c, tid, nt); // uniform
        }
    }
    rank_and_write(s_first);
}


// The workgroups of a launch share out the segments of one class; a launch has no more
// workgroups than can be resident, so a class without segments costs next to nothing.
// (The lidar's eight-entry instantiation took 82 registers, two more than six resident wavefronts
// per SIMD allow; held to 80 it spills nothing: lidar step 0.367 -> 0.365 ms.)
template <int ER, bool TIES>
__global__ void __attribute__((amdgpu_waves_per_eu(ER == 8 && TIES ? 6 : 1, ER == 8 && TIES ? 6 : 8)))
isect_small_segment_sort_kernel(uint32_t n_segments, uint32_t n_tiles, uint32_t sshift,
                                                uint32_t tile_n_bits, uint32_t lds_words,
                                                uint32_t bucket_cap, int64_t n_isects,
                                                const uint32_t *__restrict__ seg_count,
                                                const uint32_t *__restrict__ seg_list,
                                                const int32_t *__restrict__ tile_starts,
                                                const uint64_t *__restrict__ pairs,
                                                int64_t *__restrict__ isect_ids,
                                                int32_t *__restrict__ flatten_ids) {
    extern __shared__ uint64_t lds_staged[];
    __shared__ uint32_t s_wave[2 * (1024 / SPLATAD_WAVE)];
    __shared__ uint32_t s_big;
    const uint32_t count = *seg_count;
    for (uint32_t k = blockIdx.x; k < count; k += gridDim.x) { // uniform across the workgroup
        sort_segment_small<ER, TIES>(seg_list[k], n_segments, n_tiles, sshift, tile_n_bits, lds_words,
                                     bucket_cap, n_isects, tile_starts, pairs, isect_ids, flatten_ids,
                                     lds_staged, s_wave, s_big);
        __syncthreads(); // the next segment reuses the LDS
    }
}

// ---------------------------------------------------------------------------------------------
// Cameras: the coarse lists are sorted, and the tile lists written in order.
//
// A Gaussian that covers many tiles is one entry of a coarse block's list and up to sixteen
// intersections (6.3 on a 1080p driving frame).  Instead of expanding the coarse lists into
// unordered tile segments and sorting every segment (each such Gaussian sorted sixteen times
// over), a workgroup sorts a piece of a coarse list by (depth bits, flatten id) in LDS and then
// walks the sorted piece once per tile of the block: the entries whose mask names the tile, in
// their sorted order, are the piece's share of the tile's list.  Pieces are runs of consecutive
// depth slabs of one block (the slab is a non-decreasing function of the depth bits, so the
// pieces of a block follow each other in the tile lists as they do in depth); where a piece
// lands in a tile's list follows from the tile's start (the scan of the per-tile counts) plus
// the entries of the block's earlier slabs that name the tile, counted per list and tile
// beforehand.  Coarse blocks differ wildly in length -- a block at the horizon of a driving
// frame holds ten times the average -- which the depth slabs even out: their bounds are
// quantiles of the visible Gaussians' depths.
constexpr uint32_t kBlockSortCap = 10240;   // longest (block, slab) list the LDS sort takes
constexpr uint32_t kBlockMergeCap = 4096;   // slabs of a block are sorted together up to this many entries,
constexpr uint32_t kBlockPairsCap = 32768;  // and about this many intersections
// (a lidar's wide tiles: an entry names four tiles on average where a camera's names six, but its
// lists come out evenly long, and pieces of 4096 entries all fall into one class whose single
// launch then lasts 100 us: sweep intersection 0.254 ms with the camera's caps, 0.226 with these,
// 0.238 with the per-tile segment sort)
constexpr uint32_t kBlockMergeCapLidar = 2048, kBlockPairsCapLidar = 12288;
static_assert(kBlockMergeCap <= 4096 && kBlockMergeCapLidar <= 4096, "classes beyond 4096 entries hold single lists only: the host skips their launches by the longest list");
constexpr uint32_t kBlockLongMax = 8 * kBlockSortCap; // longest list the block sort takes at all (in parts)
// Calls with fewer intersections sort on one stream (measured: camera frames of 0.85 / 1.9 / 3.4 /
// 8.3M intersections take 0.21 / 0.236 / 0.284 / 0.306 ms that way against 0.21 / 0.258 / 0.305 /
// 0.31 with the helper streams, a sweep of 1.9M 0.265 against 0.31; the frame of 16.1M needs them)
constexpr int64_t kOneStreamIsects = 1 << 23;
constexpr int kBlockClasses = 6;            // five by length, and the lists beyond kBlockSortCap
constexpr int kBlockLongClass = 5;
__constant__ const uint32_t kBlockClassMax[kBlockClasses] = {512u, 2048u, 4096u, 8192u, kBlockSortCap, 0xFFFFFFFFu};

// Dynamic LDS of the block sort: the staging array and its four end markers, the masks and
// bucket numbers of the staged entries, the fine bins and two bucket tables.
__host__ __device__ inline size_t block_sort_lds_bytes(uint32_t lds_words, uint32_t bucket_cap) {
    return ((size_t)lds_words + 4) * 8 + (kSortFineBins + 2 * (size_t)bucket_cap + 1) * 4 +
           2 * (((size_t)lds_words * 2 + 7) & ~(size_t)7);
}

// Counts, for every (block, slab) list, the entries that name each of the block's sixteen tiles:
// counts[list * 16 + t], zero beforehand.  A wavefront takes 64 consecutive entries; those of
// one list (nearly always all of them) are counted with a ballot per tile and added with one
// atomic instruction of sixteen lanes.  The lists being short, no counter sees many atomics.
__global__ void __launch_bounds__(SPLATAD_THREADS)
isect_list_count_kernel(const int64_t *__restrict__ n_entries_ptr, const uint4 *__restrict__ entries,
                        int32_t *__restrict__ counts) {
    const int64_t n_entries = *n_entries_ptr;
    const uint32_t lane = threadIdx.x & (SPLATAD_WAVE - 1);
    const int64_t wave_id = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / SPLATAD_WAVE;
    const int64_t n_waves = (int64_t)gridDim.x * blockDim.x / SPLATAD_WAVE;
    for (int64_t e0 = wave_id * SPLATAD_WAVE; e0 < n_entries; e0 += n_waves * SPLATAD_WAVE) { // uniform per wavefront
        const bool has = e0 + lane < n_entries;
        const uint4 rec = has ? entries[e0 + lane] : make_uint4(0u, 0u, 0xFFFFFFFFu, 0u);
        uint64_t todo = __ballot(has);
        while (todo) {
            const int leader = __ffsll((unsigned long long)todo) - 1;
            const uint32_t list = (uint32_t)__shfl((int)rec.z, leader, SPLATAD_WAVE);
            const bool in = has && rec.z == list;
            todo &= ~__ballot(in);
            const uint32_t mask = in ? rec.w : 0u;
            uint32_t cnt = 0;
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const uint32_t n_hits = (uint32_t)__popcll(__ballot((mask >> t) & 1u)); // uniform
                asm("v_writelane_b32 %0, %1, %2" : "+v"(cnt) : "s"(n_hits), "n"(t));
            }
            if (lane < 16 && cnt) atomicAdd(&counts[(size_t)list * 16 + lane], (int32_t)cnt);
        }
    }
}

// A lane per tile: adds up the tile's counts over the slab lists of its block (the tile's number
// of intersections, which the scan behind this kernel turns into the tile's start) and leaves in
// their place the counts of the slabs before each (where a slab's entries start inside the
// tile's list).  Sixteen consecutive lanes take the sixteen tiles of one block, so that every
// load and store of a wavefront is four whole 64-byte rows of the counter table.
__global__ void __launch_bounds__(SPLATAD_THREADS)
isect_tile_totals_kernel(CoarseGrid cg, uint32_t tile_w, uint32_t tile_h, uint32_t bsshift, uint32_t n_blocks,
                         int32_t *__restrict__ counts, int32_t *__restrict__ tile_counts) {
    const uint32_t id = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t block = id >> 4, t = id & 15u;
    if (block >= n_blocks) return;
    const uint32_t per_cam = cg.cw * cg.ch, cam = block / per_cam, r = block - cam * per_cam;
    const uint32_t by = r / cg.cw, bx = r - by * cg.cw;
    const uint32_t x = (bx << 2) + (t & 3u), y = (by << kCoarseRowShift) + (t >> 2);
    if (x >= tile_w || y >= tile_h) return; // (a tile beyond the grid's edge: its counters stay zero)
    int32_t *mine = counts + ((size_t)block << bsshift) * 16 + t;
    const uint32_t slabs = 1u << bsshift;
    int32_t c[1u << kSlabShiftMax];
#pragma unroll
    for (uint32_t sl = 0; sl < (1u << kSlabShiftMax); ++sl) c[sl] = sl < slabs ? mine[(size_t)sl * 16] : 0;
    int32_t run = 0;
#pragma unroll
    for (uint32_t sl = 0; sl < (1u << kSlabShiftMax); ++sl) {
        if (sl < slabs) mine[(size_t)sl * 16] = run;
        run += c[sl];
    }
    tile_counts[cam * tile_w * tile_h + y * tile_w + x] = run;
}

// First workgroup: cuts every block's slab lists into pieces {first entry, entries, block, first
// list}, a piece being as many consecutive slabs as stay within kBlockMergeCap entries (fewer
// where the entries meet many tiles each, so that a piece writes about kBlockPairsCap
// intersections at most; a single slab's list beyond that is a piece of its own), and lists the
// pieces by size class: class c's are pieces[c * max_pieces ..] , class_count[c] of them.  The
// other workgroups scan the tile counts into the tiles' starts (seg_starts) and the tile
// offsets: each takes a stretch of the tiles and adds up, for itself, the counts of all tiles
// before it (a few thousand to some ten thousand words from L2: cheaper than a scan launch in
// the chain of dependent kernels).
__global__ void __launch_bounds__(1024)
isect_block_plan_kernel(uint32_t n_blocks, uint32_t bsshift, const int32_t *__restrict__ totals,
                        const uint32_t *__restrict__ list_starts, const int32_t *__restrict__ tile_counts,
                        CoarseGrid cg, uint32_t tile_w, uint32_t tile_h, uint32_t n_segments,
                        int32_t *__restrict__ seg_starts, int32_t *__restrict__ tile_offsets,
                        uint32_t *__restrict__ class_count, uint32_t max_pieces,
                        uint4 *__restrict__ pieces, uint32_t merge_cap, uint32_t pairs_cap) {
    const uint32_t tid = threadIdx.x, nt = blockDim.x, lane = tid & (SPLATAD_WAVE - 1);
    if (blockIdx.x != 0) { // uniform across the workgroup
        __shared__ uint32_t s_wave[1024 / SPLATAD_WAVE];
        const uint32_t workers = gridDim.x - 1, wave = tid / SPLATAD_WAVE, n_waves = nt / SPLATAD_WAVE;
        const uint32_t per = ((n_segments + workers - 1) / workers + nt - 1) / nt * nt; // whole rounds of the workgroup
        const uint32_t lo = min(n_segments, (blockIdx.x - 1) * per), hi = min(n_segments, lo + per);
        if (lo >= hi) return;
        // the counts before the stretch (lo is a multiple of the workgroup size: whole int4)
        uint32_t sum = 0;
        const int4 *counts4 = reinterpret_cast<const int4 *>(tile_counts);
        for (uint32_t i = tid; i < lo / 4; i += nt) {
            const int4 v = counts4[i];
            sum += (uint32_t)(v.x + v.y + v.z + v.w);
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, SPLATAD_WAVE);
        if (lane == 0) s_wave[wave] = sum;
        __syncthreads();
        uint32_t before = 0;
        for (uint32_t k = 0; k < n_waves; ++k) before += s_wave[k];
        for (uint32_t s0 = lo; s0 < hi; s0 += nt) { // uniform
            const uint32_t seg = s0 + tid;
            const uint32_t mine = seg < hi ? (uint32_t)tile_counts[seg] : 0u;
            uint32_t incl = mine;
#pragma unroll
            for (int off = 1; off < SPLATAD_WAVE; off <<= 1) {
                const uint32_t up = __shfl_up(incl, off, SPLATAD_WAVE);
                if (lane >= (uint32_t)off) incl += up;
            }
            __syncthreads(); // the totals of the round before have been read
            if (lane == SPLATAD_WAVE - 1) s_wave[wave] = incl;
            __syncthreads();
            uint32_t waves_before = 0, round = 0;
            for (uint32_t k = 0; k < n_waves; ++k) {
                const uint32_t v = s_wave[k];
                if (k < wave) waves_before += v;
                round += v;
            }
            if (seg < hi) {
                const int32_t start = (int32_t)(before + waves_before + incl - mine);
                seg_starts[seg] = start;
                if (tile_offsets != nullptr) tile_offsets[seg] = start;
            }
            before += round;
        }
        return;
    }
    __shared__ uint32_t s_count[kBlockClasses];
    if (tid < kBlockClasses) s_count[tid] = 0;
    __syncthreads();
    const uint32_t slabs = 1u << bsshift;
    for (uint32_t b = tid; b < n_blocks; b += nt) {
        const uint32_t list0 = b << bsshift;
        // everything the block needs is requested before any of it is used
        uint32_t v[1u << kSlabShiftMax];
        if (slabs >= 4) { // the block's totals are whole, aligned int4
            const int4 *totals4 = reinterpret_cast<const int4 *>(totals + list0);
#pragma unroll
            for (uint32_t q = 0; q < (1u << kSlabShiftMax) / 4; ++q) {
                const int4 t = 4 * q < slabs ? totals4[q] : make_int4(0, 0, 0, 0);
                v[4 * q] = (uint32_t)t.x; v[4 * q + 1] = (uint32_t)t.y; v[4 * q + 2] = (uint32_t)t.z; v[4 * q + 3] = (uint32_t)t.w;
            }
        } else {
#pragma unroll
            for (uint32_t sl = 0; sl < (1u << kSlabShiftMax); ++sl) v[sl] = sl < slabs ? (uint32_t)totals[list0 + sl] : 0u;
        }
        const uint32_t block_first = list_starts[list0];
        // the block's intersections: its tiles' counts (copies == 1 here: one counter per tile)
        uint32_t in_tiles[16];
        {
            const uint32_t per_cam = cg.cw * cg.ch, cam = b / per_cam, r = b - cam * per_cam;
            const uint32_t by = r / cg.cw, bx = r - by * cg.cw;
#pragma unroll
            for (uint32_t t = 0; t < 16; ++t) {
                const uint32_t x = (bx << 2) + (t & 3u), y = (by << kCoarseRowShift) + (t >> 2);
                in_tiles[t] = x < tile_w && y < tile_h ? (uint32_t)tile_counts[cam * tile_w * tile_h + y * tile_w + x] : 0u;
            }
        }
        uint64_t pairs = 0;
#pragma unroll
        for (uint32_t t = 0; t < 16; ++t) pairs += in_tiles[t];
        uint32_t block_n = 0;
#pragma unroll
        for (uint32_t sl = 0; sl < (1u << kSlabShiftMax); ++sl) block_n += v[sl];
        if (block_n == 0) continue;
        uint32_t cap = merge_cap;
        if (pairs * cap > (uint64_t)pairs_cap * block_n)
            cap = max(512u, (uint32_t)((uint64_t)pairs_cap * block_n / pairs));
        uint32_t piece_first = block_first, piece_n = 0, piece_list = list0;
        auto emit = [&](uint32_t next_list) {
            if (piece_n != 0) {
                int c = 0;
                while (c + 1 < kBlockClasses && piece_n > kBlockClassMax[c]) ++c;
                const uint32_t k = atomicAdd(&s_count[c], 1u);
                pieces[(size_t)c * max_pieces + k] = make_uint4(piece_first, piece_n, b, piece_list);
                piece_first += piece_n;
                piece_n = 0;
            }
            piece_list = next_list;
        };
#pragma unroll
        for (uint32_t sl = 0; sl < (1u << kSlabShiftMax); ++sl) {
            if (sl < slabs) {
                if (piece_n != 0 && piece_n + v[sl] > cap) emit(list0 + sl);
                if (piece_n == 0) piece_list = list0 + sl;
                piece_n += v[sl];
            }
        }
        emit(0u);
    }
    __syncthreads();
    if (tid < kBlockClasses) class_count[tid] = s_count[tid];
}

// Sorts one piece (n <= ER * blockDim.x entries, n <= lds_words) in LDS -- sort_segment_small's
// method, with the tile masks travelling beside the keys -- and writes its share of the lists
// of the block's sixteen tiles.
template <int ER, bool TIES>
__device__ __forceinline__ void sort_expand_piece(uint4 piece, CoarseGrid cg, uint32_t tile_w, uint32_t tile_h,
                                                  uint32_t n_tiles, uint32_t tile_n_bits, uint32_t lds_words,
                                                  uint32_t bucket_cap, int64_t n_isects,
                                                  const uint4 *__restrict__ entries,
                                                  const int32_t *__restrict__ seg_starts,
                                                  const int32_t *__restrict__ slabs_before,
                                                  int64_t *__restrict__ isect_ids,
                                                  int32_t *__restrict__ flatten_ids,
                                                  uint64_t *lds_staged, uint32_t *s_wave, uint32_t &s_big,
                                                  uint32_t (*s_cnt)[16], bool gathered = false,
                                                  uint32_t n_gathered = 0, uint32_t *carried = nullptr) {
    // gathered: the piece is the first n_gathered entries of the staging array and their masks (a
    // part of a long list, see sort_expand_long_list); *carried (lane t < 16) then holds the
    // entries of the list's nearer parts and of the block's earlier slabs that name tile t, and
    // takes this part's on top
    const uint32_t n = gathered ? n_gathered : piece.y;
    uint32_t *s_fine = reinterpret_cast<uint32_t *>(lds_staged + lds_words + 4);
    uint32_t *s_first = s_fine + kSortFineBins;   // bucket_cap + 1 words: starts, then the end
    uint32_t *s_cursor = s_first + bucket_cap + 1;
    uint16_t *s_bucket = reinterpret_cast<uint16_t *>(s_cursor + bucket_cap);
    uint16_t *s_mask = s_bucket + ((lds_words + 3) & ~3u);
    const uint4 *g = entries + piece.x;
    const uint32_t tid = threadIdx.x, nt = blockDim.x;
    const uint32_t lane = tid & (SPLATAD_WAVE - 1), wave = tid / SPLATAD_WAVE;
    const uint32_t n_waves = nt / SPLATAD_WAVE;

    uint64_t held[ER];
    uint32_t held_mask[ER];
    uint32_t pre; // lane t < 16: the entries of the block's earlier slabs that name tile t
    if (gathered) { // uniform
#pragma unroll
        for (int k = 0; k < ER; ++k) {
            const uint32_t i = tid + k * nt;
            held[k] = i < n ? lds_staged[i] : ~0ull;
            held_mask[k] = i < n ? (uint32_t)s_mask[i] : 0u;
        }
        pre = *carried;
        __syncthreads(); // the staging array is free for the sort
    } else {
#pragma unroll
        for (int k = 0; k < ER; ++k) {
            const uint32_t i = tid + k * nt;
            const uint4 e = i < n ? g[i] : make_uint4(~0u, ~0u, 0u, 0u);
            held[k] = ((uint64_t)e.y << 32) | (uint64_t)e.x;
            held_mask[k] = e.w;
        }
        pre = lane < 16 ? (uint32_t)slabs_before[(size_t)piece.w * 16 + lane] : 0u;
    }
    auto count16 = [&](uint32_t mask) -> uint32_t {
        uint32_t cnt = 0;
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const uint32_t n_hits = (uint32_t)__popcll(__ballot((mask >> t) & 1u)); // uniform
            asm("v_writelane_b32 %0, %1, %2" : "+v"(cnt) : "s"(n_hits), "n"(t));
        }
        return cnt;
    };
    uint32_t lo = 0xFFFFFFFFu, hi = 0u, id_lo = 0xFFFFFFFFu, id_hi = 0u;
#pragma unroll
    for (int k = 0; k < ER; ++k)
        if (tid + k * nt < n) {
            const uint32_t d = (uint32_t)(held[k] >> 32), id = (uint32_t)held[k];
            lo = min(lo, d);
            hi = max(hi, d);
            id_lo = min(id_lo, id);
            id_hi = max(id_hi, id);
        }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        lo = min(lo, (uint32_t)__shfl_xor((int)lo, off, SPLATAD_WAVE));
        hi = max(hi, (uint32_t)__shfl_xor((int)hi, off, SPLATAD_WAVE));
        id_lo = min(id_lo, (uint32_t)__shfl_xor((int)id_lo, off, SPLATAD_WAVE));
        id_hi = max(id_hi, (uint32_t)__shfl_xor((int)id_hi, off, SPLATAD_WAVE));
    }
    if (lane == 0) {
        s_wave[4 * wave] = lo; s_wave[4 * wave + 1] = hi;
        s_wave[4 * wave + 2] = id_lo; s_wave[4 * wave + 3] = id_hi;
    }
    if (tid == 0) s_big = 0;
    if (tid < 4) lds_staged[n + tid] = ~0ull;

    // Places of the staged entries: an entry's bucket is first[b] .. first[b + 1], its place the
    // bucket's start plus the bucket's smaller keys.  The keys (depth bits, flatten id) of a
    // coarse list are distinct.  Kept in registers (with the mask above the place), for the
    // staging array is where the sorted piece goes.
    uint64_t placed[ER];
    uint32_t place_mask[ER];
    auto rank_all = [&](const uint32_t *first) {
#pragma unroll
        for (int k = 0; k < ER; ++k) {
            const uint32_t i = tid + k * nt;
            placed[k] = 0;
            place_mask[k] = 0;
            if (i < n) {
                const uint64_t p = lds_staged[i];
                const uint32_t b = s_bucket[i];
                const uint32_t s0 = first[b], s1 = first[b + 1];
                uint32_t place = s0;
                for (uint32_t j = s0; j < s1; j += 4) {
                    const uint64_t q0 = lds_staged[j], q1 = lds_staged[j + 1];
                    const uint64_t q2 = lds_staged[j + 2], q3 = lds_staged[j + 3];
                    if constexpr (TIES)
                        place += (q0 < p || (q0 == p && j < i) ? 1u : 0u) + (q1 < p || (q1 == p && j + 1 < i) ? 1u : 0u) +
                                 (q2 < p || (q2 == p && j + 2 < i) ? 1u : 0u) + (q3 < p || (q3 == p && j + 3 < i) ? 1u : 0u);
                    else
                        place += (q0 < p ? 1u : 0u) + (q1 < p ? 1u : 0u) + (q2 < p ? 1u : 0u) + (q3 < p ? 1u : 0u);
                }
                placed[k] = p;
                place_mask[k] = place | ((uint32_t)s_mask[i] << 16);
            }
        }
    };

    uint32_t n_bins = 1;
    while (n_bins < kSortDirectBins && n_bins * kSortDirectMean < n) n_bins <<= 1;
    for (uint32_t f = tid; f < n_bins; f += nt) s_fine[f] = 0;
    __syncthreads();
    for (uint32_t w = 0; w < n_waves; ++w) {
        lo = min(lo, s_wave[4 * w]);
        hi = max(hi, s_wave[4 * w + 1]);
        id_lo = min(id_lo, s_wave[4 * w + 2]);
        id_hi = max(id_hi, s_wave[4 * w + 3]);
    }
    __syncthreads(); // s_wave is reused by the scans
    bool ranked = false;
    if (hi < 0x7F800000u) { // uniform; depths that are positive finite floats
        // Direct path, as in sort_segment_small: bins linear in the depth, and the atomic that
        // counts an entry into its bin tells its place inside the bin.  A piece whose depths are
        // all equal (a wall that faces the camera) is ordered by the flatten ids alone: bins
        // linear in the id.
        const bool by_id = hi == lo;
        const float lo_depth = __uint_as_float(lo), range = __uint_as_float(hi) - lo_depth;
        const float bin_scale = by_id ? (float)n_bins / ((float)(id_hi - id_lo) + 1.f)
                                      : (float)n_bins / range;
        uint32_t where[ER]; // bin, and above it the place inside the bin
#pragma unroll
        for (int k = 0; k < ER; ++k) {
            where[k] = 0;
            if (tid + k * nt < n) {
                const float x = by_id ? (float)((uint32_t)held[k] - id_lo) * bin_scale
                                      : (__uint_as_float((uint32_t)(held[k] >> 32)) - lo_depth) * bin_scale;
                const uint32_t f = min(n_bins - 1, (uint32_t)x);
                where[k] = f | (atomicAdd(&s_fine[f], 1u) << 16);
            }
        }
        __syncthreads();
        block_exclusive_scan(
            n_bins, tid, nt, s_wave, [&](uint32_t f) { return s_fine[f]; },
            [&](uint32_t f, uint32_t before, uint32_t v) {
                s_fine[f] = before;
                if (v > kSortDirectMax) s_big = 2;
            });
        if (s_big != 2) { // uniform
            if (tid == 0) s_fine[n_bins] = n;
#pragma unroll
            for (int k = 0; k < ER; ++k)
                if (tid + k * nt < n) {
                    const uint32_t f = where[k] & 0xFFFFu;
                    const uint32_t at = s_fine[f] + (where[k] >> 16);
                    lds_staged[at] = held[k];
                    s_bucket[at] = (uint16_t)f;
                    s_mask[at] = (uint16_t)held_mask[k];
                }
            __syncthreads();
            rank_all(s_fine);
            ranked = true;
        } else {
            __syncthreads(); // every lane has read the flag
            if (tid == 0) s_big = 0;
        }
    }
    if (!ranked) { // uniform: buckets equalised over the depth bits, as in sort_segment_small
        uint32_t n_fine = 1;
        while (n_fine < kSortFineBins && n_fine * 16 < n) n_fine <<= 1;
        for (uint32_t f = tid; f < n_fine; f += nt) s_fine[f] = 0;
        const float scale = (float)n_fine / ((float)(hi - lo) + 1.f);
        auto fine_pos = [&](uint64_t p, uint32_t &f) -> float {
            const float x = (float)((uint32_t)(p >> 32) - lo) * scale;
            f = min(n_fine - 1, (uint32_t)x);
            return x;
        };
        __syncthreads();
#pragma unroll
        for (int k = 0; k < ER; ++k)
            if (tid + k * nt < n) {
                uint32_t f;
                fine_pos(held[k], f);
                atomicAdd(&s_fine[f], 1u);
            }
        __syncthreads();
        const uint32_t mean = kSortBucketMean;
        const uint32_t nb = block_exclusive_scan(
            n_fine, tid, nt, s_wave,
            [&](uint32_t f) { return (s_fine[f] + mean - 1) / mean; },
            [&](uint32_t f, uint32_t before, uint32_t v) { s_fine[f] = before | (v << 16); });
        for (uint32_t b = tid; b < nb; b += nt) s_cursor[b] = 0;
        __syncthreads();
        uint32_t bucket[ER];
#pragma unroll
        for (int k = 0; k < ER; ++k) {
            bucket[k] = 0;
            if (tid + k * nt < n) {
                uint32_t f;
                const float x = fine_pos(held[k], f);
                const uint32_t packed = s_fine[f];
                const uint32_t c = packed >> 16;
                bucket[k] = (packed & 0xFFFFu) + min(c - 1, (uint32_t)((x - (float)f) * (float)c));
                atomicAdd(&s_cursor[bucket[k]], 1u);
            }
        }
        __syncthreads();
        block_exclusive_scan(
            nb, tid, nt, s_wave, [&](uint32_t b) { return s_cursor[b]; },
            [&](uint32_t b, uint32_t before, uint32_t) {
                s_cursor[b] = before;
                s_first[b] = before;
            });
        if (tid == 0) s_first[nb] = n;
#pragma unroll
        for (int k = 0; k < ER; ++k)
            if (tid + k * nt < n) {
                const uint32_t at = atomicAdd(&s_cursor[bucket[k]], 1u);
                lds_staged[at] = held[k];
                s_bucket[at] = (uint16_t)bucket[k];
                s_mask[at] = (uint16_t)held_mask[k];
            }
        __syncthreads();
        // (a bucket of many equal depths is ranked like any other: every entry counts the
        // bucket's smaller keys)
        rank_all(s_first);
    }
    __syncthreads(); // every place is known: the staging array takes the sorted piece
#pragma unroll
    for (int k = 0; k < ER; ++k)
        if (tid + k * nt < n) {
            const uint32_t place = place_mask[k] & 0xFFFFu;
            lds_staged[place] = placed[k];
            s_mask[place] = (uint16_t)(place_mask[k] >> 16);
        }
    __syncthreads();

    // The sorted piece, tile by tile.  A wavefront takes consecutive chunks of 64 entries; it
    // counts its chunks' entries per tile, learns from the other wavefronts' counts where its
    // first chunk starts in every tile's list, and writes.
    const uint32_t n_chunks = (n + SPLATAD_WAVE - 1) / SPLATAD_WAVE, per_wave = (n_chunks + n_waves - 1) / n_waves;
    const uint32_t c0 = min(n_chunks, wave * per_wave), c1 = min(n_chunks, c0 + per_wave);
    uint32_t mine = 0;
    for (uint32_t c = c0; c < c1; ++c) { // uniform per wavefront
        const uint32_t i = c * SPLATAD_WAVE + lane;
        mine += count16(i < n ? (uint32_t)s_mask[i] : 0u);
    }
    if (lane < 16) s_cnt[wave][lane] = mine;
    __syncthreads();
    uint32_t base = 0, tile_key = 0;
    if (lane < 16) {
        const uint32_t per_cam = cg.cw * cg.ch;
        const uint32_t cam = piece.z / per_cam, r = piece.z - cam * per_cam;
        const uint32_t by = r / cg.cw, bx = r - by * cg.cw;
        const uint32_t x = (bx << 2) + (lane & 3u), y = (by << kCoarseRowShift) + (lane >> 2);
        if (x < tile_w && y < tile_h) { // (a tile beyond the grid's edge is in no mask)
            const uint32_t tile = y * tile_w + x;
            base = (uint32_t)seg_starts[cam * n_tiles + tile];
            tile_key = (cam << tile_n_bits) | tile;
        }
        base += pre;
        for (uint32_t w = 0; w < wave; ++w) base += s_cnt[w][lane];
    }
    // Where the wavefront's next entry of every tile goes, and the tiles' keys, are the same for all
    // lanes: kept in scalar registers from here on.
    uint32_t next_of[16], key_of[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        next_of[t] = (uint32_t)__builtin_amdgcn_readlane((int)base, t);
        key_of[t] = (uint32_t)__builtin_amdgcn_readlane((int)tile_key, t);
    }
    const uint32_t cap = (uint32_t)n_isects; // below 2^31; keeps a caller's mismatch inside the lists
    for (uint32_t c = c0; c < c1; ++c) { // uniform per wavefront
        const uint32_t i = c * SPLATAD_WAVE + lane;
        const uint64_t p = i < n ? lds_staged[i] : 0ull;
        const uint32_t mask = i < n ? (uint32_t)s_mask[i] : 0u;
        const uint32_t depth = (uint32_t)(p >> 32);
        const uint32_t depth_sign = (uint32_t)((int32_t)depth >> 31);
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const bool named = (mask >> t) & 1u;
            const uint64_t hits = wave_ballot(named);
            if (hits == 0) continue; // uniform
            const uint32_t first = next_of[t];
            next_of[t] = first + (uint32_t)__popcll(hits);
            if (next_of[t] > cap) continue; // uniform: the caller's lists end before this run does
            if (wave_lanes(hits)) { // (the lanes that name the tile, from the mask at hand)
                const uint32_t at = __builtin_amdgcn_mbcnt_hi((uint32_t)(hits >> 32),
                                                              __builtin_amdgcn_mbcnt_lo((uint32_t)hits, first));
                // the key as the reference forms it: the depth bits sign-extended below the tile
                isect_ids[at] = (int64_t)(((uint64_t)(key_of[t] | depth_sign) << 32) | (uint64_t)depth);
                flatten_ids[at] = (int32_t)(uint32_t)p;
            }
        }
    }
    if (gathered) { // uniform: what this part added to the tiles' lists
        uint32_t total = pre;
        if (lane < 16)
            for (uint32_t w = 0; w < n_waves; ++w) total += s_cnt[w][lane];
        *carried = total;
    }
}

// A list too long for the LDS sort, by one workgroup, part by part in ascending key order.  The
// key intervals still to do are kept on a small stack (nearest on top).  An interval of up to
// lds_words entries is gathered from the list into the staging array (in any order), sorted and
// written like any piece, and the tiles' cursors move on by what it wrote; a longer interval is
// cut in two: a histogram of its keys (depth bits above flatten id, as one 64-bit number) over
// kLongBins bins that are linear between its smallest and largest key, with every bin's
// smallest and largest key beside the count, tells its nearest part and the rest.  The keys of
// a coarse list are distinct, so an interval that still holds too much spans more keys than
// bins, both halves of a cut are smaller than the interval, and the stack stays a few entries
// deep (every level of cutting divides the span of the keys by kLongBins).
constexpr uint32_t kLongBins = 2048;
constexpr uint32_t kLongStack = 32;
struct LongInterval { uint64_t lo, hi; uint32_t n, pad; };

template <int ER, bool TIES>
__device__ __forceinline__ void sort_expand_long_list(uint4 piece, CoarseGrid cg, uint32_t tile_w, uint32_t tile_h,
                                                      uint32_t n_tiles, uint32_t tile_n_bits, uint32_t lds_words,
                                                      uint32_t bucket_cap, int64_t n_isects,
                                                      const uint4 *__restrict__ entries,
                                                      const int32_t *__restrict__ seg_starts,
                                                      const int32_t *__restrict__ slabs_before,
                                                      int64_t *__restrict__ isect_ids,
                                                      int32_t *__restrict__ flatten_ids, uint64_t *lds_staged,
                                                      uint32_t *s_wave, uint32_t &s_big, uint32_t (*s_cnt)[16],
                                                      LongInterval *s_stack, uint32_t &s_top, uint32_t &s_kept,
                                                      unsigned long long *s_range) {
    const uint32_t tid = threadIdx.x, nt = blockDim.x, lane = tid & (SPLATAD_WAVE - 1);
    const uint4 *g = entries + piece.x;
    const uint32_t n_all = piece.y;
    uint16_t *s_mask;
    {
        uint32_t *s_fine = reinterpret_cast<uint32_t *>(lds_staged + lds_words + 4);
        uint32_t *s_cursor = s_fine + kSortFineBins + bucket_cap + 1;
        s_mask = reinterpret_cast<uint16_t *>(s_cursor + bucket_cap) + ((lds_words + 3) & ~3u);
    }
    // the histogram of an interval lies over the staging array, which is idle meanwhile
    unsigned long long *h_lo = reinterpret_cast<unsigned long long *>(lds_staged);
    unsigned long long *h_hi = h_lo + kLongBins;
    uint32_t *h_n = reinterpret_cast<uint32_t *>(h_hi + kLongBins);
    uint32_t *h_group = h_n + kLongBins; // a bin's sub-interval
    // smallest and largest key of the list
    {
        unsigned long long lo = ~0ull, hi = 0ull;
        for (uint32_t j = tid; j < n_all; j += nt) {
            const uint4 e = g[j];
            const unsigned long long key = ((unsigned long long)e.y << 32) | e.x;
            lo = min(lo, key);
            hi = max(hi, key);
        }
        if (tid == 0) { s_range[0] = ~0ull; s_range[1] = 0ull; }
        __syncthreads();
        if (lo <= hi) { atomicMin(&s_range[0], lo); atomicMax(&s_range[1], hi); }
        __syncthreads();
        if (tid == 0) {
            s_stack[0].lo = s_range[0]; s_stack[0].hi = s_range[1]; s_stack[0].n = n_all;
            s_top = 1;
        }
    }
    uint32_t carried = lane < 16 ? (uint32_t)slabs_before[(size_t)piece.w * 16 + lane] : 0u;
    for (;;) {
        __syncthreads();
        if (s_top == 0) break; // uniform
        const LongInterval cur = s_stack[s_top - 1];
        __syncthreads();
        if (tid == 0) { s_top -= 1; s_kept = 0; }
        if (cur.n <= lds_words) { // uniform: gather, sort, write
            __syncthreads();
            for (uint32_t j0 = (tid & ~(SPLATAD_WAVE - 1u)); j0 < n_all; j0 += 4 * nt) { // uniform per wavefront
                uint4 e[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t j = j0 + u * nt + lane;
                    e[u] = j < n_all ? g[j] : make_uint4(0u, 0u, 0u, 0u);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t j = j0 + u * nt + lane;
                    const unsigned long long key = ((unsigned long long)e[u].y << 32) | e[u].x;
                    const bool mine = j < n_all && key >= cur.lo && key <= cur.hi;
                    const uint64_t keep = __ballot(mine);
                    if (keep != 0) { // uniform
                        uint32_t at = 0;
                        const int leader = __ffsll((unsigned long long)keep) - 1;
                        if ((int)lane == leader) at = atomicAdd(&s_kept, (uint32_t)__popcll(keep));
                        at = (uint32_t)__shfl((int)at, leader, SPLATAD_WAVE) +
                             (uint32_t)__popcll(keep & ((1ull << lane) - 1ull));
                        if (mine && at < lds_words) { // (the interval's count says it fits)
                            lds_staged[at] = key;
                            s_mask[at] = (uint16_t)e[u].w;
                        }
                    }
                }
            }
            __syncthreads();
            sort_expand_piece<ER, TIES>(piece, cg, tile_w, tile_h, n_tiles, tile_n_bits, lds_words, bucket_cap, n_isects,
                                  entries, seg_starts, slabs_before, isect_ids, flatten_ids, lds_staged, s_wave,
                                  s_big, s_cnt, true, min(s_kept, lds_words), &carried);
            continue;
        }
        // cut the interval
        for (uint32_t f = tid; f < kLongBins; f += nt) { h_lo[f] = ~0ull; h_hi[f] = 0ull; h_n[f] = 0; }
        const float scale = (float)kLongBins / ((float)(cur.hi - cur.lo) + 1.f);
        __syncthreads();
        for (uint32_t j = tid; j < n_all; j += nt) {
            const uint4 e = g[j];
            const unsigned long long key = ((unsigned long long)e.y << 32) | e.x;
            if (key < cur.lo || key > cur.hi) continue;
            const uint32_t f = min(kLongBins - 1u, (uint32_t)((float)(key - cur.lo) * scale));
            atomicAdd(&h_n[f], 1u);
            atomicMin(&h_lo[f], key);
            atomicMax(&h_hi[f], key);
        }
        __syncthreads();
        // The nearest part: the leading bins that together fit the staging array, up to the first
        // bin of more than half of it -- or that bin alone, if it comes first, to be cut again
        // (its keys span less than this interval's: the smallest and the largest key of an
        // interval lie in its first and last bin).  The part and, under it, the rest of the
        // interval take the interval's place on the stack.
        const uint32_t half = lds_words / 2;
        if (tid == 0) { s_range[0] = ~0ull; s_range[1] = 0ull; s_kept = 0; s_big = kLongBins; }
        block_exclusive_scan(
            kLongBins, tid, nt, s_wave, [&](uint32_t f) { return h_n[f]; },
            [&](uint32_t f, uint32_t before, uint32_t c) {
                h_group[f] = before;
                if (c > half) atomicMin(&s_big, f);
            });
        const uint32_t first_big = s_big;
        __syncthreads();
        for (uint32_t f = tid; f < kLongBins; f += nt) {
            const uint32_t c = h_n[f];
            if (c == 0) continue;
            const bool leads = h_group[f] == 0; // the first bin that holds anything
            const bool in_part = leads || (f < first_big && h_group[f] + c <= lds_words);
            if (in_part) {
                atomicAdd(&s_kept, c);
                atomicMax(&s_range[1], h_hi[f]); // the part ends at its largest key
            } else {
                atomicMin(&s_range[0], h_lo[f]); // the rest begins at its smallest
            }
        }
        __syncthreads();
        if (tid == 0) {
            uint32_t top = s_top;
            const uint32_t n_part = s_kept;
            if (cur.n > n_part) { s_stack[top].lo = s_range[0]; s_stack[top].hi = cur.hi; s_stack[top].n = cur.n - n_part; ++top; }
            s_stack[top].lo = cur.lo; s_stack[top].hi = s_range[1]; s_stack[top].n = n_part; ++top;
            s_top = top;
        }
    }
}

// LONG: the launch takes the lists beyond the capacity of the LDS sort, part by part.
template <int ER, bool TIES, bool LONG = false>
__global__ void isect_block_sort_kernel(CoarseGrid cg, uint32_t tile_w, uint32_t tile_h, uint32_t n_tiles,
                                        uint32_t tile_n_bits, uint32_t lds_words, uint32_t bucket_cap,
                                        int64_t n_isects, const uint32_t *__restrict__ class_count,
                                        const uint4 *__restrict__ pieces, const uint4 *__restrict__ entries,
                                        const int32_t *__restrict__ seg_starts,
                                        const int32_t *__restrict__ slabs_before,
                                        int64_t *__restrict__ isect_ids, int32_t *__restrict__ flatten_ids) {
    extern __shared__ uint64_t lds_staged[];
    __shared__ uint32_t s_wave[4 * (1024 / SPLATAD_WAVE)];
    __shared__ uint32_t s_big;
    __shared__ uint32_t s_cnt[1024 / SPLATAD_WAVE][16];
    const uint32_t count = *class_count;
    if constexpr (LONG) {
        __shared__ LongInterval s_stack[kLongStack];
        __shared__ uint32_t s_top, s_kept;
        __shared__ unsigned long long s_range[2];
        for (uint32_t k = blockIdx.x; k < count; k += gridDim.x) { // uniform across the workgroup
            sort_expand_long_list<ER, TIES>(pieces[k], cg, tile_w, tile_h, n_tiles, tile_n_bits, lds_words, bucket_cap,
                                      n_isects, entries, seg_starts, slabs_before, isect_ids, flatten_ids,
                                      lds_staged, s_wave, s_big, s_cnt, s_stack, s_top, s_kept, s_range);
            __syncthreads();
        }
        return;
    }
    for (uint32_t k = blockIdx.x; k < count; k += gridDim.x) { // uniform across the workgroup
        sort_expand_piece<ER, TIES>(pieces[k], cg, tile_w, tile_h, n_tiles, tile_n_bits, lds_words, bucket_cap, n_isects,
                              entries, seg_starts, slabs_before, isect_ids, flatten_ids, lds_staged, s_wave,
                              s_big, s_cnt);
        __syncthreads(); // the next piece reuses the LDS
    }
}

template <int ER, bool TIES, bool LONG = false>
static int launch_block_sort(int cls, uint32_t threads, uint32_t max_n, uint32_t workgroups, uint32_t max_pieces,
                             CoarseGrid cg, uint32_t tile_w, uint32_t tile_h, uint32_t n_tiles,
                             uint32_t tile_n_bits, int64_t n_isects, const uint32_t *class_count,
                             const uint4 *pieces, const uint4 *entries, const int32_t *seg_starts,
                             const int32_t *slabs_before, int64_t *isect_ids, int32_t *flatten_ids,
                             hipStream_t stream) {
    SPLATAD_REQUIRE((uint64_t)ER * threads >= max_n && max_n <= kBlockSortCap && max_n % 512u == 0,
                    "block sort: class %d does not fit", cls);
    const uint32_t bucket_cap = sort_bucket_capacity(max_n);
    {   // the bins of the direct path: a power of two, at most max_n / kSortDirectMean of them
        uint32_t bins = 1;
        while (bins < kSortDirectBins && bins * kSortDirectMean < max_n) bins <<= 1;
        SPLATAD_REQUIRE(bins + 1 <= kSortFineBins + 2 * bucket_cap + 1 && bins <= 65536u,
                        "block sort: no room for the %u bins of class %d", bins, cls);
    }
    const size_t lds_bytes = block_sort_lds_bytes(max_n, bucket_cap);
    {   // raise the kernel's dynamic LDS limit once per instantiation and size
        static std::mutex guard;
        static size_t allowed = 0;
        std::lock_guard<std::mutex> lock(guard);
        if (lds_bytes > allowed) {
            SPLATAD_CHECK_HIP(hipFuncSetAttribute((const void *)isect_block_sort_kernel<ER, TIES, LONG>,
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
            allowed = lds_bytes;
        }
    }
    hipLaunchKernelGGL((isect_block_sort_kernel<ER, TIES, LONG>), dim3(workgroups < max_pieces ? workgroups : max_pieces),
                       dim3(threads), lds_bytes, stream, cg, tile_w, tile_h, n_tiles, tile_n_bits, max_n,
                       bucket_cap, n_isects, class_count + cls, pieces + (size_t)cls * max_pieces, entries,
                       seg_starts, slabs_before, isect_ids, flatten_ids);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

// The two upper classes (more than 12288 entries) in one launch, longest segments first.  Their
// workgroups need most of a compute unit's LDS, so even a launch that finds its class empty waits for such a unit to
// fall free once other sort kernels are running; one launch, enqueued before those, meets an
// idle GPU and costs next to nothing when the scene has no long segments (the usual case for
// cameras), while a lidar's long segments all start at once.
constexpr uint32_t kSortBigThreads = 1024;

__global__ void __launch_bounds__(kSortBigThreads)
isect_big_segment_sort_kernel(uint32_t n_segments, uint32_t n_tiles, uint32_t sshift,
                              uint32_t tile_n_bits, int64_t n_isects,
                              const uint32_t *__restrict__ seg_counts,
                              const uint32_t *__restrict__ seg_lists,
                              const int32_t *__restrict__ tile_starts,
                              const uint64_t *__restrict__ pairs, int64_t *isect_ids,
                              int32_t *__restrict__ flatten_ids) {
    extern __shared__ uint64_t lds_staged[];
    __shared__ uint32_t s_wave[2 * (1024 / SPLATAD_WAVE)];
    __shared__ uint32_t s_big;
    for (int cls = kSortClasses - 1; cls >= 5; --cls) { // uniform
        const uint32_t count = seg_counts[cls];
        const uint32_t *list = seg_lists + (size_t)cls * n_segments;
        for (uint32_t k = blockIdx.x; k < count; k += gridDim.x) { // uniform across the workgroup
            if (cls == 5)
                sort_segment<32, false>(list[k], n_segments, n_tiles, sshift, tile_n_bits, kSortWindow,
                                        sort_bucket_capacity(32768u), n_isects, tile_starts, pairs,
                                        isect_ids, flatten_ids, lds_staged, s_wave, s_big);
            else
                sort_segment<0, false>(list[k], n_segments, n_tiles, sshift, tile_n_bits, kSortWindow,
                                       sort_bucket_capacity(0x7FFFFFFFu), n_isects, tile_starts, pairs,
                                       isect_ids, flatten_ids, lds_staged, s_wave, s_big);
            __syncthreads(); // the next segment reuses the LDS
        }
    }
}

static size_t sort_lds_bytes(uint32_t lds_words, uint32_t max_n) {
    return (size_t)lds_words * 8 + (kSortFineBins + 2 * (size_t)sort_bucket_capacity(max_n)) * 4;
}

static int launch_big_segment_sort(uint32_t workgroups, uint32_t segs, uint32_t n_tiles,
                                   uint32_t sshift, uint32_t tile_n_bits, int64_t n_isects, const uint32_t *seg_counts,
                                   const uint32_t *seg_lists, const int32_t *tile_starts,
                                   const uint64_t *pairs, int64_t *isect_ids, int32_t *flatten_ids,
                                   hipStream_t stream) {
    const size_t lds_bytes = sort_lds_bytes(kSortWindow, 0x7FFFFFFFu);
    {
        static std::mutex guard;
        static bool raised = false;
        std::lock_guard<std::mutex> lock(guard);
        if (!raised) {
            SPLATAD_CHECK_HIP(hipFuncSetAttribute((const void *)isect_big_segment_sort_kernel,
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
            raised = true;
        }
    }
    hipLaunchKernelGGL(isect_big_segment_sort_kernel, dim3(workgroups < segs ? workgroups : segs),
                       dim3(kSortBigThreads), lds_bytes, stream, segs, n_tiles, sshift, tile_n_bits, n_isects,
                       seg_counts, seg_lists, tile_starts, pairs, isect_ids, flatten_ids);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

template <int ER, bool TIES>
static int launch_small_segment_sort(int cls, uint32_t threads, uint32_t max_n, uint32_t workgroups,
                                     uint32_t segs, uint32_t n_tiles, uint32_t sshift, uint32_t tile_n_bits,
                                     int64_t n_isects, const uint32_t *seg_counts,
                                     const uint32_t *seg_lists, const int32_t *tile_starts,
                                     const uint64_t *pairs, int64_t *isect_ids, int32_t *flatten_ids,
                                     hipStream_t stream) {
    SPLATAD_REQUIRE((uint64_t)ER * threads >= max_n && max_n <= 12288u &&
                        ((max_n & (max_n - 1)) == 0 || max_n % 4096u == 0),
                    "segment sort: class %d does not fit", cls);
    const uint32_t bucket_cap = sort_bucket_capacity(max_n);
    {   // the bins of the direct path: a power of two, at most max_n / kSortDirectMean of them
        const uint32_t bins = max_n / kSortDirectMean < kSortDirectBins ? max_n / kSortDirectMean : kSortDirectBins;
        SPLATAD_REQUIRE(bins + 1 <= kSortFineBins + 2 * bucket_cap + 1 && bins <= 65536u,
                        "segment sort: no room for the %u bins of class %d", bins, cls);
    }
    const size_t lds_bytes = sort_small_lds_bytes(max_n, bucket_cap);
    {   // raise the kernel's dynamic LDS limit once per instantiation and size
        static std::mutex guard;
        static size_t allowed = 0;
        std::lock_guard<std::mutex> lock(guard);
        if (lds_bytes > allowed) {
            SPLATAD_CHECK_HIP(hipFuncSetAttribute(
                (const void *)isect_small_segment_sort_kernel<ER, TIES>,
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
            allowed = lds_bytes;
        }
    }
    hipLaunchKernelGGL((isect_small_segment_sort_kernel<ER, TIES>), dim3(workgroups < segs ? workgroups : segs),
                       dim3(threads), lds_bytes, stream, segs, n_tiles, sshift, tile_n_bits, max_n,
                       bucket_cap, n_isects, seg_counts + cls, seg_lists + (size_t)cls * segs,
                       tile_starts, pairs, isect_ids, flatten_ids);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
isect_offset_encode_kernel(int64_t n_isects, const int64_t *__restrict__ isect_ids,
                           uint32_t n_tiles, uint32_t tile_n_bits, int64_t total_tiles,
                           int32_t *__restrict__ offsets) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_isects) return;
    const int64_t mask = ((int64_t)1 << tile_n_bits) - 1;
    const int64_t hi = isect_ids[idx] >> 32;
    const int64_t id_curr = (hi >> tile_n_bits) * n_tiles + (hi & mask);
    int64_t first; // first table entry this intersection is responsible for
    if (idx == 0) {
        first = 0;
    } else {
        const int64_t hp = isect_ids[idx - 1] >> 32;
        if (hp == hi) {
            first = id_curr + 1; // nothing to write
        } else {
            first = (hp >> tile_n_bits) * n_tiles + (hp & mask) + 1;
        }
    }
    for (int64_t i = first; i <= id_curr && i < total_tiles; ++i) offsets[i] = (int32_t)idx;
    if (idx == n_isects - 1)
        for (int64_t i = id_curr + 1; i < total_tiles; ++i) offsets[i] = (int32_t)n_isects;
}

__global__ void fill_zero_i32_kernel(int32_t *p, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

struct IsectWorkspace {
    int64_t *n_entries;           // [1] length of the coarse lists
    int64_t *scan_total;          // [1]
    uint32_t *slab_bounds;        // [kSlabEstimates][1 << kSlabShiftMax] depth bits at which the slabs begin
    int32_t *zeroed;              // tile_counts, tile_fill, block_totals, seg_counts: contiguous, cleared together
    uint64_t n_zeroed;
    int32_t *tile_counts;         // [tile copies * segments], segments = C * n_tiles * slabs
    int32_t *tile_fill;           // same
    int32_t *block_totals;        // [C * blocks] entries per coarse block (in the cleared part)
    int32_t *coarse_counts;       // [coarse workgroups * C * blocks] run starts inside the blocks' lists
    int32_t *tile_starts;         // [tile copies * segments]
    int32_t *seg_starts;          // [segments] first entry of every segment, for the sort
    uint32_t *seg_counts;         // [kSortClasses] segments per size class (in the cleared part)
    uint32_t *seg_lists;          // [kSortClasses * segments]
    int32_t *list_tile_counts;    // [lists * 16] entries per list and tile of the block (in the cleared part)
    uint32_t *list_starts;        // [lists + 1] first entry of every (block, slab) list, and the end
    uint32_t *piece_counts;       // [kBlockClasses] pieces per size class
    uint4 *pieces;                // [kBlockClasses * lists] the pieces the block sort takes, by class
    int64_t *block_sums;          // scan scratch
    // the lists, whose size depends on the number of intersections
    int64_t *cum_before;          // [total] (sort == false)
    uint4 *entries;               // [n_isects] (sort == true), shares memory with cum_before
    uint64_t *pairs;              // [n_isects]
};

template <bool LIDAR>
static CoarseGrid coarse_grid(const TileGrid &g) {
    CoarseGrid cg;
    cg.bshift = !LIDAR ? 2 : (g.tile_w % 4 == 0 ? 2 : (g.tile_w % 2 == 0 ? 1 : 0));
    cg.cw = (g.tile_w + (1u << cg.bshift) - 1) >> cg.bshift;
    cg.ch = (g.tile_h + (1u << kCoarseRowShift) - 1) >> kCoarseRowShift;
    return cg;
}

// Copies of a counter table: a power of two chosen so that the table has about a quarter of a
// million entries, i.e. thousands of cache lines for the atomics to spread over (measured with
// one atomic per tile and workgroup of the tile binning: half as many copies as before cost
// nothing there and shorten the scan; a quarter starts to cost).
static uint32_t isect_copies(uint64_t blocks) {
    uint32_t k = 1;
    while (k < 256 && (uint64_t)(2 * k) * blocks <= (1ull << 18)) k *= 2;
    return k;
}

// Workgroups of the coarse binning (= rows of its counter table): enough to fill the GPU,
// fewer when many blocks would make the table long.
constexpr uint64_t kCoarseTable = 1ull << 19;          // entries of the [workgroup][block] table aimed at
constexpr uint64_t kCoarseTableBlockSort = 1ull << 23; // with the block sort's depth slabs
static uint32_t coarse_workgroups(uint64_t total, uint64_t blocks, uint64_t table) {
    uint64_t wgs = table / (blocks ? blocks : 1);
    // (with the block sort's lists a workgroup flushes thousands of counters with an atomic each:
    // measured on a 1080p frame of 1M Gaussians, the intersection takes 0.228 / 0.219 / 0.240 ms
    // with 512 / 256 / 128 workgroups; a workgroup per compute unit also where the lists are
    // many -- six cameras' 24480 lists: 2.43 ms a frame with 171 workgroups, 2.25 with 256; a 4M
    // frame's 32640 lists: 1.06 against 0.96 ms)
    if (wgs > (table == kCoarseTableBlockSort ? 256u : 512u)) wgs = table == kCoarseTableBlockSort ? 256 : 512;
    if (wgs < 64) wgs = 64;
    const uint64_t needed = (total + kCoarseThreads - 1) / kCoarseThreads;
    if (wgs > needed) wgs = needed ? needed : 1;
    return (uint32_t)wgs;
}

// Everything the two calls derive from the sizes alone, the same way in both.
// With depth slabs (sshift > 0), segments are (tile, slab) pairs and blocks (coarse block,
// slab) pairs.
struct IsectPlan {
    uint32_t n_tiles, tile_n_bits, sshift, per_cam, coarse_wgs, cams_per_launch;
    uint32_t bsshift;   // depth slabs of the coarse lists: sshift, or the block sort's own
    bool block_sort;    // cameras: the coarse lists are sorted and the tile lists written in order
    uint64_t segs, blocks, cslots;
    CoarseGrid cg;
};

// Depth slabs of the coarse lists for the block sort: enough that a list holds about a hundred
// Gaussians on average (the longest list of a driving frame, at its horizon, is some ten times
// the average and should fit the LDS sort, kBlockSortCap: a list taken in parts costs one
// workgroup 100 us and more -- 1M Gaussians on a 1080p frame with 8 slabs instead of 16 take
// 0.33 instead of 0.22 ms), but no more than lets the coarse binning keep all sensors' counters in
// LDS at once, down to two slabs.  (Frames of 2M and 4M Gaussians take 32 and 64 slabs: 0.648
// and 1.043 ms a frame against 0.671 and 1.052 with 16.)
static uint32_t block_slab_shift(uint64_t total, uint32_t C, uint64_t blocks_per_cam) {
    const uint64_t per_block = total / ((uint64_t)C * blocks_per_cam);
    uint32_t s = 0;
    while (s < kSlabShiftMax && (per_block >> s) > 128) ++s;
    while (s > 1 && (((uint64_t)C * blocks_per_cam) << s) > kCoarseLdsBlocks) --s;
    return s;
}

template <bool LIDAR>
static IsectPlan isect_plan(const TileGrid &g, uint64_t total, uint32_t C, int sort) {
    IsectPlan pl;
    pl.n_tiles = g.tile_w * g.tile_h;
    pl.tile_n_bits = splatad_bit_width(pl.n_tiles);
    pl.cg = coarse_grid<LIDAR>(g);
    pl.block_sort = sort && (!LIDAR || pl.cg.bshift == 2);
    pl.sshift = sort && !pl.block_sort ? slab_shift_for(total, (uint64_t)C * pl.n_tiles) : 0;
    pl.bsshift = pl.block_sort ? block_slab_shift(total, C, (uint64_t)pl.cg.cw * pl.cg.ch) : pl.sshift;
    // one sensor's block counters have to fit the LDS of the coarse binning
    while (pl.bsshift > 0 && ((uint64_t)pl.cg.cw * pl.cg.ch << pl.bsshift) > kCoarseLdsBlocks) --pl.bsshift;
    if (!pl.block_sort) pl.sshift = pl.bsshift;
    pl.segs = ((uint64_t)C * pl.n_tiles) << pl.sshift;
    pl.per_cam = (pl.cg.cw * pl.cg.ch) << pl.bsshift;
    pl.blocks = (uint64_t)C * pl.per_cam;
    pl.coarse_wgs = coarse_workgroups(total, pl.blocks, pl.block_sort ? kCoarseTableBlockSort : kCoarseTable);
    pl.cslots = pl.blocks * pl.coarse_wgs;
    pl.cams_per_launch = pl.per_cam ? kCoarseLdsBlocks / pl.per_cam : 0;
    return pl;
}

// Layout of the workspace from sizes only; cslots is the length of the coarse counter table,
// or an upper bound of it when only the number of tiles is known (workspace sizing).
static size_t carve_isect(void *ws, uint64_t total, uint64_t segs, uint64_t lists, bool block_sort,
                          uint64_t cslots, IsectWorkspace *out) {
    const uint64_t block_sort_lists = block_sort ? lists : 0; // what only the block sort uses
    const uint64_t tslots = segs * isect_copies(segs);
    const uint64_t scan_n = total > tslots ? total : tslots;
    char *p = (char *)ws;
    IsectWorkspace w = {};
    w.n_entries = (int64_t *)p;             p += 256;
    w.scan_total = (int64_t *)p;            p += 256;
    w.slab_bounds = (uint32_t *)p;          p += splatad_align256((kSlabEstimates << kSlabShiftMax) * 4);
    w.zeroed = (int32_t *)p;
    w.tile_counts = (int32_t *)p;           p += splatad_align256(tslots * 4);
    w.tile_fill = (int32_t *)p;             p += splatad_align256(tslots * 4);
    w.block_totals = (int32_t *)p;          p += splatad_align256(lists * 4);
    w.list_tile_counts = (int32_t *)p;      p += splatad_align256(block_sort_lists * 64);
    w.seg_counts = (uint32_t *)p;           p += 256;
    w.n_zeroed = (uint64_t)(p - (char *)w.zeroed) / 4;
    w.coarse_counts = (int32_t *)p;         p += splatad_align256(cslots * 4);
    w.tile_starts = (int32_t *)p;           p += splatad_align256(tslots * 4);
    w.seg_lists = (uint32_t *)p;            p += splatad_align256(segs * kSortClasses * 4);
    w.seg_starts = (int32_t *)p;            p += splatad_align256(segs * 4);
    w.list_starts = (uint32_t *)p;          p += splatad_align256((lists + 1) * 4);
    w.piece_counts = (uint32_t *)p;         p += 256;
    w.pieces = (uint4 *)p;                  p += splatad_align256(block_sort_lists * kBlockClasses * 16);
    w.block_sums = (int64_t *)p;            p += scan_workspace_bytes((int64_t)scan_n);
    if (out) *out = w;
    return (size_t)(p - (char *)ws);
}

static size_t carve_lists(void *lists, uint64_t total, int64_t n_isects, IsectWorkspace *w) {
    char *p = (char *)lists;
    const uint64_t list_bytes = splatad_align256((uint64_t)n_isects * 16);
    const uint64_t cum_bytes = splatad_align256(total * 8);
    if (w) { w->cum_before = (int64_t *)p; w->entries = (uint4 *)p; }
    p += list_bytes > cum_bytes ? list_bytes : cum_bytes;
    if (w) w->pairs = (uint64_t *)p;
    p += splatad_align256((uint64_t)n_isects * 8);
    return (size_t)(p - (char *)lists);
}

static size_t isect_ws_bytes(uint64_t total, uint32_t C, uint64_t n_tiles) {
    uint64_t segs = (uint64_t)C * n_tiles;
    // Bounds for both kinds of plan; coarse_workgroups() keeps the table at its aimed-at size
    // unless 64 rows exceed that.
    // The segment sort's plan: the most slabs a plan for these sizes uses, as many lists as segments
    // at most.  The block sort's: tiles as segments, and a sensor's ceil(w / 4) * ceil(h / 4) blocks
    // (at most a quarter of its w * h tiles, plus one) times 1 << kSlabShiftMax lists
    const uint64_t slabbed = segs << slab_shift_for(total, segs);
    const uint64_t lists = (uint64_t)C * (n_tiles / 4 + 1) << kSlabShiftMax;
    const uint64_t a = carve_isect(nullptr, total, slabbed, slabbed, false,
                                   slabbed * 64 > kCoarseTable ? slabbed * 64 : kCoarseTable, nullptr);
    const uint64_t b = carve_isect(nullptr, total, segs, lists, true,
                                   lists * 64 > kCoarseTableBlockSort ? lists * 64 : kCoarseTableBlockSort, nullptr);
    return a > b ? a : b;
}

static inline dim3 grid_for(uint64_t n) {
    return dim3((uint32_t)((n + SPLATAD_THREADS - 1) / SPLATAD_THREADS));
}

// Per device, created at first use and kept for the life of the process: the helper streams
// (default priority) and events of the segment sort.  `guard` serialises the enqueueing of the
// fork / join sequences that share them (enqueueing only: no call waits for the GPU under it).
struct IsectDevice {
    hipStream_t aux[2];
    hipEvent_t fork, join[2];
    std::mutex guard;
};

static int isect_device(IsectDevice **out) {
    static std::mutex table_guard;
    static IsectDevice *table[64] = {};
    int dev = 0;
    SPLATAD_CHECK_HIP(hipGetDevice(&dev));
    SPLATAD_REQUIRE(dev >= 0 && dev < 64, "isect: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(table_guard);
    if (!table[dev]) {
        IsectDevice *s = new IsectDevice();
        for (hipStream_t &a : s->aux) SPLATAD_CHECK_HIP(hipStreamCreateWithFlags(&a, hipStreamNonBlocking));
        SPLATAD_CHECK_HIP(hipEventCreateWithFlags(&s->fork, hipEventDisableTiming));
        for (hipEvent_t &e : s->join) SPLATAD_CHECK_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
        table[dev] = s;
    }
    *out = table[dev];
    return 0;
}

// First stage of the binning, which needs no list memory (the counters were cleared by the
// kernel before it): count the coarse lists.
template <bool LIDAR>
static int enqueue_coarse_count(const TileGrid &g, const IsectPlan &pl, const IsectWorkspace &w,
                                uint64_t total, uint32_t N, const int64_t *camera_ids,
                                const float *means2d, const void *radii, const float *depths,
                                uint32_t C, hipStream_t stream) {
    SPLATAD_REQUIRE(pl.per_cam <= kCoarseLdsBlocks, "isect: %u x %u tiles per sensor exceed the "
                    "binning capacity", g.tile_w, g.tile_h);
    SPLATAD_REQUIRE(pl.blocks < (1ull << 31) && pl.cslots < (1ull << 31), "isect: tile grid too large");
    {
        static std::mutex guard;
        static bool raised = false;
        std::lock_guard<std::mutex> lock(guard);
        if (!raised) {
            SPLATAD_CHECK_HIP(hipFuncSetAttribute(
                (const void *)isect_coarse_kernel<LIDAR, false>,
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kCoarseLdsBlocks * 4)));
            SPLATAD_CHECK_HIP(hipFuncSetAttribute(
                (const void *)isect_coarse_kernel<LIDAR, true>,
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kCoarseLdsBlocks * 4)));
            raised = true;
        }
    }
    for (uint32_t c0 = 0; c0 < C; c0 += pl.cams_per_launch) {
        const uint32_t c1 = C - c0 < pl.cams_per_launch ? C : c0 + pl.cams_per_launch;
        hipLaunchKernelGGL((isect_coarse_kernel<LIDAR, false>), dim3(pl.coarse_wgs),
                           dim3(kCoarseThreads), (size_t)(c1 - c0) * pl.per_cam * 4, stream, g, pl.cg,
                           total, N, camera_ids, means2d, radii, pl.bsshift ? depths : nullptr, c0, c1,
                           (uint32_t)pl.blocks, w.coarse_counts, (uint4 *)nullptr, pl.bsshift,
                           (const uint32_t *)w.slab_bounds, (const int32_t *)nullptr, (const int32_t *)nullptr,
                           (int32_t *)nullptr, w.block_totals, (int64_t *)nullptr, 0u, (uint32_t *)nullptr,
                           (unsigned long long *)nullptr);
    }
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

// The counting kernel's cross-workgroup counters: one set per leased host word (calls that
// overlap hold different leases), in device memory of the library itself, zero when the library
// is loaded and left at zero by every counting kernel that completes.
static __device__ __align__(256) unsigned long long count_words[kHostWordSlots * kCountWords];

// Address of the current device's copy of `count_words`, looked up once per device.  In host
// code the array's name is only a handle for this lookup, never an address a kernel could use.
static int count_words_of(int slot, unsigned long long **out) {
    static std::mutex guard;
    static unsigned long long *table[kHostWordDevices] = {};
    int dev = 0;
    SPLATAD_CHECK_HIP(hipGetDevice(&dev));
    SPLATAD_REQUIRE(dev >= 0 && dev < kHostWordDevices, "isect: device index %d out of range", dev);
    SPLATAD_REQUIRE(slot >= 0 && slot < kHostWordSlots, "isect: host word slot %d out of range", slot);
    std::lock_guard<std::mutex> lock(guard);
    if (table[dev] == nullptr) {
        void *ptr = nullptr;
        SPLATAD_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(count_words)));
        SPLATAD_REQUIRE(ptr != nullptr, "isect: the counters have no device address");
        table[dev] = (unsigned long long *)ptr;
    }
    *out = table[dev] + (size_t)slot * kCountWords;
    return 0;
}

template <bool LIDAR>
static int isect_count(TileGrid g, uint64_t total, uint32_t N, const int64_t *camera_ids,
                       const float *means2d, const void *radii, const float *depths, uint32_t C, int sort,
                       int32_t *tiles_per_gauss, void *workspace, int64_t *n_isects_host,
                       hipStream_t stream, bool known = false) {
    // known: the caller has the number of intersections from elsewhere (the packed projection
    // counts them for its rows); everything is enqueued as usual, nothing is waited for
    SPLATAD_REQUIRE(known || n_isects_host != nullptr, "isect: n_isects_host is null");
    if (n_isects_host) *n_isects_host = 0;
    if (total == 0) return 0;
    SPLATAD_REQUIRE(total < (1ull << 31), "isect: number of projected Gaussians must be below 2^31");
    // (tiles_per_gauss may be null for a caller that knows the count and wants sorted lists: the
    // rows' counts are then not made)
    SPLATAD_REQUIRE(means2d && radii && workspace && (tiles_per_gauss || (known && sort)),
                    "isect: null pointer argument");
    SPLATAD_REQUIRE(camera_ids != nullptr || N > 0, "isect: N is zero for unpacked input");
    SPLATAD_REQUIRE(!sort || depths != nullptr, "isect: depths is null");
    const IsectPlan pl = isect_plan<LIDAR>(g, total, C, sort);
    SPLATAD_REQUIRE(pl.n_tiles > 0 && C > 0, "isect: empty tile grid");
    SPLATAD_REQUIRE(pl.tile_n_bits + splatad_bit_width(C) <= 32,
                    "isect: camera and tile ids need more than 32 bits");
    IsectWorkspace w;
    carve_isect(workspace, total, pl.segs, pl.blocks, pl.block_sort, sort ? pl.cslots : 0, &w);
    // the number of intersections reaches the host through a leased pinned word
    HostWordLease lease(stream);
    unsigned long long *counters = nullptr;
    if (!known) {
        if (int rc = host_word_refuse_capture(stream, "isect")) return rc;
        if (int rc = host_word_acquire(&lease.word)) return rc;
        if (int rc = count_words_of(lease.word.slot, &counters)) return rc;
    }
    // the counting kernel clears the tile counters, the fill cursors and the class counters of
    // the binning behind it
    // (a caller that knows the count and sorts without depth slabs needs nothing of the counting
    // kernel but the cleared counters)
    const bool skip_count = known && sort && pl.bsshift == 0;
    if (!skip_count) {
        dim3 count_grid = grid_for(total);
        if (count_grid.x > 1024) count_grid.x = 1024;
        // (without the rows' counts the kernel only clears and finds the slabs' bounds)
        const bool count_rows = tiles_per_gauss != nullptr;
        if (!count_rows && count_grid.x > 256) count_grid.x = 256;
        const bool slabs = sort && pl.bsshift != 0; // one more workgroup finds the slabs' bounds
        if (slabs) count_grid.x += kSlabEstimates;
        hipLaunchKernelGGL((slabs ? isect_count_kernel<LIDAR, true> : isect_count_kernel<LIDAR, false>),
                           count_grid, dim3(SPLATAD_THREADS), 0, stream, g,
                           total, means2d, radii, tiles_per_gauss, counters, lease.word.device,
                           w.zeroed, sort ? w.n_zeroed : (uint64_t)0, depths, 1u << pl.bsshift,
                           slabs ? w.slab_bounds : (uint32_t *)nullptr,
                           // the block sort's slabs even out the coarse lists, an entry per Gaussian
                           // and block; the segment sort's the tile segments
                           pl.block_sort ? 1 : 0, count_rows ? 1 : 0);
        SPLATAD_LAUNCH_CHECK();
    } else {
        hipLaunchKernelGGL(fill_zero_i32_kernel, grid_for(w.n_zeroed), dim3(SPLATAD_THREADS), 0, stream,
                           w.zeroed, (int64_t)w.n_zeroed);
        SPLATAD_LAUNCH_CHECK();
    }
    // work for the GPU while the host learns the count and sizes the lists
    if (sort) {
        if (int rc = enqueue_coarse_count<LIDAR>(g, pl, w, total, N, camera_ids, means2d, radii, depths,
                                                 C, stream))
            return rc;
    }
    if (known) return 0;
    unsigned long long n = 0;
    if (int rc = host_word_wait(&lease, "isect", &n)) return rc;
    SPLATAD_REQUIRE(n < (1ull << 31), "isect: %llu intersections exceed the int32 offset range", n);
    *n_isects_host = (int64_t)n;
    return 0;
}

// Work of the caller's that a fill call runs beside its sort: handed one of the sort's helper
// streams right after their fork (so it is joined with them), once.
struct BesideWork {
    splatad_beside_fn fn = nullptr;
    void *context = nullptr;
    bool done = false;
    int run(hipStream_t on) {
        if (fn == nullptr || done) return 0;
        done = true;
        const int rc = fn(context, (splatad_stream_t)on);
        SPLATAD_REQUIRE(rc == 0, "isect: the caller's work beside the sort failed with %d", rc);
        return 0;
    }
};

template <bool LIDAR>
static int isect_fill_with(TileGrid g, uint64_t total, uint32_t N, const int64_t *camera_ids,
                      const float *means2d, const void *radii, const float *depths, uint32_t C,
                      int sort, int64_t n_isects, const int32_t *tiles_per_gauss,
                      void *workspace, void *lists, int64_t *isect_ids, int32_t *flatten_ids,
                      int32_t *tile_offsets, hipStream_t stream, const int32_t *remap,
                      const int32_t *remap_offsets, int32_t *tiles_out, hipStream_t beside,
                      BesideWork &beside_work);

template <bool LIDAR>
static int isect_fill(TileGrid g, uint64_t total, uint32_t N, const int64_t *camera_ids,
                      const float *means2d, const void *radii, const float *depths, uint32_t C,
                      int sort, int64_t n_isects, const int32_t *tiles_per_gauss,
                      void *workspace, void *lists, int64_t *isect_ids, int32_t *flatten_ids,
                      int32_t *tile_offsets, hipStream_t stream, const int32_t *remap = nullptr,
                      int32_t *tiles_out = nullptr, hipStream_t beside = nullptr,
                      splatad_beside_fn beside_fn = nullptr, void *beside_context = nullptr,
                      const int32_t *remap_offsets = nullptr) {
    BesideWork work;
    work.fn = beside_fn;
    work.context = beside_context;
    const int rc = isect_fill_with<LIDAR>(g, total, N, camera_ids, means2d, radii, depths, C, sort, n_isects,
                                          tiles_per_gauss, workspace, lists, isect_ids, flatten_ids, tile_offsets,
                                          stream, remap, remap_offsets, tiles_out, beside, work);
    if (rc) return rc;
    return work.run(stream); // nothing was sorted on helper streams: on the call's own stream
}

template <bool LIDAR>
static int isect_fill_with(TileGrid g, uint64_t total, uint32_t N, const int64_t *camera_ids,
                      const float *means2d, const void *radii, const float *depths, uint32_t C,
                      int sort, int64_t n_isects, const int32_t *tiles_per_gauss,
                      void *workspace, void *lists, int64_t *isect_ids, int32_t *flatten_ids,
                      int32_t *tile_offsets, hipStream_t stream, const int32_t *remap,
                      const int32_t *remap_offsets, int32_t *tiles_out, hipStream_t beside,
                      BesideWork &beside_work) {
    SPLATAD_REQUIRE(remap == nullptr || (sort && camera_ids == nullptr),
                    "isect: remapped rows need sort != 0 and a dense [C, N] layout");
    if (total == 0 || n_isects == 0) {
        if (tile_offsets && sort && (uint64_t)C * g.tile_w * g.tile_h > 0) {
            const uint64_t tiles = (uint64_t)C * g.tile_w * g.tile_h;
            hipLaunchKernelGGL(fill_zero_i32_kernel, grid_for(tiles), dim3(SPLATAD_THREADS), 0,
                               stream, tile_offsets, (int64_t)tiles);
            SPLATAD_LAUNCH_CHECK();
        }
        if (beside != nullptr && beside != stream) { // nothing to sort: ordered behind this point
            IsectDevice *ss = nullptr;
            if (int rc = isect_device(&ss)) return rc;
            std::lock_guard<std::mutex> fork_lock(ss->guard);
            SPLATAD_CHECK_HIP(hipEventRecord(ss->fork, stream));
            SPLATAD_CHECK_HIP(hipStreamWaitEvent(beside, ss->fork, 0));
        }
        return 0;
    }
    SPLATAD_REQUIRE(means2d && radii && depths && workspace && lists && isect_ids && flatten_ids,
                    "isect: null pointer argument");
    SPLATAD_REQUIRE(camera_ids != nullptr || N > 0, "isect: N is zero for unpacked input");
    const IsectPlan pl = isect_plan<LIDAR>(g, total, C, sort);
    const uint32_t n_tiles = pl.n_tiles, tile_n_bits = pl.tile_n_bits, sshift = pl.sshift;
    const uint64_t segs = pl.segs;
    const CoarseGrid cg = pl.cg;
    IsectWorkspace w;
    carve_isect(workspace, total, segs, pl.blocks, pl.block_sort, sort ? pl.cslots : 0, &w);
    carve_lists(lists, total, n_isects, &w);
    int rc;
    if (!sort) {
        SPLATAD_REQUIRE(tiles_per_gauss != nullptr, "isect: tiles_per_gauss is null");
        rc = launch_exclusive_scan<int64_t>(tiles_per_gauss, (int64_t)total, 1, 0, w.cum_before,
                                            w.scan_total, w.block_sums, stream);
        if (rc) return rc;
        hipLaunchKernelGGL(isect_emit_kernel<LIDAR>, grid_for(total), dim3(SPLATAD_THREADS), 0,
                           stream, g, total, N, camera_ids, means2d, radii, depths,
                           (const int64_t *)w.cum_before, tile_n_bits, isect_ids, flatten_ids);
        SPLATAD_LAUNCH_CHECK();
        return 0;
    }
    // The block sort takes coarse lists of up to kBlockLongMax entries.  Whether all lists are that
    // short the host learns from the filling kernel, through a pinned word as it learnt the
    // number of intersections (the wait below ends as soon as that kernel has begun: the GPU has
    // the tile binning to do meanwhile); a scene with a longer list takes the segment sort.
    HostWordLease longest(stream);
    if (pl.block_sort) {
        if ((rc = host_word_refuse_capture(stream, "isect")) != 0) return rc;
        if ((rc = host_word_acquire(&longest.word)) != 0) return rc;
    }
    // the coarse lists were counted by the counting call; fill them
    for (uint32_t c0 = 0; c0 < C; c0 += pl.cams_per_launch) {
        const uint32_t c1 = C - c0 < pl.cams_per_launch ? C : c0 + pl.cams_per_launch;
        hipLaunchKernelGGL((isect_coarse_kernel<LIDAR, true>), dim3(pl.coarse_wgs),
                           dim3(kCoarseThreads), (size_t)(c1 - c0) * pl.per_cam * 4, stream, g, cg,
                           total, N, camera_ids, means2d, radii, depths, c0, c1, (uint32_t)pl.blocks,
                           w.coarse_counts, w.entries, pl.bsshift, (const uint32_t *)w.slab_bounds, remap,
                           remap_offsets, tiles_out, w.block_totals, w.n_entries, (uint32_t)n_isects,
                           pl.block_sort ? w.list_starts : (uint32_t *)nullptr,
                           pl.block_sort ? longest.word.device : (unsigned long long *)nullptr);
    }
    SPLATAD_LAUNCH_CHECK();
    // tile segments: count, scan, fill.  The number of coarse entries stays on the device;
    // the grid is sized for the bound n_isects and strides.
    const uint32_t tcopies = pl.block_sort ? 1u : isect_copies(segs);
    uint64_t bin_wgs = ((uint64_t)n_isects + SPLATAD_THREADS - 1) / SPLATAD_THREADS;
    if (bin_wgs > 8192) bin_wgs = 8192;
    const bool square = cg.bshift == 2; // 4 x 4 tiles per block: the unrolled kernels
    if (pl.block_sort) {
        // counts per list and tile, from which both the tiles' counts and the places of the
        // lists inside the tiles' segments follow
        hipLaunchKernelGGL(isect_list_count_kernel, dim3((uint32_t)bin_wgs), dim3(SPLATAD_THREADS), 0, stream,
                           (const int64_t *)w.n_entries, (const uint4 *)w.entries, w.list_tile_counts);
        hipLaunchKernelGGL(isect_tile_totals_kernel, grid_for((uint64_t)C * cg.cw * cg.ch * 16), dim3(SPLATAD_THREADS), 0,
                           stream, cg, g.tile_w, g.tile_h, pl.bsshift, C * cg.cw * cg.ch, w.list_tile_counts,
                           w.tile_counts);
    } else
    hipLaunchKernelGGL((square ? isect_tile_bin_kernel<false, 16> : isect_tile_bin_kernel<false, 0>),
                       dim3((uint32_t)bin_wgs),
                       dim3(SPLATAD_THREADS), 0, stream, cg, g.tile_w, g.tile_h, sshift, tcopies,
                       (uint32_t)segs, (const int64_t *)w.n_entries, (const uint4 *)w.entries,
                       w.tile_counts, (const int32_t *)nullptr, (int32_t *)nullptr,
                       (uint64_t *)nullptr, (int64_t)0, (uint32_t *)nullptr, (uint32_t *)nullptr,
                       (int32_t *)nullptr, (const int64_t *)nullptr, 0u, (int32_t *)nullptr,
                       pl.bsshift - sshift);
    SPLATAD_LAUNCH_CHECK();
    IsectDevice *ss = nullptr;
    if ((rc = isect_device(&ss)) != 0) return rc;
    const uint32_t nseg = (uint32_t)segs;
    bool short_lists = false;
    unsigned long long longest_list = 0;
    if (pl.block_sort) {
        if ((rc = host_word_wait(&longest, "isect", &longest_list)) != 0) return rc;
        short_lists = longest_list <= kBlockLongMax;
    }
    // up to 128 scan blocks, i.e. any table of the size isect_copies() aims at: one scan launch,
    // and the filling pass adds the blocks before an element itself (the block sort's planning
    // kernel scans its tile counts itself)
    const int64_t scan_n = (int64_t)(segs * tcopies);
    const int scan_stride = tcopies > 1 ? -(int)tcopies : 1;
    uint32_t n_scan_blocks = 0;
    const bool local_scan = scan_n <= kScanLocalBlocks * SCAN_TILE;
    if (short_lists)
        rc = 0;
    else if (local_scan)
        rc = launch_local_scan<int32_t>(w.tile_counts, scan_n, scan_stride, w.tile_starts, w.block_sums,
                                        &n_scan_blocks, stream);
    else
        rc = launch_exclusive_scan<int32_t>(w.tile_counts, scan_n, scan_stride, 0, w.tile_starts,
                                            w.scan_total, w.block_sums, stream);
    if (rc) return rc;
    if (short_lists) {
        // Pieces of the coarse lists by size class, and the tiles' starts; then a launch per
        // class, the long pieces first, beside each other on the caller's stream and two helper
        // streams like the classes of the segment sort below.
        const uint32_t n_blocks = C * cg.cw * cg.ch;
        uint32_t plan_wgs = 1 + (nseg + 1023) / 1024;
        if (plan_wgs > 65) plan_wgs = 65;
        hipLaunchKernelGGL(isect_block_plan_kernel, dim3(plan_wgs), dim3(1024), 0, stream, n_blocks, pl.bsshift,
                           (const int32_t *)w.block_totals, (const uint32_t *)w.list_starts,
                           (const int32_t *)w.tile_counts, cg, g.tile_w, g.tile_h, nseg,
                           w.seg_starts, tile_offsets, w.piece_counts, (uint32_t)pl.blocks, w.pieces,
                           LIDAR ? kBlockMergeCapLidar : kBlockMergeCap, LIDAR ? kBlockPairsCapLidar : kBlockPairsCap);
        SPLATAD_LAUNCH_CHECK();
        // A small call (up to about half a million Gaussians) is bound by the host and by
        // launch latencies, not by the GPU: its classes go one behind the other on the caller's
        // stream, without the fork and the join of the helper streams (three event records and
        // four cross-stream waits, 45 us of host time).
        const bool one_stream = n_isects < kOneStreamIsects;
        hipStream_t const aux0 = one_stream ? stream : ss->aux[0], aux1 = one_stream ? stream : ss->aux[1];
        const bool orders_beside = beside != nullptr && beside != stream;
        std::unique_lock<std::mutex> fork_lock(ss->guard, std::defer_lock);
        if (!one_stream || orders_beside) {
            fork_lock.lock();
            SPLATAD_CHECK_HIP(hipEventRecord(ss->fork, stream));
            if (!one_stream)
                for (hipStream_t aux : ss->aux) SPLATAD_CHECK_HIP(hipStreamWaitEvent(aux, ss->fork, 0));
            if (orders_beside) SPLATAD_CHECK_HIP(hipStreamWaitEvent(beside, ss->fork, 0));
        }
        auto enqueue_block_sorts = [&]() -> int {
            int e;
            // (the caller's work first on the stream of the many mid-sized pieces: measured on a
            // packed frame, its compaction there costs the step 14 us less than behind the sort;
            // on the other helper stream 3 us less, on the caller's own 6 us more)
            if ((e = beside_work.run(aux0)) != 0) return e;
#define SPLATAD_BLOCK_CLASS(cls, ER, threads, hi, wgs, on)                                                        \
            if ((e = launch_block_sort<ER, LIDAR>(cls, threads, hi, wgs, (uint32_t)pl.blocks, cg, g.tile_w, g.tile_h,   \
                                           n_tiles, tile_n_bits, n_isects, w.piece_counts, w.pieces, w.entries,  \
                                           w.seg_starts, w.list_tile_counts, isect_ids, flatten_ids, on)) != 0)  \
                return e;
            // (the lists too long for one LDS sort first: a workgroup each, part by part)
            // Pieces beyond kBlockMergeCap entries are single lists, so the longest list tells
            // which of the upper classes are empty: their launches (5 us each on the way) are left out.
            if (longest_list > kBlockSortCap &&
                (e = launch_block_sort<10, LIDAR, true>(kBlockLongClass, 1024, kBlockSortCap, 256u, (uint32_t)pl.blocks, cg,
                                                 g.tile_w, g.tile_h, n_tiles, tile_n_bits, n_isects,
                                                 w.piece_counts, w.pieces, w.entries, w.seg_starts,
                                                 w.list_tile_counts, isect_ids, flatten_ids, stream)) != 0)
                return e;
            if (longest_list > 8192u) SPLATAD_BLOCK_CLASS(4, 10, 1024, kBlockSortCap, 256u, stream)
            if (longest_list > 4096u) SPLATAD_BLOCK_CLASS(3, 8, 1024, 8192u, 256u, aux1)
            SPLATAD_BLOCK_CLASS(2, 8, 512, 4096u, 512u, aux0)
            SPLATAD_BLOCK_CLASS(1, 8, 256, 2048u, 1024u, stream)
            SPLATAD_BLOCK_CLASS(0, 4, 128, 512u, 2048u, aux1)
#undef SPLATAD_BLOCK_CLASS
            return 0;
        };
        rc = enqueue_block_sorts();
        // (joined whatever happens: work already queued on the helper streams writes the caller's buffers)
        for (int k = 0; k < (one_stream ? 0 : 2); ++k) {
            const hipError_t r = hipEventRecord(ss->join[k], ss->aux[k]);
            const hipError_t q = r == hipSuccess ? hipStreamWaitEvent(stream, ss->join[k], 0) : r;
            if (q != hipSuccess && rc == 0) SPLATAD_CHECK_HIP(q);
        }
        if (rc) return rc;
        SPLATAD_LAUNCH_CHECK();
        return 0;
    }
    hipLaunchKernelGGL((square ? isect_tile_bin_kernel<true, 16> : isect_tile_bin_kernel<true, 0>),
                       dim3((uint32_t)bin_wgs),
                       dim3(SPLATAD_THREADS), 0, stream, cg, g.tile_w, g.tile_h, sshift, tcopies,
                       (uint32_t)segs, (const int64_t *)w.n_entries, (const uint4 *)w.entries,
                       w.tile_counts, (const int32_t *)w.tile_starts, w.tile_fill, w.pairs, n_isects,
                       w.seg_counts, w.seg_lists, tile_offsets,
                       local_scan ? (const int64_t *)w.block_sums : (const int64_t *)nullptr, n_scan_blocks,
                       w.seg_starts, pl.bsshift - sshift);
    SPLATAD_LAUNCH_CHECK();
    // Size classes: a launch per class (one for the two upper classes), so that the LDS per
    // workgroup (and with it the number of resident workgroups) fits the segment length; the
    // segments of a class come from a list made on the device.  The classes touch disjoint
    // segments; they run on two helper streams beside the caller's, forked and joined with
    // events, so that the few long workgroups of the upper classes overlap the many short ones
    // of the lower classes.
    std::lock_guard<std::mutex> fork_lock(ss->guard);
    SPLATAD_CHECK_HIP(hipEventRecord(ss->fork, stream));
    for (hipStream_t aux : ss->aux) SPLATAD_CHECK_HIP(hipStreamWaitEvent(aux, ss->fork, 0));
    // a stream of the caller's for work of its own beside the sort: ordered behind the binning
    if (beside != nullptr && beside != stream) SPLATAD_CHECK_HIP(hipStreamWaitEvent(beside, ss->fork, 0));
    // After the fork the helper streams are joined whatever happens: work already queued on
    // them reads and writes the caller's buffers, so the caller's stream must not run past it.
    auto enqueue_sorts = [&]() -> int {
        int e;
        if ((e = beside_work.run(ss->aux[0])) != 0) return e;
#define SPLATAD_SORT_CLASS(cls, ER, threads, hi, wgs, on)                                        \
        if ((e = launch_small_segment_sort<ER, LIDAR>(cls, threads, hi, wgs, nseg, n_tiles, sshift, tile_n_bits, \
                                                      n_isects, w.seg_counts, w.seg_lists, w.seg_starts, \
                                                      w.pairs, isect_ids, flatten_ids, on)) != 0) \
            return e;
        // the upper classes go first, on the caller's stream, which does not wait for the fork;
        // then the segments of 8193 to 12288 entries (a driving frame's longest, a sixth of its
        // entries), by the short-segment sort with twelve entries per lane: through the generic
        // sort of the upper classes they took 30 us at the head of this stream
        if ((e = launch_big_segment_sort(256u, nseg, n_tiles, sshift, tile_n_bits, n_isects, w.seg_counts,
                                         w.seg_lists, w.seg_starts, w.pairs, isect_ids, flatten_ids,
                                         stream)) != 0)
            return e;
        SPLATAD_SORT_CLASS(4, 12, 1024, 12288u, 256u, stream)
        SPLATAD_SORT_CLASS(2, 8, 512, 4096u, 1024u, ss->aux[0])
        SPLATAD_SORT_CLASS(3, 8, 1024, 8192u, 512u, ss->aux[1])
        SPLATAD_SORT_CLASS(1, 8, 256, 2048u, 4096u, stream)
        SPLATAD_SORT_CLASS(0, 4, 128, 512u, 4096u, stream)
#undef SPLATAD_SORT_CLASS
        return 0;
    };
    rc = enqueue_sorts();
    for (int k = 0; k < 2; ++k) {
        const hipError_t r = hipEventRecord(ss->join[k], ss->aux[k]);
        const hipError_t q = r == hipSuccess ? hipStreamWaitEvent(stream, ss->join[k], 0) : r;
        if (q != hipSuccess && rc == 0) SPLATAD_CHECK_HIP(q);
    }
    if (rc) return rc;
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

} // namespace

extern "C" size_t splatad_isect_workspace_bytes(uint64_t total, uint32_t C, uint32_t n_tiles) {
    return isect_ws_bytes(total, C, n_tiles);
}

extern "C" size_t splatad_isect_lists_bytes(uint64_t total, int64_t n_isects) {
    return carve_lists(nullptr, total, n_isects < 0 ? 0 : n_isects, nullptr);
}

extern "C" int splatad_isect_tiles_count(uint64_t total, uint32_t N, const int64_t *camera_ids,
                                         const float *means2d, const int32_t *radii,
                                         const float *depths, uint32_t C,
                                         uint32_t tile_size, uint32_t tile_width,
                                         uint32_t tile_height, int sort, int32_t *tiles_per_gauss,
                                         void *workspace, int64_t *n_isects_host,
                                         splatad_stream_t stream) {
    SPLATAD_REQUIRE(tile_size > 0, "isect_tiles: tile_size is zero");
    TileGrid g{tile_size, tile_width, tile_height, 0.f, 0.f, nullptr};
    return isect_count<false>(g, total, N, camera_ids, means2d, radii, depths, C, sort, tiles_per_gauss,
                              workspace, n_isects_host, (hipStream_t)stream);
}

extern "C" int splatad_isect_tiles_prepare(uint64_t total, uint32_t N, const int64_t *camera_ids,
                                           const float *means2d, const int32_t *radii,
                                           const float *depths, uint32_t C, uint32_t tile_size,
                                           uint32_t tile_width, uint32_t tile_height, int sort,
                                           int32_t *tiles_per_gauss, void *workspace,
                                           splatad_stream_t stream) {
    SPLATAD_REQUIRE(tile_size > 0, "isect_tiles: tile_size is zero");
    TileGrid g{tile_size, tile_width, tile_height, 0.f, 0.f, nullptr};
    return isect_count<false>(g, total, N, camera_ids, means2d, radii, depths, C, sort, tiles_per_gauss,
                              workspace, nullptr, (hipStream_t)stream, true);
}

extern "C" int splatad_isect_tiles_fill(uint64_t total, uint32_t N, const int64_t *camera_ids,
                                        const float *means2d, const int32_t *radii,
                                        const float *depths, uint32_t C, uint32_t tile_size,
                                        uint32_t tile_width, uint32_t tile_height, int sort,
                                        int64_t n_isects, const int32_t *tiles_per_gauss,
                                        void *workspace, void *lists, int64_t *isect_ids,
                                        int32_t *flatten_ids, int32_t *tile_offsets,
                                        splatad_stream_t stream) {
    return splatad_isect_tiles_fill_beside(total, N, camera_ids, means2d, radii, depths, C, tile_size, tile_width,
                                           tile_height, sort, n_isects, tiles_per_gauss, workspace, lists,
                                           isect_ids, flatten_ids, tile_offsets, nullptr, nullptr, stream);
}

extern "C" int splatad_isect_tiles_fill_beside(uint64_t total, uint32_t N, const int64_t *camera_ids,
                                               const float *means2d, const int32_t *radii,
                                               const float *depths, uint32_t C, uint32_t tile_size,
                                               uint32_t tile_width, uint32_t tile_height, int sort,
                                               int64_t n_isects, const int32_t *tiles_per_gauss,
                                               void *workspace, void *lists, int64_t *isect_ids,
                                               int32_t *flatten_ids, int32_t *tile_offsets,
                                               splatad_beside_fn beside_work, void *beside_context,
                                               splatad_stream_t stream) {
    SPLATAD_REQUIRE(tile_size > 0, "isect_tiles: tile_size is zero");
    TileGrid g{tile_size, tile_width, tile_height, 0.f, 0.f, nullptr};
    return isect_fill<false>(g, total, N, camera_ids, means2d, radii, depths, C, sort, n_isects,
                             tiles_per_gauss, workspace, lists, isect_ids, flatten_ids,
                             tile_offsets, (hipStream_t)stream, nullptr, nullptr, nullptr, beside_work,
                             beside_context);
}

extern "C" int splatad_isect_tiles_fill_remapped(uint64_t total, uint32_t N, const float *means2d,
                                                 const int32_t *radii, const float *depths, uint32_t C,
                                                 uint32_t tile_size, uint32_t tile_width,
                                                 uint32_t tile_height, int64_t n_isects,
                                                 const int32_t *tiles_per_gauss, const int32_t *remap,
                                                 const int32_t *remap_offsets, void *workspace, void *lists, int32_t *tiles_out,
                                                 int64_t *isect_ids, int32_t *flatten_ids,
                                                 int32_t *tile_offsets, splatad_stream_t beside_stream,
                                                 splatad_beside_fn beside_work, void *beside_context,
                                                 splatad_stream_t stream) {
    SPLATAD_REQUIRE(tile_size > 0, "isect_tiles: tile_size is zero");
    SPLATAD_REQUIRE(remap != nullptr, "isect_tiles: remap is null");
    TileGrid g{tile_size, tile_width, tile_height, 0.f, 0.f, nullptr};
    return isect_fill<false>(g, total, N, nullptr, means2d, radii, depths, C, 1, n_isects, tiles_per_gauss,
                             workspace, lists, isect_ids, flatten_ids, tile_offsets, (hipStream_t)stream,
                             remap, tiles_out, (hipStream_t)beside_stream, beside_work, beside_context,
                             remap_offsets);
}

extern "C" int splatad_isect_lidar_tiles_count(uint64_t total, uint32_t N,
                                               const int64_t *camera_ids, const float *means2d,
                                               const float *radii, const float *depths, uint32_t C,
                                               const float *elev_boundaries,
                                               float tile_azim_resolution, float min_azim,
                                               uint32_t tile_width, uint32_t tile_height, int sort,
                                               int32_t *tiles_per_gauss, void *workspace,
                                               int64_t *n_isects_host, splatad_stream_t stream) {
    SPLATAD_REQUIRE(elev_boundaries != nullptr, "isect_lidar_tiles: elev_boundaries is null");
    TileGrid g{0u, tile_width, tile_height, tile_azim_resolution, min_azim, elev_boundaries};
    return isect_count<true>(g, total, N, camera_ids, means2d, radii, depths, C, sort, tiles_per_gauss,
                             workspace, n_isects_host, (hipStream_t)stream);
}

extern "C" int splatad_isect_lidar_tiles_fill(uint64_t total, uint32_t N,
                                              const int64_t *camera_ids, const float *means2d,
                                              const float *radii, const float *depths, uint32_t C,
                                              const float *elev_boundaries,
                                              float tile_azim_resolution, float min_azim,
                                              uint32_t tile_width, uint32_t tile_height, int sort,
                                              int64_t n_isects, const int32_t *tiles_per_gauss,
                                              void *workspace, void *lists, int64_t *isect_ids,
                                              int32_t *flatten_ids, int32_t *tile_offsets,
                                              splatad_stream_t stream) {
    SPLATAD_REQUIRE(elev_boundaries != nullptr, "isect_lidar_tiles: elev_boundaries is null");
    TileGrid g{0u, tile_width, tile_height, tile_azim_resolution, min_azim, elev_boundaries};
    return isect_fill<true>(g, total, N, camera_ids, means2d, radii, depths, C, sort, n_isects,
                            tiles_per_gauss, workspace, lists, isect_ids, flatten_ids, tile_offsets,
                            (hipStream_t)stream);
}

extern "C" int splatad_isect_offset_encode(int64_t n_isects, const int64_t *isect_ids, uint32_t C,
                                           uint32_t n_tiles, int32_t *offsets,
                                           splatad_stream_t stream) {
    const int64_t total_tiles = (int64_t)C * n_tiles;
    if (total_tiles == 0) return 0;
    SPLATAD_REQUIRE(offsets != nullptr, "isect_offset_encode: offsets is null");
    if (n_isects == 0) {
        hipLaunchKernelGGL(fill_zero_i32_kernel, grid_for((uint64_t)total_tiles),
                           dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, offsets, total_tiles);
        SPLATAD_LAUNCH_CHECK();
        return 0;
    }
    SPLATAD_REQUIRE(isect_ids != nullptr, "isect_offset_encode: isect_ids is null");
    hipLaunchKernelGGL(isect_offset_encode_kernel, grid_for((uint64_t)n_isects),
                       dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, n_isects, isect_ids, n_tiles,
                       splatad_bit_width(n_tiles), total_tiles, offsets);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}
