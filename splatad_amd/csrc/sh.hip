// Real spherical-harmonic colour evaluation (degree 0..4) and its VJP for gfx950.
//
// One lane per direction: the basis values are computed once and contracted with the three
// colour channels.  The basis follows Sloan's "Efficient Spherical Harmonic Evaluation"
// (JCGT 2013) with the Condon-Shortley phase kept, the convention of
// gsplat/cuda/csrc/sh.cu:13-93 of the reference.  The azimuthal factors are
// C_m + i S_m = (x + i y)^m, so their derivatives are m (C_{m-1}, S_{m-1}) in x and
// m (-S_{m-1}, C_{m-1}) in y; the backward pass uses those closed forms.
#include "common.h"
#include "sh_eval.h"

namespace {

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

// f(lds_index, global_index, row, column) for every used float of the workgroup's `rows` rows
template <typename F>
__device__ __forceinline__ void sh_for_each_float(const ShRows &r, uint32_t rows, F &&f) {
    uint32_t row = threadIdx.x / r.K3, col = threadIdx.x % r.K3;
    const uint32_t total = rows * r.K3;
    for (uint32_t e = threadIdx.x; e < total; e += blockDim.x) {
        if (col < r.used) f(row * (r.used + 1) + col, e, row, col);
        row += r.dq;
        col += r.dr;
        if (col >= r.K3) { col -= r.K3; ++row; }
    }
}

// Where a kernel takes its directions, masks and coefficient rows from.  The plain operator
// reads them from tensors; the rendering pipeline (VIEW) derives them from the scene: the
// direction of row e is the Gaussian's mean minus the position of its sensor, the row is
// active when the Gaussian's projected radius is positive, and the coefficient row is the
// Gaussian's own unless every sensor has its own coefficients.  This replaces the inverse of
// the view matrices, the gathers and the mask tensor of gsplat/rendering.py:325-345.
struct ShView {
    const float *means;                       // [N, 3]
    const float *viewmats;                    // [C, 4, 4], rows [A | t], last row (0, 0, 0, 1)
    const int64_t *camera_ids, *gaussian_ids; // per row for packed input, else null
    const int32_t *radii;                     // [n, 2]
    uint32_t N;
    int coeffs_per_sensor; // coefficient rows: 1 = one per row e, 0 = one per Gaussian
};

// Direction, activity and coefficient row of row e
template <bool VIEW>
__device__ __forceinline__ bool sh_row(uint32_t e, const ShView &v, const float *dirs,
                                       const uint8_t *masks, float &dx, float &dy, float &dz,
                                       size_t &coeff_row) {
    if (!VIEW) {
        coeff_row = e;
        if (masks != nullptr && !masks[e]) return false;
        dx = dirs[(size_t)e * 3]; dy = dirs[(size_t)e * 3 + 1]; dz = dirs[(size_t)e * 3 + 2];
        return true;
    }
    const uint32_t g = v.gaussian_ids ? (uint32_t)v.gaussian_ids[e] : e % v.N;
    const uint32_t cam = v.camera_ids ? (uint32_t)v.camera_ids[e] : e / v.N;
    coeff_row = v.coeffs_per_sensor ? (v.camera_ids ? (size_t)cam * v.N + g : (size_t)e) : (size_t)g;
    // the mean is requested together with the radius, not after the test on it
    const int32_t radius = v.radii[(size_t)e * 2];
    const float mx = v.means[(size_t)g * 3], my = v.means[(size_t)g * 3 + 1], mz = v.means[(size_t)g * 3 + 2];
    float px, py, pz;
    sensor_position(v.viewmats + (size_t)cam * 16, px, py, pz);
    dx = mx - px; dy = my - py; dz = mz - pz;
    return radius > 0;
}

// Forward: every lane reads its own row; the rows are read completely, so the cache lines a
// wavefront touches are all used (measured faster than staging through LDS).  VIEW also
// applies the colour activation of the pipeline, max(c + 1/2, 0) (gsplat/rendering.py:347),
// and writes rows of `stride` floats, with the depth as fourth channel when given (:351).
template <bool VIEW>
__device__ __forceinline__ void sh_fwd_row(uint32_t e, uint32_t K, uint32_t degree, const ShView &view,
                                           const float *__restrict__ dirs, const float *__restrict__ coeffs,
                                           const uint8_t *__restrict__ masks, const float *__restrict__ depths,
                                           uint32_t stride, float *__restrict__ colors,
                                           const int32_t *__restrict__ remap,
                                           const int32_t *__restrict__ remap_offsets = nullptr) {
    float r = 0.f, g = 0.f, b = 0.f;
    float dx = 0.f, dy = 0.f, dz = 0.f;
    size_t coeff_row;
    // remap: only the active rows have a place in the output, row e at remap[e]
    uint32_t at = e;
    if (VIEW && remap != nullptr)
        at = (uint32_t)(remap[e] + (remap_offsets != nullptr ? remap_offsets[e / SPLATAD_THREADS] : 0));
    const bool active = sh_row<VIEW>(e, view, dirs, masks, dx, dy, dz, coeff_row);
    if (VIEW && remap != nullptr && !active) return;
    if (active) sh_color(degree, coeffs + coeff_row * K * 3, dx, dy, dz, r, g, b);
    float *out = colors + (size_t)at * stride;
    if (VIEW) {
        out[0] = fmaxf(r + 0.5f, 0.f);
        out[1] = fmaxf(g + 0.5f, 0.f);
        out[2] = fmaxf(b + 0.5f, 0.f);
        if (depths != nullptr) out[3] = depths[e];
    } else {
        out[0] = r; out[1] = g; out[2] = b;
    }
}

template <bool VIEW>
__global__ void __launch_bounds__(SPLATAD_THREADS)
sh_fwd_kernel(uint32_t n, uint32_t K, uint32_t degree, ShView view, const float *__restrict__ dirs,
              const float *__restrict__ coeffs, const uint8_t *__restrict__ masks,
              const float *__restrict__ depths, uint32_t stride, float *__restrict__ colors,
              const int32_t *__restrict__ remap, const int32_t *__restrict__ remap_offsets) {
    const uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    sh_fwd_row<VIEW>(e, K, degree, view, dirs, coeffs, masks, depths, stride, colors, remap, remap_offsets);
}

// The colour cache of the compositing kernel that evaluates colours itself
// (rasterize_fwd.hip): a float4 per row, NaN = not evaluated yet.  Two launches prepare it.
// The first fills it with NaN and adds up, per workgroup, opacity x tiles over the visible rows
// (tiles estimated from the radii): divided by the number of tiles, the opacity a tile's list
// carries.  Where that is large the tiles saturate on the first entries of their lists and the
// compositing kernel evaluates those few rows itself; where it is small the lists are
// consumed to their ends, every wavefront of the compositing kernel would meet a missing row
// in every batch, and evaluating all visible rows beforehand, a row per lane, is cheaper: the
// second launch does that unless the sum reaches `enough`.
constexpr uint32_t kCachePartials = 1024; // workgroups of the first launch at most

__global__ void __launch_bounds__(SPLATAD_THREADS)
sh_cache_clear_kernel(uint32_t n, ShView view, const float *__restrict__ opacities, float inv_tile,
                      float tile_w, float tile_h, float4 *__restrict__ cache, float *__restrict__ partials) {
    __shared__ float s_sum[SPLATAD_THREADS / SPLATAD_WAVE];
    const float nan = __uint_as_float(0x7FC00000u);
    float sum = 0.f;
    // four rows per trip, their radii requested together: with many rows per lane (several
    // sensors' worth) the loop is bound by the latency of its loads, not by the bytes
    const uint32_t stride = gridDim.x * blockDim.x;
    const int2 *radii2 = reinterpret_cast<const int2 *>(view.radii);
    for (uint32_t e0 = blockIdx.x * blockDim.x + threadIdx.x; e0 < n; e0 += 4 * stride) {
        int2 r[4];
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const uint64_t e = (uint64_t)e0 + (uint64_t)k * stride;
            r[k] = e < n ? radii2[e] : make_int2(0, 0);
        }
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const uint64_t e = (uint64_t)e0 + (uint64_t)k * stride;
            if (e < n) cache[e] = make_float4(nan, nan, nan, nan);
        }
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const uint32_t e = e0 + k * stride; // (below n where the radii are positive)
            if (r[k].x > 0 && r[k].y > 0) {
                const uint32_t g = view.gaussian_ids ? (uint32_t)view.gaussian_ids[e] : e % view.N;
                sum += opacities[g] * fminf(2.f * (float)r[k].x * inv_tile + 1.f, tile_w) *
                       fminf(2.f * (float)r[k].y * inv_tile + 1.f, tile_h);
            }
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, SPLATAD_WAVE);
    if ((threadIdx.x & (SPLATAD_WAVE - 1)) == 0) s_sum[threadIdx.x / SPLATAD_WAVE] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (uint32_t w = 0; w < blockDim.x / SPLATAD_WAVE; ++w) total += s_sum[w];
        partials[blockIdx.x] = total;
    }
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
sh_cache_fill_kernel(uint32_t n, uint32_t K, uint32_t degree, ShView view, const float *__restrict__ coeffs,
                     const float *__restrict__ depths, float *__restrict__ cache,
                     const float *__restrict__ partials, uint32_t n_partials, float enough) {
    __shared__ float s_sum[SPLATAD_THREADS / SPLATAD_WAVE];
    float sum = 0.f; // every workgroup adds up the same numbers in the same order
    for (uint32_t k = threadIdx.x; k < n_partials; k += blockDim.x) sum += partials[k];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, SPLATAD_WAVE);
    if ((threadIdx.x & (SPLATAD_WAVE - 1)) == 0) s_sum[threadIdx.x / SPLATAD_WAVE] = sum;
    __syncthreads();
    float total = 0.f;
    for (uint32_t w = 0; w < blockDim.x / SPLATAD_WAVE; ++w) total += s_sum[w];
    if (total >= enough) return; // uniform across the launch
    for (uint32_t e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) {
        if (view.radii[(size_t)e * 2] <= 0) continue; // rows no list names keep their NaN
        sh_fwd_row<true>(e, K, degree, view, nullptr, coeffs, nullptr, depths, 4u, cache, nullptr);
        if (depths == nullptr) cache[(size_t)e * 4 + 3] = 0.f;
    }
}

// VIEW: v_colors are rows of `stride` floats, the gradients of the activated colours
// `colors` (same layout), so a channel passes its gradient on only where it is positive.
// DIRS: the gradients of the directions are wanted too.  A compile-time switch, so that the
// coefficient loads stand outside any branch and the compiler can issue a row's loads together
// (behind a run-time test each basis function waited for its own three loads).
template <bool VIEW, bool DIRS>
__global__ void __launch_bounds__(SPLATAD_THREADS)
sh_bwd_kernel(uint32_t n, ShRows rows, uint32_t degree, ShView view, const float *__restrict__ dirs,
              const float *__restrict__ coeffs, const uint8_t *__restrict__ masks,
              const float *__restrict__ colors, uint32_t stride,
              const float *__restrict__ v_colors, float *__restrict__ v_coeffs,
              float *__restrict__ v_dirs, int scatter) {
    extern __shared__ float s_rows[];
    // scatter: v_coeffs has the layout of coeffs, cleared by the caller, and every row's
    // gradients are added at the coefficient row it read (packed rows: the Gaussian's)
    uint32_t *s_dest = reinterpret_cast<uint32_t *>(s_rows + (size_t)blockDim.x * (rows.used + 1));
    const uint32_t first = blockIdx.x * blockDim.x;
    const uint32_t here = min(blockDim.x, n - first);
    const uint32_t e = first + threadIdx.x;
    // every lane writes its row of coefficient gradients to LDS, from where the workgroup
    // stores them coalesced; rows of masked directions are zeros (their gradients are zero)
    float *row = s_rows + (size_t)threadIdx.x * (rows.used + 1);
    float dx = 0.f, dy = 0.f, dz = 0.f, vr = 0.f, vg = 0.f, vb = 0.f;
    size_t coeff_row = 0;
    bool active = false;
    if (e < n) {
        active = sh_row<VIEW>(e, view, dirs, masks, dx, dy, dz, coeff_row);
        const float *vc = v_colors + (size_t)e * stride;
        vr = vc[0]; vg = vc[1]; vb = vc[2]; // read whether active or not: no wait for the test
        if (VIEW) {
            const float *col = colors + (size_t)e * stride;
            vr = col[0] > 0.f ? vr : 0.f;
            vg = col[1] > 0.f ? vg : 0.f;
            vb = col[2] > 0.f ? vb : 0.f;
        }
        if (!active) vr = vg = vb = 0.f;
    }
    // A workgroup none of whose rows takes a gradient (rows that no pixel composited: most rows
    // of a frame that saturates in its nearest Gaussians) only has zeros to write, and writes
    // them without evaluating a basis or passing through LDS.
    if (!__syncthreads_or(vr != 0.f || vg != 0.f || vb != 0.f)) {
        if (DIRS && e < n && (active || VIEW))
            v_dirs[(size_t)e * 3] = v_dirs[(size_t)e * 3 + 1] = v_dirs[(size_t)e * 3 + 2] = 0.f;
        if (scatter) return; // nothing to add
        float *gout = v_coeffs + (size_t)first * rows.K3;
        const uint32_t total = here * rows.K3;
        if (rows.used == rows.K3 && (reinterpret_cast<uintptr_t>(gout) & 15) == 0) {
            float4 *g4 = reinterpret_cast<float4 *>(gout);
            for (uint32_t i = threadIdx.x; i < total / 4; i += blockDim.x) g4[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            for (uint32_t i = (total & ~3u) + threadIdx.x; i < total; i += blockDim.x) gout[i] = 0.f;
        } else {
            sh_for_each_float(rows, here, [&](uint32_t, uint32_t f, uint32_t, uint32_t) { gout[f] = 0.f; });
        }
        return;
    }
    if (e < n) {
        if (scatter) s_dest[threadIdx.x] = (uint32_t)coeff_row;
        const float *cf = coeffs + coeff_row * rows.K3;
        const float inorm = active ? rsqrtf(dx * dx + dy * dy + dz * dz) : 0.f;
        const float x = dx * inorm, y = dy * inorm, z = active ? dz * inorm : 1.f;
        float gx = 0.f, gy = 0.f, gz = 0.f;
        // the whole coefficient row is requested before the first use, one memory round trip
        // instead of one per degree
        // (only for rows that take a gradient: where few of the visible rows were composited
        // -- a frame that saturates in its nearest Gaussians -- the coefficient rows are most
        // of what this kernel would read)
        float c[DIRS ? 75 : 1] = {};
        if (DIRS && active && (vr != 0.f || vg != 0.f || vb != 0.f)) {
            sh_load_band<0>(c, cf);
            if (degree >= 1) sh_load_band<1>(c, cf); // uniform
            if (degree >= 2) sh_load_band<2>(c, cf);
            if (degree >= 3) sh_load_band<3>(c, cf);
            if (degree >= 4) sh_load_band<4>(c, cf);
        }
        sh_for_each_basis(degree, x, y, z, [&](int k, float v, float bx, float by, float bz) {
            if (DIRS) {
                const float w = c[k * 3] * vr + c[k * 3 + 1] * vg + c[k * 3 + 2] * vb;
                gx += w * bx; gy += w * by; gz += w * bz;
            }
            row[k * 3] = v * vr;
            row[k * 3 + 1] = v * vg;
            row[k * 3 + 2] = v * vb;
        });
        if (DIRS && (active || VIEW)) {
            // through the normalisation: (I - n n^T) g / |d|; zero for inactive rows
            const float dot = gx * x + gy * y + gz * z;
            v_dirs[(size_t)e * 3] = (gx - dot * x) * inorm;
            v_dirs[(size_t)e * 3 + 1] = (gy - dot * y) * inorm;
            v_dirs[(size_t)e * 3 + 2] = (gz - dot * z) * inorm;
        }
    }
    __syncthreads();
    if (scatter) { // uniform
        sh_for_each_float(rows, here, [&](uint32_t l, uint32_t, uint32_t row_here, uint32_t col) {
            const float v = s_rows[l];
            if (v != 0.f) atomicAdd(v_coeffs + (size_t)s_dest[row_here] * rows.K3 + col, v);
        });
        return;
    }
    float *gout = v_coeffs + (size_t)first * rows.K3;
    sh_for_each_float(rows, here, [&](uint32_t l, uint32_t f, uint32_t, uint32_t) { gout[f] = s_rows[l]; });
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
    *bytes = (size_t)SPLATAD_THREADS * (r.used + 1) * sizeof(float) + SPLATAD_THREADS * sizeof(uint32_t);
    if (*bytes > 64 * 1024)
        SPLATAD_CHECK_HIP(hipFuncSetAttribute((const void *)kernel,
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)*bytes));
    return 0;
}

static int sh_check(uint32_t K, uint32_t degree) {
    SPLATAD_REQUIRE(degree <= 4, "spherical harmonics: degree %u is above 4", degree);
    SPLATAD_REQUIRE((degree + 1) * (degree + 1) <= K, "spherical harmonics: %u bases for degree %u", K, degree);
    return 0;
}

template <bool VIEW>
static int sh_forward(uint32_t n, uint32_t K, uint32_t degree, const ShView &view, const float *dirs,
                      const float *coeffs, const uint8_t *masks, const float *depths,
                      uint32_t stride, float *colors, hipStream_t stream, const int32_t *remap = nullptr,
                      const int32_t *remap_offsets = nullptr) {
    hipLaunchKernelGGL(sh_fwd_kernel<VIEW>, dim3((n + SPLATAD_THREADS - 1) / SPLATAD_THREADS),
                       dim3(SPLATAD_THREADS), 0, stream, n, K, degree, view, dirs, coeffs, masks,
                       depths, stride, colors, remap, remap_offsets);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

template <bool VIEW>
static int sh_backward(uint32_t n, uint32_t K, uint32_t degree, const ShView &view, const float *dirs,
                       const float *coeffs, const uint8_t *masks, const float *colors,
                       uint32_t stride, const float *v_colors, float *v_coeffs, float *v_dirs,
                       hipStream_t stream, int scatter = 0) {
    const ShRows r = sh_rows(K, degree);
    size_t lds = 0;
    const dim3 grid((n + SPLATAD_THREADS - 1) / SPLATAD_THREADS);
    if (v_dirs != nullptr) {
        if (int rc = sh_lds(sh_bwd_kernel<VIEW, true>, r, &lds)) return rc;
        hipLaunchKernelGGL((sh_bwd_kernel<VIEW, true>), grid, dim3(SPLATAD_THREADS), lds, stream, n, r,
                           degree, view, dirs, coeffs, masks, colors, stride, v_colors, v_coeffs, v_dirs, scatter);
    } else {
        if (int rc = sh_lds(sh_bwd_kernel<VIEW, false>, r, &lds)) return rc;
        hipLaunchKernelGGL((sh_bwd_kernel<VIEW, false>), grid, dim3(SPLATAD_THREADS), lds, stream, n, r,
                           degree, view, dirs, coeffs, masks, colors, stride, v_colors, v_coeffs, v_dirs, scatter);
    }
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

static int sh_view_args(uint32_t n, uint32_t C, uint32_t N, const float *means, const float *viewmats,
                        const int64_t *camera_ids, const int64_t *gaussian_ids, const int32_t *radii,
                        int coeffs_per_sensor, ShView *view) {
    SPLATAD_REQUIRE(means && viewmats && radii, "view colours: null pointer argument");
    SPLATAD_REQUIRE((camera_ids == nullptr) == (gaussian_ids == nullptr),
                    "view colours: camera_ids and gaussian_ids go together");
    SPLATAD_REQUIRE(N > 0 && C > 0, "view colours: no Gaussians or no sensors");
    SPLATAD_REQUIRE(camera_ids != nullptr || (uint64_t)n == (uint64_t)C * N,
                    "view colours: %u rows for %u sensors x %u Gaussians", n, C, N);
    *view = ShView{means, viewmats, camera_ids, gaussian_ids, radii, N, coeffs_per_sensor};
    return 0;
}

} // namespace

extern "C" int splatad_sh_fwd(uint32_t n, uint32_t K, uint32_t degree, const float *dirs,
                              const float *coeffs, const uint8_t *masks, float *colors,
                              splatad_stream_t stream) {
    if (int rc = sh_check(K, degree)) return rc;
    if (n == 0) return 0;
    SPLATAD_REQUIRE(dirs && coeffs && colors, "spherical harmonics: null pointer argument");
    return sh_forward<false>(n, K, degree, ShView{}, dirs, coeffs, masks, nullptr, 3, colors,
                             (hipStream_t)stream);
}

extern "C" int splatad_sh_bwd(uint32_t n, uint32_t K, uint32_t degree, const float *dirs,
                              const float *coeffs, const uint8_t *masks, const float *v_colors,
                              float *v_coeffs, float *v_dirs, splatad_stream_t stream) {
    if (int rc = sh_check(K, degree)) return rc;
    if (n == 0) return 0;
    SPLATAD_REQUIRE(dirs && coeffs && v_colors && v_coeffs, "spherical harmonics: null pointer argument");
    return sh_backward<false>(n, K, degree, ShView{}, dirs, coeffs, masks, nullptr, 3, v_colors,
                              v_coeffs, v_dirs, (hipStream_t)stream);
}

extern "C" int splatad_view_colors_fwd(uint32_t n, uint32_t C, uint32_t N, uint32_t K,
                                       uint32_t degree, const float *means, const float *viewmats,
                                       const int64_t *camera_ids, const int64_t *gaussian_ids,
                                       const int32_t *radii, const float *coeffs,
                                       int coeffs_per_sensor, const float *depths, float *colors,
                                       splatad_stream_t stream) {
    if (int rc = sh_check(K, degree)) return rc;
    if (n == 0) return 0;
    ShView view;
    if (int rc = sh_view_args(n, C, N, means, viewmats, camera_ids, gaussian_ids, radii,
                              coeffs_per_sensor, &view)) return rc;
    SPLATAD_REQUIRE(coeffs && colors, "view colours: null pointer argument");
    return sh_forward<true>(n, K, degree, view, nullptr, coeffs, nullptr, depths, depths ? 4u : 3u,
                            colors, (hipStream_t)stream);
}

extern "C" size_t splatad_view_colors_cache_bytes(uint64_t n_rows) {
    return (size_t)n_rows * 16 + kCachePartials * sizeof(float);
}

extern "C" int splatad_view_colors_cache(uint32_t n, uint32_t C, uint32_t N, uint32_t K, uint32_t degree,
                                         const float *means, const float *viewmats,
                                         const int64_t *camera_ids, const int64_t *gaussian_ids,
                                         const int32_t *radii, const float *coeffs,
                                         int coeffs_per_sensor, const float *depths,
                                         const float *opacities,
                                         uint32_t tile_size, uint32_t tile_width, uint32_t tile_height,
                                         float min_opacity_per_tile, float *cache,
                                         splatad_stream_t stream) {
    if (int rc = sh_check(K, degree)) return rc;
    if (n == 0) return 0;
    ShView view;
    if (int rc = sh_view_args(n, C, N, means, viewmats, camera_ids, gaussian_ids, radii,
                              coeffs_per_sensor, &view)) return rc;
    SPLATAD_REQUIRE(coeffs && opacities && cache, "view colours: null pointer argument");
    SPLATAD_REQUIRE(tile_size > 0 && tile_width > 0 && tile_height > 0, "view colours: empty tile grid");
    const float n_tiles = (float)C * (float)tile_width * (float)tile_height;
    float *partials = cache + (size_t)n * 4;
    uint32_t wgs = (n + SPLATAD_THREADS - 1) / SPLATAD_THREADS;
    if (wgs > kCachePartials) wgs = kCachePartials;
    hipLaunchKernelGGL(sh_cache_clear_kernel, dim3(wgs), dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, n,
                       view, opacities, 1.f / (float)tile_size, (float)tile_width, (float)tile_height,
                       reinterpret_cast<float4 *>(cache), partials);
    SPLATAD_LAUNCH_CHECK();
    // (a launch that mostly finds nothing to do: no more workgroups than fill the GPU a few times)
    const uint32_t rows_wgs = (n + SPLATAD_THREADS - 1) / SPLATAD_THREADS;
    hipLaunchKernelGGL(sh_cache_fill_kernel, dim3(rows_wgs < 2048u ? rows_wgs : 2048u),
                       dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, n, K, degree, view, coeffs, depths, cache,
                       (const float *)partials, wgs, min_opacity_per_tile * n_tiles);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

extern "C" int splatad_view_colors_fwd_remapped(uint32_t C, uint32_t N, uint32_t K, uint32_t degree,
                                                const float *means, const float *viewmats,
                                                const int32_t *radii, const int32_t *remap,
                                                const int32_t *remap_offsets,
                                                const float *coeffs, int coeffs_per_sensor,
                                                const float *depths, float *colors,
                                                splatad_stream_t stream) {
    if (int rc = sh_check(K, degree)) return rc;
    const uint64_t n = (uint64_t)C * N;
    if (n == 0) return 0;
    SPLATAD_REQUIRE(n < (1ull << 31), "view colours: C*N must be below 2^31");
    ShView view;
    if (int rc = sh_view_args((uint32_t)n, C, N, means, viewmats, nullptr, nullptr, radii, coeffs_per_sensor,
                              &view)) return rc;
    SPLATAD_REQUIRE(coeffs && colors && remap, "view colours: null pointer argument");
    return sh_forward<true>((uint32_t)n, K, degree, view, nullptr, coeffs, nullptr, depths, depths ? 4u : 3u,
                            colors, (hipStream_t)stream, remap, remap_offsets);
}

extern "C" int splatad_view_colors_bwd(uint32_t n, uint32_t C, uint32_t N, uint32_t K,
                                       uint32_t degree, const float *means, const float *viewmats,
                                       const int64_t *camera_ids, const int64_t *gaussian_ids,
                                       const int32_t *radii, const float *coeffs,
                                       int coeffs_per_sensor, uint32_t channels, const float *colors,
                                       const float *v_colors, int scatter_coeffs, float *v_coeffs,
                                       float *v_dirs, splatad_stream_t stream) {
    if (int rc = sh_check(K, degree)) return rc;
    if (n == 0) return 0;
    ShView view;
    if (int rc = sh_view_args(n, C, N, means, viewmats, camera_ids, gaussian_ids, radii,
                              coeffs_per_sensor, &view)) return rc;
    SPLATAD_REQUIRE(channels == 3 || channels == 4, "view colours: %u channels per row", channels);
    SPLATAD_REQUIRE(coeffs && colors && v_colors && v_coeffs, "view colours: null pointer argument");
    return sh_backward<true>(n, K, degree, view, nullptr, coeffs, nullptr, colors, channels, v_colors,
                             v_coeffs, v_dirs, (hipStream_t)stream, scatter_coeffs);
}
