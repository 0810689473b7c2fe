"""CPU oracle bindings -- TEST INFRASTRUCTURE ONLY.

ctypes front-end of ``oracle/splatad_oracle.c`` (a plain-C restatement of the
reference's rendering path).  Only ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py`` may import this package; the shipped
``splatad_amd`` package never does.

All functions take and return numpy arrays (float32 inputs; outputs are
float32 for ``precision="f32"`` and float64 for ``"f64"``).  Integer outputs
(tile intersections, sort order, offsets) exist only in single precision,
because the reference computes the tile bounds in float32
(``gsplat/cuda/csrc/rasterization.cu:46-56, 321-357``).
"""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIBS = {}


def build(force: bool = False) -> None:
    """Compile both oracle libraries with gcc (``make -C oracle``)."""
    if force:
        subprocess.check_call(["make", "-C", _DIR, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _DIR], stdout=subprocess.DEVNULL)


def _lib(precision: str):
    if precision not in ("f32", "f64"):
        raise ValueError(precision)
    if precision not in _LIBS:
        path = os.path.join(_DIR, f"liboracle_{precision}.so")
        if not os.path.exists(path):
            build()
        _LIBS[precision] = ctypes.CDLL(path)
    return _LIBS[precision]


def _real(precision):
    return np.float32 if precision == "f32" else np.float64


def _f32(a):
    return None if a is None else np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _p(a):
    if a is None:
        return ctypes.c_void_p(0)
    assert a.flags["C_CONTIGUOUS"]
    return ctypes.c_void_p(a.ctypes.data)


def set_num_threads(n: int) -> None:
    """OpenMP thread count used by the oracle loops (``OMP_NUM_THREADS``)."""
    os.environ["OMP_NUM_THREADS"] = str(n)
    try:
        omp = ctypes.CDLL("libgomp.so.1")
        omp.omp_set_num_threads(int(n))
    except OSError:
        pass


# ---------------------------------------------------------------------------
# projection
# ---------------------------------------------------------------------------
def projection_fwd(means, covars, quats, scales, velocities, viewmats, Ks, width, height,
                   linear_velocity, angular_velocity, rolling_shutter_time, eps2d=0.3,
                   near_plane=0.01, far_plane=1e10, radius_clip=0.0, calc_compensations=False,
                   precision="f32"):
    """Restates ``fully_fused_projection_fwd`` (projection.cu:605-751).

    Returns (radii int32[C,N,2], means2d, depths, conics, compensations|None, pix_vels).
    """
    lib, rt = _lib(precision), _real(precision)
    means = _f32(means); covars = _f32(covars); quats = _f32(quats); scales = _f32(scales)
    velocities = _f32(velocities); viewmats = _f32(viewmats); Ks = _f32(Ks)
    lv = _f32(linear_velocity); av = _f32(angular_velocity); rs = _f32(rolling_shutter_time)
    C, N = viewmats.shape[0], means.shape[0]
    radii = np.zeros((C, N, 2), np.int32)
    means2d = np.zeros((C, N, 2), rt); depths = np.zeros((C, N), rt)
    conics = np.zeros((C, N, 3), rt); pix_vels = np.zeros((C, N, 2), rt)
    comps = np.zeros((C, N), rt) if calc_compensations else None
    fn = getattr(lib, f"oracle_{precision}_projection_fwd")
    fn.restype = None
    fn(ctypes.c_int(C), ctypes.c_int(N), _p(means), _p(covars), _p(quats), _p(scales),
       _p(velocities), _p(viewmats), _p(Ks), ctypes.c_int(width), ctypes.c_int(height), _p(lv),
       _p(av), _p(rs), ctypes.c_float(eps2d), ctypes.c_float(near_plane),
       ctypes.c_float(far_plane), ctypes.c_float(radius_clip), _p(radii), _p(means2d),
       _p(depths), _p(conics), _p(comps), _p(pix_vels))
    return radii, means2d, depths, conics, comps, pix_vels


def lidar_projection_fwd(means, covars, quats, scales, velocities, viewmats, min_elevation,
                         max_elevation, min_azimuth, max_azimuth, linear_velocity,
                         angular_velocity, rolling_shutter_time, eps2d=0.01, near_plane=0.01,
                         far_plane=1e10, radius_clip=0.0, calc_compensations=False,
                         precision="f32"):
    """Restates ``fully_fused_lidar_projection_fwd`` (projection.cu:2268-2417).

    Returns (radii[C,N,2], means2d, depths, conics, compensations|None, pix_vels[C,N,3],
    depth_compensations[C,N,2]).
    """
    lib, rt = _lib(precision), _real(precision)
    means = _f32(means); covars = _f32(covars); quats = _f32(quats); scales = _f32(scales)
    velocities = _f32(velocities); viewmats = _f32(viewmats)
    lv = _f32(linear_velocity); av = _f32(angular_velocity); rs = _f32(rolling_shutter_time)
    C, N = viewmats.shape[0], means.shape[0]
    radii = np.zeros((C, N, 2), rt)
    means2d = np.zeros((C, N, 2), rt); depths = np.zeros((C, N), rt)
    conics = np.zeros((C, N, 3), rt); pix_vels = np.zeros((C, N, 3), rt)
    dcomps = np.zeros((C, N, 2), rt)
    comps = np.zeros((C, N), rt) if calc_compensations else None
    fn = getattr(lib, f"oracle_{precision}_lidar_projection_fwd")
    fn.restype = None
    fn(ctypes.c_int(C), ctypes.c_int(N), _p(means), _p(covars), _p(quats), _p(scales),
       _p(velocities), _p(viewmats), ctypes.c_float(min_elevation), ctypes.c_float(max_elevation),
       ctypes.c_float(min_azimuth), ctypes.c_float(max_azimuth), _p(lv), _p(av), _p(rs),
       ctypes.c_float(eps2d), ctypes.c_float(near_plane), ctypes.c_float(far_plane),
       ctypes.c_float(radius_clip), _p(radii), _p(means2d), _p(depths), _p(conics), _p(comps),
       _p(pix_vels), _p(dcomps))
    return radii, means2d, depths, conics, comps, pix_vels, dcomps


def spherical_harmonics(degree, dirs, coeffs, masks=None, precision="f32"):
    """Restates ``compute_sh_fwd`` (sh.cu:13-93, 355-374); masked rows are zero."""
    lib, rt = _lib(precision), _real(precision)
    dirs = _f32(dirs); coeffs = _f32(coeffs)
    K = coeffs.shape[-2]
    n = dirs.size // 3
    m = None if masks is None else np.ascontiguousarray(np.asarray(masks, dtype=np.uint8))
    colors = np.zeros(dirs.shape, rt)
    fn = getattr(lib, f"oracle_{precision}_sh_fwd")
    fn.restype = None
    fn(ctypes.c_long(n), ctypes.c_int(K), ctypes.c_int(degree), _p(dirs), _p(coeffs), _p(m),
       _p(colors))
    return colors


# ---------------------------------------------------------------------------
# intersection / sort / offsets (single precision only)
# ---------------------------------------------------------------------------
def bit_width(v: int) -> int:
    return int(v).bit_length()


def _isect(lidar, means2d, radii, depths, tile_size, tile_w, tile_h, elev_boundaries,
           tile_azim_res, min_azim, sort, n_cameras, camera_ids):
    lib = _lib("f32")
    means2d = _f32(means2d); depths = _f32(depths)
    radii = _f32(radii) if lidar else np.ascontiguousarray(np.asarray(radii, dtype=np.int32))
    eb = _f32(elev_boundaries)
    packed = means2d.ndim == 2
    if packed:
        total = means2d.shape[0]; N = 0; C = n_cameras
        cam = np.ascontiguousarray(np.asarray(camera_ids, dtype=np.int64))
    else:
        C, N = means2d.shape[:2]; total = C * N; cam = None
    tpg = np.zeros(depths.shape, np.int32)
    lib.oracle_isect_count.restype = ctypes.c_long
    n_isects = lib.oracle_isect_count(
        ctypes.c_int(lidar), ctypes.c_long(total), _p(means2d), _p(radii),
        ctypes.c_uint32(tile_size), ctypes.c_uint32(tile_w), ctypes.c_uint32(tile_h), _p(eb),
        ctypes.c_float(tile_azim_res), ctypes.c_float(min_azim), _p(tpg))
    ids = np.zeros((n_isects,), np.int64); flat = np.zeros((n_isects,), np.int32)
    lib.oracle_isect_emit.restype = None
    lib.oracle_isect_emit(
        ctypes.c_int(lidar), ctypes.c_long(total), ctypes.c_long(N), _p(cam), _p(means2d),
        _p(radii), _p(depths), ctypes.c_uint32(tile_size), ctypes.c_uint32(tile_w),
        ctypes.c_uint32(tile_h), _p(eb), ctypes.c_float(tile_azim_res), ctypes.c_float(min_azim),
        _p(ids), _p(flat))
    if sort and n_isects:
        end_bit = 32 + bit_width(tile_w * tile_h) + bit_width(C)
        lib.oracle_sort_pairs.restype = None
        lib.oracle_sort_pairs(ctypes.c_long(n_isects), ctypes.c_int(end_bit), _p(ids), _p(flat))
    return tpg, ids, flat


def isect_tiles(means2d, radii, depths, tile_size, tile_width, tile_height, sort=True,
                n_cameras=None, camera_ids=None):
    """Restates ``isect_tiles`` (rasterization.cu:15-216)."""
    return _isect(0, means2d, radii, depths, tile_size, tile_width, tile_height, None, 0.0, 0.0,
                  sort, n_cameras, camera_ids)


def isect_lidar_tiles(means2d, radii, depths, elev_boundaries, tile_azim_resolution, min_azim,
                      sort=True, n_cameras=None, camera_ids=None, n_tiles_azim=None):
    """Restates ``isect_lidar_tiles`` (rasterization.cu:287-529).

    ``n_tiles_azim`` defaults to the reference's full turn of tile columns; a caller of the
    kernel-level interface may pass fewer (a sector)."""
    import math
    if n_tiles_azim is None:
        # rasterization.cu:435-436: float32 division, ceil
        n_tiles_azim = int(math.ceil(float(np.float32(360.0) / np.float32(tile_azim_resolution))))
    n_tiles_elev = int(np.asarray(elev_boundaries).shape[0] - 1)
    return _isect(1, means2d, radii, depths, 0, n_tiles_azim, n_tiles_elev, elev_boundaries,
                  tile_azim_resolution, min_azim, sort, n_cameras, camera_ids)


def isect_offset_encode(isect_ids, n_cameras, tile_width, tile_height):
    """Restates ``isect_offset_encode`` (rasterization.cu:218-285)."""
    lib = _lib("f32")
    ids = np.ascontiguousarray(np.asarray(isect_ids, dtype=np.int64))
    offsets = np.zeros((n_cameras, tile_height, tile_width), np.int32)
    lib.oracle_isect_offset_encode.restype = None
    lib.oracle_isect_offset_encode(ctypes.c_long(ids.shape[0]), _p(ids),
                                   ctypes.c_uint32(n_cameras),
                                   ctypes.c_uint32(tile_width * tile_height), _p(offsets))
    return offsets


# ---------------------------------------------------------------------------
# lidar point binning
# ---------------------------------------------------------------------------
def map_points_to_lidar_tiles(points2d, elev_boundaries, tile_azim_resolution, min_azim,
                              n_cameras=None, camera_ids=None, sort=True):
    """Restates ``map_points_to_lidar_tiles`` (rasterization.cu:596-770).

    Returns (tile_ids int64[total], flatten_ids int32[total])."""
    import math
    lib = _lib("f32")
    pts = _f32(points2d); eb = _f32(elev_boundaries)
    if pts.ndim == 2:
        total, N = pts.shape[0], 0
        cam = np.ascontiguousarray(np.asarray(camera_ids, dtype=np.int64))
    else:
        C, N = pts.shape[:2]; total = C * N; cam = None
    n_az = int(math.ceil(float(np.float32(360.0) / np.float32(tile_azim_resolution))))
    n_el = int(eb.shape[0] - 1)
    ids = np.zeros((total,), np.int64); flat = np.zeros((total,), np.int32)
    lib.oracle_map_points_to_lidar_tiles.restype = None
    lib.oracle_map_points_to_lidar_tiles(
        ctypes.c_long(total), ctypes.c_long(N), _p(cam), _p(pts), _p(eb),
        ctypes.c_float(tile_azim_resolution), ctypes.c_float(min_azim), ctypes.c_uint32(n_az),
        ctypes.c_uint32(n_el), _p(ids), _p(flat))
    if sort and total:
        lib.oracle_sort_pairs.restype = None
        lib.oracle_sort_pairs(ctypes.c_long(total), ctypes.c_int(64), _p(ids), _p(flat))
    return ids, flat


def points_mapping_offset_encode(point_ids, n_lidars, tile_width, tile_height):
    """Restates ``points_mapping_offset_encode`` (rasterization.cu:531-594)."""
    lib = _lib("f32")
    ids = np.ascontiguousarray(np.asarray(point_ids, dtype=np.int64))
    offsets = np.zeros((n_lidars, tile_height, tile_width), np.int32)
    lib.oracle_points_mapping_offset_encode.restype = None
    lib.oracle_points_mapping_offset_encode(
        ctypes.c_long(ids.shape[0]), _p(ids), ctypes.c_uint32(n_lidars),
        ctypes.c_uint32(tile_width * tile_height), _p(offsets))
    return offsets


def populate_image_from_points(points, image_width, image_height, tile_width, tile_height,
                               tile_offsets, flatten_ids):
    """Restates ``populate_image_from_points`` (rasterization.cu:772-833)."""
    lib = _lib("f32")
    pts = _f32(points)
    offs = np.ascontiguousarray(np.asarray(tile_offsets, dtype=np.int32))
    flat = np.ascontiguousarray(np.asarray(flatten_ids, dtype=np.int32))
    C, gh, gw = offs.shape
    image = np.zeros((C, image_height, image_width, 5), np.float32)
    lib.oracle_populate_image_from_points.restype = None
    lib.oracle_populate_image_from_points(
        ctypes.c_uint32(C), ctypes.c_long(flat.shape[0]), _p(pts), ctypes.c_uint32(image_width),
        ctypes.c_uint32(image_height), ctypes.c_uint32(tile_width), ctypes.c_uint32(tile_height),
        ctypes.c_uint32(gw), ctypes.c_uint32(gh), _p(offs), _p(flat), _p(image))
    return image


def compute_relocation(opacities, scales, ratios, binoms):
    """Restates ``compute_relocation`` (gsplat/relocation.py:10-49, relocation.cu:4-30)."""
    lib = _lib("f32")
    o = _f32(opacities); sc = _f32(scales); b = _f32(binoms)
    n_max = b.shape[0]
    r = np.ascontiguousarray(np.clip(np.asarray(ratios), 1, n_max).astype(np.int32))
    new_o = np.zeros_like(o); new_s = np.zeros_like(sc)
    lib.oracle_compute_relocation.restype = None
    lib.oracle_compute_relocation(ctypes.c_long(o.shape[0]), _p(o), _p(sc), _p(r), _p(b),
                                  ctypes.c_int(n_max), _p(new_o), _p(new_s))
    return new_o, new_s


# ---------------------------------------------------------------------------
# rasterization
# ---------------------------------------------------------------------------
class nudged_thresholds:
    """Context manager: the fused compositing functions take their discontinuous decisions
    at alpha_scale / 255, t_scale * 1e-4, median_scale * 0.5 and range - threshold +
    asum_shift instead of the reference's values.  With it a parity test finds the pixels
    whose value depends on a decision within a few rounding errors of its threshold."""

    def __init__(self, precision="f64", alpha_scale=1.0, t_scale=1.0, median_scale=1.0,
                 asum_shift=0.0):
        self.precision = precision
        self.args = (alpha_scale, t_scale, median_scale, asum_shift)

    def _set(self, a, t, m, s):
        fn = getattr(_lib(self.precision), f"oracle_{self.precision}_set_thresholds")
        fn.restype = None
        fn(ctypes.c_double(a), ctypes.c_double(t), ctypes.c_double(m), ctypes.c_double(s))

    def __enter__(self):
        self._set(*self.args)
        return self

    def __exit__(self, *exc):
        self._set(1.0, 1.0, 1.0, 0.0)
        return False


def rasterize_to_pixels_fwd(means2d, conics, colors, opacities, pix_vels, rolling_shutter_time,
                            backgrounds, width, height, tile_size, isect_offsets, flatten_ids,
                            precision="f32"):
    """Restates ``rasterize_to_pixels_fwd`` (rasterization.cu:1360-1518).

    Returns (render_colors[C,H,W,D], render_alphas[C,H,W,1], last_ids int32[C,H,W]).
    """
    lib, rt = _lib(precision), _real(precision)
    means2d = _f32(means2d); conics = _f32(conics); colors = _f32(colors)
    opacities = _f32(opacities); pix_vels = _f32(pix_vels); rs = _f32(rolling_shutter_time)
    bg = _f32(backgrounds)
    offs = np.ascontiguousarray(np.asarray(isect_offsets, dtype=np.int32))
    flat = np.ascontiguousarray(np.asarray(flatten_ids, dtype=np.int32))
    C, th, tw = offs.shape
    D = colors.shape[-1]
    rc = np.zeros((C, height, width, D), rt); ra = np.zeros((C, height, width, 1), rt)
    last = np.zeros((C, height, width), np.int32)
    fn = getattr(lib, f"oracle_{precision}_rasterize_to_pixels_fwd")
    fn.restype = None
    fn(ctypes.c_int(C), ctypes.c_long(flat.shape[0]), ctypes.c_int(D), _p(means2d), _p(conics),
       _p(colors), _p(opacities), _p(pix_vels), _p(rs), _p(bg), ctypes.c_int(width),
       ctypes.c_int(height), ctypes.c_int(tile_size), ctypes.c_int(tw), ctypes.c_int(th),
       _p(offs), _p(flat), _p(rc), _p(ra), _p(last))
    return rc, ra, last


def rasterize_to_points_fwd(means2d, conics, colors, opacities, pix_vels, depth_compensations,
                            backgrounds, raster_pts, width, height, tile_width, tile_height,
                            compute_alpha_sum_until_points, threshold, isect_offsets, flatten_ids,
                            depth_channel_idx, precision="f32"):
    """Restates ``rasterize_to_points_fwd`` (rasterization.cu:2021-2219).

    Returns (render_colors, render_alphas, last_ids, alpha_sum_until_points|None,
    median_depths), the order of the reference's C++ op.
    """
    lib, rt = _lib(precision), _real(precision)
    means2d = _f32(means2d); conics = _f32(conics); colors = _f32(colors)
    opacities = _f32(opacities); pix_vels = _f32(pix_vels); dc = _f32(depth_compensations)
    bg = _f32(backgrounds); rp = _f32(raster_pts)
    offs = np.ascontiguousarray(np.asarray(isect_offsets, dtype=np.int32))
    flat = np.ascontiguousarray(np.asarray(flatten_ids, dtype=np.int32))
    C, gh, gw = offs.shape
    D = colors.shape[-1]
    rc = np.zeros((C, height, width, D), rt); ra = np.zeros((C, height, width, 1), rt)
    asum = np.zeros((C, height, width, 1), rt) if compute_alpha_sum_until_points else None
    med = np.zeros((C, height, width, 1), rt)
    last = np.zeros((C, height, width), np.int32)
    fn = getattr(lib, f"oracle_{precision}_rasterize_to_points_fwd")
    fn.restype = None
    fn(ctypes.c_int(C), ctypes.c_long(flat.shape[0]), ctypes.c_int(D), _p(means2d), _p(conics),
       _p(colors), _p(opacities), _p(pix_vels), _p(dc), _p(bg), _p(rp), ctypes.c_int(width),
       ctypes.c_int(height), ctypes.c_int(tile_width), ctypes.c_int(tile_height),
       ctypes.c_int(gw), ctypes.c_int(gh), ctypes.c_int(bool(compute_alpha_sum_until_points)),
       ctypes.c_float(threshold), _p(offs), _p(flat), ctypes.c_int(depth_channel_idx), _p(rc),
       _p(ra), _p(asum), _p(last), _p(med))
    return rc, ra, last, asum, med


# ---------------------------------------------------------------------------
# (Gaussian, pixel) index lists and compositing over them
# ---------------------------------------------------------------------------
def _indices_in_range(lidar, range_start, range_end, transmittances, means2d, conics, opacities,
                      pix_vels, sensor, width, height, tile_width, tile_height, isect_offsets,
                      flatten_ids, precision):
    lib = _lib(precision)
    trans = _f32(transmittances); means2d = _f32(means2d); conics = _f32(conics)
    opacities = _f32(opacities); pix_vels = _f32(pix_vels); sensor = _f32(sensor)
    offs = np.ascontiguousarray(np.asarray(isect_offsets, dtype=np.int32))
    flat = np.ascontiguousarray(np.asarray(flatten_ids, dtype=np.int32))
    C, gh, gw = offs.shape
    N = means2d.shape[1]
    fn = getattr(lib, f"oracle_{precision}_rasterize_to_indices_in_range")
    fn.restype = None
    cap = 2 ** 40

    def run(counts, starts, gids, idx):
        fn(ctypes.c_int(bool(lidar)), ctypes.c_long(min(int(range_start), cap)),
           ctypes.c_long(min(int(range_end), cap)), ctypes.c_int(C), ctypes.c_long(N),
           ctypes.c_long(flat.shape[0]), _p(trans), _p(means2d), _p(conics), _p(opacities),
           _p(pix_vels), _p(sensor), ctypes.c_int(width), ctypes.c_int(height),
           ctypes.c_int(tile_width), ctypes.c_int(tile_height), ctypes.c_int(gw), ctypes.c_int(gh),
           _p(offs), _p(flat), _p(counts), _p(starts), _p(gids), _p(idx))

    counts = np.zeros(C * height * width, np.int32)
    run(counts, None, None, None)
    starts = np.ascontiguousarray(np.cumsum(counts, dtype=np.int64) - counts)
    total = int(counts.sum(dtype=np.int64))
    gids = np.zeros(total, np.int64); idx = np.zeros(total, np.int64)
    if total:
        run(None, starts, gids, idx)
    return gids, idx % (width * height), idx // (width * height)


def rasterize_to_indices_in_range(range_start, range_end, transmittances, means2d, conics,
                                  opacities, pix_vels, width, height, tile_size, isect_offsets,
                                  flatten_ids, rolling_shutter_time=None, precision="f32"):
    """Restates ``rasterize_to_indices_in_range`` (_wrapper.py:1115-1198; kernel and its two
    passes rasterization.cu:839-1092).  Returns (gaussian_ids, pixel_ids, camera_ids), int64."""
    C = np.asarray(means2d).shape[0]
    rs = np.zeros(C, np.float32) if rolling_shutter_time is None else rolling_shutter_time
    return _indices_in_range(False, range_start, range_end, transmittances, means2d, conics,
                             opacities, pix_vels, rs, width, height, tile_size, tile_size,
                             isect_offsets, flatten_ids, precision)


def rasterize_to_indices_in_range_lidar(range_start, range_end, transmittances, means2d, conics,
                                        opacities, pix_vels, raster_pts, width, height,
                                        tile_width, tile_height, isect_offsets, flatten_ids,
                                        precision="f32"):
    """Restates ``rasterize_to_indices_in_range_lidar`` (_wrapper.py:1200-1281; kernel
    rasterization.cu:1100-1358)."""
    return _indices_in_range(True, range_start, range_end, transmittances, means2d, conics,
                             opacities, pix_vels, raster_pts, width, height, tile_width,
                             tile_height, isect_offsets, flatten_ids, precision)


def _composite_rays(alphas, values, rays, n_rays):
    """Per ray, in list order: T_k = prod_{j<k} (1 - alpha_j), weight_k = T_k alpha_k; returns
    (sum_k weight_k values_k [n_rays, D], sum_k weight_k [n_rays, 1]).  This is what the
    reference obtains from nerfacc's render_weight_from_alpha and accumulate_along_rays
    (_torch_impl.py:694-704); nerfacc is not vendored by the reference and no version is
    pinned, so the published definition is restated as a scalar loop."""
    out = np.zeros((n_rays, values.shape[-1]), np.float64)
    acc = np.zeros((n_rays, 1), np.float64)
    T, prev = 1.0, -1
    for k in range(alphas.shape[0]):
        r = int(rays[k])
        if r != prev:
            T, prev = 1.0, r
        w = T * float(alphas[k])
        out[r] += w * values[k]
        acc[r, 0] += w
        T *= 1.0 - float(alphas[k])
    return out, acc


def accumulate(means2d, conics, opacities, colors, pix_vels, rolling_shutter_time, gaussian_ids,
               pixel_ids, camera_ids, width, height):
    """Restates ``accumulate`` (_torch_impl.py:610-706) in float64.  Returns
    (renders[C,H,W,D], alphas[C,H,W,1])."""
    f = lambda a: np.asarray(a, np.float64)
    means2d, conics, opacities, colors, pix_vels = map(f, (means2d, conics, opacities, colors, pix_vels))
    rs = f(rolling_shutter_time)
    g, p, c = (np.asarray(a, np.int64) for a in (gaussian_ids, pixel_ids, camera_ids))
    C, D = means2d.shape[0], colors.shape[-1]
    col, row = p % width, p // width
    roll = rs[c] * (row / (height - 1) - 0.5)
    d = means2d[c, g] + roll[:, None] * pix_vels[c, g] - (np.stack([col, row], -1) + 0.5)
    cn = conics[c, g]
    sigma = 0.5 * (cn[:, 0] * d[:, 0] ** 2 + cn[:, 2] * d[:, 1] ** 2) + cn[:, 1] * d[:, 0] * d[:, 1]
    alpha = np.minimum(opacities[c, g] * np.exp(-sigma), 0.999)
    out, acc = _composite_rays(alpha, colors[c, g], c * height * width + p, C * height * width)
    return out.reshape(C, height, width, D), acc.reshape(C, height, width, 1)


def accumulate_lidar(means2d, conics, opacities, lidar_features, pix_vels, depth_compensations,
                     raster_pts, gaussian_ids, pixel_ids, camera_ids, width, height,
                     compute_alpha_sum_until_pts, compute_alpha_sum_until_pts_threshold):
    """Restates ``accumulate_lidar`` (_torch_impl.py:709-830) in float64.  Returns
    (renders, alphas, alpha_sum_until_points | None)."""
    f = lambda a: np.asarray(a, np.float64)
    means2d, conics, opacities, feats, pix_vels, dc, pts = map(
        f, (means2d, conics, opacities, lidar_features, pix_vels, depth_compensations, raster_pts))
    g, p, c = (np.asarray(a, np.int64) for a in (gaussian_ids, pixel_ids, camera_ids))
    C, D = means2d.shape[0], feats.shape[-1]
    col, row = p % width, p // width
    pt = pts[c, row, col]
    roll = pt[:, 3]
    d = np.mod(means2d[c, g] + roll[:, None] * pix_vels[c, g][:, :2] - pt[:, :2] + 180, 360) - 180
    cn = conics[c, g]
    sigma = 0.5 * (cn[:, 0] * d[:, 0] ** 2 + cn[:, 2] * d[:, 1] ** 2) + cn[:, 1] * d[:, 0] * d[:, 1]
    alpha = np.minimum(opacities[c, g] * np.exp(-sigma), 0.999)
    vals = feats[c, g].copy()
    vals[:, -1] += (d * dc[c, g]).sum(-1) + pix_vels[c, g][:, 2] * roll
    rays, n_rays = c * height * width + p, C * height * width
    out, acc = _composite_rays(alpha, vals, rays, n_rays)
    asum = None
    if compute_alpha_sum_until_pts:
        before = feats[c, g][:, -1] < pt[:, 2] - compute_alpha_sum_until_pts_threshold
        asum = np.zeros(n_rays, np.float64)
        np.add.at(asum, rays, np.where(before, alpha, 0.0))
        asum = asum.reshape(C, height, width, 1)
    return out.reshape(C, height, width, D), acc.reshape(C, height, width, 1), asum
