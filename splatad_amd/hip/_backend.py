"""Loader of libsplatad_hip.so and the `_C`-shaped operator table built on it.

Counterpart of the reference's extension loader and pybind11 module
(gsplat/cuda/_backend.py:80-142, gsplat/cuda/csrc/ext.cpp:4-52): `_C.<name>(*args)` takes the
same positional arguments and returns the same tuples of tensors as the reference's C++ ops
(gsplat/cuda/csrc/bindings.h:123-468).  Behind it sits a plain C ABI (include/splatad_hip.h)
called through ctypes with raw device pointers; outputs and workspaces are allocated here with
torch so that they live in torch's caching allocator, on torch's current stream.

There is no CPU path: without the built library, or with non-GPU tensors, the ops raise.
"""
import ctypes
import threading
import weakref
import math
import os
from typing import Optional

import torch
from torch import Tensor

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_DIR, "libsplatad_hip.so")

_lib = None


ABI_VERSION = 11  # splatad_abi_version() of the library these bindings were written for


def load_library():
    """Returns the ctypes handle of libsplatad_hip.so; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP kernels first with "
                "`python -m splatad_amd.build` (needs hipcc). There is no CPU fallback."
            )
        lib = ctypes.CDLL(LIB_PATH)
        lib.splatad_last_error.restype = ctypes.c_char_p
        lib.splatad_abi_version.restype = ctypes.c_int
        if lib.splatad_abi_version() != ABI_VERSION:
            raise RuntimeError(
                f"{LIB_PATH} has ABI version {lib.splatad_abi_version()}, this package needs {ABI_VERSION}: "
                "rebuild it with `python -m splatad_amd.build`")
        for name in ("splatad_projection_packed_workspace_bytes", "splatad_isect_workspace_bytes",
                     "splatad_isect_lists_bytes", "splatad_view_colors_cache_bytes",
                     "splatad_map_points_to_lidar_tiles_workspace_bytes",
                     "splatad_rasterize_to_indices_workspace_bytes",
                     "splatad_rasterize_bwd_workspace_bytes"):
            getattr(lib, name).restype = ctypes.c_size_t
        _lib = lib
    return _lib


def _check(rc: int):
    if rc != 0:
        msg = load_library().splatad_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"splatad_hip error {rc}: {msg}")


def _in(t: Optional[Tensor], name: str, dtype=torch.float32) -> Optional[Tensor]:
    """Input check (bindings.h:9-13 of the reference): GPU, contiguous, expected dtype."""
    if t is None:
        return None
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if t.dtype != dtype:
        raise RuntimeError(f"{name} must have dtype {dtype}, got {t.dtype}")
    if t.data_ptr() % 16 != 0 and t.numel() > 0:
        t = t.clone()  # the kernels use 8/16-byte vector accesses
    return t


def _p(t: Optional[Tensor]):
    return ctypes.c_void_p(0 if t is None or t.numel() == 0 else t.data_ptr())


_redirect = threading.local()  # .stream: where this thread's library calls go instead, see library_stream


def _stream(device):
    """Handle of torch's current stream on the device (the raw query: the Stream object that
    torch.cuda.current_stream() builds costs several microseconds per call), or the stream that
    library_stream() has put in its place."""
    other = getattr(_redirect, "stream", None)
    if other is not None:
        return other
    index = device.index if device.index is not None else torch.cuda.current_device()
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(index))


class library_stream:
    """`with library_stream(handle)`: the calls this thread makes into the library enqueue on the
    stream `handle` (a ctypes pointer) instead of torch's current one.  For the callbacks that an
    intersection call runs beside its sort; torch's own kernels do not follow, so nothing inside
    may launch one (allocations are fine)."""

    def __init__(self, handle):
        self.handle = handle

    def __enter__(self):
        self.before = getattr(_redirect, "stream", None)
        _redirect.stream = self.handle

    def __exit__(self, *exc):
        _redirect.stream = self.before


class _on:
    """`with _on(device)`: torch.cuda.device(device), entered only when another device is current."""

    def __init__(self, device):
        self._ctx = None
        if device.index is not None and device.index != torch.cuda.current_device():
            self._ctx = torch.cuda.device(device)

    def __enter__(self):
        if self._ctx is not None:
            self._ctx.__enter__()

    def __exit__(self, *exc):
        if self._ctx is not None:
            return self._ctx.__exit__(*exc)
        return False


_u32, _i32, _i64, _u64, _f32 = ctypes.c_uint32, ctypes.c_int, ctypes.c_int64, ctypes.c_uint64, ctypes.c_float


# int (*splatad_beside_fn)(void *context, splatad_stream_t stream)
_BESIDE_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p)


def _zeros_many(device, *shapes):
    """Zero-filled float32 tensors of the given shapes (None stays None), carved out of one
    buffer that a single fill clears: gradient outputs come in groups of four to seven, and a
    fill per tensor costs more in launches than in bandwidth."""
    counts = [0 if sh is None else int(math.prod(sh)) for sh in shapes]
    sizes = [(n + 63) // 64 * 64 for n in counts]  # pieces of whole 256 bytes
    pool = torch.zeros((sum(sizes),), dtype=torch.float32, device=device)
    out, at = [], 0
    for sh, n, size in zip(shapes, counts, sizes):
        out.append(None if sh is None else pool[at:at + n].view(tuple(sh)))
        at += size
    return out


def _gathered_outputs(device, means, covars, quats, scales, viewmats, velocities):
    """Gradient outputs of a projection backward over unpacked input, by shape (None stays None):
    the kernel stores every per-Gaussian row itself, only the pose gradient is accumulated and
    has to start at zero."""
    f = dict(dtype=torch.float32, device=device)
    out = [None if sh is None else torch.empty(tuple(sh), **f) for sh in (means, covars, quats, scales)]
    out.append(None if viewmats is None else torch.zeros(tuple(viewmats), **f))
    out.append(None if velocities is None else torch.empty(tuple(velocities), **f))
    return out


def _zeros_like_many(*tensors):
    ref = next(t for t in tensors if t is not None)
    return _zeros_many(ref.device, *(None if t is None else t.shape for t in tensors))


def _bwd_workspace(lib, total: int, channels: int, lidar: bool, device) -> Optional[Tensor]:
    """Scratch for the packed gradient accumulation of the compositing backward, or None where
    it does not pay: with few channels a Gaussian's gradients fit one 64-byte record and the
    kernel, otherwise bound by its global atomics, runs twice as fast (measured: 0.57 instead of
    1.15 ms on the camera bench scene); with the 33 channels of a lidar call the kernel is
    bound by its arithmetic and clearing and unpacking 192-byte records only adds time."""
    nbytes = lib.splatad_rasterize_bwd_workspace_bytes(_u64(total), _u32(channels), _i32(bool(lidar)))
    return _workspace(nbytes, device) if nbytes <= total * 64 else None


def _workspace(nbytes: int, device) -> Tensor:
    return torch.empty((max(int(nbytes), 256),), dtype=torch.uint8, device=device)


class _Ops:
    """Operator table with the names and calling conventions of the reference's `_C`."""

    # ------------------------------------------------------------------ projection
    def fully_fused_projection_fwd(self, means, covars, quats, scales, velocities, viewmats, Ks,
                                   image_width, image_height, linear_velocity, angular_velocity,
                                   rolling_shutter_time, eps2d, near_plane, far_plane, radius_clip,
                                   calc_compensations):
        lib = load_library()
        means = _in(means, "means"); covars = _in(covars, "covars"); quats = _in(quats, "quats")
        scales = _in(scales, "scales"); velocities = _in(velocities, "velocities")
        viewmats = _in(viewmats, "viewmats"); Ks = _in(Ks, "Ks")
        lv = _in(linear_velocity, "linear_velocity"); av = _in(angular_velocity, "angular_velocity")
        rs = _in(rolling_shutter_time, "rolling_shutter_time")
        N, C, dev = means.shape[0], viewmats.shape[0], means.device
        f = dict(dtype=torch.float32, device=dev)
        radii = torch.empty((C, N, 2), dtype=torch.int32, device=dev)
        means2d = torch.empty((C, N, 2), **f); depths = torch.empty((C, N), **f)
        conics = torch.empty((C, N, 3), **f); pix_vels = torch.empty((C, N, 2), **f)
        comps = torch.empty((C, N), **f) if calc_compensations else None
        with _on(dev):
            _check(lib.splatad_projection_fwd(
                _u32(C), _u32(N), _p(means), _p(covars), _p(quats), _p(scales), _p(velocities),
                _p(viewmats), _p(Ks), _u32(image_width), _u32(image_height), _p(lv), _p(av), _p(rs),
                _f32(eps2d), _f32(near_plane), _f32(far_plane), _f32(radius_clip), _p(radii),
                _p(means2d), _p(depths), _p(conics), _p(comps), _p(pix_vels), _stream(dev)))
        return radii, means2d, depths, conics, comps, pix_vels

    def fully_fused_projection_packed_fwd(self, means, covars, quats, scales, velocities, viewmats,
                                          Ks, image_width, image_height, linear_velocity,
                                          angular_velocity, rolling_shutter_time, eps2d, near_plane,
                                          far_plane, radius_clip, calc_compensations,
                                          isect_grid=None, beside=None):
        """isect_grid = (tile_size, tile_width, tile_height): the counting call also counts the
        tile intersections of the rows it keeps, and their lists are made here, ahead of the
        packed outputs (the GPU is waiting for that work, not for the outputs); they travel with
        the returned radii, see _isect().

        beside: an object with `side` (a torch stream or None), `requests` and `results` (dicts).
        With isect_grid and a side stream, the kernels that write the packed outputs go to that
        stream, ordered behind the binning by the intersection call itself, and run beside the
        segment sort; the caller joins the stream before anything reads the outputs on its own
        stream (_isect() with the lists of these rows does not read them; without them it waits
        for the stream left on the radii).  requests["color_cache"] = (degrees_to_use, coeffs,
        with_depth, tile_size, tile_width, tile_height, min_opacity_per_tile) asks for what
        view_colors_cache() makes of the packed rows; requests["colors"] = (degrees_to_use, coeffs,
        with_depth) and requests["opacities"] = opacities [N] ask for what view_colors_fwd() and
        the gather opacities[gaussian_ids] (* compensations) would give for the returned rows;
        they are made on the same stream and left in results under the same keys."""
        lib = load_library()
        means = _in(means, "means"); covars = _in(covars, "covars"); quats = _in(quats, "quats")
        scales = _in(scales, "scales"); velocities = _in(velocities, "velocities")
        viewmats = _in(viewmats, "viewmats"); Ks = _in(Ks, "Ks")
        lv = _in(linear_velocity, "linear_velocity"); av = _in(angular_velocity, "angular_velocity")
        rs = _in(rolling_shutter_time, "rolling_shutter_time")
        N, C, dev = means.shape[0], viewmats.shape[0], means.device
        f = dict(dtype=torch.float32, device=dev)
        with _on(dev):
            ws = _workspace(lib.splatad_projection_packed_workspace_bytes(_u32(C), _u32(N)), dev)
            nnz_host, n_isects_host = _i64(0), _i64(0)
            head = (_u32(C), _u32(N), _p(means), _p(covars), _p(quats), _p(scales), _p(velocities),
                    _p(viewmats), _p(Ks), _u32(image_width), _u32(image_height), _p(lv), _p(av), _p(rs),
                    _f32(eps2d), _f32(near_plane), _f32(far_plane), _f32(radius_clip),
                    _i32(bool(calc_compensations)))
            main = _stream(dev)
            if isect_grid is None:
                _check(lib.splatad_projection_packed_count(*head, _p(ws), ctypes.byref(nnz_host), main))
            else:
                # the counting call also starts the tile intersection, on the dense rows in its
                # workspace, while the host waits for the counts
                n_tiles = int(isect_grid[1]) * int(isect_grid[2])
                assert n_tiles.bit_length() + int(C).bit_length() <= 32
                isect_ws = _workspace(lib.splatad_isect_workspace_bytes(_u64(C * N), _u32(C), _u32(n_tiles)), dev)
                _check(lib.splatad_projection_packed_count_tiles(
                    *head, *(_u32(v) for v in isect_grid), _p(ws), _p(isect_ws), ctypes.byref(nnz_host),
                    ctypes.byref(n_isects_host), main))
            nnz = int(nnz_host.value)
            isect_result = side = None
            requests = getattr(beside, "requests", None) or {}

            def write_outputs(work):
                """Allocates the packed outputs and what was asked for of them, and enqueues the
                kernels that write them on the stream `work`."""
                indptr = torch.empty((C + 1,), dtype=torch.int32, device=dev)
                camera_ids = torch.empty((nnz,), dtype=torch.int64, device=dev)
                gaussian_ids = torch.empty((nnz,), dtype=torch.int64, device=dev)
                radii = torch.empty((nnz, 2), dtype=torch.int32, device=dev)
                means2d = torch.empty((nnz, 2), **f); depths = torch.empty((nnz,), **f)
                conics = torch.empty((nnz, 3), **f); pix_vels = torch.empty((nnz, 2), **f)
                comps = torch.empty((nnz,), **f) if calc_compensations else None
                opacities = requests.get("opacities")
                row_opacities = None
                if opacities is not None:
                    opacities = _in(opacities, "opacities")
                    assert opacities.shape == (N,), opacities.shape
                    row_opacities = torch.empty((nnz,), **f)
                _check(lib.splatad_projection_packed_fill(
                    _u32(C), _u32(N), _i64(nnz), _p(ws), _p(indptr), _p(camera_ids), _p(gaussian_ids),
                    _p(radii), _p(means2d), _p(depths), _p(conics), _p(comps), _p(pix_vels),
                    _p(opacities), _p(row_opacities), work))
                results = {}
                if row_opacities is not None:
                    results["opacities"] = row_opacities
                if "colors" in requests:
                    degree, coeffs, with_depth = requests["colors"]
                    coeffs = _in(coeffs, "coeffs")
                    colors = torch.empty((nnz, 4 if with_depth else 3), **f)
                    if nnz:
                        _check(lib.splatad_view_colors_fwd_packed(
                            _u32(C), _u32(N), _u32(coeffs.shape[-2]), _u32(degree), _p(means), _p(viewmats),
                            _p(ws), _p(coeffs), _i32(coeffs.dim() == 4), _i32(bool(with_depth)), _p(colors), work))
                    results["colors"] = colors
                if "color_cache" in requests:
                    # the colour cache of rasterize_to_pixels_sh_fwd for the packed rows, see
                    # view_colors_cache(); needs requests["opacities"]
                    degree, coeffs, with_depth, tile_size, tile_w, tile_h, limit = requests["color_cache"]
                    coeffs = _in(coeffs, "coeffs")
                    assert opacities is not None
                    words = lib.splatad_view_colors_cache_bytes(_u64(nnz)) // 4
                    buf = torch.empty((words,), **f)
                    if nnz:
                        _check(lib.splatad_view_colors_cache(
                            _u32(nnz), _u32(C), _u32(N), _u32(coeffs.shape[-2]), _u32(degree), _p(means),
                            _p(viewmats), _p(camera_ids), _p(gaussian_ids), _p(radii), _p(coeffs),
                            _i32(coeffs.dim() == 4), _p(depths if with_depth else None), _p(opacities),
                            _u32(tile_size), _u32(tile_w), _u32(tile_h), _f32(limit), _p(buf), work))
                    results["color_cache"] = buf[: nnz * 4].view(nnz, 4)
                return (indptr, camera_ids, gaussian_ids, radii, means2d, depths, conics, comps, pix_vels), results

            written = None
            work = main  # the stream of the kernels that write the outputs
            if isect_grid is not None:
                # first what the GPU is waiting for: the rest of the tile intersection
                side = getattr(beside, "side", None)
                if side is not None:
                    work = ctypes.c_void_p(side.cuda_stream)
                n_isects = int(n_isects_host.value)
                tile_w, tile_h = int(isect_grid[1]), int(isect_grid[2])
                tiles_per_gauss = torch.empty((nnz,), dtype=torch.int32, device=dev)
                isect_ids = torch.empty((n_isects,), dtype=torch.int64, device=dev)
                flatten_ids = torch.empty((n_isects,), dtype=torch.int32, device=dev)
                offsets = lists = None
                if n_isects:
                    offsets = torch.empty((C, tile_h, tile_w), dtype=torch.int32, device=dev)
                    lists = _workspace(lib.splatad_isect_lists_bytes(_u64(C * N), _i64(n_isects)), dev)
                else:
                    tiles_per_gauss.zero_()
                if n_isects or side is not None:  # (without lists the call only orders the side stream)
                    # Without a side stream of the caller's, the outputs are written from inside
                    # the intersection call, on a stream of the library's that runs beside the sort
                    # and is joined with it: the call hands that stream to this callback once.
                    # (The outputs are allocated in the callback too: by then the host is ahead
                    # of the GPU, whereas before this call the GPU waits for it; allocated before,
                    # the step took 0.410 instead of 0.400 ms.)
                    caught = []

                    def beside_work(_context, stream_handle):
                        nonlocal written
                        try:
                            written = write_outputs(ctypes.c_void_p(stream_handle))
                            return 0
                        except BaseException as e:  # (an exception must not cross the C frames)
                            caught.append(e)
                            return 1

                    callback = _BESIDE_FN(beside_work) if side is None else None
                    rc = lib.splatad_isect_tiles_fill_packed(
                        _u32(C), _u32(N), *(_u32(v) for v in isect_grid), _i64(n_isects), _p(ws),
                        _p(isect_ws), _p(lists), _p(tiles_per_gauss), _p(isect_ids), _p(flatten_ids),
                        _p(offsets), work if side is not None else None, callback, None, main)
                    if caught:
                        raise caught[0]
                    _check(rc)
                if offsets is not None:
                    # isect_offset_encode() on the same, unmodified tensor is free
                    isect_ids._splatad_tile_offsets = (offsets, isect_ids._version)
                isect_result = (tiles_per_gauss, isect_ids, flatten_ids)
            if written is None:
                written = write_outputs(work)
            (indptr, camera_ids, gaussian_ids, radii, means2d, depths, conics, comps, pix_vels), results = written
            if beside is not None:
                beside.results = results
            if side is not None:
                ws.record_stream(side)  # read there after the last use here
                radii._splatad_fill_stream = side
        if isect_grid is not None:
            # valid for these very tensors as long as nobody writes to them
            radii._splatad_isect_count = (tuple(int(v) for v in isect_grid), isect_result,
                                          radii._version, weakref.ref(means2d), means2d._version,
                                          weakref.ref(depths), depths._version, C)
        return indptr, camera_ids, gaussian_ids, radii, means2d, depths, conics, comps, pix_vels

    def fully_fused_lidar_projection_fwd(self, means, covars, quats, scales, velocities, viewmats,
                                         min_elevation, max_elevation, min_azimuth, max_azimuth,
                                         linear_velocity, angular_velocity, rolling_shutter_time,
                                         eps2d, near_plane, far_plane, radius_clip,
                                         calc_compensations):
        lib = load_library()
        means = _in(means, "means"); covars = _in(covars, "covars"); quats = _in(quats, "quats")
        scales = _in(scales, "scales"); velocities = _in(velocities, "velocities")
        viewmats = _in(viewmats, "viewmats")
        lv = _in(linear_velocity, "linear_velocity"); av = _in(angular_velocity, "angular_velocity")
        rs = _in(rolling_shutter_time, "rolling_shutter_time")
        N, C, dev = means.shape[0], viewmats.shape[0], means.device
        f = dict(dtype=torch.float32, device=dev)
        radii = torch.empty((C, N, 2), **f)
        means2d = torch.empty((C, N, 2), **f); depths = torch.empty((C, N), **f)
        conics = torch.empty((C, N, 3), **f); pix_vels = torch.empty((C, N, 3), **f)
        dcomps = torch.empty((C, N, 2), **f)
        comps = torch.empty((C, N), **f) if calc_compensations else None
        with _on(dev):
            _check(lib.splatad_lidar_projection_fwd(
                _u32(C), _u32(N), _p(means), _p(covars), _p(quats), _p(scales), _p(velocities),
                _p(viewmats), _f32(min_elevation), _f32(max_elevation), _f32(min_azimuth),
                _f32(max_azimuth), _p(lv), _p(av), _p(rs), _f32(eps2d), _f32(near_plane),
                _f32(far_plane), _f32(radius_clip), _p(radii), _p(means2d), _p(depths), _p(conics),
                _p(comps), _p(pix_vels), _p(dcomps), _stream(dev)))
        return radii, means2d, depths, conics, comps, pix_vels, dcomps

    def fully_fused_projection_bwd(self, means, covars, quats, scales, velocities, viewmats, Ks,
                                   image_width, image_height, linear_velocity, angular_velocity,
                                   rolling_shutter_time, eps2d, radii, conics, compensations,
                                   v_means2d, v_depths, v_conics, v_compensations, v_pix_vels,
                                   viewmats_requires_grad, velocities_requires_grad=False):
        return self._projection_bwd(means, covars, quats, scales, velocities, viewmats, Ks,
                                    image_width, image_height, linear_velocity, angular_velocity,
                                    rolling_shutter_time, eps2d, None, None, radii, conics,
                                    compensations, v_means2d, v_depths, v_conics, v_compensations,
                                    v_pix_vels, viewmats_requires_grad, False,
                                    velocities_requires_grad)

    def fully_fused_projection_packed_bwd(self, means, covars, quats, scales, velocities, viewmats,
                                          Ks, image_width, image_height, linear_velocity,
                                          angular_velocity, rolling_shutter_time, eps2d, camera_ids,
                                          gaussian_ids, conics, compensations, pix_vels, v_means2d,
                                          v_depths, v_conics, v_compensations, v_pix_vels,
                                          viewmats_requires_grad, sparse_grad,
                                          velocities_requires_grad=False):
        return self._projection_bwd(means, covars, quats, scales, velocities, viewmats, Ks,
                                    image_width, image_height, linear_velocity, angular_velocity,
                                    rolling_shutter_time, eps2d, camera_ids, gaussian_ids, None,
                                    conics, compensations, v_means2d, v_depths, v_conics,
                                    v_compensations, v_pix_vels, viewmats_requires_grad, sparse_grad,
                                    velocities_requires_grad)

    def _projection_bwd(self, means, covars, quats, scales, velocities, viewmats, Ks, image_width,
                        image_height, linear_velocity, angular_velocity, rolling_shutter_time, eps2d,
                        camera_ids, gaussian_ids, radii, conics, compensations, v_means2d, v_depths,
                        v_conics, v_compensations, v_pix_vels, viewmats_requires_grad, sparse_grad,
                        velocities_requires_grad):
        lib = load_library()
        means = _in(means, "means"); covars = _in(covars, "covars"); quats = _in(quats, "quats")
        scales = _in(scales, "scales"); velocities = _in(velocities, "velocities")
        viewmats = _in(viewmats, "viewmats"); Ks = _in(Ks, "Ks")
        lv = _in(linear_velocity, "linear_velocity"); av = _in(angular_velocity, "angular_velocity")
        rs = _in(rolling_shutter_time, "rolling_shutter_time")
        camera_ids = _in(camera_ids, "camera_ids", torch.int64)
        gaussian_ids = _in(gaussian_ids, "gaussian_ids", torch.int64)
        radii = _in(radii, "radii", torch.int32); conics = _in(conics, "conics")
        compensations = _in(compensations, "compensations")
        v_means2d = _in(v_means2d, "v_means2d"); v_depths = _in(v_depths, "v_depths")
        v_conics = _in(v_conics, "v_conics"); v_compensations = _in(v_compensations, "v_compensations")
        v_pix_vels = _in(v_pix_vels, "v_pix_vels")
        N, C, dev = means.shape[0], viewmats.shape[0], means.device
        packed = camera_ids is not None
        nnz = camera_ids.shape[0] if packed else 0
        rows = nnz if (packed and sparse_grad) else N
        f = dict(dtype=torch.float32, device=dev)
        shapes = ((rows, 3), (rows, 6) if covars is not None else None,
                  (rows, 4) if covars is None else None, (rows, 3) if covars is None else None,
                  viewmats.shape if viewmats_requires_grad else None,
                  velocities.shape if (velocities_requires_grad and velocities is not None) else None)
        v_means, v_covars, v_quats, v_scales, v_viewmats, v_velocities = (
            _zeros_many(dev, *shapes) if packed else _gathered_outputs(dev, *shapes))
        with _on(dev):
            _check(lib.splatad_projection_bwd(
                _u32(C), _u32(N), _p(means), _p(covars), _p(quats), _p(scales), _p(velocities),
                _p(viewmats), _p(Ks), _u32(image_width), _u32(image_height), _p(lv), _p(av), _p(rs),
                _f32(eps2d), _p(camera_ids), _p(gaussian_ids), _i64(nnz), _p(radii), _p(conics),
                _p(compensations), _p(v_means2d), _p(v_depths), _p(v_conics), _p(v_compensations),
                _p(v_pix_vels), _i32(bool(sparse_grad)), _p(v_means), _p(v_covars), _p(v_quats),
                _p(v_scales), _p(v_viewmats), _p(v_velocities), _stream(dev)))
        if velocities_requires_grad:
            return v_means, v_covars, v_quats, v_scales, v_viewmats, v_velocities
        return v_means, v_covars, v_quats, v_scales, v_viewmats

    def fully_fused_lidar_projection_bwd(self, means, covars, quats, scales, velocities, viewmats,
                                         min_elevation, max_elevation, min_azimuth, max_azimuth,
                                         linear_velocity, angular_velocity, rolling_shutter_time,
                                         eps2d, radii, conics, compensations, v_means2d, v_depths,
                                         v_conics, v_compensations, v_pix_vels,
                                         v_depth_compensations, viewmats_requires_grad,
                                         velocities_requires_grad=False):
        lib = load_library()
        means = _in(means, "means"); covars = _in(covars, "covars"); quats = _in(quats, "quats")
        scales = _in(scales, "scales"); velocities = _in(velocities, "velocities")
        viewmats = _in(viewmats, "viewmats")
        lv = _in(linear_velocity, "linear_velocity"); av = _in(angular_velocity, "angular_velocity")
        rs = _in(rolling_shutter_time, "rolling_shutter_time")
        radii = _in(radii, "radii"); conics = _in(conics, "conics")
        compensations = _in(compensations, "compensations")
        v_means2d = _in(v_means2d, "v_means2d"); v_depths = _in(v_depths, "v_depths")
        v_conics = _in(v_conics, "v_conics"); v_compensations = _in(v_compensations, "v_compensations")
        v_pix_vels = _in(v_pix_vels, "v_pix_vels")
        v_dc = _in(v_depth_compensations, "v_depth_compensations")
        N, C, dev = means.shape[0], viewmats.shape[0], means.device
        v_means, v_covars, v_quats, v_scales, v_viewmats, v_velocities = _gathered_outputs(
            dev, *(None if t is None else t.shape for t in (
                means, covars, quats if covars is None else None, scales if covars is None else None,
                viewmats if viewmats_requires_grad else None,
                velocities if (velocities_requires_grad and velocities is not None) else None)))
        with _on(dev):
            _check(lib.splatad_lidar_projection_bwd(
                _u32(C), _u32(N), _p(means), _p(covars), _p(quats), _p(scales), _p(velocities),
                _p(viewmats), _p(lv), _p(av), _p(rs), _f32(eps2d), _p(radii), _p(conics),
                _p(compensations), _p(v_means2d), _p(v_depths), _p(v_conics), _p(v_compensations),
                _p(v_pix_vels), _p(v_dc), _p(v_means), _p(v_covars), _p(v_quats), _p(v_scales),
                _p(v_viewmats), _p(v_velocities), _stream(dev)))
        if velocities_requires_grad:
            return v_means, v_covars, v_quats, v_scales, v_viewmats, v_velocities
        return v_means, v_covars, v_quats, v_scales, v_viewmats

    # ------------------------------------------------------------------ spherical harmonics
    def compute_sh_fwd(self, degrees_to_use, dirs, coeffs, masks):
        lib = load_library()
        dirs = _in(dirs, "dirs"); coeffs = _in(coeffs, "coeffs")
        masks = _in(masks, "masks", torch.bool)
        if coeffs.shape[-1] != 3:
            raise RuntimeError("coeffs must have last dimension 3")
        if dirs.shape[-1] != 3:
            raise RuntimeError("dirs must have last dimension 3")
        K, n, dev = coeffs.shape[-2], dirs.numel() // 3, dirs.device
        colors = torch.empty_like(dirs)
        with _on(dev):
            _check(lib.splatad_sh_fwd(_u32(n), _u32(K), _u32(degrees_to_use), _p(dirs), _p(coeffs),
                                      _p(masks), _p(colors), _stream(dev)))
        return colors

    def compute_sh_bwd(self, K, degrees_to_use, dirs, coeffs, masks, v_colors, compute_v_dirs):
        lib = load_library()
        dirs = _in(dirs, "dirs"); coeffs = _in(coeffs, "coeffs")
        masks = _in(masks, "masks", torch.bool); v_colors = _in(v_colors, "v_colors")
        n, dev = dirs.numel() // 3, dirs.device
        # the kernel writes the floats of the bases in use; the others must read zero
        full = (degrees_to_use + 1) ** 2 == K
        v_coeffs = torch.empty_like(coeffs) if full else torch.zeros_like(coeffs)
        v_dirs = torch.zeros_like(dirs) if compute_v_dirs else None
        with _on(dev):
            _check(lib.splatad_sh_bwd(_u32(n), _u32(K), _u32(degrees_to_use), _p(dirs), _p(coeffs),
                                      _p(masks), _p(v_colors), _p(v_coeffs), _p(v_dirs),
                                      _stream(dev)))
        return v_coeffs, v_dirs

    def view_colors_fwd(self, degrees_to_use, means, viewmats, camera_ids, gaussian_ids, radii,
                        coeffs, depths):
        """Colours max(SH(mean - sensor position) + 1/2, 0) per (sensor, Gaussian), with the
        depth as fourth channel when given.  No counterpart among the reference's C++ ops: it
        replaces the tensor operations of gsplat/rendering.py:325-351."""
        lib = load_library()
        means = _in(means, "means"); viewmats = _in(viewmats, "viewmats")
        camera_ids = _in(camera_ids, "camera_ids", torch.int64)
        gaussian_ids = _in(gaussian_ids, "gaussian_ids", torch.int64)
        radii = _in(radii, "radii", torch.int32); coeffs = _in(coeffs, "coeffs")
        depths = _in(depths, "depths")
        C, N, dev = viewmats.shape[0], means.shape[0], means.device
        lead = tuple(radii.shape[:-1])
        n = int(math.prod(lead))
        colors = torch.empty(lead + (4 if depths is not None else 3,), dtype=torch.float32, device=dev)
        with _on(dev):
            _check(lib.splatad_view_colors_fwd(
                _u32(n), _u32(C), _u32(N), _u32(coeffs.shape[-2]), _u32(degrees_to_use), _p(means),
                _p(viewmats), _p(camera_ids), _p(gaussian_ids), _p(radii), _p(coeffs),
                _i32(coeffs.dim() == 4), _p(depths), _p(colors), _stream(dev)))
        return colors

    def view_colors_cache(self, degrees_to_use, means, viewmats, camera_ids, gaussian_ids, radii, coeffs,
                          depths, opacities, tile_size, tile_width, tile_height, min_opacity_per_tile):
        """The colour cache that rasterize_to_pixels_sh_fwd takes ([rows, 4] floats, NaN = not
        evaluated): all NaN where tiles will saturate early, the colours of the visible rows
        where the estimate of the opacity per tile falls below min_opacity_per_tile."""
        lib = load_library()
        means = _in(means, "means"); viewmats = _in(viewmats, "viewmats")
        camera_ids = _in(camera_ids, "camera_ids", torch.int64)
        gaussian_ids = _in(gaussian_ids, "gaussian_ids", torch.int64)
        radii = _in(radii, "radii", torch.int32); coeffs = _in(coeffs, "coeffs")
        opacities = _in(opacities, "opacities"); depths = _in(depths, "depths")
        C, N, dev = viewmats.shape[0], means.shape[0], means.device
        assert opacities.shape == (N,), opacities.shape
        assert depths is None or depths.shape == radii.shape[:-1], depths.shape
        lead = tuple(radii.shape[:-1])
        n = int(math.prod(lead))
        words = lib.splatad_view_colors_cache_bytes(_u64(n)) // 4
        buf = torch.empty((words,), dtype=torch.float32, device=dev)
        with _on(dev):
            _check(lib.splatad_view_colors_cache(
                _u32(n), _u32(C), _u32(N), _u32(coeffs.shape[-2]), _u32(degrees_to_use), _p(means),
                _p(viewmats), _p(camera_ids), _p(gaussian_ids), _p(radii), _p(coeffs),
                _i32(coeffs.dim() == 4), _p(depths), _p(opacities), _u32(tile_size), _u32(tile_width),
                _u32(tile_height), _f32(min_opacity_per_tile), _p(buf), _stream(dev)))
        return buf[: n * 4].view(lead + (4,))

    def view_colors_bwd(self, degrees_to_use, means, viewmats, camera_ids, gaussian_ids, radii,
                        coeffs, colors, v_colors, compute_v_dirs, scatter_coeffs=False):
        """Per-row gradients (v_coeffs [..., K, 3], v_dirs [..., 3] | None) of view_colors_fwd;
        with scatter_coeffs, v_coeffs is summed over the rows of a Gaussian and shaped like coeffs."""
        lib = load_library()
        means = _in(means, "means"); viewmats = _in(viewmats, "viewmats")
        camera_ids = _in(camera_ids, "camera_ids", torch.int64)
        gaussian_ids = _in(gaussian_ids, "gaussian_ids", torch.int64)
        radii = _in(radii, "radii", torch.int32); coeffs = _in(coeffs, "coeffs")
        colors = _in(colors, "colors"); v_colors = _in(v_colors, "v_colors")
        C, N, dev = viewmats.shape[0], means.shape[0], means.device
        lead = tuple(radii.shape[:-1])
        n, K = int(math.prod(lead)), coeffs.shape[-2]
        f = dict(dtype=torch.float32, device=dev)
        # the kernel writes the floats of the bases in use; the others must read zero
        full = (degrees_to_use + 1) ** 2 == K
        if scatter_coeffs:
            # gradients in the layout of coeffs: the kernel adds every row's at its Gaussian's
            v_coeffs = torch.zeros_like(coeffs)
        else:
            v_coeffs = (torch.empty if full else torch.zeros)(lead + (K, 3), **f)
        v_dirs = torch.empty(lead + (3,), **f) if compute_v_dirs else None
        with _on(dev):
            _check(lib.splatad_view_colors_bwd(
                _u32(n), _u32(C), _u32(N), _u32(K), _u32(degrees_to_use), _p(means), _p(viewmats),
                _p(camera_ids), _p(gaussian_ids), _p(radii), _p(coeffs), _i32(coeffs.dim() == 4),
                _u32(colors.shape[-1]), _p(colors), _p(v_colors), _i32(bool(scatter_coeffs)), _p(v_coeffs),
                _p(v_dirs), _stream(dev)))
        return v_coeffs, v_dirs

    # ------------------------------------------------------------------ intersection
    def _isect(self, lidar, means2d, radii, depths, camera_ids, gaussian_ids, C, grid_args,
               tile_w, tile_h, sort, beside_work=None):
        """beside_work: a callable without arguments, called once before this returns.  Where the
        call sorts (cameras), it is called from inside the fill call with this thread's library
        calls redirected to a helper stream of the sort (library_stream): what it enqueues runs
        beside the sort and is joined with it.  It must launch no torch kernel and need nothing
        but what was enqueued before this call."""
        # A packed projection that was told the tile grid has made the lists of these rows from its
        # dense copy of them (good for one call, and only for the very tensors it returned,
        # unwritten since).
        known = getattr(radii, "_splatad_isect_count", None) if not lidar and sort else None
        if known is not None:
            del radii._splatad_isect_count
            if (known[0] == (int(grid_args[0].value), tile_w, tile_h) and known[2] == radii._version
                    and known[3]() is means2d and known[4] == means2d._version
                    and known[5]() is depths and known[6] == depths._version and known[7] == C):
                if beside_work is not None:
                    beside_work()
                return known[1]
        filled = getattr(radii, "_splatad_fill_stream", None)
        if filled is not None:
            # rows of a packed projection whose outputs were written on another stream
            torch.cuda.current_stream(radii.device).wait_stream(filled)
        lib = load_library()
        means2d = _in(means2d, "means2d"); depths = _in(depths, "depths")
        radii = _in(radii, "radii", torch.float32 if lidar else torch.int32)
        camera_ids = _in(camera_ids, "camera_ids", torch.int64)
        _in(gaussian_ids, "gaussian_ids", torch.int64)
        packed = means2d.dim() == 2
        dev = means2d.device
        if packed:
            assert camera_ids is not None and gaussian_ids is not None
            total, N = means2d.shape[0], 0
        else:
            N = means2d.shape[1]
            total = C * N
            camera_ids = None
        n_tiles = tile_w * tile_h
        # reference: assert(tile_n_bits + cam_n_bits <= 32), rasterization.cu:138
        assert n_tiles.bit_length() + int(C).bit_length() <= 32
        tiles_per_gauss = torch.empty(depths.shape, dtype=torch.int32, device=dev)
        count = lib.splatad_isect_lidar_tiles_count if lidar else lib.splatad_isect_tiles_count
        fill = lib.splatad_isect_lidar_tiles_fill if lidar else lib.splatad_isect_tiles_fill
        with _on(dev):
            # the binning knows every tile's first intersection: keep that table with the
            # ids so that isect_offset_encode() on the same, unmodified tensor is free
            offsets = (torch.empty((C, tile_h, tile_w), dtype=torch.int32, device=dev)
                       if sort else None)
            # one workspace for both calls: the counting call leaves the start of the binning in it
            ws = _workspace(lib.splatad_isect_workspace_bytes(_u64(total), _u32(C), _u32(n_tiles)), dev)
            head = (_u64(total), _u32(N), _p(camera_ids), _p(means2d), _p(radii), _p(depths))
            tail = (_u32(C), *grid_args, _u32(tile_w), _u32(tile_h), _i32(bool(sort)))
            n_host = _i64(0)
            _check(count(*head, *tail, _p(tiles_per_gauss), _p(ws), ctypes.byref(n_host),
                         _stream(dev)))
            n_isects = int(n_host.value)
            isect_ids = torch.empty((n_isects,), dtype=torch.int64, device=dev)
            flatten_ids = torch.empty((n_isects,), dtype=torch.int32, device=dev)
            if n_isects:
                lists = _workspace(lib.splatad_isect_lists_bytes(_u64(total), _i64(n_isects)), dev)
                if beside_work is not None and not lidar:
                    caught = []

                    def run_beside(_context, stream_handle):
                        try:
                            with library_stream(ctypes.c_void_p(stream_handle)):
                                beside_work()
                            return 0
                        except BaseException as e:  # (an exception must not cross the C frames)
                            caught.append(e)
                            return 1

                    rc = lib.splatad_isect_tiles_fill_beside(
                        *head, *tail, _i64(n_isects), _p(tiles_per_gauss), _p(ws), _p(lists), _p(isect_ids),
                        _p(flatten_ids), _p(offsets), _BESIDE_FN(run_beside), None, _stream(dev))
                    beside_work = None
                    if caught:
                        raise caught[0]
                    _check(rc)
                else:
                    _check(fill(*head, *tail, _i64(n_isects), _p(tiles_per_gauss), _p(ws),
                                _p(lists), _p(isect_ids), _p(flatten_ids), _p(offsets), _stream(dev)))
            else:
                offsets = None
            if beside_work is not None:
                beside_work()
            if offsets is not None:
                isect_ids._splatad_tile_offsets = (offsets, isect_ids._version)
        return tiles_per_gauss, isect_ids, flatten_ids

    def isect_tiles(self, means2d, radii, depths, camera_ids, gaussian_ids, C, tile_size,
                    tile_width, tile_height, sort, double_buffer, beside_work=None):
        return self._isect(False, means2d, radii, depths, camera_ids, gaussian_ids, C,
                           (_u32(tile_size),), tile_width, tile_height, sort, beside_work)

    def isect_lidar_tiles(self, means2d, radii, depths, camera_ids, gaussian_ids, C,
                          elev_boundaries, tile_azim_resolution, min_azim, sort, double_buffer):
        eb = _in(elev_boundaries, "elev_boundaries")
        # rasterization.cu:435-436: float32 division, then ceil
        res32 = torch.tensor(tile_azim_resolution, dtype=torch.float32)
        n_tiles_azim = int(math.ceil((torch.tensor(360.0, dtype=torch.float32) / res32).item()))
        n_tiles_elev = eb.shape[0] - 1
        return self._isect(True, means2d, radii, depths, camera_ids, gaussian_ids, C,
                           (_p(eb), _f32(tile_azim_resolution), _f32(min_azim)), n_tiles_azim,
                           n_tiles_elev, sort)

    def isect_offset_encode(self, isect_ids, C, tile_width, tile_height):
        lib = load_library()
        cached = getattr(isect_ids, "_splatad_tile_offsets", None)
        if (cached is not None and cached[1] == isect_ids._version
                and tuple(cached[0].shape) == (C, tile_height, tile_width)):
            return cached[0]
        isect_ids = _in(isect_ids, "isect_ids", torch.int64)
        dev = isect_ids.device
        offsets = torch.empty((C, tile_height, tile_width), dtype=torch.int32, device=dev)
        with _on(dev):
            _check(lib.splatad_isect_offset_encode(_i64(isect_ids.shape[0]), _p(isect_ids), _u32(C),
                                                   _u32(tile_width * tile_height), _p(offsets),
                                                   _stream(dev)))
        return offsets

    # ------------------------------------------------------------------ lidar point binning
    def map_points_to_lidar_tiles(self, points2d, camera_ids, C, elev_boundaries,
                                  tile_azim_resolution, min_azim, sort, double_buffer):
        lib = load_library()
        points2d = _in(points2d, "points2d"); eb = _in(elev_boundaries, "elev_boundaries")
        camera_ids = _in(camera_ids, "camera_ids", torch.int64)
        dev = points2d.device
        packed = points2d.dim() == 2
        if packed:
            assert camera_ids is not None
            total, N = points2d.shape[0], 0
        else:
            N = points2d.shape[1]
            total = C * N
            camera_ids = None
        # rasterization.cu:689-690: float32 division, then ceil
        res32 = torch.tensor(tile_azim_resolution, dtype=torch.float32)
        n_az = int(math.ceil((torch.tensor(360.0, dtype=torch.float32) / res32).item()))
        n_el = eb.shape[0] - 1
        tile_ids = torch.empty((total,), dtype=torch.int64, device=dev)
        flatten_ids = torch.empty((total,), dtype=torch.int32, device=dev)
        if total:
            with _on(dev):
                ws = _workspace(lib.splatad_map_points_to_lidar_tiles_workspace_bytes(
                    _u64(total), _u32(C), _u32(n_az * n_el)), dev) if sort else None
                _check(lib.splatad_map_points_to_lidar_tiles(
                    _u64(total), _u32(N), _p(camera_ids), _p(points2d), _u32(C), _p(eb),
                    _f32(tile_azim_resolution), _f32(min_azim), _u32(n_az), _u32(n_el),
                    _i32(bool(sort)), _p(ws), _p(tile_ids), _p(flatten_ids), _stream(dev)))
        return tile_ids, flatten_ids

    def points_mapping_offset_encode(self, point_ids, C, tile_width, tile_height):
        lib = load_library()
        point_ids = _in(point_ids, "point_ids", torch.int64)
        dev = point_ids.device
        offsets = torch.empty((C, tile_height, tile_width), dtype=torch.int32, device=dev)
        with _on(dev):
            _check(lib.splatad_points_mapping_offset_encode(
                _i64(point_ids.shape[0]), _p(point_ids), _u32(C), _u32(tile_width * tile_height),
                _p(offsets), _stream(dev)))
        return offsets

    def populate_image_from_points(self, points, image_width, image_height, tile_width,
                                   tile_height, tile_offsets, flatten_ids):
        lib = load_library()
        points = _in(points, "points")
        tile_offsets = _in(tile_offsets, "tile_offsets", torch.int32)
        flatten_ids = _in(flatten_ids, "flatten_ids", torch.int32)
        if points.shape[-1] != 5:
            raise ValueError("populate_image_from_points: points must have 5 values each")
        dev = points.device
        C, gh, gw = tile_offsets.shape
        image = torch.empty((C, image_height, image_width, 5), dtype=torch.float32, device=dev)
        with _on(dev):
            _check(lib.splatad_populate_image_from_points(
                _u32(C), _i64(flatten_ids.shape[0]), _p(points), _u32(image_width),
                _u32(image_height), _u32(tile_width), _u32(tile_height), _u32(gw), _u32(gh),
                _p(tile_offsets), _p(flatten_ids), _p(image), _stream(dev)))
        return image

    # ------------------------------------------------------------------ unfused projection ops
    def quat_scale_to_covar_preci_fwd(self, quats, scales, compute_covar, compute_preci, triu):
        lib = load_library()
        quats = _in(quats, "quats"); scales = _in(scales, "scales")
        N, dev = quats.shape[0], quats.device
        shape = (N, 6) if triu else (N, 3, 3)
        covars = torch.empty(shape, dtype=torch.float32, device=dev) if compute_covar else None
        precis = torch.empty(shape, dtype=torch.float32, device=dev) if compute_preci else None
        with _on(dev):
            _check(lib.splatad_quat_scale_to_covar_preci_fwd(
                _u32(N), _p(quats), _p(scales), _i32(bool(triu)), _p(covars), _p(precis), _stream(dev)))
        return covars, precis

    def quat_scale_to_covar_preci_bwd(self, quats, scales, v_covars, v_precis, triu):
        lib = load_library()
        quats = _in(quats, "quats"); scales = _in(scales, "scales")
        v_covars = _in(v_covars, "v_covars"); v_precis = _in(v_precis, "v_precis")
        dev = quats.device
        v_quats = torch.empty_like(quats); v_scales = torch.empty_like(scales)
        with _on(dev):
            _check(lib.splatad_quat_scale_to_covar_preci_bwd(
                _u32(quats.shape[0]), _p(quats), _p(scales), _p(v_covars), _p(v_precis),
                _i32(bool(triu)), _p(v_quats), _p(v_scales), _stream(dev)))
        return v_quats, v_scales

    def world_to_cam_fwd(self, means, covars, viewmats):
        lib = load_library()
        means = _in(means, "means"); covars = _in(covars, "covars"); viewmats = _in(viewmats, "viewmats")
        C, N, dev = viewmats.shape[0], means.shape[0], means.device
        means_c = torch.empty((C, N, 3), dtype=torch.float32, device=dev)
        covars_c = torch.empty((C, N, 3, 3), dtype=torch.float32, device=dev)
        with _on(dev):
            _check(lib.splatad_world_to_cam_fwd(_u32(C), _u32(N), _p(means), _p(covars), _p(viewmats),
                                                _p(means_c), _p(covars_c), _stream(dev)))
        return means_c, covars_c

    def world_to_cam_bwd(self, means, covars, viewmats, v_means_c, v_covars_c, means_grad,
                         covars_grad, viewmats_grad):
        lib = load_library()
        means = _in(means, "means"); covars = _in(covars, "covars"); viewmats = _in(viewmats, "viewmats")
        v_means_c = _in(v_means_c, "v_means_c"); v_covars_c = _in(v_covars_c, "v_covars_c")
        C, N, dev = viewmats.shape[0], means.shape[0], means.device
        v_means = torch.zeros_like(means) if means_grad else None
        v_covars = torch.zeros_like(covars) if covars_grad else None
        v_viewmats = torch.zeros_like(viewmats) if viewmats_grad else None
        with _on(dev):
            _check(lib.splatad_world_to_cam_bwd(
                _u32(C), _u32(N), _p(means), _p(covars), _p(viewmats), _p(v_means_c), _p(v_covars_c),
                _p(v_means), _p(v_covars), _p(v_viewmats), _stream(dev)))
        return v_means, v_covars, v_viewmats

    def persp_proj_fwd(self, means, covars, Ks, width, height):
        lib = load_library()
        means = _in(means, "means"); covars = _in(covars, "covars"); Ks = _in(Ks, "Ks")
        C, N, dev = means.shape[0], means.shape[1], means.device
        means2d = torch.empty((C, N, 2), dtype=torch.float32, device=dev)
        covars2d = torch.empty((C, N, 2, 2), dtype=torch.float32, device=dev)
        with _on(dev):
            _check(lib.splatad_persp_proj_fwd(_u32(C), _u32(N), _p(means), _p(covars), _p(Ks), _u32(width),
                                              _u32(height), _p(means2d), _p(covars2d), _stream(dev)))
        return means2d, covars2d

    def persp_proj_bwd(self, means, covars, Ks, width, height, v_means2d, v_covars2d):
        lib = load_library()
        means = _in(means, "means"); covars = _in(covars, "covars"); Ks = _in(Ks, "Ks")
        v_means2d = _in(v_means2d, "v_means2d"); v_covars2d = _in(v_covars2d, "v_covars2d")
        C, N, dev = means.shape[0], means.shape[1], means.device
        v_means = torch.empty_like(means); v_covars = torch.empty_like(covars)
        with _on(dev):
            _check(lib.splatad_persp_proj_bwd(
                _u32(C), _u32(N), _p(means), _p(covars), _p(Ks), _u32(width), _u32(height),
                _p(v_means2d), _p(v_covars2d), _p(v_means), _p(v_covars), _stream(dev)))
        return v_means, v_covars

    def compute_pix_velocity_fwd(self, p_view, lin_vel, ang_vel, velocities, Ks, width, height):
        lib = load_library()
        p_view = _in(p_view, "p_view"); lin_vel = _in(lin_vel, "lin_vel"); ang_vel = _in(ang_vel, "ang_vel")
        velocities = _in(velocities, "velocities"); Ks = _in(Ks, "Ks")
        C, N, dev = p_view.shape[0], p_view.shape[1], p_view.device
        vel = torch.empty((C, N, 2), dtype=torch.float32, device=dev)
        with _on(dev):
            _check(lib.splatad_compute_pix_velocity_fwd(
                _u32(C), _u32(N), _p(p_view), _p(lin_vel), _p(ang_vel), _p(velocities), _p(Ks),
                _u32(width), _u32(height), _p(vel), _stream(dev)))
        return vel

    def compute_pix_velocity_bwd(self, p_view, lin_vel, ang_vel, velocities, Ks, width, height, v_vel):
        lib = load_library()
        p_view = _in(p_view, "p_view"); lin_vel = _in(lin_vel, "lin_vel"); ang_vel = _in(ang_vel, "ang_vel")
        velocities = _in(velocities, "velocities"); Ks = _in(Ks, "Ks"); v_vel = _in(v_vel, "v_vel")
        C, N, dev = p_view.shape[0], p_view.shape[1], p_view.device
        v_p_view = torch.empty_like(p_view); v_velocities = torch.empty_like(velocities)
        with _on(dev):
            _check(lib.splatad_compute_pix_velocity_bwd(
                _u32(C), _u32(N), _p(p_view), _p(lin_vel), _p(ang_vel), _p(velocities), _p(Ks),
                _u32(width), _u32(height), _p(v_vel), _p(v_p_view), _p(v_velocities), _stream(dev)))
        return v_p_view, v_velocities

    def lidar_proj_fwd(self, means, covars, eps2d):
        lib = load_library()
        means = _in(means, "means"); covars = _in(covars, "covars")
        C, N, dev = means.shape[0], means.shape[1], means.device
        means2d = torch.empty((C, N, 2), dtype=torch.float32, device=dev)
        covars2d = torch.empty((C, N, 2, 2), dtype=torch.float32, device=dev)
        depth_comps = torch.empty((C, N, 2), dtype=torch.float32, device=dev)
        with _on(dev):
            _check(lib.splatad_lidar_proj_fwd(_u32(C), _u32(N), _p(means), _p(covars), _f32(eps2d),
                                              _p(means2d), _p(covars2d), _p(depth_comps), _stream(dev)))
        return means2d, covars2d, depth_comps

    def lidar_proj_bwd(self, means, covars, eps2d, v_means2d, v_covars2d, v_depth_compensations):
        lib = load_library()
        means = _in(means, "means"); covars = _in(covars, "covars")
        v_means2d = _in(v_means2d, "v_means2d"); v_covars2d = _in(v_covars2d, "v_covars2d")
        v_dc = _in(v_depth_compensations, "v_depth_compensations")
        C, N, dev = means.shape[0], means.shape[1], means.device
        v_means = torch.empty_like(means); v_covars = torch.empty_like(covars)
        with _on(dev):
            _check(lib.splatad_lidar_proj_bwd(
                _u32(C), _u32(N), _p(means), _p(covars), _f32(eps2d), _p(v_means2d), _p(v_covars2d),
                _p(v_dc), _p(v_means), _p(v_covars), _stream(dev)))
        return v_means, v_covars

    def compute_lidar_velocity_fwd(self, p_view, lin_vel, ang_vel, velocities):
        lib = load_library()
        p_view = _in(p_view, "p_view"); lin_vel = _in(lin_vel, "lin_vel"); ang_vel = _in(ang_vel, "ang_vel")
        velocities = _in(velocities, "velocities")
        C, N, dev = p_view.shape[0], p_view.shape[1], p_view.device
        vel = torch.empty((C, N, 3), dtype=torch.float32, device=dev)
        with _on(dev):
            _check(lib.splatad_compute_lidar_velocity_fwd(
                _u32(C), _u32(N), _p(p_view), _p(lin_vel), _p(ang_vel), _p(velocities), _p(vel),
                _stream(dev)))
        return vel

    def compute_lidar_velocity_bwd(self, p_view, lin_vel, ang_vel, velocities, v_vel):
        lib = load_library()
        p_view = _in(p_view, "p_view"); lin_vel = _in(lin_vel, "lin_vel"); ang_vel = _in(ang_vel, "ang_vel")
        velocities = _in(velocities, "velocities"); v_vel = _in(v_vel, "v_vel")
        C, N, dev = p_view.shape[0], p_view.shape[1], p_view.device
        v_p_view = torch.empty_like(p_view); v_velocities = torch.empty_like(velocities)
        with _on(dev):
            _check(lib.splatad_compute_lidar_velocity_bwd(
                _u32(C), _u32(N), _p(p_view), _p(lin_vel), _p(ang_vel), _p(velocities), _p(v_vel),
                _p(v_p_view), _p(v_velocities), _stream(dev)))
        return v_p_view, v_velocities

    # ------------------------------------------------------------------ densification helper
    def compute_relocation(self, opacities, scales, ratios, binoms, n_max):
        lib = load_library()
        opacities = _in(opacities, "opacities"); scales = _in(scales, "scales")
        ratios = _in(ratios, "ratios", torch.int32); binoms = _in(binoms, "binoms")
        dev = opacities.device
        new_opacities = torch.empty_like(opacities)
        new_scales = torch.empty_like(scales)
        with _on(dev):
            _check(lib.splatad_compute_relocation(
                _u32(opacities.shape[0]), _p(opacities), _p(scales), _p(ratios), _p(binoms),
                _i32(n_max), _p(new_opacities), _p(new_scales), _stream(dev)))
        return new_opacities, new_scales

    # ------------------------------------------------------------------ rasterization
    def rasterize_to_pixels_fwd(self, means2d, conics, colors, opacities, pix_vels,
                                rolling_shutter_time, backgrounds, image_width, image_height,
                                tile_size, tile_offsets, flatten_ids, tile_batches=None, tile_cycles=None):
        """tile_batches: optional int32 [C, tile_height, tile_width] tensor that receives the number
        of list entries every tile staged (a diagnostic, not part of the reference's op)."""
        lib = load_library()
        means2d = _in(means2d, "means2d"); conics = _in(conics, "conics")
        colors = _in(colors, "colors"); opacities = _in(opacities, "opacities")
        pix_vels = _in(pix_vels, "pix_vels"); rs = _in(rolling_shutter_time, "rolling_shutter_time")
        backgrounds = _in(backgrounds, "backgrounds")
        tile_offsets = _in(tile_offsets, "tile_offsets", torch.int32)
        flatten_ids = _in(flatten_ids, "flatten_ids", torch.int32)
        C, th, tw = tile_offsets.shape
        D, dev = colors.shape[-1], means2d.device
        f = dict(dtype=torch.float32, device=dev)
        renders = torch.empty((C, image_height, image_width, D), **f)
        alphas = torch.empty((C, image_height, image_width, 1), **f)
        last_ids = torch.empty((C, image_height, image_width), dtype=torch.int32, device=dev)
        with _on(dev):
            _check(lib.splatad_rasterize_to_pixels_fwd(
                _u32(C), _i64(flatten_ids.shape[0]), _u32(D), _p(means2d), _p(conics), _p(colors),
                _p(opacities), _p(pix_vels), _p(rs), _p(backgrounds), _u32(image_width),
                _u32(image_height), _u32(tile_size), _u32(tw), _u32(th), _p(tile_offsets),
                _p(flatten_ids), _p(renders), _p(alphas), _p(last_ids),
                _p(_in(tile_batches, "tile_batches", torch.int32)),
                _p(_in(tile_cycles, "tile_cycles", torch.int64)), _stream(dev)))
        return renders, alphas, last_ids

    def rasterize_to_pixels_sh_fwd(self, sh_degree, means, viewmats, coeffs, gaussian_ids, depths,
                                   means2d, conics, opacities, pix_vels, rolling_shutter_time,
                                   backgrounds, image_width, image_height, tile_size, tile_offsets,
                                   flatten_ids, cache=None, want_last_ids=True):
        """rasterize_to_pixels_fwd for rows whose colours are the view-dependent colours of
        `coeffs` ([N, K, 3] or [C, N, K, 3]): the kernel evaluates them for the entries it
        stages.  Rows are dense [C, N], or packed [nnz] with gaussian_ids [nnz]; depths, if
        given, is rendered as a fourth channel.  want_last_ids=False: the third result is None
        and the kernel does not keep track of them."""
        lib = load_library()
        means = _in(means, "means"); viewmats = _in(viewmats, "viewmats"); coeffs = _in(coeffs, "coeffs")
        depths = _in(depths, "depths"); gaussian_ids = _in(gaussian_ids, "gaussian_ids", torch.int64)
        means2d = _in(means2d, "means2d"); conics = _in(conics, "conics")
        opacities = _in(opacities, "opacities")
        pix_vels = _in(pix_vels, "pix_vels"); rs = _in(rolling_shutter_time, "rolling_shutter_time")
        backgrounds = _in(backgrounds, "backgrounds")
        tile_offsets = _in(tile_offsets, "tile_offsets", torch.int32)
        flatten_ids = _in(flatten_ids, "flatten_ids", torch.int32)
        C, th, tw = tile_offsets.shape
        N, dev = means.shape[0], means2d.device
        rows = (C, N) if gaussian_ids is None else tuple(gaussian_ids.shape)
        assert means2d.shape == rows + (2,) and coeffs.shape[-1] == 3, (means2d.shape, coeffs.shape)
        assert coeffs.shape[:-2] in ((N,), (C, N)), coeffs.shape
        D = 3 if depths is None else 4
        f = dict(dtype=torch.float32, device=dev)
        renders = torch.empty((C, image_height, image_width, D), **f)
        alphas = torch.empty((C, image_height, image_width, 1), **f)
        last_ids = (torch.empty((C, image_height, image_width), dtype=torch.int32, device=dev)
                    if want_last_ids else None)
        # colours of the rows that tiles stage, left by the first for the others; NaN = not yet
        if cache is None:
            cache = torch.full(rows + (4,), float("nan"), **f)
        cache = _in(cache, "cache")
        assert cache.shape == rows + (4,), cache.shape
        with _on(dev):
            _check(lib.splatad_rasterize_to_pixels_fwd_sh(
                _u32(C), _u32(N), _i64(flatten_ids.shape[0]), _u32(coeffs.shape[-2]), _u32(sh_degree),
                _p(means), _p(viewmats), _p(coeffs), _i32(coeffs.dim() == 4), _p(gaussian_ids),
                _p(depths), _p(cache), _p(means2d),
                _p(conics), _p(opacities), _p(pix_vels), _p(rs), _p(backgrounds), _u32(image_width),
                _u32(image_height), _u32(tile_size), _u32(tw), _u32(th), _p(tile_offsets),
                _p(flatten_ids), _p(renders), _p(alphas), _p(last_ids), _stream(dev)))
        return renders, alphas, last_ids

    def rasterize_to_pixels_lane_stats(self, means2d, conics, opacities, pix_vels, rolling_shutter_time,
                                       image_width, image_height, tile_size, tile_offsets, flatten_ids):
        """Diagnostic: the eight lane-utilisation counters of the camera compositing loop
        (include/splatad_hip.h) as an int64 tensor."""
        lib = load_library()
        means2d = _in(means2d, "means2d"); conics = _in(conics, "conics")
        opacities = _in(opacities, "opacities"); pix_vels = _in(pix_vels, "pix_vels")
        rs = _in(rolling_shutter_time, "rolling_shutter_time")
        tile_offsets = _in(tile_offsets, "tile_offsets", torch.int32)
        flatten_ids = _in(flatten_ids, "flatten_ids", torch.int32)
        C, th, tw = tile_offsets.shape
        dev = means2d.device
        stats = torch.zeros((8,), dtype=torch.int64, device=dev)
        with _on(dev):
            _check(lib.splatad_rasterize_to_pixels_lane_stats(
                _u32(C), _i64(flatten_ids.shape[0]), _p(means2d), _p(conics), _p(opacities), _p(pix_vels),
                _p(rs), _u32(image_width), _u32(image_height), _u32(tile_size), _u32(tw), _u32(th),
                _p(tile_offsets), _p(flatten_ids), _p(stats), _stream(dev)))
        return stats

    def rasterize_to_pixels_bwd(self, means2d, conics, colors, opacities, pix_vels,
                                rolling_shutter_time, backgrounds, image_width, image_height,
                                tile_size, tile_offsets, flatten_ids, render_alphas, last_ids,
                                v_render_colors, v_render_alphas, absgrad, colors_from_cache=False):
        """colors_from_cache: `colors` is the colour cache rasterize_to_pixels_sh_fwd left behind
        (NaN rows = never staged, taken as zero); with its four channels the gradient of the
        fourth, the depth, comes back as a seventh, contiguous tensor of one value per row (what
        the projection's backward pass takes) and v_colors[..., 3] stays zero."""
        lib = load_library()
        means2d = _in(means2d, "means2d"); conics = _in(conics, "conics")
        colors = _in(colors, "colors"); opacities = _in(opacities, "opacities")
        pix_vels = _in(pix_vels, "pix_vels"); rs = _in(rolling_shutter_time, "rolling_shutter_time")
        backgrounds = _in(backgrounds, "backgrounds")
        tile_offsets = _in(tile_offsets, "tile_offsets", torch.int32)
        flatten_ids = _in(flatten_ids, "flatten_ids", torch.int32)
        render_alphas = _in(render_alphas, "render_alphas")
        last_ids = _in(last_ids, "last_ids", torch.int32)
        v_render_colors = _in(v_render_colors, "v_render_colors")
        v_render_alphas = _in(v_render_alphas, "v_render_alphas")
        C, th, tw = tile_offsets.shape
        D, dev = colors.shape[-1], means2d.device
        split_depth = colors_from_cache and D == 4
        v_means2d, v_conics, v_colors, v_opacities, v_pix_vels, v_means2d_abs, v_depths = _zeros_like_many(
            means2d, conics, colors, opacities, pix_vels, means2d if absgrad else None,
            opacities if split_depth else None)
        if flatten_ids.shape[0]:
            total = means2d.numel() // 2
            with _on(dev):
                ws = _bwd_workspace(lib, total, D, False, dev)
                head = (_u32(C), _i64(flatten_ids.shape[0]), _u32(D), _p(means2d), _p(conics),
                        _p(colors), _p(opacities), _p(pix_vels), _p(rs), _p(backgrounds),
                        _u32(image_width), _u32(image_height), _u32(tile_size), _u32(tw), _u32(th),
                        _p(tile_offsets), _p(flatten_ids), _p(render_alphas), _p(last_ids),
                        _p(v_render_colors), _p(v_render_alphas), _p(v_means2d_abs), _p(v_means2d),
                        _p(v_conics), _p(v_colors))
                tail = (_p(v_opacities), _p(v_pix_vels), _u64(total), _p(ws),
                        ctypes.c_size_t(0 if ws is None else ws.numel()), _stream(dev))
                if colors_from_cache:
                    _check(lib.splatad_rasterize_to_pixels_bwd_sh(*head, _p(v_depths), *tail))
                else:
                    _check(lib.splatad_rasterize_to_pixels_bwd(*head, *tail))
        if split_depth:
            return v_means2d_abs, v_means2d, v_conics, v_colors, v_opacities, v_pix_vels, v_depths
        return v_means2d_abs, v_means2d, v_conics, v_colors, v_opacities, v_pix_vels

    def rasterize_to_points_fwd(self, means2d, conics, colors, opacities, pix_vels,
                                depth_compensations, backgrounds, raster_pts, image_width,
                                image_height, tile_width, tile_height,
                                compute_alpha_sum_until_points,
                                compute_alpha_sum_until_points_threshold, tile_offsets, flatten_ids,
                                depth_channel_idx, tile_batches=None, range_channel=None, tile_cycles=None):
        """With range_channel ([C, N] or [nnz]) the last channel is read from it and `colors`
        holds the other channels only (depth_channel_idx counts it: colors.shape[-1])."""
        lib = load_library()
        means2d = _in(means2d, "means2d"); conics = _in(conics, "conics")
        colors = _in(colors, "colors"); opacities = _in(opacities, "opacities")
        range_channel = _in(range_channel, "range_channel")
        pix_vels = _in(pix_vels, "pix_vels"); dc = _in(depth_compensations, "depth_compensations")
        backgrounds = _in(backgrounds, "backgrounds"); raster_pts = _in(raster_pts, "raster_pts")
        tile_offsets = _in(tile_offsets, "tile_offsets", torch.int32)
        flatten_ids = _in(flatten_ids, "flatten_ids", torch.int32)
        C, gh, gw = tile_offsets.shape
        D, dev = colors.shape[-1] + (range_channel is not None), means2d.device
        f = dict(dtype=torch.float32, device=dev)
        renders = torch.empty((C, image_height, image_width, D), **f)
        alphas = torch.empty((C, image_height, image_width, 1), **f)
        medians = torch.empty((C, image_height, image_width, 1), **f)
        asum = (torch.empty((C, image_height, image_width, 1), **f)
                if compute_alpha_sum_until_points else None)
        last_ids = torch.empty((C, image_height, image_width), dtype=torch.int32, device=dev)
        with _on(dev):
            _check(lib.splatad_rasterize_to_points_fwd(
                _u32(C), _i64(flatten_ids.shape[0]), _u32(D), _p(means2d), _p(conics), _p(colors),
                _p(range_channel), _p(opacities), _p(pix_vels), _p(dc), _p(backgrounds),
                _p(raster_pts),
                _u32(image_width), _u32(image_height), _u32(tile_width), _u32(tile_height),
                _u32(gw), _u32(gh), _i32(bool(compute_alpha_sum_until_points)),
                _f32(compute_alpha_sum_until_points_threshold), _p(tile_offsets), _p(flatten_ids),
                _u32(depth_channel_idx), _p(renders), _p(alphas), _p(asum), _p(last_ids),
                _p(medians), _p(_in(tile_batches, "tile_batches", torch.int32)),
                _p(_in(tile_cycles, "tile_cycles", torch.int64)), _stream(dev)))
        return renders, alphas, last_ids, asum, medians

    def rasterize_to_points_bwd(self, means2d, conics, colors, opacities, pix_vels,
                                depth_compensations, backgrounds, raster_pts, image_width,
                                image_height, tile_width, tile_height, tile_offsets, flatten_ids,
                                render_alphas, last_ids, v_render_colors, v_render_alphas,
                                v_alpha_sum_until_points, absgrad, compute_alpha_sum_until_points,
                                compute_alpha_sum_until_points_threshold, depth_channel_idx,
                                range_channel=None):
        """With range_channel, an eighth result follows: its gradient."""
        lib = load_library()
        means2d = _in(means2d, "means2d"); conics = _in(conics, "conics")
        colors = _in(colors, "colors"); opacities = _in(opacities, "opacities")
        range_channel = _in(range_channel, "range_channel")
        pix_vels = _in(pix_vels, "pix_vels"); dc = _in(depth_compensations, "depth_compensations")
        backgrounds = _in(backgrounds, "backgrounds"); raster_pts = _in(raster_pts, "raster_pts")
        tile_offsets = _in(tile_offsets, "tile_offsets", torch.int32)
        flatten_ids = _in(flatten_ids, "flatten_ids", torch.int32)
        render_alphas = _in(render_alphas, "render_alphas")
        last_ids = _in(last_ids, "last_ids", torch.int32)
        v_render_colors = _in(v_render_colors, "v_render_colors")
        v_render_alphas = _in(v_render_alphas, "v_render_alphas")
        v_asum = _in(v_alpha_sum_until_points, "v_alpha_sum_until_points")
        C, gh, gw = tile_offsets.shape
        D, dev = colors.shape[-1] + (range_channel is not None), means2d.device
        (v_means2d, v_conics, v_colors, v_opacities, v_pix_vels, v_dc, v_means2d_abs,
         v_range) = _zeros_like_many(means2d, conics, colors, opacities, pix_vels, dc,
                                     means2d if absgrad else None, range_channel)
        if flatten_ids.shape[0]:
            total = means2d.numel() // 2
            with _on(dev):
                ws = _bwd_workspace(lib, total, D, True, dev)
                _check(lib.splatad_rasterize_to_points_bwd(
                    _u32(C), _i64(flatten_ids.shape[0]), _u32(D), _p(means2d), _p(conics),
                    _p(colors), _p(range_channel), _p(opacities), _p(pix_vels), _p(dc), _p(backgrounds),
                    _p(raster_pts), _u32(image_width), _u32(image_height), _u32(tile_width),
                    _u32(tile_height), _u32(gw), _u32(gh),
                    _i32(bool(compute_alpha_sum_until_points)),
                    _f32(compute_alpha_sum_until_points_threshold), _p(tile_offsets),
                    _p(flatten_ids), _u32(depth_channel_idx), _p(render_alphas), _p(last_ids),
                    _p(v_render_colors), _p(v_render_alphas), _p(v_asum), _p(v_means2d_abs),
                    _p(v_means2d), _p(v_conics), _p(v_colors), _p(v_range), _p(v_opacities),
                    _p(v_pix_vels), _p(v_dc), _u64(total), _p(ws), ctypes.c_size_t(0 if ws is None else ws.numel()),
                    _stream(dev)))
        if range_channel is not None:
            return v_means2d_abs, v_means2d, v_conics, v_colors, v_opacities, v_pix_vels, v_dc, v_range
        return v_means2d_abs, v_means2d, v_conics, v_colors, v_opacities, v_pix_vels, v_dc

    # ------------------------------------------------------------------ index lists
    def _indices_in_range(self, lidar, range_start, range_end, transmittances, means2d, conics,
                          opacities, pix_vels, sensor, image_width, image_height, tile_width,
                          tile_height, tile_offsets, flatten_ids):
        lib = load_library()
        transmittances = _in(transmittances, "transmittances")
        means2d = _in(means2d, "means2d"); conics = _in(conics, "conics")
        opacities = _in(opacities, "opacities"); pix_vels = _in(pix_vels, "pix_vels")
        sensor = _in(sensor, "raster_pts" if lidar else "rolling_shutter_time")
        tile_offsets = _in(tile_offsets, "tile_offsets", torch.int32)
        flatten_ids = _in(flatten_ids, "flatten_ids", torch.int32)
        C, N = means2d.shape[0], means2d.shape[1]
        gh, gw = tile_offsets.shape[1], tile_offsets.shape[2]
        dev = means2d.device
        i64 = dict(dtype=torch.int64, device=dev)
        n_pixels, n_isects = C * image_height * image_width, flatten_ids.shape[0]
        if n_pixels == 0 or n_isects == 0:
            return torch.empty((0,), **i64), torch.empty((0,), **i64)
        count = (lib.splatad_rasterize_to_indices_in_range_lidar_count if lidar
                 else lib.splatad_rasterize_to_indices_in_range_count)
        fill = (lib.splatad_rasterize_to_indices_in_range_lidar_fill if lidar
                else lib.splatad_rasterize_to_indices_in_range_fill)
        tiles = ((_u32(tile_width), _u32(tile_height), _u32(gw), _u32(gh)) if lidar
                 else (_u32(tile_width), _u32(gw), _u32(gh)))
        head = (_i64(int(min(range_start, 2 ** 62))), _i64(int(min(range_end, 2 ** 62))), _u32(C),
                _u32(N), _i64(n_isects), _p(transmittances), _p(means2d), _p(conics), _p(opacities),
                _p(pix_vels), _p(sensor), _u32(image_width), _u32(image_height), *tiles,
                _p(tile_offsets), _p(flatten_ids))
        with _on(dev):
            nbytes = lib.splatad_rasterize_to_indices_workspace_bytes(
                _u32(C), _u32(image_width), _u32(image_height))
            ws = _workspace(nbytes, dev)
            chunk_starts = torch.empty((n_pixels,), **i64)
            n_elems = torch.empty((1,), **i64)
            _check(count(*head, _p(ws), ctypes.c_size_t(ws.numel()), _p(chunk_starts), _p(n_elems),
                         _stream(dev)))
            total = int(n_elems.item())  # the one host read: sizes the outputs
            gaussian_ids = torch.empty((total,), **i64)
            indices = torch.empty((total,), **i64)
            if total:
                _check(fill(*head, _p(chunk_starts), _p(gaussian_ids), _p(indices), _stream(dev)))
        return gaussian_ids, indices

    def rasterize_to_indices_in_range(self, range_start, range_end, transmittances, means2d,
                                      conics, opacities, pix_vels, rolling_shutter_time,
                                      image_width, image_height, tile_size, tile_offsets,
                                      flatten_ids):
        return self._indices_in_range(False, range_start, range_end, transmittances, means2d,
                                      conics, opacities, pix_vels, rolling_shutter_time,
                                      image_width, image_height, tile_size, tile_size,
                                      tile_offsets, flatten_ids)

    def rasterize_to_indices_in_range_lidar(self, range_start, range_end, transmittances, means2d,
                                            conics, opacities, pix_vels, raster_pts, image_width,
                                            image_height, tile_width, tile_height, tile_offsets,
                                            flatten_ids):
        return self._indices_in_range(True, range_start, range_end, transmittances, means2d,
                                      conics, opacities, pix_vels, raster_pts, image_width,
                                      image_height, tile_width, tile_height, tile_offsets,
                                      flatten_ids)


_C = _Ops()
