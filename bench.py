"""Benchmark of the forward rendering path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--n N]

A step is one complete forward call of `rasterization()` (projection + SH + tile intersection
+ sort + offsets + rasterize) on the driving-camera workload: 1M Gaussians, 1920x1080 pinhole,
SH degree 3, rolling shutter, RGB+D.  All inputs are resident in HBM before the timed region.
The same is done for `lidar_rasterization()` on the 128x2048 lidar sweep and reported in the
"lidar" object of the same JSON line.  "roofline" describes the dominant kernel
(rasterize_to_pixels forward, which in a forward-only call also evaluates the colours of the
Gaussians it composites), timed with events on the launch stream; "cpu_baseline" times the
CPU oracle (a C restatement of the reference's algorithm, OpenMP) on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

VALU_CLOCK_HZ = 2.4e9  # MI355X peak engine clock, published
N_SIMDS = 256 * 4      # 256 compute units, four SIMDs each; a wave64 vector instruction issues over 4 cycles
# vector instructions a (pixel, composited Gaussian) pair costs the camera compositing kernel at
# the least in its formulation (exact float32, no packed FP32): five multiply-adds of the exponent
# polynomial, one v_exp_f32, the alpha test, the next transmittance and its test and update (4),
# the weight and four channel multiply-adds (5) = 15
MIN_VALU_PER_PIXEL_AND_GAUSSIAN = 15

PROFILE = os.path.join(ROOT, "profiles", "kernels_counters_camera_1M_1080p_lidar_128x2048.txt")


def profiled_counters():
    """Per-kernel hardware counters of the default workloads, read from the committed rocprofv3
    summary (its lines `@ kernel | FETCH_SIZE KiB | WRITE_SIZE KiB | SQ_INSTS_VALU`, averages per
    dispatch, and `@ calibration | fetch factor | write factor` from a 1 GiB copy).  They describe
    the 1M-Gaussian default only.  Returns {} when the summary is missing."""
    out = {}
    try:
        with open(PROFILE) as f:
            for line in f:
                if not line.startswith("@ "):
                    continue
                parts = [x.strip() for x in line[2:].split("|")]
                if parts[0] == "calibration":
                    out["calibration"] = (float(parts[1]), float(parts[2]))
                elif len(parts) == 4:
                    out[parts[0]] = dict(fetch_kib=float(parts[1]), write_kib=float(parts[2]), insts_valu=float(parts[3]))
    except OSError:
        return {}
    return out


def hbm_traffic_bytes(counters, kernel):
    """FETCH_SIZE and WRITE_SIZE of a kernel scaled by what the same counters read for a copy of
    known size; None when the summary does not hold the kernel."""
    if kernel not in counters or "calibration" not in counters:
        return None
    ff, wf = counters["calibration"]
    c = counters[kernel]
    return int((c["fetch_kib"] * ff + c["write_kib"] * wf) * 1024)


def valu_roofline(counters, kernel, kernel_ms, pairs=None):
    """The bound that holds the compositing kernels: vector instruction issue.  achieved = the
    fraction of the GPU's issue cycles (four per wave64 instruction and SIMD) the kernel's
    SQ_INSTS_VALU fill during its event-timed duration; floor_ms = the time the (pixel,
    Gaussian) pairs that composite need at MIN_VALU_PER_PIXEL_AND_GAUSSIAN instructions each."""
    if kernel not in counters:
        return None
    insts = counters[kernel]["insts_valu"]
    busy_s = insts * 4.0 / (N_SIMDS * VALU_CLOCK_HZ)
    out = {"kernel": kernel, "bound": "valu_issue", "achieved": busy_s / (kernel_ms * 1e-3), "peak": 1.0,
           "unit": "fraction of vector issue cycles", "frac": busy_s / (kernel_ms * 1e-3),
           "insts_valu_per_launch": insts, "issue_ms": busy_s * 1e3, "kernel_ms": kernel_ms}
    if pairs is not None:
        floor_s = pairs / 64.0 * MIN_VALU_PER_PIXEL_AND_GAUSSIAN * 4.0 / (N_SIMDS * VALU_CLOCK_HZ)
        out.update(pixel_gaussian_pairs=int(pairs), min_insts_per_pair=MIN_VALU_PER_PIXEL_AND_GAUSSIAN,
                   floor_ms=floor_s * 1e3, floor_over_kernel=floor_s / (kernel_ms * 1e-3))
    return out


def _sync():
    import torch

    torch.cuda.synchronize()


def time_steps(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    _sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    _sync()
    return (time.perf_counter() - t0) / steps


def time_kernel(fn, iters, warmup=2):
    """Average duration in ms of the work fn() enqueues on torch's current stream."""
    import torch

    for _ in range(warmup):
        fn()
    _sync()
    # one pair of events around all launches: a pair per launch adds the dispatch latency behind
    # each start marker (4-5 us) to every kernel, which the kernel trace does not count
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(iters):
        fn()
    stop.record()
    _sync()
    return start.elapsed_time(stop) / iters


def time_kernel_on(make, fn, iters, warmup=2):
    """As time_kernel, for fn(x) with x = make() made afresh for every call (a kernel that changes
    its input), right before the call as in a step, so that fn meets x as warm in the caches as a
    step's kernel does: the time of make(); fn(x) less the time of make() alone."""
    import torch

    def timed(body):
        for _ in range(warmup):
            body()
        _sync()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):  # enqueued back to back, so that the GPU never waits for the host
            body()
        stop.record()
        _sync()
        return start.elapsed_time(stop) / iters

    return timed(lambda: fn(make())) - timed(make)


def staged_isects(tile_entries):
    """List entries the compositing kernel staged: whole batches until every pixel / point of a
    tile has saturated, clipped to the tile's list, as counted by the kernel itself."""
    return int(tile_entries.sum().item())


def cycle_spread(cycles):
    """Spread of the per-tile run times of a compositing kernel (shader clock cycles of each
    tile's workgroup): the kernel lasts as long as its slowest tiles."""
    import torch

    c = cycles.flatten().double()
    c = c[c > 0]
    q = torch.quantile(c, torch.tensor([0.5, 0.9, 0.99], dtype=torch.float64, device=c.device)).tolist()
    return {"tiles": int(c.numel()), "mean": round(c.mean().item()), "p50": round(q[0]), "p90": round(q[1]),
            "p99": round(q[2]), "max": round(c.max().item()), "max_over_mean": round((c.max() / c.mean()).item(), 3)}


def stage_rooflines(leg):
    """Per stage of a forward call: event-timed duration of the stage's launches in isolation, the
    bytes any implementation of the stage has to move, and what that makes of the HBM peak."""
    out = {}
    for k, ms in leg["stages"].items():
        b = leg["stage_bytes"].get(k)
        if b is None:
            continue
        gbs = b / (ms * 1e-3) / 1e9
        out[k[:-3]] = {"ms": round(ms, 4), "algorithmic_bytes": int(b), "achieved_GBps": round(gbs, 1),
                       "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
    return out


def bench_camera(args):
    import torch

    from splatad_amd import rasterization, workloads
    from splatad_amd.hip._backend import _C

    dev = torch.device("cuda:0")
    s = workloads.to_device(workloads.camera_driving(n=args.n), dev)

    def run(packed=False):
        return rasterization(
            s["means"], s["quats"], s["scales"], s["opacities"], s["colors"], s["velocities"],
            s["viewmats"], s["Ks"], s["width"], s["height"], s["linear_velocity"],
            s["angular_velocity"], s["rolling_shutter_time"], sh_degree=s["sh_degree"],
            packed=packed, render_mode="RGB+D", near_plane=s["near_plane"],
            far_plane=s["far_plane"], eps2d=s["eps2d"], tile_size=s["tile_size"])

    with torch.no_grad():
        sec = time_steps(run, args.steps, args.warmup)
        sec_packed = time_steps(lambda: run(True), args.steps, args.warmup)
        rc, ra, meta = run()
        C, H, W = 1, s["height"], s["width"]
        # dominant kernel, isolated
        colors = None

        # rebuild the rasterizer's inputs exactly as rasterization() does
        from splatad_amd import spherical_harmonics
        camtoworlds = torch.inverse(s["viewmats"])
        dirs = s["means"][None] - camtoworlds[:, None, :3, 3]
        cols = spherical_harmonics(3, dirs, s["colors"].expand(C, -1, -1, -1), masks=meta["radii"][..., 0] > 0)
        cols = torch.cat([torch.clamp_min(cols + 0.5, 0.0), meta["depths"][..., None]], -1).contiguous()
        ts = s["tile_size"]

        def raster():
            return _C.rasterize_to_pixels_fwd(
                meta["means2d"], meta["conics"], cols, meta["opacities"], meta["pix_vels"],
                s["rolling_shutter_time"], None, W, H, ts, meta["isect_offsets"], meta["flatten_ids"])

        # what the step runs: the same kernel evaluating the colours of the entries it stages,
        # on a colour cache that two short launches prepare (left empty for this frame)
        from splatad_amd.hip._wrapper import MIN_OPACITY_PER_TILE

        def color_cache():
            return _C.view_colors_cache(3, s["means"], s["viewmats"], None, None, meta["radii"], s["colors"],
                                        meta["depths"], s["opacities"], ts, meta["tile_width"],
                                        meta["tile_height"], MIN_OPACITY_PER_TILE)

        def raster_sh(cache):
            return _C.rasterize_to_pixels_sh_fwd(
                3, s["means"], s["viewmats"], s["colors"], None, meta["depths"], meta["means2d"],
                meta["conics"], meta["opacities"], meta["pix_vels"], s["rolling_shutter_time"], None,
                W, H, ts, meta["isect_offsets"], meta["flatten_ids"], cache=cache, want_last_ids=False)

        first = color_cache()
        cache_left_empty = bool(torch.isnan(first).all().item())
        assert torch.equal(raster_sh(first)[0], raster()[0]) and torch.equal(raster()[0], rc)
        k_ms = time_kernel_on(color_cache, raster_sh, iters=max(5, args.steps))
        k_plain_ms = time_kernel(raster, iters=max(5, args.steps))
        n_isects = int(meta["flatten_ids"].shape[0])
        batches = torch.zeros_like(meta["isect_offsets"])
        _C.rasterize_to_pixels_fwd(
            meta["means2d"], meta["conics"], cols, meta["opacities"], meta["pix_vels"],
            s["rolling_shutter_time"], None, W, H, ts, meta["isect_offsets"], meta["flatten_ids"],
            tile_batches=batches)
        i_need = staged_isects(batches)
        cycles = torch.zeros(meta["isect_offsets"].shape, dtype=torch.int64, device=dev)
        _C.rasterize_to_pixels_fwd(
            meta["means2d"], meta["conics"], cols, meta["opacities"], meta["pix_vels"],
            s["rolling_shutter_time"], None, W, H, ts, meta["isect_offsets"], meta["flatten_ids"],
            tile_cycles=cycles)
        tile_cycles = cycle_spread(cycles)
        D = cols.shape[-1]
        P, T = C * H * W, meta["isect_offsets"].numel()
        N, K = s["means"].shape[0], s["colors"].shape[-2]
        # rows (camera, Gaussian) among the staged entries: each one's mean and coefficients
        # have to be read at least once
        first = meta["isect_offsets"].flatten().long()
        marks = torch.zeros(n_isects + 1, dtype=torch.int32, device=dev)
        marks.index_add_(0, first, torch.ones_like(first, dtype=torch.int32))
        marks.index_add_(0, first + batches.flatten().long(), -torch.ones_like(first, dtype=torch.int32))
        staged = torch.cumsum(marks[:-1], 0) > 0
        rows_staged = int(torch.unique(meta["flatten_ids"][staged]).numel())
        plain_bytes = i_need * (36 + 4 * D) + P * (4 * D + 8) + T * 4
        # per staged entry its geometry and cache row, per staged row the evaluation (mean,
        # coefficients, depth) and the cache row written back
        alg_bytes = i_need * (36 + 16) + rows_staged * (12 + 12 * K + 4 + 16) + P * (4 * D + 8) + T * 4
        # per-stage times of the same call
        stages = {}
        proj = lambda: _C.fully_fused_projection_fwd(
            s["means"], None, s["quats"], s["scales"], s["velocities"], s["viewmats"], s["Ks"], W, H,
            s["linear_velocity"], s["angular_velocity"], s["rolling_shutter_time"], s["eps2d"],
            s["near_plane"], s["far_plane"], 0.0, False)
        stages["projection_ms"] = time_kernel(proj, 5)
        isect = lambda: _C.isect_tiles(meta["means2d"], meta["radii"], meta["depths"], None, None, C,
                                       ts, meta["tile_width"], meta["tile_height"], True, True)
        stages["isect_sort_ms"] = time_kernel(isect, 5)
        # on a copy: the tensor returned by isect_tiles carries the table the binning made
        ids_copy = meta["isect_ids"].clone()
        stages["offset_encode_ms"] = time_kernel(
            lambda: _C.isect_offset_encode(ids_copy, C, meta["tile_width"], meta["tile_height"]), 5)
        stages["view_colors_ms"] = time_kernel(
            lambda: _C.view_colors_fwd(3, s["means"], s["viewmats"], None, None, meta["radii"],
                                       s["colors"], meta["depths"]), 5)
        stages["color_cache_ms"] = time_kernel(color_cache, 5)
        stages["rasterize_ms"] = k_ms
        stages["rasterize_given_colors_ms"] = k_plain_ms
        nnz = int((meta["radii"][..., 0] > 0).sum().item())
        stage_bytes = {
            "projection_ms": N * 52 + C * N * 40,
            # what any implementation has to move: read the projected (mean, radii, depth) rows, write
            # a key and an id per intersection and the offsets
            "isect_sort_ms": C * N * 20 + n_isects * 12 + T * 4,
            "offset_encode_ms": n_isects * 8 + T * 4,
            "view_colors_ms": nnz * (12 + 12 * K + 1 + 12),
            "color_cache_ms": C * N * (8 + 16) + N * 4,
            "rasterize_ms": alg_bytes,
            "rasterize_given_colors_ms": plain_bytes,
        }
        st = _C.rasterize_to_pixels_lane_stats(
            meta["means2d"], meta["conics"], meta["opacities"], meta["pix_vels"], s["rolling_shutter_time"], W, H,
            ts, meta["isect_offsets"], meta["flatten_ids"]).tolist()
        lanes = dict(iterations=st[0], pixels_per_lane=st[6],
                     compositing_lane_fraction=st[1] / max(1, st[0] * 64 * st[6]),
                     footprint_test_pass_fraction=st[5] / max(1, st[4]),
                     iterations_without_a_compositing_lane=st[3] / max(1, st[0]))
    return dict(sec=sec, sec_packed=sec_packed, pixels=P, kernel_ms=k_ms, alg_bytes=alg_bytes,
                n_isects=n_isects, i_need=i_need, rows_staged=rows_staged, cache_left_empty=cache_left_empty,
                nnz=nnz, stages=stages,
                stage_bytes=stage_bytes,
                channels=D, lanes=lanes, tile_cycles=tile_cycles)


def bench_lidar(args):
    import torch

    from splatad_amd import lidar_rasterization, workloads
    from splatad_amd.hip._backend import _C

    dev = torch.device("cuda:0")
    s = workloads.to_device(workloads.lidar_sweep(n=args.n), dev)

    def run(chunk=33):
        return lidar_rasterization(
            s["means"], s["quats"], s["scales"], s["opacities"], s["lidar_features"],
            s["velocities"], s["viewmats"], s["raster_pts"], s["tile_elevation_boundaries"],
            s["linear_velocity"], s["angular_velocity"], s["rolling_shutter_time"],
            min_azimuth=s["min_azimuth"], max_azimuth=s["max_azimuth"],
            min_elevation=s["min_elevation"], max_elevation=s["max_elevation"],
            n_elevation_channels=s["n_elevation_channels"],
            azimuth_resolution=s["azimuth_resolution"], tile_width=s["tile_width"],
            tile_height=s["tile_height"], near_plane=s["near_plane"], far_plane=s["far_plane"],
            eps2d=s["eps2d"], channel_chunk=chunk)

    with torch.no_grad():
        sec = time_steps(run, args.steps, args.warmup)
        sec_chunk32 = time_steps(lambda: run(32), max(2, args.steps // 2), 1)
        rf, ra, asum, meta = run()
        C, H, W = ra.shape[:3]
        proj = _C.fully_fused_lidar_projection_fwd(
            s["means"], None, s["quats"], s["scales"], s["velocities"], s["viewmats"],
            s["min_elevation"], s["max_elevation"], s["min_azimuth"], s["max_azimuth"],
            s["linear_velocity"], s["angular_velocity"], s["rolling_shutter_time"], s["eps2d"],
            s["near_plane"], s["far_plane"], 0.0, False)
        # the compositing kernel as lidar_rasterization() calls it: features and ranges apart
        feats, ranges = s["lidar_features"], meta["depths"]
        D = feats.shape[-1] + 1

        def raster(**kw):
            return _C.rasterize_to_points_fwd(
                meta["means2d"], meta["conics"], feats, meta["opacities"], meta["pix_vels"], proj[6],
                None, s["raster_pts"], W, H, s["tile_width"], s["tile_height"], True, 0.2,
                meta["isect_offsets"], meta["flatten_ids"], D - 1, range_channel=ranges, **kw)

        k_ms = time_kernel(raster, iters=max(5, args.steps))
        n_isects = int(meta["flatten_ids"].shape[0])
        batches = torch.zeros_like(meta["isect_offsets"])
        raster(tile_batches=batches)
        i_need = staged_isects(batches)
        cycles = torch.zeros(meta["isect_offsets"].shape, dtype=torch.int64, device=dev)
        raster(tile_cycles=cycles)
        tile_cycles = cycle_spread(cycles)
        P, T = C * H * W, meta["isect_offsets"].numel()
        # staged per list entry: id, mean, angular velocity, conic, opacity (40 bytes); the features
        # of the Gaussians a wavefront composites are read on demand and not counted here
        alg_bytes = i_need * 40 + P * (4 * D + 32) + T * 4
        # the figure with a staged entry's features counted too (4 * D bytes more per entry): what a
        # kernel that stages whole Gaussians, as the reference's does, has to read
        alg_bytes_features = i_need * (40 + 4 * D) + P * (4 * D + 32) + T * 4
        stages = {}
        stages["projection_ms"] = time_kernel(lambda: _C.fully_fused_lidar_projection_fwd(
            s["means"], None, s["quats"], s["scales"], s["velocities"], s["viewmats"],
            s["min_elevation"], s["max_elevation"], s["min_azimuth"], s["max_azimuth"],
            s["linear_velocity"], s["angular_velocity"], s["rolling_shutter_time"], s["eps2d"],
            s["near_plane"], s["far_plane"], 0.0, False), 5)
        stages["isect_sort_ms"] = time_kernel(lambda: _C.isect_lidar_tiles(
            meta["means2d"], meta["radii"], meta["depths"], None, None, C,
            s["tile_elevation_boundaries"], s["azimuth_resolution"] * s["tile_width"], s["min_azimuth"],
            True, True), 5)
        stages["rasterize_ms"] = k_ms
        N = s["means"].shape[0]
        stage_bytes = {"projection_ms": N * 52 + C * N * 52,
                       "isect_sort_ms": C * N * 20 + n_isects * 12 + T * 4,
                       "rasterize_ms": alg_bytes}
    return dict(sec=sec, sec_chunk32=sec_chunk32, points=P, kernel_ms=k_ms, alg_bytes=alg_bytes,
                n_isects=n_isects, i_need=i_need, channels=D, stages=stages, stage_bytes=stage_bytes,
                tile_cycles=tile_cycles, alg_bytes_features=alg_bytes_features)


def bench_backward(args):
    """Forward + backward (L1 losses on colour, depth and alpha against random targets, the
    shape of a training step) of the camera and the lidar call, ms per step."""
    import torch

    from splatad_amd import lidar_rasterization, rasterization, workloads

    dev = torch.device("cuda:0")
    out = {}
    s = workloads.to_device(workloads.camera_driving(n=args.n), dev)
    names = ("means", "quats", "scales", "opacities", "colors")
    p = {k: s[k].clone().requires_grad_(True) for k in names}
    g = torch.Generator(device=dev).manual_seed(7)
    target = torch.rand((1, s["height"], s["width"], 4), device=dev, generator=g)

    def cam_step():
        rc, ra, _ = rasterization(
            p["means"], p["quats"], p["scales"], p["opacities"], p["colors"], s["velocities"],
            s["viewmats"], s["Ks"], s["width"], s["height"], s["linear_velocity"],
            s["angular_velocity"], s["rolling_shutter_time"], sh_degree=s["sh_degree"],
            packed=False, render_mode="RGB+D", near_plane=s["near_plane"],
            far_plane=s["far_plane"], eps2d=s["eps2d"], tile_size=s["tile_size"])
        ((rc - target).abs().mean() + ra.mean()).backward()
        for t in p.values():
            t.grad = None

    out["camera_fwd_bwd_ms"] = time_steps(cam_step, max(3, args.steps // 2), 2) * 1e3
    del s, p, target
    l = workloads.to_device(workloads.lidar_sweep(n=args.n), dev)
    lnames = ("means", "quats", "scales", "opacities", "lidar_features")
    q = {k: l[k].clone().requires_grad_(True) for k in lnames}

    def lidar_step():
        rf, ra, _, _ = lidar_rasterization(
            q["means"], q["quats"], q["scales"], q["opacities"], q["lidar_features"],
            l["velocities"], l["viewmats"], l["raster_pts"], l["tile_elevation_boundaries"],
            l["linear_velocity"], l["angular_velocity"], l["rolling_shutter_time"],
            min_azimuth=l["min_azimuth"], max_azimuth=l["max_azimuth"],
            min_elevation=l["min_elevation"], max_elevation=l["max_elevation"],
            n_elevation_channels=l["n_elevation_channels"],
            azimuth_resolution=l["azimuth_resolution"], tile_width=l["tile_width"],
            tile_height=l["tile_height"], near_plane=l["near_plane"], far_plane=l["far_plane"],
            eps2d=l["eps2d"], channel_chunk=33)
        (rf.abs().mean() + ra.mean()).backward()
        for t in q.values():
            t.grad = None

    out["lidar_fwd_bwd_ms"] = time_steps(lidar_step, max(3, args.steps // 2), 2) * 1e3

    # the compositing backward in isolation: gradient of the compositing call alone with respect
    # to its per-Gaussian inputs (kernels, clearing and unpacking of the gradient records), on
    # the forward call's own lists
    from splatad_amd.hip import _wrapper as ops

    def leaves(*ts):
        return [t.detach().clone().requires_grad_(True) for t in ts]

    with torch.no_grad():
        _, ra, _, meta = lidar_rasterization(
            l["means"], l["quats"], l["scales"], l["opacities"], l["lidar_features"], l["velocities"],
            l["viewmats"], l["raster_pts"], l["tile_elevation_boundaries"], l["linear_velocity"],
            l["angular_velocity"], l["rolling_shutter_time"], min_azimuth=l["min_azimuth"],
            max_azimuth=l["max_azimuth"], min_elevation=l["min_elevation"], max_elevation=l["max_elevation"],
            n_elevation_channels=l["n_elevation_channels"], azimuth_resolution=l["azimuth_resolution"],
            tile_width=l["tile_width"], tile_height=l["tile_height"], near_plane=l["near_plane"],
            far_plane=l["far_plane"], eps2d=l["eps2d"], channel_chunk=33)
        from splatad_amd.hip._backend import _C
        dcomp = _C.fully_fused_lidar_projection_fwd(
            l["means"], None, l["quats"], l["scales"], l["velocities"], l["viewmats"], l["min_elevation"],
            l["max_elevation"], l["min_azimuth"], l["max_azimuth"], l["linear_velocity"], l["angular_velocity"],
            l["rolling_shutter_time"], l["eps2d"], l["near_plane"], l["far_plane"], 0.0, False)[6]
    H, W = ra.shape[1:3]
    ins = leaves(meta["means2d"], meta["conics"], l["lidar_features"], meta["opacities"], meta["depths"])
    rf, ra, asum, med = ops.rasterize_to_points(
        ins[0], ins[1], ins[2], ins[3], meta["pix_vels"], dcomp, l["raster_pts"], W, H,
        l["tile_width"], l["tile_height"], meta["isect_offsets"], meta["flatten_ids"], True, 0.2, ranges=ins[4])
    loss = rf.abs().mean() + ra.mean()
    out["lidar_rasterize_bwd_ms"] = time_kernel(lambda: torch.autograd.grad(loss, ins, retain_graph=True), 5)
    del l, q, ins, rf, ra, asum, med, loss, meta

    s = workloads.to_device(workloads.camera_driving(n=args.n), dev)
    with torch.no_grad():
        _, _, meta = rasterization(
            s["means"], s["quats"], s["scales"], s["opacities"], s["colors"], s["velocities"], s["viewmats"],
            s["Ks"], s["width"], s["height"], s["linear_velocity"], s["angular_velocity"],
            s["rolling_shutter_time"], sh_degree=s["sh_degree"], packed=False, render_mode="RGB+D",
            near_plane=s["near_plane"], far_plane=s["far_plane"], eps2d=s["eps2d"], tile_size=s["tile_size"])
        cols = torch.rand((1, s["means"].shape[0], 4), device=dev)
        target = torch.rand((1, s["height"], s["width"], 4), device=dev)
    ins = leaves(meta["means2d"], meta["conics"], cols, meta["opacities"])
    rc, ra = ops.rasterize_to_pixels(
        ins[0], ins[1], ins[2], ins[3], meta["pix_vels"], s["width"], s["height"], s["tile_size"],
        meta["isect_offsets"], meta["flatten_ids"], rolling_shutter_time=s["rolling_shutter_time"])
    loss = (rc - target).abs().mean() + ra.mean()
    out["camera_rasterize_bwd_ms"] = time_kernel(lambda: torch.autograd.grad(loss, ins, retain_graph=True), 5)
    return out


def bench_configs(args):
    """Driver-timed legs for the benchmark's other forward configurations: configs[0] (10k
    Gaussians, 320x240, RGB, packed and unpacked) and configs[3] (2M Gaussians around the sensor:
    six 1920x1080 rolling-shutter cameras in one call, and the 128x2048 sweep), each with its
    step time, its intersections and the event-timed stages of the call."""
    import torch

    from splatad_amd import lidar_rasterization, rasterization, workloads
    from splatad_amd.hip._backend import _C

    dev = torch.device("cuda:0")
    out = {}
    steps, warmup = max(5, args.steps // 2), max(2, args.warmup // 5)

    def camera_leg(s, label, render_mode):
        C = s["viewmats"].shape[0]

        def run(packed=False):
            return rasterization(
                s["means"], s["quats"], s["scales"], s["opacities"], s["colors"], s["velocities"],
                s["viewmats"], s["Ks"], s["width"], s["height"], s["linear_velocity"],
                s["angular_velocity"], s["rolling_shutter_time"], sh_degree=s["sh_degree"],
                packed=packed, render_mode=render_mode, near_plane=s["near_plane"],
                far_plane=s["far_plane"], eps2d=s["eps2d"], tile_size=s["tile_size"])

        sec = time_steps(run, steps, warmup)
        sec_packed = time_steps(lambda: run(True), steps, warmup)
        _, _, meta = run()
        W, H, ts = s["width"], s["height"], s["tile_size"]
        zeros = torch.zeros((C, 3), device=dev)  # a sensor at rest, as rasterization() passes it
        lin = s["linear_velocity"] if s["linear_velocity"] is not None else zeros
        ang = s["angular_velocity"] if s["angular_velocity"] is not None else zeros
        rs = s["rolling_shutter_time"] if s["rolling_shutter_time"] is not None else zeros[:, 0].contiguous()
        stages = {
            "projection_ms": time_kernel(lambda: _C.fully_fused_projection_fwd(
                s["means"], None, s["quats"], s["scales"], s["velocities"], s["viewmats"], s["Ks"], W, H,
                lin, ang, rs, s["eps2d"], s["near_plane"], s["far_plane"], 0.0, False), 5),
            "isect_sort_ms": time_kernel(lambda: _C.isect_tiles(
                meta["means2d"], meta["radii"], meta["depths"], None, None, C, ts, meta["tile_width"],
                meta["tile_height"], True, True), 5),
        }
        stages["rest_ms (colours + compositing + host gaps)"] = sec * 1e3 - sum(stages.values())
        return {"workload": label, "ms": sec * 1e3, "ms_packed": sec_packed * 1e3,
                "Mpix_per_s": C * W * H / sec / 1e6, "n_isects": int(meta["flatten_ids"].shape[0]),
                "visible_rows": int((meta["radii"][..., 0] > 0).sum().item()),
                "stage_ms": {k: round(v, 4) for k, v in stages.items()}}

    if args.only_configs == "rig":
        with torch.no_grad():
            s = workloads.to_device(workloads.camera_driving(n=2 * args.n, n_cameras=6), dev)
            run = lambda: rasterization(
                s["means"], s["quats"], s["scales"], s["opacities"], s["colors"], s["velocities"],
                s["viewmats"], s["Ks"], s["width"], s["height"], s["linear_velocity"],
                s["angular_velocity"], s["rolling_shutter_time"], sh_degree=s["sh_degree"],
                packed=False, render_mode="RGB+D", near_plane=s["near_plane"],
                far_plane=s["far_plane"], eps2d=s["eps2d"], tile_size=s["tile_size"])
            sec = time_steps(run, steps, warmup)
            return {"config3_cameras": {"ms": sec * 1e3, "steps": steps, "warmup": warmup,
                                        "n_isects": int(run()[2]["flatten_ids"].shape[0])}}
    with torch.no_grad():
        s = workloads.to_device(workloads.camera_small(), dev)
        out["config0"] = camera_leg(s, "10000 Gaussians, 320x240, RGB, no rolling shutter (BASELINE configs[0])", "RGB")
        del s
        s = workloads.to_device(workloads.camera_driving(n=2 * args.n, n_cameras=6), dev)
        out["config3_cameras"] = camera_leg(
            s, "%d Gaussians around the sensor, six 1920x1080 rolling-shutter cameras in one call, SH degree 3, "
               "RGB+D (BASELINE configs[3])" % (2 * args.n), "RGB+D")
        del s
        torch.cuda.empty_cache()
        l = workloads.to_device(workloads.lidar_sweep(n=2 * args.n), dev)

        def lidar_run():
            return lidar_rasterization(
                l["means"], l["quats"], l["scales"], l["opacities"], l["lidar_features"],
                l["velocities"], l["viewmats"], l["raster_pts"], l["tile_elevation_boundaries"],
                l["linear_velocity"], l["angular_velocity"], l["rolling_shutter_time"],
                min_azimuth=l["min_azimuth"], max_azimuth=l["max_azimuth"],
                min_elevation=l["min_elevation"], max_elevation=l["max_elevation"],
                n_elevation_channels=l["n_elevation_channels"],
                azimuth_resolution=l["azimuth_resolution"], tile_width=l["tile_width"],
                tile_height=l["tile_height"], near_plane=l["near_plane"], far_plane=l["far_plane"],
                eps2d=l["eps2d"], channel_chunk=33)

        sec = time_steps(lidar_run, steps, warmup)
        rf, ra, _, meta = lidar_run()
        stages = {"isect_sort_ms": time_kernel(lambda: _C.isect_lidar_tiles(
            meta["means2d"], meta["radii"], meta["depths"], None, None, 1, l["tile_elevation_boundaries"],
            l["azimuth_resolution"] * l["tile_width"], l["min_azimuth"], True, True), 5)}
        out["config3_lidar"] = {
            "workload": "%d Gaussians, 128x2048 sweep, 32 features + range (BASELINE configs[3])" % (2 * args.n),
            "ms": sec * 1e3, "Mpts_per_s": ra.numel() / sec / 1e6, "n_isects": int(meta["flatten_ids"].shape[0]),
            "stage_ms": {k: round(v, 4) for k, v in stages.items()}}
        out["config3_frame_ms"] = out["config3_cameras"]["ms"] + out["config3_lidar"]["ms"]
    return out


def cpu_baseline_camera(args):
    """The CPU oracle on the same camera workload (same seed and distributions), OpenMP over
    all host cores given to the process; bounded by using fewer Gaussians when needed."""
    import numpy as np

    import oracle
    from splatad_amd import workloads

    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    oracle.set_num_threads(cores)
    n = args.cpu_n
    s = workloads.camera_driving(n=n)
    npy = lambda t: t.numpy()
    W, H, ts = s["width"], s["height"], s["tile_size"]
    tw, th = -(-W // ts), -(-H // ts)
    def frame():
        radii, m2, depths, conics, _, pv = oracle.projection_fwd(
            npy(s["means"]), None, npy(s["quats"]), npy(s["scales"]), None, npy(s["viewmats"]),
            npy(s["Ks"]), W, H, npy(s["linear_velocity"]), npy(s["angular_velocity"]),
            npy(s["rolling_shutter_time"]), eps2d=s["eps2d"], near_plane=s["near_plane"],
            far_plane=s["far_plane"], precision="f32")
        c2w = np.linalg.inv(npy(s["viewmats"]))
        dirs = npy(s["means"])[None] - c2w[:, None, :3, 3]
        cols = oracle.spherical_harmonics(3, dirs, np.broadcast_to(npy(s["colors"])[None], (1, n, 16, 3)),
                                          masks=radii[..., 0] > 0, precision="f32")
        cols = np.concatenate([np.maximum(cols + 0.5, 0.0), depths[..., None]], -1)
        _, ids, flat = oracle.isect_tiles(m2, radii, depths, ts, tw, th)
        offs = oracle.isect_offset_encode(ids, 1, tw, th)
        opac = npy(s["opacities"])[None]
        oracle.rasterize_to_pixels_fwd(m2, conics, cols, opac, pv, npy(s["rolling_shutter_time"]), None,
                                       W, H, ts, offs, flat, precision="f32")

    # whole frames for about ten seconds (three at least), the first one included
    frames, t0 = 0, time.perf_counter()
    while frames < 3 or (time.perf_counter() - t0 < 10.0 and frames < 64):
        frame()
        frames += 1
    dt = (time.perf_counter() - t0) / frames
    return dict(value=W * H / dt / 1e6, unit="Mpix/s", cores=cores, kind="port",
                sample=f"{frames} full {W}x{H} forward frames of the same workload with {n} Gaussians "
                       f"({dt:.2f} s each; C oracle, OpenMP in projection/SH/compositing, serial "
                       "intersection and merge sort)")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--n", type=int, default=1_000_000, help="Gaussians (default: the benchmark's 1M)")
    ap.add_argument("--cpu-n", type=int, default=1_000_000, help="Gaussians of the CPU baseline sample")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-lidar", action="store_true")
    ap.add_argument("--no-bwd", action="store_true", help="skip the forward + backward timing")
    ap.add_argument("--no-configs", action="store_true", help="skip the legs for configs[0] and configs[3]")
    ap.add_argument("--only-configs", nargs="?", const="all", default=None, choices=["all", "rig"],
                    help="run the legs for configs[0] and configs[3] alone and print their JSON object; "
                         "'rig' runs only the unpacked six-camera call of configs[3] (what the kernel "
                         "trace of the rig under profiles/ was made with)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three 1 GiB device-to-device copies (known HBM traffic, used "
                         "to scale FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build renders on one GPU; --gpus must be 1 "
              "(with more GPUs each would render its own share of the sensors)", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.only_configs:
        print(json.dumps({"configs": bench_configs(args)}))
        return
    cam = bench_camera(args)
    lid = None if args.no_lidar else bench_lidar(args)
    achieved = cam["alg_bytes"] / (cam["kernel_ms"] * 1e-3) / 1e9
    plain = cam["stage_bytes"]["rasterize_given_colors_ms"] / (cam["stages"]["rasterize_given_colors_ms"] * 1e-3) / 1e9
    counters = profiled_counters() if args.n == 1_000_000 else {}
    # (template arguments: channels, pixels per lane, diagnostic, colours evaluated in the kernel,
    # last ids kept)
    cam_kernel = "rasterize_to_pixels_fwd_kernel<%d, 2, false, true, false>" % cam["channels"]
    cam_plain_kernel = "rasterize_to_pixels_fwd_kernel<%d, 2, false, false, true>" % cam["channels"]
    lanes = cam["lanes"]
    pairs = lanes["iterations"] * 64 * lanes["pixels_per_lane"] * lanes["compositing_lane_fraction"]
    out = {
        "metric": "camera Mpix/s (fwd)",
        "value": cam["pixels"] / cam["sec"] / 1e6,
        "unit": "Mpix/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": cam["sec"] * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "driving camera, rolling shutter: %d Gaussians, 1920x1080, SH degree 3, "
                        "RGB+D, packed=False (BASELINE configs[1])" % args.n,
            "n_isects": cam["n_isects"], "n_isects_consumed": cam["i_need"],
            "visible_gaussians": cam["nnz"], "ms_per_step_packed": cam["sec_packed"] * 1e3,
            "stage_ms": {k: round(v, 4) for k, v in cam["stages"].items()},
            "lane_utilisation": {k: (round(v, 4) if isinstance(v, float) else v) for k, v in cam["lanes"].items()},
            "tile_cycles": cam["tile_cycles"],
        },
        "stages": stage_rooflines(cam),
        "roofline": {
            # the compositing kernel that evaluates the spherical-harmonic colours of the entries
            # it stages: the entries' geometry and depth, the mean and coefficient row of every
            # (camera, Gaussian) among them once, the image.  `frac` is this kernel against these
            # bytes; `given_colors` is the same kernel handed the colours (as calls that want
            # gradients run it) against the bytes of that formulation.
            "kernel": cam_kernel,
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": hbm_traffic_bytes(counters, cam_kernel),
            "algorithmic_bytes": cam["alg_bytes"], "kernel_ms": cam["kernel_ms"],
            "rows_staged": cam["rows_staged"], "color_cache_left_empty": cam["cache_left_empty"],
            "given_colors": {"kernel": cam_plain_kernel, "achieved": plain, "frac": plain / HBM_PEAK_GBS,
                             "algorithmic_bytes": cam["stage_bytes"]["rasterize_given_colors_ms"],
                             "kernel_ms": cam["stages"]["rasterize_given_colors_ms"],
                             "traffic": hbm_traffic_bytes(counters, cam_plain_kernel)},
            # what actually bounds the kernel: vector instruction issue
            "valu_issue": valu_roofline(counters, cam_kernel, cam["kernel_ms"], pairs),
            "valu_issue_given_colors": valu_roofline(counters, cam_plain_kernel,
                                                     cam["stages"]["rasterize_given_colors_ms"], pairs),
        },
    }
    if lid is not None:
        l_ach = lid["alg_bytes"] / (lid["kernel_ms"] * 1e-3) / 1e9
        lid_kernel = "rasterize_to_points_fwd_kernel<%d, %s>" % (lid["channels"], "true" if lid["channels"] in (32, 33) else "false")
        out["lidar"] = {
            "metric": "lidar Mpts/s (fwd)", "value": lid["points"] / lid["sec"] / 1e6,
            "unit": "Mpts/s", "ms_per_step": lid["sec"] * 1e3,
            "ms_per_step_channel_chunk_32": lid["sec_chunk32"] * 1e3,
            "workload": "128x2048 lidar sweep, %d Gaussians, 32 features + range, tile 64x4, "
                        "channel_chunk=33 (BASELINE configs[2])" % args.n,
            "n_isects": lid["n_isects"], "n_isects_consumed": lid["i_need"],
            "stage_ms": {k: round(v, 4) for k, v in lid["stages"].items()},
            "stages": stage_rooflines(lid),
            "tile_cycles": lid["tile_cycles"],
            "roofline": {"kernel": lid_kernel,
                         "bound": "hbm", "achieved": l_ach, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": l_ach / HBM_PEAK_GBS,
                         "traffic": hbm_traffic_bytes(counters, lid_kernel),
                         "algorithmic_bytes": lid["alg_bytes"], "kernel_ms": lid["kernel_ms"],
                         # (the kernel reads the features of the Gaussians it composites only, about
                         # an eighth of those it stages: its traffic lies between the two figures)
                         "algorithmic_bytes_with_staged_features": lid["alg_bytes_features"],
                         # the kernel lasts as long as its slowest tile (all tiles resident at once):
                         # vector issue fills less than half of it
                         "valu_issue": valu_roofline(counters, lid_kernel, lid["kernel_ms"])},
        }
    if not args.no_configs:
        out["configs"] = bench_configs(args)
    if not args.no_bwd:
        bwd = bench_backward(args)
        out["backward"] = {k: round(v, 4) for k, v in bwd.items()}
        for key, kernel in (("camera_rasterize_bwd_ms", "rasterize_bwd_kernel<4, false, 2, false>"),
                            ("lidar_rasterize_bwd_ms", "rasterize_bwd_kernel<33, true, 1, true>")):
            # (the timed interval also holds the clearing and unpacking launches around the kernel)
            r = valu_roofline(counters, kernel, bwd[key])
            if r is not None:
                out["backward"][key.replace("_ms", "_valu_issue")] = r
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_camera(args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
