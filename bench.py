#!/usr/bin/env python3
"""Benchmark of the rasterizer hot path on one MI355X.

A step is one training-style view: preprocess forward -> render forward (tile
count and histogram, scatter by tile, per-tile sorts, blend) -> render backward ->
preprocess backward, driven through the Python operator API with N(0,1)
upstream gradients on colour, the 5-channel map and plane depth.  Workload:
BASELINE config 1 (1M Gaussians, 1152x864, SH degree 3), synthetic, seed 0,
inputs resident in HBM before the timed region.

Prints one JSON line (see --help for flags).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "citygs-x_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))  # the seeded scene generator (gs_scenes) is shared with the tests

HBM_PEAK_GBS = 8000.0

# Algorithmic bytes per unit of each HBM-bound stage (G = Gaussian, I = (Gaussian,tile) instance).
BYTES_PER_GAUSSIAN = {
    # What the kernel moves in a training step: 44 B geometry in + 192 B SH in + 32 B geometry out (the 56 B of the
    # reference's interface less the 24 B of cov3D, which the backward kernel forms again from scales and rotations)
    # + 12 B rgb + 3 B clamped + 36 B: the derivative of the colour with respect to the view direction, which the
    # backward kernel reads instead of the 192 B of coefficients.  (The reference's interface: 307 B.)
    "preprocess_fwd": 307 - 24 + 36,
    "tile_count": 16,
    # radius 4 + centre 8 + conic and opacity 16 + colour 12 + geometry channels 20 + depth 4 in, one 64 B record out
    # (visible Gaussians only: the figure is an upper bound)
    "pack_operands": 64 + 64,
    "inclusive_sum": 8,
    "preprocess_bwd": 560 - 192 + 36 - 24,
    "all_map_fwd": 60,   # means 12 + scales 12 + rotations 16 in, 20 out
    "all_map_bwd": 88,   # the same 40 + 20 B of upstream gradient in, 12 + 16 out
}
# sort: one 8 B histogram read + 5 passes (9-bit digits over the 44 key bits) x (12 B read + 12 B write)
# tile ranges: 8 B key read, plus the gather of the sorted Gaussian ids fused into it (index, table, output: 12 B)
# tile_sort: one 16 B record (Gaussian, emission index, depth bits) in, 8 B key + 4 B emission index + 4 B Gaussian
# id out.
# sort_pairs: the radix sort (5 passes of 9-bit digits over 44 key bits), timed on its own on keys of the same
# distribution: only a view whose tile grid has more than 30000 tiles builds its lists with it.
BYTES_PER_INSTANCE = {"sort_pairs": 128, "identify_tile_ranges": 20, "tile_sort": 32}
# simple-knn (distCUDA2) per point: bounding box 24 B (12 read, twice: partial and final are one pass over the
# points plus a small second one: the figure the reference's two reduction passes give), curve keys 16 B (12 in, 4 out), 32-bit radix sort with
# index payload 68 B (4 B histogram read + 4 passes x (8 in + 8 out)), gather into sorted order 32 B (4 B index +
# 12 B point in, 16 B out), box bounds 32 B (the 1024-point boxes and the 64-point leaves each read the 16 B points).
BYTES_PER_POINT = {"knn_minmax": 24, "knn_keys": 16, "knn_sort": 68, "knn_gather": 32, "knn_boxes": 32}
# The binning stage as a whole, in per-unit figures of the reference's algorithm on the same job:
# per Gaussian tile count 16 + prefix sum 8 + key emission 20 B; per instance 12 B of key/value written, 152 B
# for a radix sort with 8-bit digits over the 44 key bits, 8 B for the tile ranges.  The per-tile route here moves
# less: per instance a 16 B record written and read once, then 16 B of sorted keys, emission indices and ids.
BINNING_REFERENCE_BYTES = (44, 172)   # per Gaussian, per instance
BINNING_OWN_BYTES = (44, 48)
BINNING_STAGES = ("tile_count", "inclusive_sum", "bucket_scatter", "tile_sort", "duplicate_with_keys",
                  "identify_tile_ranges")
BINNING_KERNELS = ("bucket_count_kernel", "bucket_columns_kernel", "bucket_ranges_kernel",
                   "bucket_scatter_staged_kernel",  # (bucket_scatter_kernel beyond one round per workgroup)
                   "tile_sort_registers_kernel")  # (views with lists above 2048 records: + tile_radix_sort_kernel)
FP32_MATRIX_PEAK_TFLOPS = 157.3
# Neural-Gaussian generation with 10 offsets: (bytes per anchor, bytes per selected Gaussian, flops per anchor).
#   opacity:   feat 128 + anchor 12 in; 10 opacities, 10 mask bytes, 1 count out;      2 (35*32 + 32*10) flops
#   gaussians: feat, anchor, offsets 120, scaling 24, opacities 40, first 4 in; 72 B per Gaussian out (xyz, color,
#              opacity, scaling, rot, aux);                                            2 (2*35*32 + 32*100) flops
#   backward:  the same inputs; per Gaussian 56 B of upstream gradients + color, rot, aux 44 B; per anchor
#              284 B of gradients out; layer 1 again, dH, dX, dW2, dW1:                34240 flops
NEURAL_COST = {"neural_opacity": (191, 0, 2880), "neural_gaussians": (328, 72, 10880),
               "neural_backward": (328 + 284, 100, 34240)}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=1, help="BASELINE config index (1 = the headline workload)")
    ap.add_argument("--gaussians", type=int, default=None, help="override the Gaussian count (debugging only)")
    ap.add_argument("--all-views", action="store_true",
                    help="time the step for every camera of the configuration's batch and print one JSON object "
                         "with a per-view list (ms per view, per-stage times, instances, longest list, route); "
                         "the other BASELINE configurations are parity cases, this is how their figures are made")
    ap.add_argument("--interleave", action="store_true",
                    help="with --all-views: after the per-view measurements, render the cameras of the batch one "
                         "after the other, step by step, as a training loop does (every view is launched on what the "
                         "previous, different view needed), and report the share of views whose list kernels ran "
                         "ahead of the instance count, the time per view, and the time per view when no view may "
                         "run ahead (the cost of a miss)")
    ap.add_argument("--with-all-map", action="store_true",
                    help="with --all-views: build the geometry channels inside every step with the fused op, forward "
                         "and backward, linked to the preprocess outputs as a caller links them "
                         "(build_all_map(..., blend_records_of=means2D)), instead of preparing them once per camera")
    ap.add_argument("--vary-gaussians", action="store_true",
                    help="with --interleave: every other step renders only the first 90 %% of the Gaussians, as the "
                         "count changes at every densification of a training run")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-views-in-flight", action="store_true",
                    help="skip the supplementary measurement with two views in flight on two streams (profiling "
                         "runs: kernels that overlap there would blur the per-kernel averages)")
    ap.add_argument("--cpu-runs", type=int, default=3)
    ap.add_argument("--copy-calibration-mib", type=int, default=0,
                    help="also run three plain device-to-device copies of this many MiB after the timed regions: "
                         "a kernel of known traffic against which FETCH_SIZE / WRITE_SIZE counters are scaled")
    return ap.parse_args()


def cpu_baseline(g, cam, am, ug, runs):
    """Times the CPU oracle on the same view with the host's cores."""
    import numpy as np
    from oracle import oracle as orc
    threads = min(16, os.cpu_count() or 1)
    orc.set_num_threads(threads)
    n = lambda t: t.numpy()
    W, H = cam.image_width, cam.image_height
    gx, gy = orc.tile_grid(W, H)
    cl = np.ones(gx * gy, bool)
    bg = np.zeros(3, np.float32)
    times = []
    for _ in range(runs):
        t0 = time.perf_counter()
        pre = orc.preprocess_fwd(n(g["means3D"]), n(g["scales"]), n(g["rotations"]), n(g["opacities"]), n(g["shs"]),
                                 n(cam.world_view_transform), n(cam.full_proj_transform), n(cam.camera_center), W, H,
                                 cam.tanfovx, cam.tanfovy)
        b = orc.bin_and_sort(pre["radii"], pre["means2D"], pre["depths"], cl, W, H)
        f = orc.render_fwd(b["ranges"], b["point_list"], pre["means2D"], pre["rgb"], am, pre["conic_opacity"], cl, bg,
                           W, H, cam.tanfovx, cam.tanfovy)
        rb = orc.render_bwd(b["ranges"], b["point_list"], pre["means2D"], pre["conic_opacity"], pre["rgb"], am,
                            f["out_all_map"], f["final_T"], f["n_contrib"], cl, bg, n(ug["color"]), n(ug["all_map"]),
                            n(ug["plane_depth"]), W, H, cam.tanfovx, cam.tanfovy)
        orc.preprocess_bwd(n(g["means3D"]), pre["radii"], n(g["shs"]), pre["clamped"], n(g["scales"]),
                           n(g["rotations"]), pre["cov3D"], n(cam.world_view_transform), n(cam.full_proj_transform),
                           n(cam.camera_center), W, H, cam.tanfovx, cam.tanfovy, rb["dL_dmeans2D"],
                           rb["dL_dconic_opacity"], rb["dL_dcolors"])
        times.append((time.perf_counter() - t0) * 1e3)
    times.sort()
    return {"value": round(times[len(times) // 2], 2), "unit": "ms/view", "cores": threads, "kind": "port",
            "sample": f"{runs} full views of the same workload (median); C++/OpenMP oracle incl. python glue"}


FORWARD_STAGES = ("preprocess_fwd", "tile_count", "inclusive_sum", "pack_operands", "bucket_scatter", "tile_sort",
                  "duplicate_with_keys", "identify_tile_ranges", "render_fwd")


def all_views(args):
    """The same step as the headline measurement, for every camera of the configuration: per view the time of
    `steps` steps, the per-stage event times of another `steps` steps, and what the view looks like."""
    import torch
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import GaussianRasterizationSettings, GaussianRasterizer, _C, build_all_map
    dev = "cuda:0"
    g, cams = gs_scenes.make_scene(args.config, P=args.gaussians)
    P = g["means3D"].shape[0]
    leaf = {k: g[k].to(dev).requires_grad_(True) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
    per_view = []
    steppers = []
    for v, cam in enumerate(cams):
        W, H = cam.image_width, cam.image_height
        rs = GaussianRasterizationSettings(
            image_height=H, image_width=W, tanfovx=cam.tanfovx, tanfovy=cam.tanfovy, bg=torch.zeros(3, device=dev),
            scale_modifier=1.0, viewmatrix=cam.world_view_transform.to(dev),
            projmatrix=cam.full_proj_transform.to(dev), sh_degree=3, campos=cam.camera_center.to(dev),
            prefiltered=False, render_geo=True, debug=False)
        rast = GaussianRasterizer(rs)
        am = _C.build_all_map(leaf["means3D"].detach(), leaf["scales"].detach(), leaf["rotations"].detach(),
                              rs.viewmatrix, rs.campos)
        ug = {k: t.to(dev) for k, t in gs_scenes.upstream_grads(cam, seed=v).items()}
        gx, gy = (W + 15) // 16, (H + 15) // 16
        cl = torch.ones(gy, gx, dtype=torch.bool, device=dev)
        m2abs = torch.zeros(P, 3, device=dev, requires_grad=True)
        ca = {"avoid_pixel_all2all": False, "stats_collector": {}}
        info = {}

        def step(n_gaussians=None, rast=rast, rs=rs, am=am, ug=ug, cl=cl, m2abs=m2abs, ca=ca, info=info):
            """One view; n_gaussians: render only the first so many Gaussians (a scene between two densifications)."""
            lf = leaf if n_gaussians is None else {k: t[:n_gaussians] for k, t in leaf.items()}
            a_m = am if n_gaussians is None else am[:n_gaussians]
            m2 = m2abs if n_gaussians is None else m2abs[:n_gaussians]
            for t in leaf.values():
                t.grad = None
            m2abs.grad = None
            means2D, rgb, co, radii, depths = rast.preprocess_gaussians(
                lf["means3D"], lf["scales"], lf["rotations"], lf["shs"], lf["opacities"], ca)
            if args.with_all_map:
                a_m = build_all_map(lf["means3D"], lf["scales"], lf["rotations"], rs.viewmatrix, rs.campos,
                                    blend_records_of=means2D)
            color, n_render, _, _, _, oam, opd = rast.render_gaussians(means2D, m2, co, rgb, a_m, depths, radii, cl,
                                                                       cl, ca)
            torch.autograd.backward([color, oam, opd], [ug["color"], ug["all_map"], ug["plane_depth"]])
            info["n_render"], info["radii"] = n_render, radii
            return bool(ca["stats_collector"].get("launched_ahead", False))

        steppers.append(step)
        for _ in range(max(args.warmup, 60 if v == 0 else 3)):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        gn.stage_timing(True)
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        gn.stage_timing(False)
        st = gn.stage_timing_collect()
        stages = {k: round(tot / max(cnt, 1), 4) for k, (tot, cnt) in st.items()}
        per_view.append({
            "view": v, "image": f"{W}x{H}", "ms_per_view": round(ms, 4), "instances_R": int(info["n_render"].sum()),
            "longest_list": int(info["n_render"].max()), "visible_gaussians": int((info["radii"] > 0).sum()),
            "route": "radix sort over all keys" if "sort_pairs" in stages else "per-tile lists",
            "stages_ms": stages})
    out = {"metric": "fwd+bwd ms/view, every camera of the batch", "config": args.config, "gaussians": P,
           "all_map_built_inside_the_step": bool(args.with_all_map),
           "steps": args.steps, "n_gpus": 1, "dtype": "f32", "data": "synthetic", "per_view": per_view}
    if args.interleave:
        out["interleaved"] = interleaved(args, steppers, P)
    print(json.dumps(out))


def interleaved(args, steppers, P):
    """The cameras of the batch one after the other, `steps` rounds: every view is launched on the expectation the
    previous, different view left (and, with --vary-gaussians, every other step on nine tenths of the Gaussians).
    Per camera the time of its steps by an event pair around each; then the same rounds with the expectation
    cleared before every step, so that no view runs ahead: the difference is what a miss costs."""
    import torch
    import diff_gaussian_rasterization as dgr
    n_views = len(steppers)

    def rounds(clear):
        per_cam = [[] for _ in steppers]
        ahead = 0
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        k = 0
        for _ in range(args.steps):
            for v, step in enumerate(steppers):
                if clear:
                    dgr._expectations.clear()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                ahead += int(step(int(P * 0.9) if (args.vary_gaussians and k % 2 == 1) else None))
                e1.record()
                per_cam[v].append((e0, e1))
                k += 1
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / k
        cam_ms = [round(sum(a.elapsed_time(b) for a, b in evs) / len(evs), 4) for evs in per_cam]
        return wall, ahead / k, cam_ms

    rounds(False)  # (one untimed pass: allocator pools for the alternating sizes)
    wall, rate, cam_ms = rounds(False)
    wall_miss, rate_miss, cam_miss = rounds(True)
    return {"views_per_round": n_views, "rounds": args.steps, "vary_gaussians": bool(args.vary_gaussians),
            "ms_per_view_mean": round(wall, 4), "launched_ahead_rate": round(rate, 4),
            "ms_per_view_by_camera": cam_ms,
            "never_ahead": {"ms_per_view_mean": round(wall_miss, 4), "launched_ahead_rate": round(rate_miss, 4),
                            "ms_per_view_by_camera": cam_miss},
            "miss_cost_ms_per_view": round(wall_miss - wall, 4) if rate > 0 else None,
            "note": "a view whose expectation does not hold (more instances than the previous view's figure plus 25 % "
                    "+ 65536, or a longer list than its sort variant takes) runs the launched-ahead kernels as "
                    "no-ops and then the ordinary route; never_ahead is that ordinary route for every view"}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives are part of it); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import GaussianRasterizationSettings, GaussianRasterizer

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the rasterizer has no CPU path", file=sys.stderr)
        sys.exit(2)
    if args.all_views:
        all_views(args)
        return
    dev = "cuda:0"
    g, cams = gs_scenes.make_scene(args.config, P=args.gaussians, n_views=1)
    cam = cams[0]
    P = g["means3D"].shape[0]
    W, H = cam.image_width, cam.image_height
    am_cpu = gs_scenes.build_all_map(g["means3D"], g["scales"], g["rotations"], cam)
    ug_cpu = gs_scenes.upstream_grads(cam)

    rs = GaussianRasterizationSettings(
        image_height=H, image_width=W, tanfovx=cam.tanfovx, tanfovy=cam.tanfovy, bg=torch.zeros(3, device=dev),
        scale_modifier=1.0, viewmatrix=cam.world_view_transform.to(dev), projmatrix=cam.full_proj_transform.to(dev),
        sh_degree=3, campos=cam.camera_center.to(dev), prefiltered=False, render_geo=True, debug=False)
    rast = GaussianRasterizer(rs)
    leaf = {k: g[k].to(dev).requires_grad_(True) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
    am = am_cpu.to(dev)
    ug = {k: v.to(dev) for k, v in ug_cpu.items()}
    gx, gy = (W + 15) // 16, (H + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=dev)
    m2abs = torch.zeros(P, 3, device=dev, requires_grad=True)
    ca = {"avoid_pixel_all2all": False, "stats_collector": {}}
    info = {}

    from diff_gaussian_rasterization import build_all_map
    vmat, cpos = rs.viewmatrix, rs.campos  # (the camera's own tensors, as the caller passes them to both ops)

    def step(leaf=leaf, m2abs=m2abs, with_all_map=False):
        """with_all_map: the geometry channels are built inside the step by the fused op, forward and backward, as
        the caller builds them for every view between the two rasterizer ops
        (gaussian_renderer/__init__.py:1501-1518); otherwise they are an input prepared once."""
        for t in leaf.values():
            t.grad = None
        m2abs.grad = None
        means2D, rgb, co, radii, depths = rast.preprocess_gaussians(leaf["means3D"], leaf["scales"],
                                                                    leaf["rotations"], leaf["shs"],
                                                                    leaf["opacities"], ca)
        a_m = (build_all_map(leaf["means3D"], leaf["scales"], leaf["rotations"], vmat, cpos, blend_records_of=means2D)
               if with_all_map else am)
        color, n_render, _, _, _, oam, opd = rast.render_gaussians(means2D, m2abs, co, rgb, a_m, depths, radii, cl, cl,
                                                                   ca)
        torch.autograd.backward([color, oam, opd], [ug["color"], ug["all_map"], ug["plane_depth"]])
        info["n_render"] = n_render

    # inputs of the neural-Gaussian generation stage (timed further down), and one untimed call.  All set-up
    # that keeps the host busy and the GPU idle comes before the warm-up steps, so that the timed region follows
    # them directly.
    import gs_neural
    N_a, k_a = 200_000, 10
    sc_a = gs_scenes.make_anchor_scene(N_a, k_a, 7)
    na = {k: sc_a[k].to(dev).requires_grad_(True) for k in ("anchor", "feat", "offsets", "scaling")}
    na_cam = sc_a["campos"].to(dev)
    na_mlps = [tuple(x.to(dev).requires_grad_(True) for x in m) for m in sc_a["mlps"]]
    na_leaves = list(na.values()) + [x for m in na_mlps for x in m]
    no = gs_neural.neural_gaussians(na["anchor"], na["feat"], na["offsets"], na["scaling"], na_cam, *na_mlps)
    torch.autograd.backward(list(no[:5]), [torch.ones_like(o) for o in no[:5]])
    del no
    # The GPU has idled while the host built the scenes, and it takes some 30 ms of sustained work before its
    # clocks are back at their steady level: with five warm-up steps (4 ms) the first of twenty timed steps still
    # run during that ramp (0.835 ms per view against 0.794 measured after 60 or 200 warm-up steps).  The steps
    # below bring the clocks up; then come the W warm-up steps proper.
    ramp_steps = max(0, 60 - args.warmup)
    for _ in range(ramp_steps):
        step()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # timed region: exactly `steps` steps, nothing but the work itself on the stream
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    # Beside `value`: the same steps with the geometry channels built inside each step (forward and backward of the
    # fused all_map op), which is what a caller's view costs from parameters to gradients.
    for _ in range(max(3, args.warmup)):
        step(with_all_map=True)
    torch.cuda.synchronize()
    t0a = time.perf_counter()
    for _ in range(args.steps):
        step(with_all_map=True)
    torch.cuda.synchronize()
    ms_per_step_with_all_map = (time.perf_counter() - t0a) * 1e3 / args.steps
    # Not `value`: the same steps with two views in flight, alternating between two streams (default priority)
    # as a caller would run the views of a batch, so that one view's bandwidth-bound stages overlap the other's
    # blend kernels.  Every view has its own parameter copies here because each step resets and refills `.grad`.
    ms_per_view_two_in_flight = None
    if not args.no_views_in_flight:
        leaf_b = {k: v.detach().clone().requires_grad_(True) for k, v in leaf.items()}
        m2abs_b = torch.zeros(P, 3, device=dev, requires_grad=True)
        lanes = [(torch.cuda.Stream(), leaf, m2abs), (torch.cuda.Stream(), leaf_b, m2abs_b)]
        for s_, _, _ in lanes:
            s_.wait_stream(torch.cuda.current_stream())

        def in_flight(n):
            for i in range(n):
                s_, lf, m2 = lanes[i % 2]
                with torch.cuda.stream(s_):
                    step(lf, m2)
            for s_, _, _ in lanes:
                s_.synchronize()

        in_flight(max(20, args.warmup))  # (each stream's allocator pool has to fill before the rate is steady)
        t0b = time.perf_counter()
        in_flight(args.steps)
        ms_per_view_two_in_flight = (time.perf_counter() - t0b) * 1e3 / args.steps
        torch.cuda.synchronize()
        del leaf_b, m2abs_b, lanes
    # the same `steps` steps again with an event pair around every stage on its stream: the per-kernel
    # durations below come from this region (the event records cost a few microseconds of idle time between
    # kernels, which is why `value` is taken from the region above)
    gn.stage_timing(True)
    t2 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t3 = time.perf_counter()
    # the fused geometry-channel op that sits between the two rasterizer ops in the caller (inside
    # `value_with_all_map`, not inside `value`, whose step takes a prepared all_map): same event pairs
    g_am = torch.randn(P, 5, device=dev)
    # these kernels are shorter than a Python launch: keep the stream busy first so the launches queue up
    # behind it and the event pairs bracket kernels, not host latency
    torch.cuda._sleep(int(4e7))
    for _ in range(args.steps):
        for k in ("means3D", "rotations"):
            leaf[k].grad = None
        build_all_map(leaf["means3D"], leaf["scales"], leaf["rotations"], vmat, cpos).backward(g_am)
    # the optimizer step over the same five parameter tensors (59 M elements), fused into one launch
    from gs_optim import FusedAdam
    opt = FusedAdam([{"params": [leaf[k]], "lr": 1e-5, "name": k} for k in leaf], lr=0.0, eps=1e-15)
    for t in leaf.values():
        t.grad = torch.randn_like(t) * 1e-3
    n_adam = sum(t.numel() for t in leaf.values())
    for _ in range(args.steps):
        opt.step()
    # densification statistics of one view: 1 M anchors x 10 offsets, 40 % visible, 60 % selected, 90 % kept
    import gs_densify
    gen = torch.Generator(device=dev).manual_seed(5)
    A_s, k_s = 1_000_000, 10
    s_vis = torch.rand(A_s, generator=gen, device=dev) < 0.4
    s_sel = torch.rand(int(s_vis.sum()) * k_s, generator=gen, device=dev) < 0.6
    s_flt = torch.rand(int(s_sel.sum()), generator=gen, device=dev) < 0.9
    s_grad = torch.randn(s_flt.numel(), 3, generator=gen, device=dev)
    s_op = torch.randn(s_sel.numel(), 1, generator=gen, device=dev)
    s_acc = [torch.zeros(A_s, 1, device=dev), torch.zeros(A_s, 1, device=dev), torch.zeros(A_s * k_s, 1, device=dev),
             torch.zeros(A_s * k_s, 1, device=dev)]
    stats_bytes = (A_s + 5 * s_sel.numel() + 13 * s_flt.numel() + 16 * int(s_vis.sum()) + 16 * int(s_flt.sum()))
    torch.cuda._sleep(int(4e7))
    for _ in range(args.steps):
        gs_densify.training_statis(s_acc[0], s_acc[1], s_acc[2], s_acc[3], k_s, s_grad, s_op, s_flt, s_sel, s_vis)
    # the masked L1 + SSIM loss maps on the rendered image, forward and backward
    import gs_loss
    gt = torch.rand(3, H, W, device=dev)
    pm = torch.rand(H, W, device=dev) < 0.9
    img_l = torch.rand(3, H, W, device=dev, requires_grad=True)
    torch.cuda._sleep(int(4e7))
    for _ in range(args.steps):
        img_l.grad = None
        l1m, ssm = gs_loss.pixelwise_l1_ssim_with_mask(img_l, gt, pm)
        torch.autograd.backward([l1m, ssm], [gt, gt])
    del l1m, ssm
    # the radix sort on its own: (tile << 32 | depth bits) keys with this view's number of instances per tile, in
    # random order, 32-bit payload
    import ctypes as C
    n_per_tile = info["n_render"].to(torch.int64)
    R_s = int(n_per_tile.sum().item())
    gen_s = torch.Generator(device=dev).manual_seed(11)
    s_tiles = torch.repeat_interleave(torch.arange(n_per_tile.numel(), device=dev), n_per_tile)
    s_depth = (torch.rand(R_s, generator=gen_s, device=dev) * 99.0 + 1.0).view(torch.int32).to(torch.int64)
    s_keys = ((s_tiles << 32) | s_depth)[torch.randperm(R_s, generator=gen_s, device=dev)].contiguous()
    s_vals = torch.arange(R_s, dtype=torch.int32, device=dev)
    s_kout, s_vout = torch.empty_like(s_keys), torch.empty_like(s_vals)
    s_ws_bytes = gn.lib.gs_sort_workspace_bytes(R_s)
    s_ws = torch.empty(s_ws_bytes, dtype=torch.uint8, device=dev)
    s_end_bit = 32 + gn.lib.gs_higher_msb(gx * gy)
    s_ptr = lambda t: C.c_void_p(t.data_ptr())
    torch.cuda._sleep(int(4e7))
    for _ in range(args.steps):
        gn.check(gn.lib.gs_sort_pairs_u64(R_s, s_ptr(s_keys), s_ptr(s_kout), s_ptr(s_vals), s_ptr(s_vout), s_end_bit,
                                          s_ptr(s_ws), s_ws_bytes,
                                          C.c_void_p(torch.cuda.current_stream().cuda_stream)), "gs_sort_pairs_u64")
    assert bool((s_kout[1:] >= s_kout[:-1]).all())
    del s_tiles, s_depth, s_keys, s_vals, s_kout, s_vout, s_ws
    # simple-knn over the 1 M means of this configuration (distCUDA2, run once at initialisation by the caller)
    from simple_knn._C import distCUDA2
    knn_pts = leaf["means3D"].detach()
    torch.cuda._sleep(int(4e7))
    for _ in range(args.steps):
        knn_out = distCUDA2(knn_pts)
    del knn_out
    # neural-Gaussian generation for one view: 200 k visible anchors x 10 offsets through the three MLPs,
    # forward (opacity MLP, scan, color/cov MLPs + post-processing) and backward
    torch.cuda._sleep(int(4e7))
    for _ in range(args.steps):
        for t in na_leaves:
            t.grad = None
        no = gs_neural.neural_gaussians(na["anchor"], na["feat"], na["offsets"], na["scaling"], na_cam, *na_mlps)
        S_a = no[0].shape[0]
        if "na_up" not in info:
            info["na_up"] = [torch.randn_like(o) for o in no[:5]]
        torch.autograd.backward(list(no[:5]), info["na_up"])
    torch.cuda.synchronize()
    gn.stage_timing(False)
    stages = gn.stage_timing_collect()
    torch_neural_ms = []
    for _ in range(5):
        for t in na_leaves:
            t.grad = None
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        ro = gs_scenes.neural_gaussians_torch(na["anchor"], na["feat"], na["offsets"], na["scaling"], na_cam, na_mlps)
        ups = info["na_up"] if ro[0].shape[0] == S_a else [torch.ones_like(o) for o in ro[:5]]
        torch.autograd.backward(list(ro[:5]), ups)
        ev1.record()
        torch.cuda.synchronize()
        torch_neural_ms.append(ev0.elapsed_time(ev1))
    del no, ro, ups, na, na_mlps, na_leaves
    info.pop("na_up")
    ms_per_step_instrumented = (t3 - t2) * 1e3 / args.steps
    # the reference's conv2d formulation of the same maps, forward + backward, for reference
    import math
    import torch.nn.functional as F
    gwin = torch.Tensor([math.exp(-((x - 5) ** 2) / float(2 * 1.5 ** 2)) for x in range(11)])
    gwin = (gwin / gwin.sum()).unsqueeze(1)
    win2 = gwin.mm(gwin.t()).float().unsqueeze(0).unsqueeze(0).expand(3, 1, 11, 11).contiguous().to(dev)
    torch_ssim_ms = []
    for _ in range(5):
        img_l.grad = None
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        mu1 = F.conv2d(img_l, win2, padding=5, groups=3)
        mu2 = F.conv2d(gt, win2, padding=5, groups=3)
        mu1_sq, mu2_sq, mu12 = mu1.pow(2), mu2.pow(2), mu1 * mu2
        sg1 = F.conv2d(img_l * img_l, win2, padding=5, groups=3) - mu1_sq
        sg2 = F.conv2d(gt * gt, win2, padding=5, groups=3) - mu2_sq
        sg12 = F.conv2d(img_l * gt, win2, padding=5, groups=3) - mu12
        smap = ((2 * mu12 + 0.01 ** 2) * (2 * sg12 + 0.03 ** 2)) / ((mu1_sq + mu2_sq + 0.01 ** 2) * (sg1 + sg2 + 0.03 ** 2))
        smap = smap * pm.unsqueeze(0)
        lmap = torch.abs(img_l - gt) * pm.unsqueeze(0)
        torch.autograd.backward([lmap, smap], [gt, gt])
        ev1.record()
        torch.cuda.synchronize()
        torch_ssim_ms.append(ev0.elapsed_time(ev1))
    del gt, pm, img_l
    # the torch statements training_statis consists of, for reference
    torch_stats_ms = []
    for _ in range(5):
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        temp = s_op.clone().view(-1)
        temp[temp < 0] = 0
        s_acc[0][s_vis] += temp.view(-1, k_s).sum(dim=1, keepdim=True)
        s_acc[1][s_vis] += 1
        vis_rep = s_vis.unsqueeze(1).repeat(1, k_s).view(-1)
        combined = torch.zeros(A_s * k_s, dtype=torch.bool, device=dev)
        combined[vis_rep] = s_sel
        temp_mask = combined.clone()
        combined[temp_mask] = s_flt
        s_acc[2][combined] += torch.norm(s_grad[s_flt, :2], dim=-1, keepdim=True)
        s_acc[3][combined] += 1
        ev1.record()
        torch.cuda.synchronize()
        torch_stats_ms.append(ev0.elapsed_time(ev1))
    del s_acc, s_grad, s_op, s_sel, s_flt, s_vis
    # the torch lines it replaces, timed the same way for reference
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch_am_ms = []
    for _ in range(5):
        for k in ("means3D", "rotations"):
            leaf[k].grad = None
        e0.record()
        gs_scenes.build_all_map(leaf["means3D"], leaf["scales"], leaf["rotations"], cam).backward(g_am)
        e1.record()
        torch.cuda.synchronize()
        torch_am_ms.append(e0.elapsed_time(e1))
    for t in leaf.values():
        t.grad = None
    if args.copy_calibration_mib > 0:
        src = torch.empty(args.copy_calibration_mib << 20, dtype=torch.uint8, device=dev).random_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    R = int(info["n_render"].sum().item())

    stage_report = {}
    for name, (tot, cnt) in stages.items():
        ms = tot / max(cnt, 1)
        e = {"ms": round(ms, 4), "launches_per_step": cnt / args.steps}
        nbytes = None
        if name in BYTES_PER_GAUSSIAN:
            nbytes = BYTES_PER_GAUSSIAN[name] * P
        elif name in BYTES_PER_INSTANCE:
            nbytes = BYTES_PER_INSTANCE[name] * R
        elif name in BYTES_PER_POINT:
            nbytes = BYTES_PER_POINT[name] * P
        elif name == "duplicate_with_keys":
            nbytes = 20 * P + 12 * R
        elif name == "bucket_scatter":
            nbytes = 24 * P + 16 * R  # radius, centre, depth, tile count in, prefix sum out; one 16 B record out
        elif name == "ssim_l1_fwd":
            nbytes = (8 + 8 + 12) * 3 * H * W + H * W  # two images in, two maps + three derivative maps out, mask
        elif name == "ssim_l1_bwd":
            nbytes = (8 + 8 + 12 + 4) * 3 * H * W + H * W  # images, two upstream maps, three derivative maps in; one out
        elif name == "training_stats":
            nbytes = stats_bytes  # masks, opacities, gradient rows and the read-modify-write of the touched accumulators
        elif name == "adam_step":
            nbytes = 28 * n_adam  # p, g, m, v in; p, m, v out
        elif name in NEURAL_COST:
            per_anchor_b, per_gaussian_b, per_anchor_flop = NEURAL_COST[name]
            nbytes = per_anchor_b * N_a + per_gaussian_b * S_a
            e["algorithmic_flops"] = per_anchor_flop * N_a
            if ms > 0:
                e["TFLOPs"] = round(per_anchor_flop * N_a / (ms * 1e-3) / 1e12, 2)
                e["frac_of_fp32_matrix_peak"] = round(e["TFLOPs"] / FP32_MATRIX_PEAK_TFLOPS, 4)
        if nbytes is not None and ms > 0:
            e["algorithmic_bytes"] = nbytes
            e["GBps"] = round(nbytes / (ms * 1e-3) / 1e9, 1)
            e["frac_of_hbm_peak"] = round(e["GBps"] / HBM_PEAK_GBS, 4)
        stage_report[name] = e

    traffic = None
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath):
        try:
            tj0 = json.load(open(tpath))
            traffic = (tj0.get("preprocess_fwd_kernel<true, false>") or tj0.get("preprocess_fwd_kernel<true>")
                       or {}).get("bytes_per_launch")
        except (OSError, ValueError):
            traffic = None
    pf = stage_report.get("preprocess_fwd", {})
    # The kernel's bytes are counted as the reference's interface has them (307 B per Gaussian: 44 geometry in, 192
    # SH in, 56 + 12 + 3 out).  In a training step the kernel moves 319 B: it leaves out the 24 B of cov3D (formed
    # again by the backward kernel) and writes 36 B of colour derivative for that kernel (which reads them instead
    # of the 192 B of coefficients); the figure on those bytes is given beside it.
    ref_bytes = 307 * P
    roofline = {"kernel": "preprocess_fwd_kernel", "bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": None, "traffic": traffic, "algorithmic_bytes_per_launch": ref_bytes,
                "note": "307 B per Gaussian, the bytes of the reference's interface; in a training step the kernel "
                        "moves 319 B (no cov3D store, 36 B of colour derivative for the backward kernel): "
                        "achieved_on_bytes_moved counts those"}
    if pf.get("ms"):
        roofline["achieved"] = round(ref_bytes / (pf["ms"] * 1e-3) / 1e9, 1)
        roofline["frac"] = round(roofline["achieved"] / HBM_PEAK_GBS, 4)
        roofline["achieved_on_bytes_moved"] = pf.get("GBps")
    # The other half of the metric: everything between preprocess and the blend (count, prefix sum, per-tile
    # lists), one figure for the stage as a whole.
    bin_ms = sum(stage_report[k]["ms"] * stage_report[k]["launches_per_step"] for k in BINNING_STAGES
                 if k in stage_report)
    if "duplicate_with_keys" in stage_report and "sort_pairs" in stage_report:
        bin_ms += stage_report["sort_pairs"]["ms"]  # (a view on the radix route: one sort of its keys as well)
    bin_traffic = None
    if os.path.exists(tpath):
        try:
            tj = json.load(open(tpath))
            if all(k in tj for k in BINNING_KERNELS):
                bin_traffic = sum(tj[k]["bytes_per_launch"] for k in BINNING_KERNELS)
        except (OSError, ValueError, KeyError):
            bin_traffic = None
    if bin_ms > 0:
        ref_b = BINNING_REFERENCE_BYTES[0] * P + BINNING_REFERENCE_BYTES[1] * R
        own_b = BINNING_OWN_BYTES[0] * P + BINNING_OWN_BYTES[1] * R
        own_gbps = own_b / (bin_ms * 1e-3) / 1e9
        ref_gbps = ref_b / (bin_ms * 1e-3) / 1e9
        roofline["sort"] = {
            "kernel": "binning: " + " + ".join(BINNING_KERNELS), "bound": "hbm", "ms": round(bin_ms, 4),
            "achieved": round(own_gbps, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(own_gbps / HBM_PEAK_GBS, 4), "traffic": bin_traffic,
            "algorithmic_bytes_per_launch": own_b,
            "note": "achieved = the bytes this route moves (44 B per Gaussian, 48 B per instance: a 16 B record "
                    "written and read, 16 B of sorted lists written) / the time of the whole stage; "
                    "reference_equivalent_* divides the bytes the reference's algorithm moves for the same job "
                    "(44 B per Gaussian + 172 B per instance: 8-bit radix sort of 44-bit keys) by the same time",
            "reference_equivalent_bytes_per_launch": ref_b,
            "reference_equivalent_GBps": round(ref_gbps, 1),
            "reference_equivalent_frac": round(ref_gbps / HBM_PEAK_GBS, 4)}

    out = {
        "metric": "fwd+bwd ms/view @1M Gaussians 1152x864; preprocess+sort HBM GB/s vs peak",
        "value": round(ms_per_step, 4), "unit": "ms/view", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        # the same view with the geometry channels built inside the step (all_map forward + backward)
        "value_with_all_map": round(ms_per_step_with_all_map, 4),
        "clock_ramp_steps_before_warmup": ramp_steps,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"BASELINE config {args.config}: {P} Gaussians, {W}x{H}, SH degree 3, render_geo, "
                               f"1 view per step, seed 0", "instances_R": R, "tiles": gx * gy},
        "gaussian_views_per_s": round(P / (ms_per_step * 1e-3), 1),
        # the forward half of a step (preprocess, per-tile lists, blend): sum of its stages' event times
        "forward_ms_per_view": round(sum(stage_report[k]["ms"] * stage_report[k].get("launches_per_step", 1.0)
                                         for k in FORWARD_STAGES if k in stage_report)
                                     # (a view on the radix route: one sort of its keys as well)
                                     + (stage_report["sort_pairs"]["ms"] if "duplicate_with_keys" in stage_report
                                        and "sort_pairs" in stage_report else 0.0), 4),
        "roofline": roofline,
        # two views in flight on two streams (how the views of a batch can be issued); `value` is one view at a time
        "ms_per_view_two_views_in_flight": (round(ms_per_view_two_in_flight, 4)
                                            if ms_per_view_two_in_flight is not None else None),
        "ms_per_step_with_stage_events": round(ms_per_step_instrumented, 4),
        "stages": stage_report,
        "ssim_l1_torch_reference_ms": round(sorted(torch_ssim_ms)[len(torch_ssim_ms) // 2], 4),
        "training_stats_torch_reference_ms": round(sorted(torch_stats_ms)[len(torch_stats_ms) // 2], 4),
        "all_map_torch_reference_ms": round(sorted(torch_am_ms)[len(torch_am_ms) // 2], 4),
        "neural_gaussians_torch_reference_ms": round(sorted(torch_neural_ms)[len(torch_neural_ms) // 2], 4),
        "neural_gaussians_workload": {"anchors": N_a, "n_offsets": k_a, "selected": S_a},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(g, cam, am_cpu.numpy(), ug_cpu, args.cpu_runs)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
