#!/usr/bin/env python3
"""Benchmark of the hot path: forward trace + backward trace of one ray batch.

Default workload (config3): 1,000,000 surfels in a 10 m room, 1920x1080 pinhole rays, SH degree 3,
max_trace_depth 0, fp32, training mode (a_weights atomics on), seed 0, synthetic data.
A step = one forward launch + one backward launch through the launcher boundary (output allocation and
zero-initialisation of the gradient buffers included, as in the reference launcher); inputs are resident in HBM.

Prints ONE JSON line.  value = rays / (t_fwd + t_bwd) over the timed steps.  Extra keys: BVH build / refit ms,
the forward without a record in evaluation mode and the backward that walks the BVH again (what a caller without a
hit record gets), algorithmic bytes and their fraction of the 8 TB/s HBM peak, `roofline` for the dominant kernel
(measured with events on the launch stream right around the kernel), `cpu_baseline` (the CPU oracle on a bounded
sample of the same workload, timed on this box's host cores), and - in the default run - `other_workloads`: the other
four benchmark configurations, a few steps each (config2 as its 30-view build-once-then-refit loop, config5 as its
20-frame perturb-and-refit loop).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "diff-surfel-tracing_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0


def algorithmic_bytes(aux, slots, sh_degree=3, training=True):
    """Bytes per ray and per evaluated / composited hit that the path must move whatever the implementation
    (BVH traffic excluded): (fwd_ray, fwd_proc, fwd_con), (bwd_ray, bwd_proc, bwd_con), per-surfel zero-fill.
    `aux` channels, `slots` = mid_val slots per ray.  With aux 2, two slots, SH3, training:
    (204, 40, 208), (272, 40, 764), 316."""
    mid = 11 + aux + 3
    sh = 12 * (sh_degree + 1) ** 2
    fwd = (24 + 4 * (11 + aux + mid * slots), 40, sh + 4 * aux + (8 if training else 0))
    bwd = (24 + 4 * (11 + aux) + 4 * mid * slots + 4 * (9 + aux) + 24, 40,
           sh + 4 * aux + 36 + 8 * (16 + aux + 3 * (sh_degree + 1) ** 2))
    per_surfel = 4 * (3 + 3 + 3 + 3 * (sh_degree + 1) ** 2 + 3 + aux + 1 + 2 + 4 + 9) + 4
    return fwd, bwd, per_surfel


def replay_bytes(R, bwd_ray, n_proc, n_con, blocks, surfels_touched, P, cols, aux_in):
    """What the replaying backward has to move by its own design, in place of the reference-shaped count above (which
    prices 66 atomics and an SH gather per hit that this kernel does not perform): per ray as before; per stored chunk
    its 16x64 entries and 64 admission counts; 12 bytes of recorded colour per composited hit; per evaluated entry
    the surfel's mean, scale, rotation and opacity (40 bytes); per composited hit its triangle's three corners (36) and
    its auxiliary values; one read-modify-write of the gradient row of every surfel that received a gradient; and
    the closing kernel's pass over all rows (read) and gradient tensors (read-modify-write)."""
    return (R * bwd_ray + blocks * (16 * 64 * 8 + 64 * 4 + 8) + n_con * 12 + n_proc * 40 + n_con * (36 + 4 * aux_in)
            + surfels_touched * cols * 8 + P * cols * (4 + 8))


def workloads():
    import dst_scenes as S
    return {
        "config1": dict(name="cfg1 cube P=10k 128x128 SH3 depth0", scene=lambda: S.scene_cube(10000),
                        rays=lambda: S.rays_cube(128, 128)),
        "config2": dict(name="cfg2 sphere P=100k 800x800 SH3 depth0", scene=lambda: S.scene_sphere(100000),
                        rays=lambda: S.rays_sphere(800, 800), views=30),
        "config3": dict(name="cfg3 room P=1M 1920x1080 SH3 depth0", scene=lambda: S.scene_room(1000000),
                        rays=lambda: S.rays_room(1080, 1920)),
        "config4": dict(name="cfg4 room P=500k 1280x720 SH3 aux8 depth2 threshold0.1",
                        scene=lambda: S.scene_room(500000, aux=8), rays=lambda: S.rays_room(720, 1280),
                        aux=8, depth=2, threshold=0.1),
        "config5": dict(name="cfg5 lidar P=2M (1,131072,3) SH3 aux4 depth0", scene=lambda: S.scene_lidar(2000000),
                        rays=lambda: S.rays_lidar(), aux=4, frames=20),
    }


def traffic_of(workload, which):
    """HBM bytes per launch from the committed counter runs (not measured by this run)."""
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath):
        rec = json.load(open(tpath)).get("%s/%s" % (workload, which))
        if rec:
            return rec["bytes_per_launch"]
    return None


def roofline_of(workload, which, kernel, a_bytes, ms, basis):
    achieved = a_bytes / (ms * 1e-3) / 1e9
    traffic = traffic_of(workload, which)
    r = {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS,
         "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5), "traffic": traffic,
         # `traffic` is not measured by this run: it is the FETCH_SIZE + WRITE_SIZE figure of the committed
         # counter runs of the same command (profiles/), which goes stale when the kernels change
         "traffic_source": None if traffic is None else "profiles/hbm_traffic.json (rocprofv3 --pmc runs of this command)",
         "algorithmic_bytes_per_launch": int(a_bytes), "algorithmic_bytes_basis": basis, "avg_launch_ms": round(ms, 4)}
    if traffic is not None:   # what actually crossed the HBM interface, as a share of its peak
        r["hbm_measured_frac"] = round(traffic / (ms * 1e-3) / (HBM_PEAK_GBS * 1e9), 5)
    return r


def run_workload(key, steps, warmup, main, args):
    import torch

    import diff_surfel_tracing as dst
    import dst_scenes as S
    from diff_surfel_tracing import _C

    dev = "cuda"
    wl = workloads()[key]
    sc_cpu = wl["scene"]()
    o_cpu, d_cpu = wl["rays"]()
    H, W = o_cpu.shape[:2]
    R, P = H * W, sc_cpu["means3D"].shape[0]
    g = {k: v.to(dev) for k, v in sc_cpu.items()}
    ro, rd = o_cpu.to(dev), d_cpu.to(dev)
    aux, depth, threshold = wl.get("aux", 0), wl.get("depth", 0), wl.get("threshold", 0.0)
    aux_out = aux if aux else 2                 # channels of the aux output (2 when the scene has none)
    slots = max(1, depth) + 1                   # mid_val slots per ray
    (FWD_RAY, FWD_PROC, FWD_CON), (BWD_RAY, BWD_PROC, BWD_CON), PER_SURFEL_INIT = algorithmic_bytes(aux_out, slots)
    ug = {k: v.to(dev) for k, v in S.upstream_grads(H, W, aux_out).items()}
    ug["dist"] = torch.zeros(H, W, 1, device=dev)
    tracer = dst.SurfelTracer()
    ctx = tracer.optix_context
    ev = lambda: torch.cuda.Event(enable_timing=True)  # noqa: E731

    def timed(fn):
        a, b = ev(), ev()
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b)

    def median(fn, n=5):
        return sorted(timed(fn) for _ in range(n))[n // 2]

    # --- acceleration structure: build and refit times (median of 5, after one warm-up that sizes the buffers)
    build = lambda rebuild: tracer.build_acceleration_structure(g["vertices"], g["faces"], rebuild)  # noqa: E731
    timed(lambda: build(True))
    build_ms = median(lambda: build(True))
    refit_ms = median(lambda: build(False))
    # a dynamic frame's geometry update, two ways: the reference's (tensor operations make the quads, then a refit
    # from them) and this library's extension (one kernel makes the quads and refits)
    quads = lambda: S.get_triangles(g["means3D"], g["scales"], g["rotations"])  # noqa: E731
    timed(quads)
    quads_ms = median(quads)
    v_out = torch.empty_like(g["vertices"])
    fused = lambda: tracer.refit_from_surfels(g["means3D"], g["scales"], g["rotations"], v_out)  # noqa: E731
    timed(fused)
    refit_fused_ms = median(fused)
    build(False)   # back to the scene's own quads

    e = torch.empty(0, device=dev)
    bg = torch.zeros(3, device=dev)
    eye = torch.eye(4, device=dev)
    cam = torch.zeros(3, device=dev)
    counters = torch.zeros(2, dtype=torch.int64, device=dev)

    def common(sc):
        return (sc["vertices"], bg, sc["means3D"], sc["shs"], 3, e, sc.get("others_precomp", e), sc["opacities"],
                sc["scales"], 1.0, sc["rotations"], e, eye, eye, cam, False, False, depth, threshold)

    def step(fwd_events=None, bwd_events=None, count=False, record=True, rays=None, sc=None, keep=None):
        # what the autograd function does: the forward trace records its hit buffers, backward replays them
        o_, d_ = rays if rays is not None else (ro, rd)
        cm = common(sc if sc is not None else g)
        rec = ctx.acquire_record(H, W, max(1, depth), dev, max_trace_depth=depth) if record else None
        out = _C.trace_surfels(ctx, True, True, o_, d_, *cm, counters=counters if count else None,
                               events=fwd_events, hit_record=rec)
        grads = _C.trace_surfels_backward(ctx, True, o_, d_, *cm, *out[:7], ug["rgb"], ug["dpt"], ug["acc"],
                                          ug["norm"], ug["dist"], ug["aux"], events=bwd_events, hit_record=rec)
        if keep is not None and rec is not None:
            keep["blocks"] = rec.requested_blocks()
            keep["complete"] = keep["blocks"] <= rec.blocks
            keep["record_bytes"] = rec.words.numel() * 8
            keep["surfels_touched"] = int((grads[8] != 0).sum())
        ctx.release_record(rec)
        return out, grads

    # --- the frames of the workload: one ray batch over a static scene, the 30 views of config2 (refit before each,
    # as its definition says: build once, then rebuild=False), or the 20 perturbed frames of config5 (quads from the
    # moved means by tensor operations, then a refit)
    frames = []
    if wl.get("views"):
        for view in range(wl["views"]):
            o_v, d_v = S.rays_sphere(H, W, view=view)
            frames.append(dict(rays=(o_v.to(dev), d_v.to(dev)), sc=None))
    elif wl.get("frames"):
        cur = sc_cpu
        for frame in range(1, wl["frames"] + 1):
            gen = torch.Generator().manual_seed(3000 + frame)   # dst_scenes.perturb_means, without its CPU quads
            pick = torch.randperm(P, generator=gen)[: int(0.1 * P)]
            means = cur["means3D"].clone()
            means[pick] += 0.05 * torch.randn(pick.shape[0], 3, generator=gen)
            cur = dict(cur)
            cur["means3D"] = means
            frames.append(dict(rays=None, means=means.to(dev)))

    for _ in range(warmup):
        step()
    if main and args.traffic_probe:
        probe_src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        probe_dst = torch.empty_like(probe_src)
        torch.mul(probe_src, 2.0, out=probe_dst)   # reads 2^30 bytes, writes 2^30 bytes
        torch.cuda.synchronize()
        del probe_src, probe_dst
    torch.cuda.synchronize()
    ctx.update_record_estimate()   # the warm-up's forward traces have said how many blocks a record needs
    info = {}
    step(count=True, keep=info)
    torch.cuda.synchronize()
    n_proc, n_con = counters.tolist()

    n_steps = len(frames) if frames else steps
    handed_before = ctx.trace_info().tiles_handed_over
    fe = [(ev(), ev()) for _ in range(n_steps)]
    be = [(ev(), ev()) for _ in range(n_steps)]
    geo_ms = []
    torch.cuda.synchronize()
    trace_s = 0.0
    for k in range(n_steps):
        fr = frames[k] if frames else {}
        sc_k = None
        if "means" in fr:      # config5: the frame's quads, then a refit (both timed as the frame's geometry update)
            sc_k = dict(g)
            sc_k["means3D"] = fr["means"]
            def update():
                sc_k["vertices"], _ = S.get_triangles(sc_k["means3D"], g["scales"], g["rotations"])
                tracer.build_acceleration_structure(sc_k["vertices"], g["faces"], False)
            geo_ms.append(timed(update))
        elif frames:           # config2: the structure is refitted before every view
            geo_ms.append(timed(lambda: build(False)))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        step(fe[k], be[k], rays=fr.get("rays"), sc=sc_k)
        torch.cuda.synchronize()
        trace_s += time.perf_counter() - t0
    if not frames:             # one timed region around all steps, as the contract asks
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(n_steps):
            step(fe[k], be[k])
        torch.cuda.synchronize()
        trace_s = time.perf_counter() - t0
    ms_per_step = trace_s * 1e3 / n_steps
    trace_info = ctx.trace_info()
    handed = (trace_info.tiles_handed_over - handed_before) / n_steps
    fwd_ms = sum(a.elapsed_time(b) for a, b in fe) / n_steps   # kernel launch -> kernel end, on the launch stream
    bwd_ms = sum(a.elapsed_time(b) for a, b in be) / n_steps
    if frames and "means" in frames[-1]:
        build(False)           # back to the scene's own quads

    # --- the same step for a caller without a hit record: evaluation-mode forward (no record, no a_weights) and the
    # backward that walks the BVH again
    def eval_forward(events):
        _C.trace_surfels(ctx, False, True, ro, rd, *common(g), events=events)
    n_alt = max(3, min(steps, 10))
    alt = [(ev(), ev()) for _ in range(n_alt)]
    eval_forward(None)
    for k in range(n_alt):
        eval_forward(alt[k])
    torch.cuda.synchronize()
    fwd_eval_ms = sum(a.elapsed_time(b) for a, b in alt) / n_alt
    alt = [(ev(), ev()) for _ in range(n_alt)]
    step(record=False)
    for k in range(n_alt):
        step(None, alt[k], record=False)
    torch.cuda.synchronize()
    bwd_retrace_ms = sum(a.elapsed_time(b) for a, b in alt) / n_alt

    # --- the same step with the SH coefficients read from their binary16 copy (DST_FLAG_SH_HALF; the copy is made by
    # a packing kernel in front of every trace, timed on its own)
    sh_half = None
    if main:
        pack_ms = median(lambda: _C.pack_sh_half(g["shs"]))
        ctx.sh_half = True
        alt_f = [(ev(), ev()) for _ in range(n_alt)]
        alt_b = [(ev(), ev()) for _ in range(n_alt)]
        step()
        for k in range(n_alt):
            step(alt_f[k], alt_b[k])
        torch.cuda.synchronize()
        ctx.sh_half = False
        sh_half = {"fwd_kernel_ms": round(sum(a.elapsed_time(b) for a, b in alt_f) / n_alt, 4),
                   "bwd_kernel_ms": round(sum(a.elapsed_time(b) for a, b in alt_b) / n_alt, 4),
                   "pack_ms": round(pack_ms, 4)}

    A_fwd = R * FWD_RAY + n_proc * FWD_PROC + n_con * FWD_CON
    A_bwd = R * BWD_RAY + n_proc * BWD_PROC + n_con * BWD_CON
    A_total = A_fwd + A_bwd + PER_SURFEL_INIT * P
    cols = 64 + aux_out
    A_replay = replay_bytes(R, BWD_RAY, n_proc, n_con, info.get("blocks", 0), info.get("surfels_touched", 0), P, cols,
                            aux)
    rays_per_s = R / (ms_per_step * 1e-3)

    aux_max = 2 if aux_out <= 2 else (4 if aux_out <= 4 else 8)
    mixed = "true" if (depth > 0 or H < 8) else "false"   # kernels with the per-lane walk built in
    # (image grids at depth 0 run the kernels without the tile hand-over unless the scene has many small quads)
    fwd_name = ("k_trace_fwd_plain<%d,true>" % aux_max if mixed == "false" and not trace_info.handover_active
                else "k_trace_fwd<%d,true,%s,false>" % (aux_max, mixed))
    fwd_roof = roofline_of(key, "forward", fwd_name, A_fwd, fwd_ms,
                           "per ray / evaluated entry / composited hit, reference-shaped")
    bwd_roof = roofline_of(key, "backward", "k_trace_bwd<%d,true,false,false>" % aux_max, A_replay, bwd_ms,
                           "what the replaying kernel moves by design: record, per-hit geometry, gradient rows")
    # the reference-shaped count (66 atomics and an SH gather per hit) describes the work the kernel stands in for,
    # not bytes it moves: above the HBM peak it is no utilisation figure
    bwd_roof["reference_equivalent"] = {"algorithmic_bytes_per_launch": int(A_bwd),
                                        "GB/s": round(A_bwd / (bwd_ms * 1e-3) / 1e9, 2)}
    retrace_roof = roofline_of(key, "backward_retrace", "k_trace_bwd<%d,false,%s,false>" % (aux_max, mixed), A_bwd,
                               bwd_retrace_ms, "per ray / evaluated entry / composited hit, reference-shaped")
    per_kernel = {"forward": fwd_roof, "backward": bwd_roof, "backward_retrace": retrace_roof}

    result = {
        "ms_per_step": round(ms_per_step, 4), "rays_per_s": round(rays_per_s, 1), "steps": n_steps,
        "config": {"workload": wl["name"], "surfels": P, "rays": R, "sh_degree": 3, "max_trace_depth": depth,
                   "aux_channels": aux, "training": True, "seed": 0},
        "fwd_kernel_ms": round(fwd_ms, 4), "bwd_kernel_ms": round(bwd_ms, 4),
        "fwd_eval_kernel_ms": round(fwd_eval_ms, 4), "bwd_retrace_kernel_ms": round(bwd_retrace_ms, 4),
        "bvh_build_ms": round(build_ms, 4), "bvh_refit_ms": round(refit_ms, 4),
        "quads_by_tensor_ops_ms": round(quads_ms, 4), "bvh_refit_from_surfels_ms": round(refit_fused_ms, 4),
        "hits_evaluated_per_ray": round(n_proc / R, 3), "hits_composited_per_ray": round(n_con / R, 3),
        "hit_record": {"blocks_used": info.get("blocks"), "complete": info.get("complete"),
                       "allocated_bytes": info.get("record_bytes")},
        # forward tiles whose packet walk ran into the step limit and were traced ray by ray by the second launch
        "tile_handover": {"active": bool(trace_info.handover_active), "small_quads": trace_info.small_quads,
                          "step_limit": trace_info.handover_steps, "tiles_per_forward": round(handed, 2)},
        "algorithmic_bytes": int(A_total),
        "reference_equivalent_hbm_frac": round(A_total / (ms_per_step * 1e-3) / (HBM_PEAK_GBS * 1e9), 5),
        "roofline_kernels": per_kernel,
    }
    if sh_half is not None:
        result["sh_half"] = sh_half
    if geo_ms:
        result["geometry_update_ms_per_frame"] = round(sum(geo_ms) / len(geo_ms), 4)
        result["frame_loop"] = ("%d views, structure built once and refitted before each" % len(frames) if wl.get("views")
                                else "%d frames: 10 %% of the means moved, quads by tensor operations, refit" % len(frames))
    keep = dict(sc_cpu=sc_cpu, o_cpu=o_cpu, d_cpu=d_cpu, ug=ug, depth=depth, threshold=threshold, P=P)
    del tracer, ctx
    return result, keep


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="config3", choices=["config1", "config2", "config3", "config4", "config5"])
    ap.add_argument("--cpu-stride", type=int, default=1, help="CPU baseline traces every n-th pixel row and column")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the short runs of the other four configurations (default run only)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run one plain 1 GiB read + 1 GiB write kernel (a yardstick for HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (rays would be sharded across "
              "GPUs with one all-reduce of the per-surfel gradients)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch

    torch.cuda.set_device(0)
    res, keep = run_workload(args.workload, args.steps, args.warmup, True, args)
    per_kernel = res["roofline_kernels"]
    # `roofline` is the kernel of the step that takes longer; within 3 % of each other, the forward
    fwd_k, bwd_k = per_kernel["forward"], per_kernel["backward"]
    roofline = bwd_k if bwd_k["avg_launch_ms"] > 1.03 * fwd_k["avg_launch_ms"] else fwd_k

    result = {
        "metric": "rays/s fwd+bwd at 1M surfels 1080p" if args.workload == "config3" else "rays/s fwd+bwd",
        "value": res["rays_per_s"], "unit": "rays/s", "n_gpus": 1, "steps": res["steps"], "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic", "config": res["config"],
    }
    for k, v in res.items():
        if k not in ("ms_per_step", "rays_per_s", "steps", "config", "roofline_kernels"):
            result[k] = v
    result["roofline"] = roofline
    result["roofline_kernels"] = per_kernel

    if not args.no_cpu_baseline:
        from oracle import surfel_oracle as O
        st = max(1, args.cpu_stride)
        o_cpu, d_cpu, sc_cpu, ug = keep["o_cpu"], keep["d_cpu"], keep["sc_cpu"], keep["ug"]
        so, sd = o_cpu[::st, ::st].contiguous(), d_cpu[::st, ::st].contiguous()
        n = {k: v.numpy() for k, v in sc_cpu.items()}
        s = O.Scene(so.numpy(), sd.numpy(), n["vertices"], n["faces"], n["means3D"], n["opacities"], n["scales"],
                    n["rotations"], shs=n["shs"], others_precomp=n.get("others_precomp"),
                    max_trace_depth=keep["depth"], specular_threshold=keep["threshold"])
        cores = min(O.num_threads(), int(os.environ.get("OMP_NUM_THREADS", "0") or O.num_threads()))
        f = O.forward(s, O.HITS_BVH_LEXI, counters=False)
        tf = s.trace_seconds
        ugs = {k: v.cpu()[::st, ::st].contiguous().numpy() for k, v in ug.items() if k != "dist"}
        O.backward(s, f, ugs, O.HITS_BVH_LEXI)
        tb = s.trace_seconds
        rs = so.shape[0] * so.shape[1]
        result["cpu_baseline"] = {
            "value": round(rs / (tf + tb), 1), "unit": "rays/s", "cores": cores, "kind": "port",
            "sample": "%s of the same image (%d rays) against the full %d-surfel scene; CPU BVH build excluded; "
                      "fwd %.2f s + bwd %.2f s" % ("every pixel" if st == 1 else "every %d-th pixel row and column" % st,
                                                   rs, keep["P"], tf, tb)}
        del s, f, n
    del keep

    if args.workload == "config3" and not args.no_other_workloads and not args.traffic_probe:
        # the other benchmark configurations, a few steps each, no CPU leg (parity-test cases; their times for the record)
        others = {}
        for key in ("config1", "config2", "config4", "config5"):
            torch.cuda.empty_cache()
            r, _ = run_workload(key, 5, 2, False, args)
            others[key] = r
        result["other_workloads"] = others
    print(json.dumps(result))


if __name__ == "__main__":
    main()
