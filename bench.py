#!/usr/bin/env python3
"""Benchmark of the hot path: forward trace + backward re-trace of one ray batch.

Default workload (config3): 1,000,000 surfels in a 10 m room, 1920x1080 pinhole rays, SH degree 3,
max_trace_depth 0, fp32, training mode (a_weights atomics on), seed 0, synthetic data.
A step = one forward launch + one backward launch through the launcher boundary (output allocation and
zero-initialisation of the gradient buffers included, as in the reference launcher); inputs are resident in HBM.

Prints ONE JSON line.  value = rays / (t_fwd + t_bwd) over the timed steps.  Extra keys: BVH build / refit ms,
algorithmic bytes and their fraction of the 8 TB/s HBM peak, `roofline` for the dominant kernel (measured with
events on the launch stream right around the kernel), `cpu_baseline` (the CPU oracle on a bounded sample of the
same workload, timed on this box's host cores).
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


def workloads():
    import dst_scenes as S
    return {
        "config1": dict(name="cfg1 cube P=10k 128x128 SH3 depth0", scene=lambda: S.scene_cube(10000),
                        rays=lambda: S.rays_cube(128, 128)),
        "config2": dict(name="cfg2 sphere P=100k 800x800 SH3 depth0", scene=lambda: S.scene_sphere(100000),
                        rays=lambda: S.rays_sphere(800, 800)),
        "config3": dict(name="cfg3 room P=1M 1920x1080 SH3 depth0", scene=lambda: S.scene_room(1000000),
                        rays=lambda: S.rays_room(1080, 1920)),
        "config4": dict(name="cfg4 room P=500k 1280x720 SH3 aux8 depth2 threshold0.1",
                        scene=lambda: S.scene_room(500000, aux=8), rays=lambda: S.rays_room(720, 1280),
                        aux=8, depth=2, threshold=0.1),
        "config5": dict(name="cfg5 lidar P=2M (1,131072,3) SH3 aux4 depth0", scene=lambda: S.scene_lidar(2000000),
                        rays=lambda: S.rays_lidar(), aux=4),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="config3", choices=["config1", "config2", "config3", "config4", "config5"])
    ap.add_argument("--cpu-stride", type=int, default=1, help="CPU baseline traces every n-th pixel row and column")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run one plain 1 GiB read + 1 GiB write kernel (a yardstick for HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (rays would be sharded across "
              "GPUs with one all-reduce of the per-surfel gradients)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch

    import diff_surfel_tracing as dst
    import dst_scenes as S
    from diff_surfel_tracing import _C

    torch.cuda.set_device(0)
    dev = "cuda"
    wl = workloads()[args.workload]
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

    # --- acceleration structure: build and refit times (median of 5, after one warm-up that sizes the buffers)
    def timed_build(rebuild):
        a, b = ev(), ev()
        a.record()
        tracer.build_acceleration_structure(g["vertices"], g["faces"], rebuild)
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b)
    timed_build(True)
    build_ms = sorted(timed_build(True) for _ in range(5))[2]
    refit_ms = sorted(timed_build(False) for _ in range(5))[2]

    # a dynamic frame's geometry update, two ways: the reference's (tensor operations make the quads, then a refit
    # from them) and this library's extension (one kernel makes the quads and refits)
    def timed(fn):
        a, b = ev(), ev()
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b)
    timed(lambda: S.get_triangles(g["means3D"], g["scales"], g["rotations"]))
    quads_ms = sorted(timed(lambda: S.get_triangles(g["means3D"], g["scales"], g["rotations"])) for _ in range(5))[2]
    v_out = torch.empty_like(g["vertices"])
    fused = lambda: tracer.refit_from_surfels(g["means3D"], g["scales"], g["rotations"], v_out)  # noqa: E731
    timed(fused)
    refit_fused_ms = sorted(timed(fused) for _ in range(5))[2]
    tracer.build_acceleration_structure(g["vertices"], g["faces"], False)   # back to the scene's own quads

    e = torch.empty(0, device=dev)
    bg = torch.zeros(3, device=dev)
    eye = torch.eye(4, device=dev)
    cam = torch.zeros(3, device=dev)
    common = (g["vertices"], bg, g["means3D"], g["shs"], 3, e, g.get("others_precomp", e), g["opacities"], g["scales"],
              1.0, g["rotations"], e, eye, eye, cam, False, False, depth, threshold)
    counters = torch.zeros(2, dtype=torch.int64, device=dev)

    def step(fwd_events=None, bwd_events=None, count=False):
        # what the autograd function does: the forward trace records its hit buffers, backward replays them
        rec = ctx.acquire_record(H, W, max(1, depth), dev)
        out = _C.trace_surfels(ctx, True, True, ro, rd, *common, counters=counters if count else None,
                               events=fwd_events, hit_record=rec)
        grads = _C.trace_surfels_backward(ctx, True, ro, rd, *common, *out[:7], ug["rgb"], ug["dpt"], ug["acc"],
                                          ug["norm"], ug["dist"], ug["aux"], events=bwd_events, hit_record=rec)
        ctx.release_record(rec)
        return out, grads

    for _ in range(args.warmup):
        step()
    if args.traffic_probe:
        probe_src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        probe_dst = torch.empty_like(probe_src)
        torch.mul(probe_src, 2.0, out=probe_dst)   # reads 2^30 bytes, writes 2^30 bytes
        torch.cuda.synchronize()
        del probe_src, probe_dst
    step(count=True)
    torch.cuda.synchronize()
    n_proc, n_con = counters.tolist()

    fe = [(ev(), ev()) for _ in range(args.steps)]
    be = [(ev(), ev()) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        step(fe[k], be[k])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    fwd_ms = sum(a.elapsed_time(b) for a, b in fe) / args.steps   # kernel launch -> kernel end, on the launch stream
    bwd_ms = sum(a.elapsed_time(b) for a, b in be) / args.steps

    A_fwd = R * FWD_RAY + n_proc * FWD_PROC + n_con * FWD_CON
    A_bwd = R * BWD_RAY + n_proc * BWD_PROC + n_con * BWD_CON
    A_total = A_fwd + A_bwd + PER_SURFEL_INIT * P
    rays_per_s = R / (ms_per_step * 1e-3)

    def roofline_of(which, kernel, a_bytes, ms):
        achieved = a_bytes / (ms * 1e-3) / 1e9
        traffic = None
        tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
        if os.path.exists(tpath):
            rec = json.load(open(tpath)).get("%s/%s" % (args.workload, which))
            if rec:
                traffic = rec["bytes_per_launch"]
        return {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5), "traffic": traffic,
                # `traffic` is not measured by this run: it is the FETCH_SIZE + WRITE_SIZE figure of the committed
                # counter runs of the same command (profiles/), which goes stale when the kernels change
                "traffic_source": None if traffic is None else "profiles/hbm_traffic.json (rocprofv3 --pmc runs of this command)",
                "algorithmic_bytes_per_launch": int(a_bytes), "avg_launch_ms": round(ms, 4)}
    aux_max = 2 if aux_out <= 2 else (4 if aux_out <= 4 else 8)
    mixed = "true" if (depth > 0 or H < 8) else "false"   # kernels with the per-lane walk built in
    per_kernel = {"forward": roofline_of("forward", "k_trace_fwd<%d,true,%s,false>" % (aux_max, mixed), A_fwd, fwd_ms),
                  "backward": roofline_of("backward", "k_trace_bwd<%d,true,false,false>" % aux_max, A_bwd, bwd_ms)}
    # The two kernels take about the same time on this workload, so "the slower one" flips from run to run.  `roofline`
    # is the one further from its bound (the lower fraction: the one to work on); both are under `roofline_kernels`.
    roofline = min(per_kernel.values(), key=lambda r: r["frac"])

    result = {
        "metric": "rays/s fwd+bwd at 1M surfels 1080p" if args.workload == "config3" else "rays/s fwd+bwd",
        "value": round(rays_per_s, 1), "unit": "rays/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": wl["name"], "surfels": P, "rays": R, "sh_degree": 3, "max_trace_depth": depth,
                   "aux_channels": aux, "training": True, "seed": 0},
        "fwd_kernel_ms": round(fwd_ms, 4), "bwd_kernel_ms": round(bwd_ms, 4),
        "bvh_build_ms": round(build_ms, 4), "bvh_refit_ms": round(refit_ms, 4),
        "quads_by_tensor_ops_ms": round(quads_ms, 4), "bvh_refit_from_surfels_ms": round(refit_fused_ms, 4),
        "hits_evaluated_per_ray": round(n_proc / R, 3), "hits_composited_per_ray": round(n_con / R, 3),
        "algorithmic_bytes": int(A_total), "hbm_peak_frac": round(A_total / (ms_per_step * 1e-3) / (HBM_PEAK_GBS * 1e9), 5),
        "roofline": roofline, "roofline_kernels": per_kernel,
    }

    if not args.no_cpu_baseline:
        from oracle import surfel_oracle as O
        st = max(1, args.cpu_stride)
        so, sd = o_cpu[::st, ::st].contiguous(), d_cpu[::st, ::st].contiguous()
        n = {k: v.numpy() for k, v in sc_cpu.items()}
        s = O.Scene(so.numpy(), sd.numpy(), n["vertices"], n["faces"], n["means3D"], n["opacities"], n["scales"],
                    n["rotations"], shs=n["shs"], others_precomp=n.get("others_precomp"), max_trace_depth=depth,
                    specular_threshold=threshold)
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
                                                   rs, P, tf, tb)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
