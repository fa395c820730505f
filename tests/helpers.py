"""Shared plumbing of the tests: scene dict -> oracle scene, scene dict -> GPU call."""
import numpy as np
import torch

import dst_scenes as S


def to_numpy(scene):
    return {k: v.detach().cpu().numpy() for k, v in scene.items()}


def oracle_scene(O, scene, ray_o, ray_d, **kw):
    n = to_numpy(scene)
    return O.Scene(ray_o.numpy(), ray_d.numpy(), n["vertices"], n["faces"], n["means3D"], n["opacities"], n["scales"],
                   n["rotations"], shs=n.get("shs"), colors_precomp=n.get("colors_precomp"),
                   others_precomp=n.get("others_precomp"), **kw)


def settings(dst, H, W, dev, bg=(0.0, 0.0, 0.0), sh_degree=3, max_trace_depth=0, specular_threshold=0.0, debug=False):
    eye = torch.eye(4, device=dev)
    return dst.SurfelTracingSettings(H, W, 1.0, 1.0, torch.tensor(bg, dtype=torch.float32, device=dev), 1.0, eye, eye,
                                     sh_degree, torch.zeros(3, device=dev), False, debug, max_trace_depth,
                                     specular_threshold)


PARAM_NAMES = ("means3D", "shs", "colors_precomp", "others_precomp", "opacities", "scales", "rotations")
OUT_NAMES = ("rgb", "dpt", "acc", "norm", "dist", "aux", "mid", "wet")


def gpu_trace(tracer, scene, ray_o, ray_d, upstream=None, rebuild=True, build=True, dev="cuda", **kw):
    """Build the BVH, trace forward through the public API and (with `upstream`) backward.
    Returns (outputs dict of numpy arrays, gradients dict of numpy arrays or None)."""
    import diff_surfel_tracing as dst
    start_from_first = kw.pop("start_from_first", True)
    training = kw.pop("training", True)
    g = {k: v.to(dev) for k, v in scene.items()}
    if build:
        tracer.build_acceleration_structure(g["vertices"], g["faces"], rebuild)
    H, W = ray_o.shape[0], ray_o.shape[1]
    st = settings(dst, H, W, dev, **kw)
    leaf = {k: g[k].clone().requires_grad_(upstream is not None) for k in PARAM_NAMES if k in g}
    ro = ray_o.to(dev).clone().requires_grad_(upstream is not None)
    rd = ray_d.to(dev).clone().requires_grad_(upstream is not None)
    grads3D = torch.zeros_like(leaf["means3D"], requires_grad=upstream is not None)
    tracer.train(training)
    out = tracer(ro, rd, g["vertices"], leaf["means3D"], grads3D, shs=leaf.get("shs"),
                 colors_precomp=leaf.get("colors_precomp"), others_precomp=leaf.get("others_precomp"),
                 opacities=leaf["opacities"], scales=leaf["scales"], rotations=leaf["rotations"],
                 tracer_settings=st, start_from_first=start_from_first)
    tracer.train(True)
    outs = {n: t.detach().cpu().numpy() for n, t in zip(OUT_NAMES, out)}
    grads = None
    if upstream is not None:
        idx = {"rgb": 0, "dpt": 1, "acc": 2, "norm": 3, "aux": 5}
        loss = sum((out[idx[k]] * v.to(dev)).sum() for k, v in upstream.items() if k in idx)
        loss.backward()
        grads = {"ray_o": ro.grad, "ray_d": rd.grad, "grads3D": grads3D.grad}
        grads.update({k: v.grad for k, v in leaf.items()})
        grads = {k: (None if v is None else v.cpu().numpy()) for k, v in grads.items()}
    torch.cuda.synchronize()
    return outs, grads


def assert_forward_exact(gpu, ref, skip=("wet",)):
    """Per-ray outputs are the same sequence of fp32 operations on both sides: equal bit for bit."""
    for k in ("rgb", "dpt", "acc", "norm", "aux", "mid"):
        if k in skip:
            continue
        a, b = gpu[k], ref[k]
        assert a.shape == b.shape, (k, a.shape, b.shape)
        same = (a.view(np.uint32) == b.view(np.uint32)) | (np.isnan(a) & np.isnan(b))
        assert same.all(), "%s differs in %d of %d values, max abs diff %g" % (
            k, (~same).sum(), same.size, np.nanmax(np.abs(a - b)))
    assert np.array_equal(gpu["dist"], ref["dist"][..., :1])


def assert_close_sum(a, b, rel, name):
    """Atomically accumulated sums: order differs, so compare against the largest magnitude (north star: 1e-3)."""
    assert a.shape == b.shape, (name, a.shape, b.shape)
    scale = max(float(np.abs(b).max()), 1e-30)
    err = float(np.abs(a - b).max()) / scale
    assert err <= rel, "%s: max error %.3g of max |ref| %.3g exceeds %.1g" % (name, err, scale, rel)


GRAD_REL = 1e-3   # north star: gradients within 1e-3 relative
OUT_ABS = 1e-4    # north star: rendered outputs within 1e-4 absolute (we get bit equality)


def upstream(H, W, aux, seed=0, acc=True):
    ug = S.upstream_grads(H, W, aux, seed)
    if not acc:
        ug.pop("acc")
    return ug
