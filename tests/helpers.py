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


NOISE_FACTOR = 4.0


def _report(name, a, b, err, tol, bad, noisy):
    k = np.unravel_index(np.argmax(err / np.maximum(tol, 1e-300)), err.shape)
    return ("%s: %d of %d elements off (%d of them carry a rounding-noise allowance); worst at %s: got %.9g, "
            "want %.9g (|diff| %.3g, allowed %.3g)" % (name, bad.sum(), bad.size, (bad & noisy).sum(), k, a[k], b[k],
                                                       err[k], tol[k]))


# What the noise allowance was actually used for, per compared tensor: (name, elements, needing the noise term,
# whose noise term alone exceeds LOUD_NOISE of the value).  conftest prints it at the end of a run.
NOISE_LOG = []
LOUD_NOISE = 0.3


def _same_nonfinite(a, b, name):
    """NaN / +inf / -inf must sit in the same places on both sides; returns the mask of finite elements."""
    fa, fb = np.isfinite(a), np.isfinite(b)
    assert np.array_equal(fa, fb), "%s: %d elements are finite on one side only" % (name, int((fa != fb).sum()))
    if not fa.all():
        bad = ~fa
        same = (np.isnan(a[bad]) & np.isnan(b[bad])) | (a[bad] == b[bad])
        assert same.all(), "%s: %d non-finite elements differ in kind (nan, +inf, -inf)" % (name, int((~same).sum()))
    return fa


def _noise_rules(name, err, base, extra, ref_abs, max_noisy, finite):
    """The two rules that keep the rounding-noise allowance from hiding a defect: few elements may need it at all,
    and only a handful may carry an allowance that is itself a sizeable part of the value."""
    noisy = (err > base) & finite
    loud = np.zeros_like(noisy) if np.isscalar(extra) else ((extra > LOUD_NOISE * ref_abs) & (ref_abs > base) & finite)
    NOISE_LOG.append((name, int(noisy.size), int(noisy.sum()), int(loud.sum())))
    assert noisy.sum() <= max(max_noisy * noisy.size, MIN_NOISY), (
        "%s: %d of %d elements (%.3g) pass only through the noise allowance; they miss the plain bound by factors of %s, "
        "relative errors %s" % (name, noisy.sum(), noisy.size, noisy.mean(),
                                np.round(np.sort((err / np.maximum(base, 1e-300))[noisy])[-8:], 2).tolist(),
                                ["%.2g" % x for x in np.sort((err / np.maximum(ref_abs, 1e-300))[noisy])[-8:]]))
    assert loud.sum() <= max(MAX_LOUD * loud.size, MIN_NOISY), (
        "%s: the noise allowance alone exceeds %.0f %% of the value on %d of %d elements" % (
            name, 100 * LOUD_NOISE, loud.sum(), loud.size))
    return noisy


def assert_close_sum(a, b, rel, name, noise=None, max_noisy=None):
    """Sums accumulated in a different order on the two sides (atomics on the GPU, double accumulators in the
    oracle): ELEMENT-WISE |a - b| <= rel * |b| + floor + NOISE_FACTOR * noise.
    floor: rel/20 of the root-mean-square of the channel's nonzero entries (a sum that cancels keeps the rounding
    of its summands while its value shrinks; the columns of one tensor can differ by orders of magnitude).
    noise: what fp32 rounding alone does to this element of the reference's formula, from the oracle: |b - b64|
    (b64 = its gradient algebra evaluated in double on the same fp32 inputs and decisions) plus, for the
    geometric gradients, its first-order sensitivity to one unit of rounding in the plane-hit chain (a grazing
    hit at 50 m divides a difference of two 50 m vectors by n.d twice: one ulp in t = n.(v1-o)/n.d moves such an
    element by tens of per cent).  No fp32 implementation, the reference's included, is closer to another than that.
    At most MAX_NOISY of the elements (or MIN_NOISY of them, for a small tensor) may owe their pass to the noise
    term, and at most MAX_LOUD of them may carry a noise term above LOUD_NOISE of the value itself.  NaN and
    infinities must sit at the same places on both sides."""
    max_noisy = MAX_NOISY if max_noisy is None else max_noisy
    assert a.shape == b.shape, (name, a.shape, b.shape)
    a64, b64 = np.asarray(a, np.float64), np.asarray(b, np.float64)
    flat_b = b64.reshape(-1, b64.shape[-1]) if b64.ndim > 1 else b64.reshape(-1, 1)
    flat_a = a64.reshape(flat_b.shape)
    finite = _same_nonfinite(flat_a, flat_b, name)
    fb = np.where(finite, flat_b, 0.0)
    live = fb != 0
    rms = np.sqrt((fb ** 2).sum(0) / np.maximum(live.sum(0), 1))
    base = rel * np.abs(fb) + rel / 20 * rms[None, :]
    extra = 0.0 if noise is None else NOISE_FACTOR * np.nan_to_num(np.asarray(noise, np.float64).reshape(flat_b.shape),
                                                                    nan=0.0, posinf=0.0, neginf=0.0)
    err = np.where(finite, np.abs(np.where(finite, flat_a, 0.0) - fb), 0.0)
    tol = base + extra
    bad = err > tol
    if bad.any():
        raise AssertionError(_report(name, flat_a, flat_b, err, tol, bad, err > base))
    _noise_rules(name, err, base, extra, np.abs(fb), max_noisy, finite)


def assert_same_sums(a, b, rel, name):
    """Two GPU results of the same sums whose float atomics ran in different orders (one image against its parts, one
    call against the same call made another way).  Not the parity bar - that one has the oracle's noise estimate to
    lean on: element-wise |a - b| <= rel * |b| + rel * (root mean square of the channel's nonzero entries)."""
    assert a.shape == b.shape, (name, a.shape, b.shape)
    a64 = np.asarray(a, np.float64).reshape(a.shape[0], -1)
    b64 = np.asarray(b, np.float64).reshape(a.shape[0], -1)
    rms = np.sqrt((b64 ** 2).sum(0) / np.maximum((b64 != 0).sum(0), 1))
    err, tol = np.abs(a64 - b64), rel * np.abs(b64) + rel * rms[None, :]
    bad = err > tol
    assert not bad.any(), "%s: %d of %d elements off, worst %.2f of its tolerance" % (
        name, int(bad.sum()), bad.size, float((err / np.maximum(tol, 1e-300)).max()))


def assert_close_rays(a, b, rel, name, noise=None, max_noisy=None):
    """Per-ray gradients are plain stores (no atomics): element-wise |a - b| <= rel * |b| + rel/10 * (largest
    component of that ray's gradient) + NOISE_FACTOR * noise (see assert_close_sum, also for the rules on how many
    elements may lean on the noise term and on non-finite values)."""
    max_noisy = MAX_NOISY if max_noisy is None else max_noisy
    assert a.shape == b.shape, (name, a.shape, b.shape)
    a64, b64 = np.asarray(a, np.float64), np.asarray(b, np.float64)
    finite = _same_nonfinite(a64, b64, name)
    fb = np.where(finite, b64, 0.0)
    row = np.abs(fb).max(-1, keepdims=True)
    base = rel * np.abs(fb) + rel / 10 * row + 1e-30
    extra = 0.0 if noise is None else NOISE_FACTOR * np.nan_to_num(np.asarray(noise, np.float64), nan=0.0, posinf=0.0,
                                                                    neginf=0.0)
    err = np.where(finite, np.abs(np.where(finite, a64, 0.0) - fb), 0.0)
    tol = base + extra
    bad = err > tol
    if bad.any():
        raise AssertionError(_report(name, a64, b64, err, tol, bad, err > base))
    _noise_rules(name, err, base, extra, np.abs(fb), max_noisy, finite)


def assert_gradients(got, ref32, ref64, rel, tag=""):
    """Every gradient tensor of `got` (GPU) against the oracle's (`ref32`).  `ref64` = oracle.backward(...,
    noise=True): its double-precision values and its sensitivity estimate together give the rounding-noise allowance."""
    est = {} if ref64 is None else ref64.get("noise", {})
    for k, want in ref32.items():
        if k == "noise":
            continue
        if got.get(k) is None:
            assert k in ("shs", "colors_precomp", "others_precomp"), k
            continue
        if np.abs(want).max() == 0 and k not in est:
            assert np.abs(got[k]).max() == 0, k
            continue
        noise = None
        if ref64 is not None:
            noise = np.abs(want.astype(np.float64) - ref64[k].astype(np.float64))
            if k in est:
                noise = noise + est[k].astype(np.float64)
        (assert_close_rays if k in ("ray_o", "ray_d") else assert_close_sum)(got[k], want, rel, tag + k, noise=noise)


MAX_NOISY = 2e-3  # share of a tensor's elements that may need the noise term (observed: 1.1e-3 on the sphere of config 2,
                  # whose silhouette is all grazing hits; at most 7e-5 on configs 3, 4 and 5 at full size)
MAX_LOUD = 2e-2   # share whose noise term alone may exceed LOUD_NOISE of the value (observed: 9e-3 on config 2, 9e-4 on 3)
MIN_NOISY = 4     # a share is no measure on a tensor of 80 elements
GRAD_REL = 1e-3   # north star: gradients within 1e-3 relative
OUT_ABS = 1e-4    # north star: rendered outputs within 1e-4 absolute (we get bit equality)


def upstream(H, W, aux, seed=0, acc=True):
    ug = S.upstream_grads(H, W, aux, seed)
    if not acc:
        ug.pop("acc")
    return ug
