"""Seeded random configurations, HIP path against the oracle with the checks of test_gpu_parity.check_case: scene kind,
surfel count from 3 to 40 000, surfel size x0.3 to x10, image from 1x1 to 71x71 (or the same rays as a list, or
unrelated rays), aux channels, SH degree, depth 0 to 2 with thresholds, background, `start_from_first`; a degenerate
trait (all surfels at one point, zero scales, a scene 3 km from the origin, 25:1 quads, a scene of 0.1 mm or 30 km,
opacities of exactly 0 and 1, a flat scene seen head-on and edge-on, NaN and infinite parameters, a few surfels a
thousand to a million scene sizes away); and the mode of the
call (plain, deterministic, without a hit record, without gradient rows, after a refit, after a refit from the
surfel parameters).  Drawn from generators of their own, so that the cases above stay what they were: surfels another
30 times smaller in a third of the cases (quads of a millimetre and less seen from metres away), and the forward's
tile hand-over forced to 1 or to 48 steps in half of them.  The cases are small; their value is in the combinations no
hand-written test makes."""
import os
import warnings

import numpy as np
import pytest
import torch

import dst_scenes as S
from test_gpu_parity import _with_scales, check_case

pytestmark = pytest.mark.gpu

TRAITS = ("none", "none", "samepoint", "zero_scale", "far_away", "elongated", "tiny", "huge", "opacity", "flat_z", "nonfinite",
          "outliers")
MODES = ("plain", "plain", "det", "norec", "norows", "refit", "refit_surfels")


def _scene(rng, case, fine):
    P = int(rng.choice([3, 40, 300, 2500, 12000, 40000]))
    kind = str(rng.choice(["cube", "room", "sphere", "lidar"]))
    aux = int(rng.choice([0, 2, 4, 8]))
    colors = bool(rng.rand() < 0.4)
    factor = float(rng.choice([0.3, 1.0, 1.0, 3.0, 10.0]))
    depth = int(rng.choice([0, 0, 0, 1, 2]))
    if depth > 0 and aux == 0:
        aux = 4
    if kind == "cube":
        sc = S.scene_cube(P=P, seed=case, colors=colors, aux=aux)
    elif kind == "room":
        sc = S.scene_room(P=P, seed=case, aux=aux, half=1.5)
    elif kind == "sphere":
        sc = S.scene_sphere(P=P, seed=case)
    else:
        sc = S.scene_lidar(P=P, seed=case, aux=aux)
    if kind in ("cube", "sphere") and P <= 40:
        factor *= 8
    if fine:
        factor *= 1.0 / 30.0
    if factor != 1.0:
        sc = _with_scales(sc, factor)
    if "others_precomp" not in sc:
        depth = 0
    return sc, kind, depth, P


def _apply_trait(sc, trait, gen):
    """Returns the shift / scale the camera has to follow."""
    P = sc["means3D"].shape[0]
    move, zoom = None, 1.0
    if trait == "samepoint":
        sc["means3D"] = (sc["means3D"][:1] * 0.2).repeat(P, 1).contiguous()
        if P > 2500:
            sc["scales"] = sc["scales"] * 0.2
    elif trait == "zero_scale":
        z = torch.rand(sc["scales"].shape, generator=gen) < 0.15
        sc["scales"] = torch.where(z, torch.zeros_like(sc["scales"]), sc["scales"]).contiguous()
    elif trait == "far_away":
        move = torch.tensor([3000.0, -2000.0, 1000.0])
        sc["means3D"] = (sc["means3D"] + move).contiguous()
    elif trait == "elongated":
        sc["scales"] = (sc["scales"] * torch.tensor([5.0, 0.2])).contiguous()
    elif trait in ("tiny", "huge"):
        zoom = 1e-4 if trait == "tiny" else 3e4
        sc["means3D"] = (sc["means3D"] * zoom).contiguous()
        sc["scales"] = (sc["scales"] * zoom).contiguous()
    elif trait == "opacity":
        r = torch.rand(sc["opacities"].shape, generator=gen)
        sc["opacities"] = torch.where(r < 0.3, torch.zeros_like(r),
                                      torch.where(r < 0.6, torch.ones_like(r), sc["opacities"])).contiguous()
    elif trait == "flat_z":
        sc["means3D"][:, 2] = 0.0
        sc["rotations"] = torch.tensor([1.0, 0.0, 0.0, 0.0]).repeat(P, 1).contiguous()
    elif trait == "outliers":
        k = max(1, P // 500)
        dirs = torch.nn.functional.normalize(torch.randn(k, 3, generator=gen), dim=-1)
        far = 10.0 ** (3.0 + 3.0 * torch.rand(k, 1, generator=gen))       # 1e3 to 1e6 scene sizes away
        sc["means3D"][:k] = dirs * far * float(sc["means3D"].abs().max())
    elif trait == "nonfinite":
        r = torch.rand(P, generator=gen)
        sc["means3D"][r < 0.02, 0] = float("nan")
        sc["means3D"][(r >= 0.02) & (r < 0.04), 1] = float("inf")
        sc["scales"][(r >= 0.05) & (r < 0.06), 0] = float("inf")
        sc["scales"][(r >= 0.06) & (r < 0.07), 1] = float("nan")
        sc["rotations"][(r >= 0.07) & (r < 0.08)] = 0.0
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    return move, zoom


def _rays(rng, case, kind, sc, H, W):
    ray_kind = str(rng.choice(["image", "image", "list", "random"]))
    if ray_kind == "random":
        gen = torch.Generator().manual_seed(case)
        m = sc["means3D"]
        ext = float(m[torch.isfinite(m).all(-1)].abs().max())
        o = ((torch.rand(H, W, 3, generator=gen) * 2 - 1) * ext * 0.8).contiguous()
        d = torch.nn.functional.normalize(torch.randn(H, W, 3, generator=gen), dim=-1).contiguous()
        return o, d, True
    if kind == "room":
        o, d = S.pinhole_rays(H, W, 70.0, (-0.6, -0.3, 0.15), (0.9, 0.45, -0.15))
    elif kind == "lidar":
        o, d = S.pinhole_rays(H, W, 80.0, (0.0, 0.0, 1.8), (30.0, 10.0, 0.0))
    elif kind == "sphere":
        o, d = S.rays_sphere(H, W, view=case)
    else:
        o, d = S.rays_cube(H, W, view=case % 5)
    if ray_kind == "list":
        o, d = o.reshape(1, H * W, 3).contiguous(), d.reshape(1, H * W, 3).contiguous()
    return o, d, False


class _Rebuilding:
    """The tracer, but every build is a refit (or nothing at all): check_case then traces on the structure the test
    prepared."""

    def __init__(self, tracer, refit):
        self._tracer, self._refit = tracer, refit

    def __getattr__(self, name):
        return getattr(self._tracer, name)

    def __call__(self, *a, **k):
        return self._tracer(*a, **k)

    def build_acceleration_structure(self, v, f, rebuild=True):
        if self._refit:
            self._tracer.build_acceleration_structure(v, f, False)


N_CASES = int(os.environ.get("DST_SWEEP_CASES", "36"))   # more on demand (10 800 pass)
FIRST_CASE = int(os.environ.get("DST_SWEEP_FIRST", "5000"))


@pytest.mark.parametrize("case", range(FIRST_CASE, FIRST_CASE + N_CASES))
def test_random_configuration(oracle, tracer, case):
    rng = np.random.RandomState(case)
    fine = bool(np.random.RandomState(case + 9999).rand() < 0.33)
    sc, kind, depth, P = _scene(rng, case, fine)
    trait, mode = str(rng.choice(TRAITS)), str(rng.choice(MODES))
    H, W = int(rng.randint(1, 72)), int(rng.randint(1, 72))
    if trait == "samepoint" and P > 12000:
        # every ray meets every quad, tens of thousands of entries per ray in a thousand chunks: a few rays are minutes of
        # oracle time already
        H, W = min(H, 3), min(W, 3)
    gen = torch.Generator().manual_seed(case + 77)
    sc = {k: v.clone() for k, v in sc.items()}
    move, zoom = _apply_trait(sc, trait, gen)
    if depth > 0:
        sc["others_precomp"][:, 0] = sc["others_precomp"][:, 0] * 0.8 + 0.1   # the reference divides by the specular
    o, d, own_origins = _rays(rng, case, kind, sc, H, W)
    if not own_origins:
        o = (o * zoom + (0.0 if move is None else move)).contiguous()
    kw = dict(bg=tuple(float(x) for x in rng.rand(3).round(2)), sh_degree=int(rng.choice([0, 1, 2, 3, 3])),
              start_from_first=bool(rng.rand() < 0.5))
    if depth > 0:
        kw.update(max_trace_depth=depth, specular_threshold=float(rng.choice([0.0, 0.1, 0.4])))
    grads = True
    if trait == "outliers":
        # its builds go over to two-level keys for good: a context of its own, the session's keeps its one-level keys
        import diff_surfel_tracing as dst
        tracer = dst.SurfelTracer()
    ctx = tracer.optix_context
    saved = (ctx.record_max_bytes, ctx.gradient_rows)
    hand = str(np.random.RandomState(case + 4242).choice(["auto", "auto", "always_1", "always_48"]))
    if trait == "samepoint" and P > 12000:
        # every ray meets every quad, tens of thousands of entries per ray in a thousand chunks: minutes for the oracle
        # as it is, and ten times the packet walk's time with every ray walking on its own
        hand = "auto"
    import helpers
    shares = (helpers.MAX_LOUD, helpers.MAX_NOISY, helpers.MIN_NOISY)
    try:
        if hand != "auto":
            ctx.set_handover(2, int(hand.split("_")[1]))
        # The shares of elements that may lean on the rounding allowance are set for the benchmark scenes.  Here the
        # traits make ill-conditioned gradients the rule (a surfel of a tenth of a millimetre, a scene 3 km from the
        # origin: the hit point is known to 1e-7 of its distance, whoever computes it), so many elements carry a wide
        # allowance; the element-wise bound itself is the same as everywhere.  Eight elements of a small tensor may
        # lean on it: forty surfels far larger than their scene and stretched 25:1 had six of their eighty scale
        # gradients there (sums that cancel to a hundredth of their terms: the oracle in float is 2.6 % from the oracle
        # in double on the worst of them, the GPU 0.4 %).
        helpers.MAX_LOUD, helpers.MAX_NOISY, helpers.MIN_NOISY = 1.0, 2e-2, 8
        if mode == "det":
            tracer.deterministic = True
            ctx.check_deterministic_range()                                       # (whatever earlier cases left)
            with warnings.catch_warnings(record=True) as caught:
                warnings.simplefilter("always")
                try:
                    check_case(oracle, tracer, sc, o, d, grads=grads, **kw)       # sizes the record
                    a, _ = check_case(oracle, tracer, sc, o, d, grads=grads, **kw)
                    b, _ = check_case(oracle, tracer, sc, o, d, grads=grads, **kw)
                except AssertionError:
                    # gradients beyond the mode's fixed range (a 0.1 mm scene of surfels 30 times smaller still: 7.7e7
                    # on a mean; a 30 km scene: 1e9) come out clamped, and the binding has to have said so; such a scene is traced without
                    # the mode, as the warning advises
                    if not any("left the fixed-point range" in str(w.message) for w in caught):
                        raise
                    a = b = {}
                    tracer.deterministic = False
                    check_case(oracle, tracer, sc, o, d, grads=grads, **kw)
            for k, v in (a.get("grads_gpu") or {}).items():
                if v is not None:
                    assert np.array_equal(v.view(np.uint32), b["grads_gpu"][k].view(np.uint32)), k
        elif mode in ("refit", "refit_surfels") and trait != "nonfinite":
            check_case(oracle, tracer, sc, o, d, grads=False, **kw)
            moved = dict(sc)
            ext = float(sc["means3D"].abs().max())
            moved["means3D"] = (sc["means3D"] + 0.2 * ext * torch.randn(sc["means3D"].shape, generator=gen)).contiguous()
            moved["scales"] = (sc["scales"] * (0.5 + 1.5 * torch.rand(sc["scales"].shape, generator=gen))).contiguous()
            moved["rotations"] = (sc["rotations"] + 0.3 * torch.randn(sc["rotations"].shape, generator=gen)).contiguous()
            if mode == "refit":
                moved["vertices"], moved["faces"] = S.get_triangles(moved["means3D"], moved["scales"], moved["rotations"])
                check_case(oracle, _Rebuilding(tracer, True), moved, o, d, grads=grads, **kw)
            else:
                moved["vertices"] = tracer.refit_from_surfels(moved["means3D"].cuda(), moved["scales"].cuda(),
                                                              moved["rotations"].cuda()).cpu()
                check_case(oracle, _Rebuilding(tracer, False), moved, o, d, grads=grads, **kw)
        else:
            if mode == "norec":
                ctx.record_max_bytes = 0
            elif mode == "norows":
                ctx.gradient_rows = False
            check_case(oracle, tracer, sc, o, d, grads=grads, **kw)
    finally:
        tracer.deterministic = False
        ctx.record_max_bytes, ctx.gradient_rows = saved
        ctx.set_handover(1, 2048)
        helpers.MAX_LOUD, helpers.MAX_NOISY, helpers.MIN_NOISY = shares
