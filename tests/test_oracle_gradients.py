"""Pins the oracle's backward pass (backward.cu) against gradients that torch autograd derives from an
independent float64 restatement of the FORWARD math.  Nothing here re-types a backward formula.

The reference's backward deviates from the true gradient in documented ways; the comparison is made on
the subset where it does not, or against a forward adjusted to express the deviation:
  - background: mid_val's colour already contains T*bg and backward adds the background term again
    (backward.cu:545-548), which is the exact gradient of a forward whose background weight is doubled;
  - accumulated weight: W is never accumulated (backward.cu:568), so the gradient of acc w.r.t. a hit's alpha is
    T_i - acc/(1-alpha_i) instead of T_i - (acc - W_i)/(1-alpha_i); that is the exact gradient of the surrogate
    acc - sum_i stopgrad(W_i/(1-alpha_i)) * alpha_i, which is what the dL/dacc test differentiates;
  - reflection origin: forward offsets the next origin by START_OFFSET (0.06) along the reflected direction, backward
    chains STEP_EPSILON (1e-5) instead (backward.cu:782 vs forward.cu:422): the exact gradient of a forward whose
    next origin is E + 1e-5 d' + stopgrad((0.06 - 1e-5) d');
  - SH mode overwrites the ray-direction gradient per hit (backward.cu:165,631) -> ray_d is compared in
    colour mode only;
  - quaternion gradients omit the normalisation Jacobian (auxiliary.h:433-477) -> compared after
    projecting the oracle's gradient with (I - q q^T) for unit q.
"""
import os

import numpy as np
import pytest
import torch

import dst_scenes as S
from helpers import oracle_scene

C0 = 0.28209479177387814
C1 = 0.4886025119029199
C2 = [1.0925484305920792, -1.0925484305920792, 0.31539156525252005, -1.0925484305920792, 0.5462742152960396]
C3 = [-0.5900435899266435, 2.890611442640554, -0.4570457994644658, 0.3731763325901154, -0.4570457994644658,
      1.445305721320277, -0.5900435899266435]


def sh_basis(d):
    """(R,3) directions -> (R,16) basis values, degree 3, direction used as given."""
    x, y, z = d.unbind(-1)
    xx, yy, zz, xy, yz, xz = x * x, y * y, z * z, x * y, y * z, x * z
    return torch.stack([
        torch.full_like(x, C0), -C1 * y, C1 * z, -C1 * x,
        C2[0] * xy, C2[1] * yz, C2[2] * (2 * zz - xx - yy), C2[3] * xz, C2[4] * (xx - yy),
        C3[0] * y * (3 * xx - yy), C3[1] * xy * z, C3[2] * y * (4 * zz - xx - yy),
        C3[3] * z * (2 * zz - 3 * xx - 3 * yy), C3[4] * x * (4 * zz - xx - yy), C3[5] * z * (xx - yy),
        C3[6] * x * (xx - 3 * yy)], dim=-1)


def forward64(ro, rd, means, scales, quats, opac, bg, colors=None, shs=None, others=None, near=0.2, bg_weight=1.0):
    """Differentiable float64 forward for depth 0.  ro, rd: (R,3).  Returns rgb (R,3), dpt (R,), norm (R,3), aux."""
    Rm = S.build_rotation(quats)                 # columns: tangent u, tangent v, normal
    Ru, Rv, Rn = Rm[:, :, 0], Rm[:, :, 1], Rm[:, :, 2]
    sx, sy = scales[:, 0], scales[:, 1]
    corner = lambda a, b: means + a * sx[:, None] * Ru + b * sy[:, None] * Rv  # noqa: E731
    A, B, C, D = corner(-3, 3), corner(-3, -3), corner(3, 3), corner(3, -3)

    def tri(v1, v2, v3):
        n = torch.linalg.cross(v2 - v1, v3 - v1)                          # (P,3)
        p = ((v1[None] - ro[:, None]) * n[None]).sum(-1)                  # (R,P)
        q = (rd[:, None] * n[None]).sum(-1)
        t = p / q
        hit = ro[:, None] + t[..., None] * rd[:, None]                    # (R,P,3)
        # barycentric inside test on detached values (a mask, not a differentiable quantity)
        with torch.no_grad():
            e1, e2, w = (v2 - v1)[None], (v3 - v1)[None], hit - v1[None]
            d11, d12, d22 = (e1 * e1).sum(-1), (e1 * e2).sum(-1), (e2 * e2).sum(-1)
            w1, w2 = (w * e1).sum(-1), (w * e2).sum(-1)
            den = d11 * d22 - d12 * d12
            b1, b2 = (d22 * w1 - d12 * w2) / den, (d11 * w2 - d12 * w1) / den
            inside = (b1 >= 0) & (b2 >= 0) & (b1 + b2 <= 1)
            margin = torch.minimum(torch.minimum(b1, b2), 1 - b1 - b2).abs()
        return t, inside, margin

    t0, in0, m0 = tri(A, B, C)
    t1, in1, m1 = tri(B, C, D)
    t = torch.where(in0, t0, t1)
    hit = (in0 | in1) & (t > 0)
    xyz = ro[:, None] + t[..., None] * rd[:, None]
    rel = xyz - means[None]
    u = (rel * Ru[None]).sum(-1) / sx[None]
    v = (rel * Rv[None]).sum(-1) / sy[None]
    G = torch.exp(-0.5 * (u * u + v * v))
    alpha = torch.clamp(opac[None, :, 0] * G, max=0.99)
    cos = -(rd[:, None] * Rn[None]).sum(-1)
    normal = torch.where(cos[..., None] > 0, Rn[None], -Rn[None])
    valid = hit & (t >= near) & (alpha >= 1.0 / 255.0) & (cos != 0)
    # front-to-back order per ray; invalid entries pushed to the end with alpha 0
    key = torch.where(valid, t.detach(), torch.full_like(t, 1e30))
    order = key.argsort(dim=1)
    gat = lambda x: torch.gather(x, 1, order)  # noqa: E731
    a_s = torch.where(gat(valid), gat(alpha), torch.zeros_like(alpha))
    Tn = torch.cumprod(1 - a_s, dim=1)
    keep = torch.cummin((Tn.detach() >= 1e-4).to(torch.int8), dim=1).values.bool()   # stop at the first crossing
    a_s = torch.where(keep, a_s, torch.zeros_like(a_s))
    Tn = torch.cumprod(1 - a_s, dim=1)
    Tp = torch.cat([torch.ones_like(Tn[:, :1]), Tn[:, :-1]], dim=1)
    w = a_s * Tp
    Tfin = Tn[:, -1]
    if colors is not None:
        col = colors[None].expand(ro.shape[0], -1, -1)
    else:
        col = torch.clamp((sh_basis(rd)[:, None, :, None] * shs[None]).sum(2) + 0.5, min=0.0)   # (R,P,3)
    col = torch.gather(col, 1, order[..., None].expand(-1, -1, 3))
    rgb = (w[..., None] * col).sum(1) + bg_weight * Tfin[:, None] * bg[None]
    dpt = (w * gat(t)).sum(1)
    nrm = (w[..., None] * torch.gather(normal, 1, order[..., None].expand(-1, -1, 3))).sum(1)
    aux = None
    if others is not None:
        oth = others[None].expand(ro.shape[0], -1, -1)
        aux = (w[..., None] * torch.gather(oth, 1, order[..., None].expand(-1, -1, others.shape[1]))).sum(1)
    edge = torch.where(in0 | in1, torch.where(in0, m0, m1), torch.minimum(m0, m1))
    info = {"n_con": (w > 0).sum(1), "w": w, "alpha": a_s, "acc": w.sum(1), "t_sorted": gat(t), "edge_margin": torch.where(t > 0, edge, torch.ones_like(edge)).min(),
            "thresh_margin": torch.where(hit, (alpha - 1 / 255).abs(), torch.ones_like(alpha)).min()}
    return rgb, dpt, nrm, aux, info


def make_case(seed, P=60, R=40, sh=False, aux=2):
    gen = torch.Generator().manual_seed(seed)
    means = (torch.rand(P, 3, generator=gen) * 2 - 1) * 0.35
    scales = torch.exp(-2.2 + 0.3 * torch.randn(P, 2, generator=gen))
    q = torch.randn(P, 4, generator=gen)
    q = q / q.norm(dim=-1, keepdim=True)
    sc = {"means3D": means, "scales": scales, "rotations": q,
          "opacities": torch.sigmoid(0.5 + torch.randn(P, 1, generator=gen))}
    if sh:
        sc["shs"] = 0.4 * torch.randn(P, 16, 3, generator=gen)
    else:
        sc["colors_precomp"] = torch.rand(P, 3, generator=gen)
    if aux:
        sc["others_precomp"] = torch.rand(P, aux, generator=gen)
    sc = {k: v.float().contiguous() for k, v in sc.items()}
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    ro = torch.tensor([0.0, 0.0, 2.0]) + 0.05 * torch.randn(R, 3, generator=gen)
    target = (torch.rand(R, 3, generator=gen) * 2 - 1) * 0.3
    rd = target - ro
    rd = rd / rd.norm(dim=-1, keepdim=True) * (0.8 + 0.4 * torch.rand(R, 1, generator=gen))   # not unit length on purpose
    up = {"rgb": torch.randn(R, 3, generator=gen), "dpt": torch.randn(R, 1, generator=gen),
          "norm": torch.randn(R, 3, generator=gen), "aux": torch.randn(R, max(aux, 2), generator=gen)}
    return sc, ro.float().contiguous(), rd.float().contiguous(), up


@pytest.mark.parametrize("seed,sh,bg", [(0, False, 0.0), (1, False, 0.0), (2, True, 0.0), (3, False, 0.6), (6, True, 0.3)])
def test_backward_matches_autograd_of_float64_forward(oracle, seed, sh, bg):
    sc, ro, rd, up = make_case(seed, sh=sh)
    R = ro.shape[0]
    bgv = (bg, 0.5 * bg, 0.25 * bg)
    s = oracle_scene(oracle, sc, ro.reshape(1, R, 3), rd.reshape(1, R, 3), bg=bgv)
    fwd = oracle.forward(s, oracle.HITS_BRUTE_LEXI)
    grads = {k: v.reshape(1, R, -1).numpy() for k, v in up.items()}
    got = oracle.backward(s, fwd, grads, oracle.HITS_BRUTE_LEXI)

    leaf = {k: sc[k].double().requires_grad_(True) for k in sc if k not in ("vertices", "faces")}
    ro64, rd64 = ro.double().requires_grad_(True), rd.double().requires_grad_(True)
    bg64 = torch.tensor(bgv, dtype=torch.float64)
    args = dict(colors=leaf.get("colors_precomp"), shs=leaf.get("shs"), others=leaf.get("others_precomp"))
    rgb, dpt, nrm, aux, info = forward64(ro64, rd64, leaf["means3D"], leaf["scales"], leaf["rotations"],
                                         leaf["opacities"], bg64, **args)
    # the two forwards agree (so the float64 model is the same function, not just a similar one)
    np.testing.assert_allclose(fwd["rgb"].reshape(R, 3), rgb.detach().numpy(), atol=2e-5)
    np.testing.assert_allclose(fwd["dpt"].reshape(R), dpt.detach().numpy(), atol=5e-5)
    np.testing.assert_allclose(fwd["norm"].reshape(R, 3), nrm.detach().numpy(), atol=2e-5)
    np.testing.assert_allclose(fwd["aux"].reshape(R, 2), aux.detach().numpy(), atol=2e-5)
    np.testing.assert_array_equal(fwd["n_con"].reshape(R), info["n_con"].numpy())
    assert fwd["n_con"].sum() > 3 * R
    # (equal per-ray contributor counts above: both sides took the same side of every threshold)

    # gradient of the forward with the background counted twice = what the reference computes (see module doc)
    rgb2, dpt2, nrm2, aux2, _ = forward64(ro64, rd64, leaf["means3D"], leaf["scales"], leaf["rotations"],
                                          leaf["opacities"], bg64, bg_weight=2.0, **args)
    loss = (rgb2 * up["rgb"].double()).sum() + (dpt2 * up["dpt"].double()[:, 0]).sum() + \
        (nrm2 * up["norm"].double()).sum() + (aux2 * up["aux"].double()).sum()
    loss.backward()

    def check(name, mine, want, rel=2e-3):
        want = want.numpy()
        scale = np.abs(want).max()
        assert scale > 0, name
        err = np.abs(mine.reshape(want.shape) - want).max() / scale
        assert err < rel, "%s: relative error %.3g" % (name, err)

    check("means3D", got["means3D"], leaf["means3D"].grad)
    check("scales", got["scales"], leaf["scales"].grad)
    check("opacities", got["opacities"], leaf["opacities"].grad)
    check("others", got["others_precomp"], leaf["others_precomp"].grad)
    check("ray_o", got["ray_o"], ro64.grad)
    q = sc["rotations"].double().numpy()
    proj = got["rotations"].astype(np.float64) - q * (q * got["rotations"]).sum(-1, keepdims=True)
    check("rotations", proj, leaf["rotations"].grad)
    if sh:
        check("shs", got["shs"], leaf["shs"].grad)
    else:
        check("colors", got["colors_precomp"], leaf["colors_precomp"].grad)
        check("ray_d", got["ray_d"], rd64.grad)
    # densification signal: sum over hits of dL/dmean * depth / 2 (backward.cu:624-626); with one hit per surfel
    # it is the mean gradient times half the hit depth -> checked in the single-hit test below


def test_grads3D_is_half_depth_times_mean_gradient(oracle):
    means = torch.tensor([[0.0, 0.0, 0.0]])
    scales = torch.tensor([[0.3, 0.4]])
    q = torch.tensor([[0.9, 0.1, -0.3, 0.2]])
    q = q / q.norm()
    v, f = S.get_triangles(means, scales, q)
    sc = {"means3D": means, "scales": scales, "rotations": q, "opacities": torch.tensor([[0.6]]),
          "colors_precomp": torch.tensor([[0.3, 0.5, 0.7]]), "vertices": v, "faces": f}
    ro = torch.tensor([[[0.1, -0.05, 2.5]]])
    rd = torch.tensor([[[-0.02, 0.03, -1.0]]])
    s = oracle_scene(oracle, sc, ro, rd)
    fwd = oracle.forward(s)
    got = oracle.backward(s, fwd, {"rgb": np.ones((1, 1, 3), np.float32), "dpt": np.ones((1, 1, 1), np.float32)})
    depth = fwd["dpt"].item() / fwd["acc"].item()
    np.testing.assert_allclose(got["grads3D"], got["means3D"] * 0.5 * depth, rtol=1e-5)
    assert np.abs(got["means3D"]).max() > 0


def test_sh_mode_replaces_ray_direction_gradient(oracle):
    """Reference quirk kept: in SH mode the last composited hit's SH direction gradient is what ray_d receives."""
    sc, ro, rd, up = make_case(5, P=1, R=1, sh=True, aux=0)
    sc["means3D"] = torch.zeros(1, 3)
    sc["scales"] = torch.full((1, 2), 0.5)
    sc["opacities"] = torch.full((1, 1), 0.8)
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    ro = torch.tensor([[0.0, 0.0, 2.0]])
    rd = torch.tensor([[0.01, 0.02, -1.0]])
    s = oracle_scene(oracle, sc, ro.reshape(1, 1, 3), rd.reshape(1, 1, 3))
    fwd = oracle.forward(s)
    assert fwd["n_con"].item() == 1
    g = {"rgb": up["rgb"].reshape(1, 1, 3).numpy()}
    got = oracle.backward(s, fwd, g)
    w = fwd["acc"].item()   # single hit: weight = alpha
    shs = sc["shs"].double()
    d64 = rd.double().requires_grad_(True)
    col = torch.clamp((sh_basis(d64)[:, None, :, None] * shs[None]).sum(2) + 0.5, min=0.0)[0, 0]
    (col * up["rgb"].double()[0] * w).sum().backward()
    np.testing.assert_allclose(got["ray_d"].ravel(), d64.grad.numpy().ravel(), rtol=1e-4, atol=1e-7)


def test_second_bounce_gradients_match_autograd_with_the_reflected_rays_held_fixed(oracle):
    """Pins how the bounces are combined in the backward pass (backward.cu:658-790: the weights f_i * prod s_j, the
    per-bounce upstream gradients) and the compositing gradients of a bounce > 0.

    Scene: a "mirror" cluster A around z = 0 facing a camera at z = 2, and a cluster B above the camera that only
    the reflected rays can reach.  The float64 model renders bounce 0 from the camera rays and bounce 1 from the
    reflected rays the oracle itself reports in mid_val, held fixed; out = C0 (1 - O0[0]) + C1 O0[0].  Holding the
    reflected rays fixed removes exactly the part of the gradient that flows through the reflection geometry (and
    that the reference approximates), so the comparison is made where that part is absent: every parameter of the
    surfels that only bounce 1 hits, and the colours and aux channels of all surfels."""
    gen = torch.Generator().manual_seed(11)
    PA, PB, R = 40, 60, 48
    meansA = torch.cat([(torch.rand(PA, 2, generator=gen) * 2 - 1) * 0.45, 0.02 * torch.randn(PA, 1, generator=gen)], -1)
    qA = torch.tensor([1.0, 0.0, 0.0, 0.0]) + 0.08 * torch.randn(PA, 4, generator=gen)     # normals close to +z
    meansB = torch.cat([(torch.rand(PB, 2, generator=gen) * 2 - 1) * 0.9, 3.2 + 0.3 * torch.rand(PB, 1, generator=gen)], -1)
    qB = torch.randn(PB, 4, generator=gen)
    means = torch.cat([meansA, meansB])
    q = torch.cat([qA, qB])
    q = q / q.norm(dim=-1, keepdim=True)
    scales = torch.cat([torch.exp(-1.6 + 0.2 * torch.randn(PA, 2, generator=gen)),
                        torch.exp(-1.3 + 0.3 * torch.randn(PB, 2, generator=gen))])
    opac = torch.sigmoid(1.0 + torch.randn(PA + PB, 1, generator=gen))
    others = torch.rand(PA + PB, 2, generator=gen)
    others[:PA, 0] = 0.5 + 0.4 * others[:PA, 0]                                            # specular of the mirror
    sc = {"means3D": means, "scales": scales, "rotations": q, "opacities": opac,
          "colors_precomp": torch.rand(PA + PB, 3, generator=gen), "others_precomp": others}
    sc = {k: v.float().contiguous() for k, v in sc.items()}
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    ro = torch.tensor([0.0, 0.0, 2.0]) + 0.03 * torch.randn(R, 3, generator=gen)
    target = torch.cat([(torch.rand(R, 2, generator=gen) * 2 - 1) * 0.3, torch.zeros(R, 1)], -1)
    rd = target - ro
    rd = (rd / rd.norm(dim=-1, keepdim=True)).float().contiguous()
    ro = ro.float().contiguous()
    g_rgb = torch.randn(R, 3, generator=gen)

    s = oracle_scene(oracle, sc, ro.reshape(1, R, 3), rd.reshape(1, R, 3), max_trace_depth=1, specular_threshold=0.1)
    fwd = oracle.forward(s, oracle.HITS_BRUTE_LEXI)
    got = oracle.backward(s, fwd, {"rgb": g_rgb.reshape(1, R, 3).numpy()}, oracle.HITS_BRUTE_LEXI)
    MID = 14 + 2
    mid = torch.from_numpy(fwd["mid"].reshape(R, 2, MID)).double()
    o1, d1 = mid[:, 1, 0:3], mid[:, 1, 3:6]
    bounced = d1.norm(dim=-1) > 0
    assert bounced.sum() > R // 2, "the mirror must reflect most rays"

    leaf = {k: sc[k].double().requires_grad_(True) for k in sc if k not in ("vertices", "faces")}
    zero_bg = torch.zeros(3, dtype=torch.float64)
    args = dict(colors=leaf["colors_precomp"], others=leaf["others_precomp"])
    geo = (leaf["means3D"], leaf["scales"], leaf["rotations"], leaf["opacities"], zero_bg)
    C0, D0, N0, O0, info0 = forward64(ro.double(), rd.double(), *geo, **args)
    d1_safe = torch.where(bounced[:, None], d1, torch.tensor([0.0, 0.0, 1.0], dtype=torch.float64).expand(R, 3))
    C1, _, _, _, info1 = forward64(o1, d1_safe, *geo, near=0.06, **args)
    C1 = torch.where(bounced[:, None], C1, torch.zeros_like(C1))
    out = C0 * (1 - O0[:, :1]) + C1 * O0[:, :1]
    # same function: bounce colours, the combined colour and the hit counts of both bounces agree
    np.testing.assert_allclose(fwd["rgb"].reshape(R, 3), out.detach().numpy(), atol=3e-5)
    np.testing.assert_allclose(mid[:, 0, 13:16].numpy(), C0.detach().numpy(), atol=3e-5)
    np.testing.assert_allclose(mid[bounced][:, 1, 13:16].numpy(), C1[bounced].detach().numpy(), atol=3e-5)
    n1 = torch.where(bounced, info1["n_con"], torch.zeros_like(info1["n_con"]))
    np.testing.assert_array_equal(fwd["n_con"].reshape(R), (info0["n_con"] + n1).numpy())
    assert n1.sum() > R, "bounce 1 must composite hits"

    (out * g_rgb.double()).sum().backward()

    def check(name, mine, want, rows, rel=2e-3):
        mine, want = np.asarray(mine, np.float64).reshape(want.shape)[rows], want.numpy()[rows]
        scale = np.abs(want).max()
        assert scale > 0, name
        err = np.abs(mine - want).max() / scale
        assert err < rel, "%s: relative error %.3g" % (name, err)

    B = slice(PA, PA + PB)   # never seen by the camera rays: z > 3 is behind their origin
    check("means3D of B", got["means3D"], leaf["means3D"].grad, B)
    check("scales of B", got["scales"], leaf["scales"].grad, B)
    check("opacities of B", got["opacities"], leaf["opacities"].grad, B)
    qn = sc["rotations"].double().numpy()
    proj = got["rotations"].astype(np.float64) - qn * (qn * got["rotations"]).sum(-1, keepdims=True)
    check("rotations of B", proj, leaf["rotations"].grad, B)
    check("colours of all", got["colors_precomp"], leaf["colors_precomp"].grad, slice(0, PA + PB))
    # the specular channel of the mirror weighs the two bounces against each other: d out / d O0 = C1 - C0
    check("aux channels of all", got["others_precomp"], leaf["others_precomp"].grad, slice(0, PA + PB))


def acc_surrogate(info):
    """acc as the reference's backward differentiates it (W never accumulated, backward.cu:568)."""
    w, a = info["w"], info["alpha"]
    W = torch.cumsum(w, dim=1)
    return info["acc"] - ((W / (1 - a)).detach() * a).sum(1)


def reference_like_loss(ro64, rd64, leaf, bg64, up, args, bg_weight=2.0, with_acc=True):
    rgb, dpt, nrm, aux, info = forward64(ro64, rd64, leaf["means3D"], leaf["scales"], leaf["rotations"],
                                         leaf["opacities"], bg64, bg_weight=bg_weight, **args)
    loss = (rgb * up["rgb"].double()).sum() + (dpt * up["dpt"].double()[:, 0]).sum() + \
        (nrm * up["norm"].double()).sum() + (aux * up["aux"].double()).sum()
    if with_acc:
        loss = loss + (acc_surrogate(info) * up["acc"].double()[:, 0]).sum()
    return loss


def relcheck(name, mine, want, rel=3e-4, rows=slice(None)):
    want = want.numpy()[rows] if hasattr(want, "numpy") else np.asarray(want)[rows]
    mine = np.asarray(mine, np.float64).reshape(-1, *want.shape[1:])[rows] if want.ndim > 1 else np.asarray(mine, np.float64).reshape(-1)[rows]
    scale = np.abs(want).max()
    assert scale > 0, name
    err = np.abs(mine.reshape(want.shape) - want).max() / scale
    if os.environ.get("DST_SHOW_ERR"):
        print("%-14s relative error %.3g" % (name, err))
    assert err < rel, "%s: relative error %.3g" % (name, err)


@pytest.mark.parametrize("seed,only_acc", [(21, True), (22, False)])
def test_dL_dacc_flow_matches_autograd_of_the_surrogate(oracle, seed, only_acc):
    """Pins the dL/dacc path of bounce_backward: upstream gradient on acc alone, then mixed with the others."""
    sc, ro, rd, up = make_case(seed, sh=False)
    R = ro.shape[0]
    gen = torch.Generator().manual_seed(seed + 100)
    up["acc"] = torch.randn(R, 1, generator=gen)
    if only_acc:
        up = {k: (v if k == "acc" else torch.zeros_like(v)) for k, v in up.items()}
    s = oracle_scene(oracle, sc, ro.reshape(1, R, 3), rd.reshape(1, R, 3))
    fwd = oracle.forward(s, oracle.HITS_BRUTE_LEXI)
    got = oracle.backward(s, fwd, {k: v.reshape(1, R, -1).numpy() for k, v in up.items()}, oracle.HITS_BRUTE_LEXI)
    leaf = {k: sc[k].double().requires_grad_(True) for k in sc if k not in ("vertices", "faces")}
    ro64, rd64 = ro.double().requires_grad_(True), rd.double().requires_grad_(True)
    args = dict(colors=leaf.get("colors_precomp"), others=leaf.get("others_precomp"))
    bg64 = torch.zeros(3, dtype=torch.float64)
    _, _, _, _, info = forward64(ro64, rd64, leaf["means3D"], leaf["scales"], leaf["rotations"], leaf["opacities"],
                                 bg64, **args)
    np.testing.assert_allclose(fwd["acc"].reshape(R), info["acc"].detach().numpy(), atol=2e-5)
    np.testing.assert_array_equal(fwd["n_con"].reshape(R), info["n_con"].numpy())
    assert (info["n_con"] >= 2).sum() > R // 2      # W_i differs from 0 and from acc on most rays
    reference_like_loss(ro64, rd64, leaf, bg64, up, args).backward()
    relcheck("means3D", got["means3D"], leaf["means3D"].grad)
    relcheck("scales", got["scales"], leaf["scales"].grad)
    relcheck("opacities", got["opacities"], leaf["opacities"].grad)
    relcheck("ray_o", got["ray_o"], ro64.grad)
    relcheck("ray_d", got["ray_d"], rd64.grad)
    q = sc["rotations"].double().numpy()
    proj = got["rotations"].astype(np.float64) - q * (q * got["rotations"]).sum(-1, keepdims=True)
    relcheck("rotations", proj, leaf["rotations"].grad)
    # the true gradient of acc is a different vector: the surrogate is not a no-op
    leaf2 = {k: sc[k].double().requires_grad_(True) for k in sc if k not in ("vertices", "faces")}
    _, _, _, _, info2 = forward64(ro.double(), rd.double(), leaf2["means3D"], leaf2["scales"], leaf2["rotations"],
                                  leaf2["opacities"], bg64, colors=leaf2["colors_precomp"], others=leaf2["others_precomp"])
    (info2["acc"] * up["acc"].double()[:, 0]).sum().backward()
    if only_acc:
        true_g = leaf2["opacities"].grad.numpy()
        assert np.abs(true_g - got["opacities"]).max() > 0.05 * np.abs(true_g).max()


def test_reflection_helpers_are_the_jacobians_they_claim(oracle):
    """dnormvdv = J_normalize(v)^T g;  ddotndndn / ddotndndd = vjp of f(n, d) = (n.d) n w.r.t. n / d
    (auxiliary.h:111-121, 234-252)."""
    gen = torch.Generator().manual_seed(31)
    for _ in range(20):
        v = torch.randn(3, generator=gen, dtype=torch.float64) * 3
        d = torch.randn(3, generator=gen, dtype=torch.float64)
        g = torch.randn(3, generator=gen, dtype=torch.float64)
        v1 = v.clone().requires_grad_(True)
        ((v1 / v1.norm()) * g).sum().backward()
        np.testing.assert_allclose(oracle.reflection_vjp("dnormvdv", v.numpy(), d.numpy(), g.numpy()), v1.grad.numpy(),
                                   rtol=2e-5, atol=1e-6)
        n = (v / v.norm()).clone().requires_grad_(True)
        d1 = d.clone().requires_grad_(True)
        (((n * d1).sum() * n) * g).sum().backward()
        np.testing.assert_allclose(oracle.reflection_vjp("ddotndndn", n.detach().numpy(), d.numpy(), g.numpy()),
                                   n.grad.numpy(), rtol=2e-5, atol=1e-6)
        np.testing.assert_allclose(oracle.reflection_vjp("ddotndndd", n.detach().numpy(), d.numpy(), g.numpy()),
                                   d1.grad.numpy(), rtol=2e-5, atol=1e-6)


def mirror_scene(seed, PA=40, PB=60, R=48):
    """A "mirror" cluster A around z = 0 facing a camera at z = 2 and a cluster B above the camera that only the
    reflected rays can reach."""
    gen = torch.Generator().manual_seed(seed)
    meansA = torch.cat([(torch.rand(PA, 2, generator=gen) * 2 - 1) * 0.45, 0.02 * torch.randn(PA, 1, generator=gen)], -1)
    qA = torch.tensor([1.0, 0.0, 0.0, 0.0]) + 0.08 * torch.randn(PA, 4, generator=gen)
    meansB = torch.cat([(torch.rand(PB, 2, generator=gen) * 2 - 1) * 0.9, 3.2 + 0.3 * torch.rand(PB, 1, generator=gen)], -1)
    qB = torch.randn(PB, 4, generator=gen)
    q = torch.cat([qA, qB])
    q = q / q.norm(dim=-1, keepdim=True)
    scales = torch.cat([torch.exp(-1.6 + 0.2 * torch.randn(PA, 2, generator=gen)),
                        torch.exp(-1.3 + 0.3 * torch.randn(PB, 2, generator=gen))])
    others = torch.rand(PA + PB, 2, generator=gen)
    others[:PA, 0] = 0.5 + 0.4 * others[:PA, 0]
    sc = {"means3D": torch.cat([meansA, meansB]), "scales": scales, "rotations": q,
          "opacities": torch.sigmoid(1.0 + torch.randn(PA + PB, 1, generator=gen)),
          "colors_precomp": torch.rand(PA + PB, 3, generator=gen), "others_precomp": others}
    sc = {k: v.float().contiguous() for k, v in sc.items()}
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    ro = torch.tensor([0.0, 0.0, 2.0]) + 0.03 * torch.randn(R, 3, generator=gen)
    target = torch.cat([(torch.rand(R, 2, generator=gen) * 2 - 1) * 0.3, torch.zeros(R, 1)], -1)
    rd = target - ro
    rd = (rd / rd.norm(dim=-1, keepdim=True)).float().contiguous()
    up = {"rgb": torch.randn(R, 3, generator=gen), "dpt": torch.randn(R, 1, generator=gen),
          "norm": torch.randn(R, 3, generator=gen), "aux": torch.randn(R, 2, generator=gen),
          "acc": torch.randn(R, 1, generator=gen)}
    return sc, ro.float().contiguous(), rd, up


@pytest.mark.parametrize("seed", [42, 43, 44, 45])
def test_full_two_bounce_chain_matches_autograd_with_the_reflected_rays_free(oracle, seed):
    """Pins the reflection-geometry chain of path_backward (backward.cu:700-790): the reflected ray of bounce 1 is a
    differentiable function of bounce 0's depth, normal, origin and direction,
        E = o + D d,  n = N/|N|,  d' = d - 2 (n.d) n,  o' = E + 1e-5 d' + stopgrad((0.06 - 1e-5) d'),
    and the float64 model renders bounce 1 from (o', d').  Every gradient the oracle returns, for every surfel and
    every ray, is compared with autograd of that model (the acc output through its surrogate)."""
    sc, ro, rd, up = mirror_scene(seed)
    R, PA = ro.shape[0], 40
    s = oracle_scene(oracle, sc, ro.reshape(1, R, 3), rd.reshape(1, R, 3), max_trace_depth=1, specular_threshold=0.0)
    fwd = oracle.forward(s, oracle.HITS_BRUTE_LEXI)
    got = oracle.backward(s, fwd, {k: v.reshape(1, R, -1).numpy() for k, v in up.items()}, oracle.HITS_BRUTE_LEXI)
    mid = torch.from_numpy(fwd["mid"].reshape(R, 2, 16)).double()
    bounced = mid[:, 1, 3:6].norm(dim=-1) > 0

    leaf = {k: sc[k].double().requires_grad_(True) for k in sc if k not in ("vertices", "faces")}
    ro64, rd64 = ro.double().requires_grad_(True), rd.double().requires_grad_(True)
    zero_bg = torch.zeros(3, dtype=torch.float64)
    args = dict(colors=leaf["colors_precomp"], others=leaf["others_precomp"])
    geo = (leaf["means3D"], leaf["scales"], leaf["rotations"], leaf["opacities"], zero_bg)
    C0, D0, N0, O0, info0 = forward64(ro64, rd64, *geo, **args)
    hit0 = info0["n_con"] > 0
    np.testing.assert_array_equal(bounced.numpy(), hit0.numpy())     # threshold 0: every ray that hits bounces
    assert hit0.sum() > R // 2
    Nsafe = torch.where(hit0[:, None], N0, torch.tensor([0.0, 0.0, 1.0], dtype=torch.float64).expand(R, 3))
    n = Nsafe / Nsafe.norm(dim=-1, keepdim=True)
    d1 = rd64 - 2 * (n * rd64).sum(-1, keepdim=True) * n
    E = ro64 + D0[:, None] * rd64
    o1 = E + 1e-5 * d1 + ((0.06 - 1e-5) * d1).detach()
    np.testing.assert_allclose(mid[bounced][:, 1, 0:3].numpy(), o1[bounced].detach().numpy(), atol=2e-5)
    np.testing.assert_allclose(mid[bounced][:, 1, 3:6].numpy(), d1[bounced].detach().numpy(), atol=2e-5)
    C1, _, _, _, info1 = forward64(o1, d1, *geo, near=0.06, **args)
    C1 = torch.where(hit0[:, None], C1, torch.zeros_like(C1))
    s0 = O0[:, :1]
    out = C0 * (1 - s0) + C1 * s0
    np.testing.assert_allclose(fwd["rgb"].reshape(R, 3), out.detach().numpy(), atol=3e-5)
    n1 = torch.where(hit0, info1["n_con"], torch.zeros_like(info1["n_con"]))
    np.testing.assert_array_equal(fwd["n_con"].reshape(R), (info0["n_con"] + n1).numpy())
    assert n1.sum() > R

    loss = (out * up["rgb"].double()).sum() + (D0 * up["dpt"].double()[:, 0]).sum() + \
        (N0 * up["norm"].double()).sum() + (O0 * up["aux"].double()).sum() + \
        (acc_surrogate(info0) * up["acc"].double()[:, 0]).sum()
    loss.backward()
    # the chain really carries weight: with the reflected rays held fixed the mirror's gradients are different
    relcheck("means3D", got["means3D"], leaf["means3D"].grad)
    relcheck("scales", got["scales"], leaf["scales"].grad)
    relcheck("opacities", got["opacities"], leaf["opacities"].grad)
    relcheck("colours", got["colors_precomp"], leaf["colors_precomp"].grad)
    relcheck("aux channels", got["others_precomp"], leaf["others_precomp"].grad)
    qn = sc["rotations"].double().numpy()
    proj = got["rotations"].astype(np.float64) - qn * (qn * got["rotations"]).sum(-1, keepdims=True)
    relcheck("rotations", proj, leaf["rotations"].grad)
    relcheck("ray_o", got["ray_o"], ro64.grad)
    relcheck("ray_d", got["ray_d"], rd64.grad)


def test_three_bounce_weights_and_chained_reflections(oracle):
    """Depth 2 (beyond the reference's shipped MAX_TRACE_DEPTH = 1; the oracle follows the reference's loop as if
    compiled for it).  Two facing mirrors: camera -> A -> B -> A.  On rays that are traced through all three
    bounces the reference's weights are the true ones (g C_i: f_i prod s_j; d out/d s_1) except for d out/d s_0,
    where its running colour is updated with a specular product that was already divided (backward.cu:762-774):
    it yields s_1 (C_2 - C_1) + (C_1 - C_0)/s_0 instead of s_1 (C_2 - C_1) + (C_1 - C_0).  That difference is added
    to the model as a stop-gradient coefficient on s_0; everything else (per-bounce colour weights, the gradient
    w.r.t. s_1, two chained reflections) is autograd of the float64 forward.  Rays that end early get no upstream
    gradient here (the reference scales them by a skipped specular, backward.cu:724-725)."""
    gen = torch.Generator().manual_seed(51)
    PA, PB, R = 50, 70, 40
    meansA = torch.cat([(torch.rand(PA, 2, generator=gen) * 2 - 1) * 0.5, 0.02 * torch.randn(PA, 1, generator=gen)], -1)
    meansB = torch.cat([(torch.rand(PB, 2, generator=gen) * 2 - 1) * 0.9, 3.4 + 0.02 * torch.randn(PB, 1, generator=gen)], -1)
    q = torch.tensor([1.0, 0.0, 0.0, 0.0]) + 0.05 * torch.randn(PA + PB, 4, generator=gen)
    q = q / q.norm(dim=-1, keepdim=True)
    scales = torch.cat([torch.exp(-1.5 + 0.2 * torch.randn(PA, 2, generator=gen)),
                        torch.exp(-1.2 + 0.2 * torch.randn(PB, 2, generator=gen))])
    others = torch.rand(PA + PB, 2, generator=gen)
    others[:, 0] = 0.5 + 0.4 * others[:, 0]
    sc = {"means3D": torch.cat([meansA, meansB]), "scales": scales, "rotations": q,
          "opacities": torch.sigmoid(0.5 + torch.randn(PA + PB, 1, generator=gen)),
          "colors_precomp": torch.rand(PA + PB, 3, generator=gen), "others_precomp": others}
    sc = {k: v.float().contiguous() for k, v in sc.items()}
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    ro = (torch.tensor([0.0, 0.0, 2.0]) + 0.03 * torch.randn(R, 3, generator=gen)).float().contiguous()
    target = torch.cat([(torch.rand(R, 2, generator=gen) * 2 - 1) * 0.25, torch.zeros(R, 1)], -1)
    rd = target - ro
    rd = (rd / rd.norm(dim=-1, keepdim=True)).float().contiguous()

    s = oracle_scene(oracle, sc, ro.reshape(1, R, 3), rd.reshape(1, R, 3), max_trace_depth=2, specular_threshold=0.0)
    fwd = oracle.forward(s, oracle.HITS_BRUTE_LEXI)
    mid = torch.from_numpy(fwd["mid"].reshape(R, 3, 16)).double()
    full = mid[:, 2, 3:6].norm(dim=-1) > 0                      # traced through all three bounces
    assert full.sum() > R // 2
    up = {"rgb": torch.randn(R, 3, generator=gen) * full[:, None], "dpt": torch.randn(R, 1, generator=gen) * full[:, None],
          "norm": torch.randn(R, 3, generator=gen) * full[:, None], "aux": torch.randn(R, 2, generator=gen) * full[:, None]}
    got = oracle.backward(s, fwd, {k: v.reshape(1, R, -1).numpy() for k, v in up.items()}, oracle.HITS_BRUTE_LEXI)

    leaf = {k: sc[k].double().requires_grad_(True) for k in sc if k not in ("vertices", "faces")}
    ro64, rd64 = ro.double().requires_grad_(True), rd.double().requires_grad_(True)
    geo = (leaf["means3D"], leaf["scales"], leaf["rotations"], leaf["opacities"], torch.zeros(3, dtype=torch.float64))
    args = dict(colors=leaf["colors_precomp"], others=leaf["others_precomp"])
    o, d, near = ro64, rd64, 0.2
    Cs, Ss, first, n_total = [], [], None, 0
    for i in range(3):
        C, D, N, O, info = forward64(o, d, *geo, near=near, **args)
        if i == 0:
            first = (D, N, O)
        np.testing.assert_allclose(mid[full][:, i, 13:16].numpy(), C[full].detach().numpy(), atol=5e-5)
        n_total = n_total + info["n_con"]
        Cs.append(C)
        Ss.append(O[:, :1])
        if i < 2:
            Nsafe = torch.where(full[:, None], N, torch.tensor([0.0, 0.0, 1.0], dtype=torch.float64).expand(R, 3))
            n = Nsafe / Nsafe.norm(dim=-1, keepdim=True)
            d_next = d - 2 * (n * d).sum(-1, keepdim=True) * n
            o = o + D[:, None] * d + 1e-5 * d_next + ((0.06 - 1e-5) * d_next).detach()
            d, near = d_next, 0.06
    np.testing.assert_array_equal(fwd["n_con"].reshape(R)[full.numpy()], n_total[full].numpy())
    s0, s1 = Ss[0], Ss[1]
    out = Cs[0] * (1 - s0) + s0 * Cs[1] * (1 - s1) + s0 * s1 * Cs[2]
    np.testing.assert_allclose(fwd["rgb"].reshape(R, 3)[full.numpy()], out[full].detach().numpy(), atol=5e-5)
    g = up["rgb"].double()
    quirk = (((Cs[1] - Cs[0]) * (1 / s0 - 1)).detach() * g).sum(-1, keepdim=True) * s0      # see the docstring
    loss = (out * g).sum() + quirk.sum() + (first[0] * up["dpt"].double()[:, 0]).sum() + \
        (first[1] * up["norm"].double()).sum() + (first[2] * up["aux"].double()).sum()
    loss.backward()
    relcheck("means3D", got["means3D"], leaf["means3D"].grad)
    relcheck("scales", got["scales"], leaf["scales"].grad)
    relcheck("opacities", got["opacities"], leaf["opacities"].grad)
    relcheck("colours", got["colors_precomp"], leaf["colors_precomp"].grad)
    relcheck("aux channels", got["others_precomp"], leaf["others_precomp"].grad)
    qn = sc["rotations"].double().numpy()
    proj = got["rotations"].astype(np.float64) - qn * (qn * got["rotations"]).sum(-1, keepdims=True)
    relcheck("rotations", proj, leaf["rotations"].grad)
    relcheck("ray_o", got["ray_o"], ro64.grad)
    relcheck("ray_d", got["ray_d"], rd64.grad)


def test_rounding_sensitivity_estimate_covers_the_float_evaluation_and_stays_small(oracle):
    """The comparison of the HIP path with the oracle allows each geometric gradient element a multiple of the
    oracle's sensitivity estimate (helpers.assert_gradients).  Here: that estimate covers what fp32 rounding does
    to the oracle's own float evaluation (float vs double algebra), on a LiDAR scene (hits 50 m away at grazing
    angles: many noisy elements) and on the unit-cube scene, where it exceeds the plain 1e-3 relative bound on a
    small share of the elements only, so the comparison keeps its teeth."""
    from helpers import NOISE_FACTOR
    lidar = S.perturb_means(S.scene_lidar(P=60000, seed=0, aux=4), 1)
    cases = ((lidar, S.rays_lidar(beams=32, azimuths=256), 4, 0.2), (S.scene_cube(P=3000, seed=1), S.rays_cube(48, 48), 2, 0.06))
    for sc, (o, d), aux, share in cases:
        up = {k: v.numpy() for k, v in S.upstream_grads(o.shape[0], o.shape[1], aux).items()}
        s = oracle_scene(oracle, sc, o, d)
        fwd = oracle.forward(s, oracle.HITS_BVH_LEXI)
        g32 = oracle.backward(s, fwd, up, oracle.HITS_BVH_LEXI)
        g64 = oracle.backward(s, fwd, up, oracle.HITS_BVH_LEXI, noise=True)
        assert fwd["n_con"].sum() > 1000
        for k in ("scales", "rotations", "means3D", "grads3D", "ray_o"):
            b, est = g32[k].astype(np.float64), g64["noise"][k].astype(np.float64)
            diff = np.abs(b - g64[k])
            assert (diff <= 1e-3 * np.abs(b) + NOISE_FACTOR * est + 1e-6 * np.abs(b).max()).all(), k
            assert (est > 1e-3 * np.abs(b))[b != 0].mean() < share, k
