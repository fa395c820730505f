"""Pins the oracle's compositing (forward.cu:136-424) with closed forms and invariants:
hand-computable scenes, the chunk boundary at 16 hits, every rejection threshold, the
256-contributor cap, permutation equivariance, the mid_val layout and a two-bounce mirror."""
import math

import numpy as np
import pytest
import torch

import dst_scenes as S
from helpers import oracle_scene

IDQ = (1.0, 0.0, 0.0, 0.0)  # identity rotation: tangent u = x, tangent v = y, normal = z


def stack_scene(zs, opac, scale=0.5, colors=None, xy=(0.0, 0.0), others=None):
    """Axis-aligned surfels (normal +z) at heights zs, all centred at xy."""
    P = len(zs)
    means = torch.tensor([[xy[0], xy[1], z] for z in zs], dtype=torch.float32)
    scales = torch.full((P, 2), scale)
    rot = torch.tensor([IDQ] * P, dtype=torch.float32)
    op = torch.as_tensor(opac, dtype=torch.float32).reshape(-1, 1).expand(P, 1).contiguous() if np.ndim(opac) else \
        torch.full((P, 1), float(opac))
    col = torch.as_tensor(colors, dtype=torch.float32) if colors is not None else torch.full((P, 3), 0.5)
    v, f = S.get_triangles(means, scales, rot)
    sc = {"means3D": means, "scales": scales, "rotations": rot, "opacities": op, "colors_precomp": col,
          "vertices": v, "faces": f}
    if others is not None:
        sc["others_precomp"] = torch.as_tensor(others, dtype=torch.float32)
    return sc


def one_ray(o, d):
    return torch.tensor(o, dtype=torch.float32).reshape(1, 1, 3), torch.tensor(d, dtype=torch.float32).reshape(1, 1, 3)


def run(oracle, sc, o, d, mode=None, **kw):
    return oracle.forward(oracle_scene(oracle, sc, o, d, **kw), oracle.HITS_BRUTE_LEXI if mode is None else mode)


def test_single_surfel_head_on(oracle):
    sc = stack_scene([0.0], 0.7, colors=[[0.2, 0.4, 0.9]])
    out = run(oracle, sc, *one_ray([0, 0, 2], [0, 0, -1]), bg=(0.1, 0.2, 0.3))
    a = np.float32(0.7)
    np.testing.assert_allclose(out["acc"].ravel(), [0.7], rtol=1e-6)
    np.testing.assert_allclose(out["rgb"].ravel(), 0.7 * np.array([0.2, 0.4, 0.9]) + 0.3 * np.array([0.1, 0.2, 0.3]),
                               rtol=1e-6)
    np.testing.assert_allclose(out["dpt"].ravel(), [a * 2.0], rtol=1e-6)
    np.testing.assert_allclose(out["norm"].ravel(), [0, 0, 0.7], atol=1e-7)  # faces the ray
    np.testing.assert_allclose(out["wet"].ravel(), [0.7], rtol=1e-6)
    assert out["n_con"].item() == 1 and out["n_proc"].item() == 1
    assert (out["dist"] == 0).all()
    # from below: the normal is flipped towards the ray (DUAL_VISIABLE)
    out = run(oracle, sc, *one_ray([0, 0, -2], [0, 0, 1]))
    np.testing.assert_allclose(out["norm"].ravel(), [0, 0, -0.7], atol=1e-7)


def test_gaussian_falloff_uses_uv_over_scale(oracle):
    sc = stack_scene([0.0], 0.7, scale=0.5)
    out = run(oracle, sc, *one_ray([0.5, 0.25, 2], [0, 0, -1]))  # u = 1, v = 0.5
    want = 0.7 * math.exp(-0.5 * (1.0 + 0.25))
    np.testing.assert_allclose(out["acc"].ravel(), [want], rtol=2e-6)
    # anisotropic scales and a rotated frame: 90 degrees about z maps u to y
    q = (math.cos(math.pi / 4), 0.0, 0.0, math.sin(math.pi / 4))
    means = torch.zeros(1, 3)
    scales = torch.tensor([[0.5, 0.1]])
    rot = torch.tensor([q], dtype=torch.float32)
    v, f = S.get_triangles(means, scales, rot)
    sc = {"means3D": means, "scales": scales, "rotations": rot, "opacities": torch.full((1, 1), 0.7),
          "colors_precomp": torch.ones(1, 3), "vertices": v, "faces": f}
    out = run(oracle, sc, *one_ray([0.05, 0.25, 2], [0, 0, -1]))  # u = y/0.5 = 0.5, v = -x/0.1 = -0.5
    np.testing.assert_allclose(out["acc"].ravel(), [0.7 * math.exp(-0.5 * 0.5)], rtol=3e-6)


def test_alpha_clamp_and_scale_modifier_absent(oracle):
    out = run(oracle, stack_scene([0.0], 1.0), *one_ray([0, 0, 2], [0, 0, -1]))
    np.testing.assert_allclose(out["acc"].ravel(), [0.99], rtol=1e-6)


def test_two_stacked_surfels_front_to_back(oracle):
    cols = [[1.0, 0.0, 0.0], [0.0, 1.0, 0.0]]
    sc = stack_scene([0.0, -1.0], [0.6, 0.5], colors=cols)
    out = run(oracle, sc, *one_ray([0, 0, 2], [0, 0, -1]), bg=(0, 0, 1.0))
    w0, w1 = 0.6, 0.4 * 0.5
    np.testing.assert_allclose(out["rgb"].ravel(), [w0, w1, 1 - w0 - w1], rtol=1e-6)
    np.testing.assert_allclose(out["dpt"].ravel(), [w0 * 2 + w1 * 3], rtol=1e-6)
    np.testing.assert_allclose(out["acc"].ravel(), [1 - 0.4 * 0.5], rtol=1e-6)
    np.testing.assert_allclose(out["wet"].ravel(), [w0, w1], rtol=1e-6)
    # order of the surfels in memory is irrelevant
    sc2 = stack_scene([-1.0, 0.0], [0.5, 0.6], colors=cols[::-1])
    out2 = run(oracle, sc2, *one_ray([0, 0, 2], [0, 0, -1]), bg=(0, 0, 1.0))
    np.testing.assert_array_equal(out["rgb"], out2["rgb"])


def test_near_plane_only_for_primary_rays_from_the_first_surface(oracle):
    sc = stack_scene([0.0], 0.7)
    o, d = one_ray([0, 0, 0.1], [0, 0, -1])  # hit at depth 0.1 < near_n = 0.2
    assert run(oracle, sc, o, d, start_from_first=True)["acc"].item() == 0.0
    np.testing.assert_allclose(run(oracle, sc, o, d, start_from_first=False)["acc"].item(), 0.7, rtol=1e-6)
    o, d = one_ray([0, 0, 0.25], [0, 0, -1])
    np.testing.assert_allclose(run(oracle, sc, o, d, start_from_first=True)["acc"].item(), 0.7, rtol=1e-6)


def test_alpha_below_one_255th_is_skipped(oracle):
    out = run(oracle, stack_scene([0.0, -1.0], [0.0039, 0.5]), *one_ray([0, 0, 2], [0, 0, -1]))
    np.testing.assert_allclose(out["acc"].ravel(), [0.5], rtol=1e-6)
    assert out["n_proc"].item() == 2 and out["n_con"].item() == 1
    out = run(oracle, stack_scene([0.0, -1.0], [0.004, 0.5]), *one_ray([0, 0, 2], [0, 0, -1]))
    np.testing.assert_allclose(out["acc"].ravel(), [1 - 0.996 * 0.5], rtol=1e-6)


def test_transmittance_threshold_drops_the_hit_that_crosses_it(oracle):
    # alpha = 0.99 each: T = 1e-2 after one, 1e-4 * (1 - 1.2e-7 ...) after two -> the second crosses 1e-4 (fp32) or the third does
    sc = stack_scene([0.0, -1.0, -2.0, -3.0], 1.0, colors=[[1, 0, 0], [0, 1, 0], [0, 0, 1], [1, 1, 1]])
    out = run(oracle, sc, *one_ray([0, 0, 2], [0, 0, -1]))
    T1 = np.float32(1) * (np.float32(1) - np.float32(0.99))
    T2 = T1 * (np.float32(1) - np.float32(0.99))
    kept = 1 if T2 < np.float32(1e-4) else 2
    assert out["n_con"].item() == kept
    want_T = T1 if kept == 1 else T2
    np.testing.assert_allclose(out["acc"].ravel(), [1 - want_T], rtol=1e-6)
    assert out["rgb"].ravel()[2] == 0.0  # nothing behind the crossing point is blended


@pytest.mark.parametrize("n", [15, 16, 17, 33, 40])
def test_chunk_boundary(oracle, n):
    """More than 16 surfels on one ray need several traversals (forward.cu:299-306); the result must not depend on it."""
    zs = [-0.01 * k for k in range(n)]
    rng = np.random.default_rng(n)
    op = rng.uniform(0.02, 0.08, n).astype(np.float32)
    col = rng.uniform(0, 1, (n, 3)).astype(np.float32)
    out = run(oracle, stack_scene(zs, op, colors=col), *one_ray([0, 0, 2], [0, 0, -1]))
    T, rgb, dpt = 1.0, np.zeros(3), 0.0
    for k in range(n):
        w = T * float(op[k])
        rgb += w * col[k]
        dpt += w * (2.0 + 0.01 * k)
        T *= 1 - float(op[k])
    assert out["n_con"].item() == n and out["n_proc"].item() == n
    np.testing.assert_allclose(out["acc"].ravel(), [1 - T], rtol=2e-6)
    np.testing.assert_allclose(out["rgb"].ravel(), rgb, rtol=2e-6)
    np.testing.assert_allclose(out["dpt"].ravel(), [dpt], rtol=2e-6)
    np.testing.assert_allclose(out["wet"].sum(), 1 - T, rtol=2e-6)


def test_coplanar_surfels_beyond_sixteen_are_lost_to_the_restart_step(oracle):
    """Reference behaviour, kept: a chunk restarts 1e-5 behind its last hit, so further hits at the same depth vanish."""
    n = 24
    sc = stack_scene([0.0] * n, 0.05)
    out = run(oracle, sc, *one_ray([0, 0, 2], [0, 0, -1]))
    assert out["n_con"].item() == 16
    np.testing.assert_allclose(out["acc"].ravel(), [1 - 0.95 ** 16], rtol=2e-6)


def test_contributor_cap_256(oracle):
    n = 300
    sc = stack_scene([-0.001 * k for k in range(n)], 0.004, scale=1.0)
    out = run(oracle, sc, *one_ray([0, 0, 2], [0, 0, -1]))
    assert out["n_con"].item() == 256
    np.testing.assert_allclose(out["acc"].ravel(), [1 - 0.996 ** 256], rtol=1e-4)


@pytest.mark.parametrize("colors", [False, True])
def test_invariants_on_a_random_scene(oracle, colors):
    sc = S.scene_cube(P=3000, seed=1, colors=colors, aux=2)
    o, d = S.rays_cube(24, 24)
    s = oracle_scene(oracle, sc, o, d)
    out = oracle.forward(s, oracle.HITS_BVH_LEXI)
    acc = out["acc"].astype(np.float64)
    assert (acc >= 0).all() and (acc <= 1).all()
    # sum over rays of the accumulated weight = sum over surfels of their accumulated weight
    np.testing.assert_allclose(acc.sum(), out["wet"].astype(np.float64).sum(), rtol=1e-5)
    assert (out["n_con"] <= out["n_proc"]).all() and out["n_con"].max() > 16
    # aux composites like colour: constant channel c gives c * acc
    sc1 = dict(sc)
    sc1["others_precomp"] = torch.full((3000, 2), 0.25)
    out1 = oracle.forward(oracle_scene(oracle, sc1, o, d), oracle.HITS_BVH_LEXI)
    np.testing.assert_allclose(out1["aux"][..., 0], 0.25 * out1["acc"][..., 0], rtol=1e-5, atol=1e-7)
    # the three hit enumerations give identical images
    for mode in (oracle.HITS_BRUTE_LITERAL, oracle.HITS_BRUTE_LEXI):
        other = oracle.forward(s, mode)
        for k in ("rgb", "dpt", "acc", "norm", "aux", "mid", "n_proc", "n_con"):
            np.testing.assert_array_equal(other[k], out[k])
    # background enters as T * bg
    outb = oracle.forward(oracle_scene(oracle, sc, o, d, bg=(1.0, 0.5, 0.25)), oracle.HITS_BVH_LEXI)
    np.testing.assert_allclose(outb["rgb"] - out["rgb"], (1 - out["acc"]) * np.array([1.0, 0.5, 0.25], np.float32),
                               atol=2e-6)


def test_permutation_equivariance(oracle):
    sc = S.scene_cube(P=2000, seed=3)
    o, d = S.rays_cube(16, 16)
    out = oracle.forward(oracle_scene(oracle, sc, o, d), oracle.HITS_BVH_LEXI)
    perm = torch.randperm(2000, generator=torch.Generator().manual_seed(0))
    sp = {k: v[perm] for k, v in sc.items() if k not in ("vertices", "faces")}
    sp["vertices"], sp["faces"] = S.get_triangles(sp["means3D"], sp["scales"], sp["rotations"])
    outp = oracle.forward(oracle_scene(oracle, sp, o, d), oracle.HITS_BVH_LEXI)
    for k in ("rgb", "dpt", "acc", "norm"):
        np.testing.assert_array_equal(out[k], outp[k])
    np.testing.assert_allclose(out["wet"][perm.numpy()], outp["wet"], rtol=1e-6)


def test_mid_val_layout(oracle):
    sc = stack_scene([0.0], 0.7, colors=[[0.2, 0.4, 0.9]], others=[[0.3, 0.6]])
    o, d = one_ray([0.1, 0, 2], [0, 0, -1])
    out = run(oracle, sc, o, d, bg=(0.1, 0.1, 0.1))
    m = out["mid"].ravel()
    assert m.shape == (32,)  # two slots of 16 channels, like the reference's MID_CHANNELS * (MAX_TRACE_DEPTH + 1)
    np.testing.assert_array_equal(m[0:3], np.array([0.1, 0, 2], np.float32))
    np.testing.assert_array_equal(m[3:6], [0, 0, -1])
    assert m[6] == out["dpt"].item() and m[7] == out["acc"].item()
    np.testing.assert_array_equal(m[8:11], out["norm"].ravel())
    np.testing.assert_array_equal(m[11:13], out["aux"].ravel())
    np.testing.assert_array_equal(m[13:16], out["rgb"].ravel())  # includes T * bg
    assert (m[16:] == 0).all()
    np.testing.assert_allclose(out["aux"].ravel(), out["acc"].item() * np.array([0.3, 0.6]), rtol=1e-6)


def test_mirror_bounce(oracle):
    """Depth 1: a horizontal mirror (specular 0.8) under a slanted ray, a red card where the reflection goes.
    c_out = (1 - s) c_0 + s c_1 with s the composited specular (forward.cu:388-393)."""
    means = torch.tensor([[0.0, 0.0, 0.0], [1.0, 0.0, 1.0]])
    scales = torch.tensor([[2.0, 2.0], [0.5, 0.5]])
    # card: normal along -x (faces the reflected ray travelling in +x,+z): rotate z to -x => about y by -90 deg
    qy = (math.cos(-math.pi / 4), 0.0, math.sin(-math.pi / 4), 0.0)
    rot = torch.tensor([IDQ, qy], dtype=torch.float32)
    v, f = S.get_triangles(means, scales, rot)
    sc = {"means3D": means, "scales": scales, "rotations": rot, "opacities": torch.tensor([[0.9], [0.8]]),
          "colors_precomp": torch.tensor([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]]),
          "others_precomp": torch.tensor([[0.8, 0.1], [0.0, 0.0]]), "vertices": v, "faces": f}
    s2 = math.sqrt(0.5)
    o, d = one_ray([-1.0, 0.0, 1.0], [s2, 0.0, -s2])  # hits the mirror at the origin, depth sqrt(2)
    out = run(oracle, sc, o, d, max_trace_depth=1, specular_threshold=0.1)
    a0 = 0.9
    spec = a0 * 0.8
    m = out["mid"].reshape(2, 16)
    np.testing.assert_allclose(m[0, 6], a0 * math.sqrt(2.0), rtol=1e-6)
    # reflected ray: origin = o + D d + 0.06 d', direction d' = (s2, 0, s2)
    dprime = np.array([s2, 0.0, s2])
    E = np.array([-1.0, 0.0, 1.0]) + a0 * math.sqrt(2.0) * np.array([s2, 0.0, -s2])
    np.testing.assert_allclose(m[1, 3:6], dprime, atol=1e-6)
    np.testing.assert_allclose(m[1, 0:3], E + 0.06 * dprime, atol=1e-6)
    # the card is hit at x = 1: |uv| small?  compute its alpha from the geometry
    t1 = (1.0 - m[1, 0]) / dprime[0]
    hit = m[1, 0:3] + t1 * dprime
    u_card = (hit - np.array([1.0, 0.0, 1.0]))
    rows = oracle.quat_to_rows(np.array(qy, np.float32)).astype(np.float64)
    uu, vv = rows[0] @ u_card / 0.5, rows[1] @ u_card / 0.5
    a1 = 0.8 * math.exp(-0.5 * (uu * uu + vv * vv))
    c0 = a0 * np.array([0.0, 0.0, 1.0])
    c1 = a1 * np.array([1.0, 0.0, 0.0])
    np.testing.assert_allclose(out["rgb"].ravel(), (1 - spec) * c0 + spec * c1, rtol=2e-5, atol=1e-6)
    np.testing.assert_allclose(out["aux"].ravel(), [spec, a0 * 0.1], rtol=1e-6)
    np.testing.assert_allclose(out["acc"].ravel(), [a0], rtol=1e-6)  # dpt/acc/norm/aux come from the first bounce only
    # below the threshold the path stops after the first bounce and the second slot stays zero
    out0 = run(oracle, sc, o, d, max_trace_depth=1, specular_threshold=0.9)
    assert (out0["mid"].reshape(2, 16)[1] == 0).all()
    np.testing.assert_allclose(out0["rgb"].ravel(), (1 - spec) * c0, rtol=1e-6)


def test_reference_stale_slot_switch_changes_nothing_without_repeated_hits(oracle):
    sc = S.scene_cube(P=3000, seed=8)
    o, d = S.rays_cube(16, 16)
    s = oracle_scene(oracle, sc, o, d)
    a = oracle.forward(s, oracle.HITS_BRUTE_LEXI, literal_stale=False)
    b = oracle.forward(s, oracle.HITS_BRUTE_LEXI, literal_stale=True)
    for k in ("rgb", "dpt", "acc", "norm", "n_con"):
        np.testing.assert_array_equal(a[k], b[k])


def _stale_slot_share(oracle, sc, o, d):
    s = oracle_scene(oracle, sc, o, d)
    a = oracle.forward(s, oracle.HITS_BVH_LEXI, literal_stale=False)
    b = oracle.forward(s, oracle.HITS_BVH_LEXI, literal_stale=True)
    differ = np.zeros(a["rgb"].shape[:2], bool)
    for k in ("rgb", "dpt", "acc", "norm"):
        differ |= (a[k].view(np.uint32) != b[k].view(np.uint32)).any(-1)
    return int(differ.sum()), differ.size, float(np.abs(a["rgb"] - b["rgb"]).max())


def test_share_of_rays_the_reference_stale_slot_touches_on_the_large_scenes(oracle):
    """The reference leaves a buffer entry that repeats the last composited surfel in place (forward.cu:207-216), and
    the entry then takes part in the next chunk's 16; the library (and the oracle by default) clears it.  On the two
    BASELINE scenes where repeated hits can arise - the 1M-surfel room (coplanar walls, every third pixel row and
    column of the 1080p image) and the 2M-surfel lidar scene (140 m ground, all 131,072 rays) - the switch changes
    few rays: 5 of the room's 230,400 sampled rays (2.2e-5; 13 of 518,400 at every second row and column), with a
    largest colour change of 3e-3, and none of the lidar rays.  The bound below is what keeps that statement true."""
    n, size, worst = _stale_slot_share(oracle, S.scene_lidar(P=2000000, seed=0, aux=4), *S.rays_lidar())
    print("stale slot, lidar scene: %d of %d rays differ" % (n, size))
    assert n == 0
    o, d = S.rays_room(1080, 1920)
    n, size, worst = _stale_slot_share(oracle, S.scene_room(P=1000000, seed=0), o[::3, ::3].contiguous(),
                                       d[::3, ::3].contiguous())
    print("stale slot, room scene: %d of %d rays differ, largest colour change %.3g" % (n, size, worst))
    assert n <= 1e-4 * size and worst < 0.02


def test_malformed_requests_are_rejected(oracle):
    sc = S.scene_cube(P=10, seed=0)
    o, d = S.rays_cube(2, 2)
    with pytest.raises(RuntimeError):
        oracle.forward(oracle_scene(oracle, sc, o, d, max_trace_depth=2, mtd_alloc=1))
    bad = dict(sc)
    bad["faces"] = sc["faces"].clone()
    bad["faces"][1, 0] = 3
    with pytest.raises(RuntimeError):
        oracle.forward(oracle_scene(oracle, bad, o, d))


def test_depth_distortion_is_the_pairwise_sum_it_stands_for(oracle):
    """compute_dist (an extension: the reference leaves `dist` at zero, forward.cu:286): the running-moment form
    equals sum_i sum_{j<i} w_i w_j (m_i - m_j)^2 with m = far/(far-near) (1 - near/depth); M1, M2 are the weighted
    moments.  Checked against a float64 evaluation from the per-hit weights of the independent forward model."""
    from test_oracle_gradients import forward64, make_case
    sc, ro, rd, _ = make_case(7, P=80, R=50)
    rd = rd / rd.norm(dim=-1, keepdim=True)       # unit directions: depth = distance
    R = ro.shape[0]
    s = oracle_scene(oracle, sc, ro.reshape(1, R, 3), rd.reshape(1, R, 3))
    plain = oracle.forward(s, oracle.HITS_BRUTE_LEXI)
    assert (plain["dist"] == 0).all()
    out = oracle.forward(s, oracle.HITS_BRUTE_LEXI, compute_dist=True)
    for k in ("rgb", "dpt", "acc", "norm", "aux", "mid"):
        np.testing.assert_array_equal(out[k], plain[k])
    leaf = {k: sc[k].double() for k in sc if k not in ("vertices", "faces")}
    # per-hit depths in compositing order: recompute them from the model's weights (w) and ordered t
    Rm = S.build_rotation(leaf["rotations"])
    rgb, dpt, nrm, aux, info = forward64(ro.double(), rd.double(), leaf["means3D"], leaf["scales"], leaf["rotations"],
                                         leaf["opacities"], torch.zeros(3, dtype=torch.float64),
                                         colors=leaf["colors_precomp"], others=leaf["others_precomp"])
    np.testing.assert_array_equal(out["n_con"].reshape(R), info["n_con"].numpy())
    w, t = info["w"], info["t_sorted"]
    m = 100.0 / (100.0 - 0.2) * (1 - 0.2 / t)
    m = torch.where(w > 0, m, torch.zeros_like(m))
    pair = (w[:, :, None] * w[:, None, :] * (m[:, :, None] - m[:, None, :]) ** 2)
    want = torch.tril(pair, diagonal=-1).sum((1, 2))
    got = out["dist"].reshape(R, 3)
    np.testing.assert_allclose(got[:, 0], want.numpy(), rtol=2e-3, atol=1e-7)
    np.testing.assert_allclose(got[:, 1], (w * m).sum(1).numpy(), rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(got[:, 2], (w * m * m).sum(1).numpy(), rtol=1e-4, atol=1e-7)
    assert want.max() > 1e-6
