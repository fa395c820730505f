"""Pins the scalar building blocks of the CPU oracle against independent references:
library routines (numpy exp, scipy spherical harmonics, scipy rotations) and a float64
ray/triangle test.  None of these re-type the oracle's formula."""
import numpy as np
import pytest
import torch
from scipy.spatial.transform import Rotation

import dst_scenes as S


def ulp_err(got32, want64):
    want32 = want64.astype(np.float32)
    ulp = np.spacing(np.abs(want32)).astype(np.float64)
    return np.abs(got32.astype(np.float64) - want64) / ulp


def test_expf_within_one_ulp_of_true_exp(oracle):
    x = np.concatenate([np.linspace(-87, 0, 40001), -np.logspace(-8, 1.9, 4000), [0.0, -0.5, -1.0, -2.7725887]])
    x = x.astype(np.float32)
    got = oracle.expf(x)
    err = ulp_err(got, np.exp(x.astype(np.float64)))
    assert err.max() <= 1.0, err.max()
    assert oracle.expf([0.0])[0] == 1.0
    # monotone on a fine grid: a dropped polynomial term or wrong reduction constant breaks this
    xs = np.linspace(-20, 0, 200001).astype(np.float32)
    assert (np.diff(oracle.expf(xs)) >= 0).all()


def test_expf_tails(oracle):
    assert oracle.expf([-100.0])[0] == 0.0
    assert oracle.expf([np.nan])[0] == 0.0
    assert oracle.expf([-87.0])[0] > 0.0


def _real_sh(l, m, d):
    """Real spherical harmonic without Condon-Shortley phase, from scipy's complex ones."""
    import scipy.special as sp
    x, y, z = d
    polar, azim = np.arccos(z / np.linalg.norm(d)), np.arctan2(y, x)
    if hasattr(sp, "sph_harm_y"):
        Y = sp.sph_harm_y(l, abs(m), polar, azim)
    else:
        Y = sp.sph_harm(abs(m), l, azim, polar)
    if m == 0:
        return Y.real
    return np.sqrt(2.0) * (-1) ** m * (Y.real if m > 0 else Y.imag)


@pytest.mark.parametrize("deg", [0, 1, 2, 3])
def test_sh_basis_is_the_real_spherical_harmonics(oracle, deg):
    """colour = sum_j basis_j(d) sh_j + 0.5 with basis_j = (-1)^m Y_lm(d): every constant, sign and
    polynomial of forward.cu:18-58 is checked against scipy, one coefficient at a time."""
    rng = np.random.default_rng(deg)
    lm = [(l, m) for l in range(4) for m in range(-l, l + 1)]
    for _ in range(5):
        d = rng.normal(size=3)
        d /= np.linalg.norm(d)
        for j, (l, m) in enumerate(lm):
            sh = np.zeros((16, 3), np.float32)
            sh[j] = (1.0, 2.0, -1.0)
            rgb, clamped = oracle.sh_color(deg, sh, d.astype(np.float32))
            basis = (-1) ** m * _real_sh(l, m, d) if l <= deg else 0.0
            want = np.array([1.0, 2.0, -1.0]) * basis + 0.5
            np.testing.assert_allclose(rgb, np.maximum(want, 0.0), atol=2e-6)
            assert list(clamped) == [float(w < 0) for w in want] or np.abs(want).min() < 1e-5


def test_sh_uses_the_direction_as_given(oracle):
    """The reference feeds the un-normalised ray direction (forward.cu:267): degree-l terms scale with |d|^l."""
    rng = np.random.default_rng(7)
    d = rng.normal(size=3).astype(np.float32)
    for j, l in [(2, 1), (6, 2), (12, 3)]:
        sh = np.zeros((16, 3), np.float32)
        sh[j] = 0.1
        a, _ = oracle.sh_color(3, sh, d)
        b, _ = oracle.sh_color(3, sh, 2 * d)
        np.testing.assert_allclose(b - 0.5, (a - 0.5) * 2 ** l, rtol=1e-5, atol=5e-7)
    sh = np.zeros((16, 3), np.float32)
    sh[0] = (1.0, -3.0, 0.0)
    rgb, clamped = oracle.sh_color(0, sh, d)
    np.testing.assert_allclose(rgb, [0.28209479177387814 + 0.5, 0.0, 0.5], atol=1e-7)
    assert list(clamped) == [0.0, 1.0, 0.0]


def test_quaternion_rows_match_scipy(oracle):
    rng = np.random.default_rng(3)
    for _ in range(50):
        q = rng.normal(size=4) * rng.uniform(0.1, 5.0)  # (w,x,y,z), any norm
        R = Rotation.from_quat([q[1], q[2], q[3], q[0]]).as_matrix()
        rows = oracle.quat_to_rows(q.astype(np.float32))
        np.testing.assert_allclose(rows, R.T, atol=3e-6)  # rows = tangent u, tangent v, normal = columns of R
    np.testing.assert_array_equal(oracle.quat_to_rows(np.array([1, 0, 0, 0], np.float32)), np.eye(3, dtype=np.float32))


def test_scene_quads_follow_the_rotation_rows(oracle):
    """get_triangles and the device math must agree on the frame: corner k = mean + a_k sx Ru + b_k sy Rv."""
    sc = S.scene_cube(P=20, seed=5)
    v = sc["vertices"].numpy().reshape(20, 4, 3)
    ab = [(-3, 3), (-3, -3), (3, 3), (3, -3)]
    for g in range(20):
        rows = oracle.quat_to_rows(sc["rotations"][g].numpy()).astype(np.float64)
        sx, sy = sc["scales"][g].numpy().astype(np.float64)
        for k, (a, b) in enumerate(ab):
            want = sc["means3D"][g].numpy() + a * sx * rows[0] + b * sy * rows[1]
            np.testing.assert_allclose(v[g, k], want, atol=2e-6)
    f = sc["faces"].numpy().reshape(20, 2, 3)
    base = 4 * np.arange(20)[:, None]
    np.testing.assert_array_equal(f[:, 0], base + [0, 1, 2])
    np.testing.assert_array_equal(f[:, 1], base + [1, 2, 3])


def _mt64(o, d, v0, v1, v2):
    """Moller-Trumbore in float64: (t, u, v) or None when parallel."""
    e1, e2 = v1 - v0, v2 - v0
    pv = np.cross(d, e2)
    det = e1 @ pv
    if abs(det) < 1e-300:
        return None
    tv = o - v0
    u = (tv @ pv) / det
    qv = np.cross(tv, e1)
    v = (d @ qv) / det
    return (e2 @ qv) / det, u, v


def test_ray_quad_matches_float64_triangle_tests(oracle):
    rng = np.random.default_rng(11)
    sc = S.scene_cube(P=200, seed=2)
    V = sc["vertices"].numpy().reshape(200, 4, 3).astype(np.float64)
    n_hit = n_checked = 0
    for _ in range(4000):
        g = rng.integers(200)
        A, B, C, D = V[g]
        # aim near the quad so that a good share of the rays hit
        target = A + rng.uniform(-0.3, 1.3) * (B - A) + rng.uniform(-0.3, 1.3) * (C - A)
        o = rng.normal(size=3) * 2.0
        d = target - o
        d /= np.linalg.norm(d)
        if rng.random() < 0.2:
            d = -d  # behind the origin: must be rejected
        o32, d32 = o.astype(np.float32), d.astype(np.float32)
        hit, t, tri = oracle.ray_quad(o32, d32, *[x.astype(np.float32) for x in (A, B, C, D)])
        o64, d64 = o32.astype(np.float64), d32.astype(np.float64)
        r0, r1 = _mt64(o64, d64, A, B, C), _mt64(o64, d64, B, C, D)
        inside, margin = [], []
        for r in (r0, r1):
            if r is None:
                inside.append(False)
                margin.append(0.0)
                continue
            tt, u, v = r
            m = min(u, v, 1 - u - v)
            inside.append(m >= 0 and tt > 0)
            margin.append(abs(m) if tt > 0 else min(abs(m), abs(tt)))
        if min(margin) < 1e-4:
            continue  # too close to an edge for fp32 and fp64 to have to agree
        n_checked += 1
        assert hit == (inside[0] or inside[1])
        if hit:
            n_hit += 1
            assert tri == (0 if inside[0] else 1)
            want_t = (r0 if tri == 0 else r1)[0]
            nrm = np.cross(B - A, C - A)
            cos = abs(nrm @ d64) / np.linalg.norm(nrm)  # fp32 rounding of n.(v-o)/n.d grows as the ray grazes the plane
            assert abs(t - want_t) <= 1e-5 * max(1.0, abs(want_t)) / max(cos, 1e-3)
    assert n_hit > 500 and n_checked > 3000


def test_ray_quad_decides_millimetre_quads_seen_from_metres_like_float64(oracle):
    """The edge tests are formed from one cross product with the ray and the quad's edge vectors, so their error is
    that of the way to the quad (eps * distance), not of its square over the edge: a 1 mm quad 3 to 6 m away is decided
    like float64 decides it as soon as the ray is 1 % of the quad away from an edge.  (With the four corners relative to
    the origin in every product, rays half a quad outside counted as hits at these sizes.)"""
    rng = np.random.default_rng(5)
    n_checked = n_hit = n_near = 0
    for _ in range(6000):
        c = rng.uniform(-2, 2, 3)
        e1 = rng.normal(size=3)
        e1 *= 1e-3 / np.linalg.norm(e1)
        e2 = np.cross(e1, rng.normal(size=3))
        e2 *= 1e-3 / np.linalg.norm(e2)
        A, B, C = c, c + e1, c + e2
        D = B + (C - A) + 2e-5 * rng.normal(size=3)          # a parallelogram, a little bent
        A, B, C, D = [x.astype(np.float32).astype(np.float64) for x in (A, B, C, D)]
        o = c + rng.normal(size=3) * 2.5
        if np.linalg.norm(o - c) < 3.0:
            o = c + (o - c) * 3.0 / np.linalg.norm(o - c)
        target = A + rng.uniform(-0.5, 1.5) * (B - A) + rng.uniform(-0.5, 1.5) * (C - A)
        d = (target - o) / np.linalg.norm(target - o)
        o32, d32 = o.astype(np.float32), d.astype(np.float32)
        hit, t, tri = oracle.ray_quad(o32, d32, *[x.astype(np.float32) for x in (A, B, C, D)])
        o64, d64 = o32.astype(np.float64), d32.astype(np.float64)
        inside, margin = [], []
        for r in (_mt64(o64, d64, A, B, C), _mt64(o64, d64, B, C, D)):
            tt, u, v = r
            m = min(u, v, 1 - u - v)
            inside.append(m >= 0 and tt > 0)
            margin.append(abs(m))
        if abs(np.cross(B - A, C - A) @ d64) < 0.2 * 1e-6:   # grazing: the plane hit itself is ill-conditioned
            continue
        if min(margin) < 1e-2:
            continue
        n_checked += 1
        n_near += min(margin) < 0.3
        assert hit == (inside[0] or inside[1]), (margin, inside, hit)
        if hit:
            n_hit += 1
            assert tri == (0 if inside[0] else 1)
    assert n_checked > 4000 and n_hit > 1000 and n_near > 2000


def test_ray_quad_known_answers(oracle):
    A, B, C, D = [np.array(p, np.float32) for p in ([-3, 3, 0], [-3, -3, 0], [3, 3, 0], [3, -3, 0])]
    down = np.array([0, 0, -1], np.float32)
    hit, t, tri = oracle.ray_quad(np.array([-1, 1, 2], np.float32), down, A, B, C, D)
    assert (hit, t, tri) == (True, 2.0, 0)  # v > u: triangle 0
    hit, t, tri = oracle.ray_quad(np.array([1, -1, 5], np.float32), down, A, B, C, D)
    assert (hit, t, tri) == (True, 5.0, 1)  # v < u: triangle 1
    hit, t, tri = oracle.ray_quad(np.array([1, 1, 2], np.float32), down, A, B, C, D)
    assert (hit, t, tri) == (True, 2.0, 0)  # on the shared diagonal: one hit, triangle 0
    assert not oracle.ray_quad(np.array([3.5, 0, 2], np.float32), down, A, B, C, D)[0]  # outside
    assert not oracle.ray_quad(np.array([0, 0, -2], np.float32), down, A, B, C, D)[0]  # behind the origin
    assert not oracle.ray_quad(np.array([0, 0, 2], np.float32), np.array([1, 0, 0], np.float32), A, B, C, D)[0]
    hit, t, _ = oracle.ray_quad(np.array([0, 0, -2], np.float32), -down, A, B, C, D)
    assert hit and t == 2.0  # both faces are hit (no culling)


def _tie_scene(P=60, seed=0):
    """Axis-aligned coplanar quads on two planes with coordinates on a coarse binary grid: equal depths are exact."""
    rng = np.random.default_rng(seed)
    means = np.zeros((P, 3), np.float32)
    means[:, 0] = rng.integers(-8, 9, P) / 16.0
    means[:, 1] = rng.integers(-8, 9, P) / 16.0
    means[:, 2] = rng.integers(0, 2, P) * 0.5
    scales = np.full((P, 2), 0.125, np.float32)
    rot = np.tile(np.array([1, 0, 0, 0], np.float32), (P, 1))
    v, f = S.get_triangles(torch.from_numpy(means), torch.from_numpy(scales), torch.from_numpy(rot))
    return {"means3D": torch.from_numpy(means), "scales": torch.from_numpy(scales), "rotations": torch.from_numpy(rot),
            "opacities": torch.full((P, 1), 0.3), "colors_precomp": torch.rand(P, 3), "vertices": v, "faces": f}


def test_k_nearest_literal_rule_equals_lexicographic_rule_and_bvh(oracle):
    from helpers import oracle_scene
    for name, sc in (("random", S.scene_cube(P=3000, seed=4, colors=True)), ("ties", _tie_scene(400, 1))):
        o, d = S.rays_cube(8, 8) if name == "random" else (
            torch.tensor([0.03125, 0.03125, 3.0]).expand(8, 8, 3).contiguous(),
            torch.tensor([0.0, 0.0, -1.0]).expand(8, 8, 3).contiguous())
        s = oracle_scene(oracle, sc, o, d)
        n_full = n_tied = 0
        for r in range(0, 64, 3):
            oo, dd = o.reshape(-1, 3)[r].numpy(), d.reshape(-1, 3)[r].numpy()
            c0, t0, i0 = oracle.k_nearest(s, oo, dd, oracle.HITS_BRUTE_LITERAL)
            c1, t1, i1 = oracle.k_nearest(s, oo, dd, oracle.HITS_BRUTE_LEXI)
            c2, t2, i2 = oracle.k_nearest(s, oo, dd, oracle.HITS_BVH_LEXI)
            assert min(c0, 16) == min(c1, 16) == min(c2, 16)
            np.testing.assert_array_equal(t0, t1)
            np.testing.assert_array_equal(i0, i1)
            np.testing.assert_array_equal(t1, t2)
            np.testing.assert_array_equal(i1, i2)
            k = min(c1, 16)
            assert (np.diff(t1[:k]) >= 0).all() and (t1[k:] == np.float32(1e16)).all()
            n_full += c1 >= 16
            n_tied += int((np.diff(t1[:k]) == 0).sum())
        if name == "ties":
            assert n_tied > 0 and n_full > 0  # the case the rule exists for is exercised
