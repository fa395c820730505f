"""Structure of the HIP-built LBVH (downloaded through the C ABI) and the error paths of the boundary."""
import ctypes as C

import numpy as np
import pytest
import torch

import dst_scenes as S

pytestmark = pytest.mark.gpu

LEAF = 0x80000000

NODE = np.dtype([("lo0", "<f4", 3), ("hi0", "<f4", 3), ("lo1", "<f4", 3), ("hi1", "<f4", 3), ("c0", "<u4"),
                 ("c1", "<u4"), ("first", "<u4"), ("last", "<u4")])
LEAFT = np.dtype([("A", "<f4", 3), ("AB", "<f4", 3), ("AC", "<f4", 3), ("AD", "<f4", 3), ("n1", "<f4", 3),
                  ("g", "<u4"), ("n0", "<f4", 3), ("n2", "<f4", 3), ("c1", "<f4"), ("pad", "<u4")])


def download(tracer):
    import diff_surfel_tracing._C as binding
    ctx = tracer.optix_context
    info = ctx.accel_info()
    assert info.node_bytes == NODE.itemsize == 64 and info.leaf_bytes == LEAFT.itemsize == 96
    n = info.n_surfels
    nodes = np.zeros(max(n - 1, 1), NODE)
    leaves = np.zeros(n, LEAFT)
    npar, lpar, keys = np.zeros(max(n - 1, 1), np.uint32), np.zeros(n, np.uint32), np.zeros(n, np.uint32)
    rc = binding.load_library().dst_accel_download(
        ctx.handle, nodes.ctypes.data, leaves.ctypes.data, npar.ctypes.data, lpar.ctypes.data, keys.ctypes.data,
        C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    return info, nodes[: n - 1], leaves, npar[: n - 1], lpar, keys


def own_tracer(hierarchy):
    """A tracer of its own whose builds make the hierarchy by agglomeration (the default) or read it off the Morton
    codes (`DST_HIERARCHY=morton` in the environment when the context is created)."""
    import os

    import diff_surfel_tracing as dst
    saved = os.environ.get("DST_HIERARCHY")
    try:
        if hierarchy == "morton":
            os.environ["DST_HIERARCHY"] = "morton"
        else:
            os.environ.pop("DST_HIERARCHY", None)
        return dst.SurfelTracer()
    finally:
        if saved is None:
            os.environ.pop("DST_HIERARCHY", None)
        else:
            os.environ["DST_HIERARCHY"] = saved


def check_tree(info, nodes, leaves, npar, lpar, keys, vertices):
    n = info.n_surfels
    assert (np.diff(keys.astype(np.int64)) >= 0).all()                 # the sort's result: Morton codes ascending
    for i in range(n - 1):                                             # a node's leaves are consecutive; the numbering
        f, l, c0, c1 = (int(nodes[k][i]) for k in ("first", "last", "c0", "c1"))   # of its children follows from them
        split = c0 & ~LEAF
        assert f <= split < l and (c1 & ~LEAF) == split + 1
        assert bool(c0 & LEAF) == (split == f) and bool(c1 & LEAF) == (split + 1 == l)
    assert sorted(leaves["g"].tolist()) == list(range(n))              # every surfel exactly once
    V = vertices.reshape(n, 4, 3)
    corners = {name: V[leaves["g"], k] for name, k in (("A", 0), ("B", 1), ("C", 2), ("D", 3))}
    np.testing.assert_array_equal(leaves["A"], corners["A"])           # corner A and the edge vectors from it, as
    with np.errstate(invalid="ignore"):                                # the fp32 differences of the corners
        for name, k in (("AB", "B"), ("AC", "C"), ("AD", "D")):
            np.testing.assert_array_equal(leaves[name], corners[k] - corners["A"])
    A, B, C, D = (corners[c].astype(np.float64) for c in "ABCD")
    with np.errstate(invalid="ignore"):
        np.testing.assert_allclose(leaves["n0"], np.cross(B - A, C - A), rtol=1e-4, atol=1e-7)   # plane normals
        np.testing.assert_allclose(leaves["n1"], np.cross(C - B, D - B), rtol=1e-4, atol=1e-7)
        np.testing.assert_allclose(leaves["n2"], np.cross(C - A, D - A), rtol=1e-4, atol=1e-7)
        n1 = np.cross(C - B, D - B)                                    # (c1 = n1.AB is all cancellation on a flat quad)
        scale = np.linalg.norm(n1, axis=1) * np.linalg.norm(B - A, axis=1)
        ok = np.isfinite(scale)
        assert (np.abs(leaves["c1"] - (n1 * (B - A)).sum(1))[ok] <= 1e-5 * scale[ok] + 1e-30).all()
    # a leaf's box: its corners, widened by 4e-6 of the quad's largest coordinate (the quad's share of the slack the
    # box tests need; computed in fp32 like the kernel does)
    with np.errstate(invalid="ignore"):
        mag = np.zeros(n, np.float32)
        for c in "ABCD":
            a = np.abs(corners[c])
            mag = np.maximum(mag, np.where(np.isfinite(a), a, np.float32(0)).max(1))
    pad = (np.float32(4e-6) * mag)[:, None]
    llo = np.minimum.reduce([corners[c] for c in "ABCD"]) - pad
    lhi = np.maximum.reduce([corners[c] for c in "ABCD"]) + pad
    assert llo.dtype == np.float32 and lhi.dtype == np.float32
    # walk from the root: every node and leaf reached once, parents consistent, boxes = exact union of content
    seen_nodes, seen_leaves = np.zeros(n - 1, bool), np.zeros(n, bool)
    box_lo, box_hi = {}, {}
    stack, order, depth, maxdepth = [(0, 0)], [], {}, 0
    while stack:
        i, dep = stack.pop()
        assert not seen_nodes[i]
        seen_nodes[i] = True
        order.append(i)
        maxdepth = max(maxdepth, dep)
        for which, c in enumerate((int(nodes["c0"][i]), int(nodes["c1"][i]))):
            if c & LEAF:
                j = c & ~LEAF
                assert not seen_leaves[j] and lpar[j] == ((i << 1) | which)
                seen_leaves[j] = True
            else:
                assert npar[c] == ((i << 1) | which)
                stack.append((c, dep + 1))
    assert seen_nodes.all() and seen_leaves.all() and npar[0] == 0xFFFFFFFF
    assert maxdepth < 62                                                 # the traversal stack holds 64 entries
    for i in reversed(order):
        los, his = [], []
        for c in (int(nodes["c0"][i]), int(nodes["c1"][i])):
            if c & LEAF:
                los.append(llo[c & ~LEAF]); his.append(lhi[c & ~LEAF])
            else:
                los.append(box_lo[c]); his.append(box_hi[c])
        np.testing.assert_array_equal(nodes["lo0"][i], los[0]); np.testing.assert_array_equal(nodes["hi0"][i], his[0])
        np.testing.assert_array_equal(nodes["lo1"][i], los[1]); np.testing.assert_array_equal(nodes["hi1"][i], his[1])
        box_lo[i], box_hi[i] = np.minimum(los[0], los[1]), np.maximum(his[0], his[1])
    return maxdepth


@pytest.mark.parametrize("hierarchy", ["agglomerated", "morton"])
@pytest.mark.parametrize("maker,P", [(S.scene_cube, 5000), (S.scene_room, 20000), (S.scene_cube, 2), (S.scene_cube, 1025),
                                     (S.scene_cube, 64), (S.scene_room, 3333)])
def test_tree_invariants_after_build_and_refit(maker, P, hierarchy):
    tracer = own_tracer(hierarchy)
    sc = maker(P=P, seed=1)
    v, f = sc["vertices"].cuda(), sc["faces"].cuda()
    tracer.build_acceleration_structure(v, f, True)
    info, *arrs = download(tracer)
    assert info.n_surfels == P and info.n_internal == P - 1
    cen = 0.5 * (sc["vertices"].reshape(P, 4, 3).amin(1) + sc["vertices"].reshape(P, 4, 3).amax(1)).numpy()
    np.testing.assert_allclose(list(info.scene_lo), cen.min(0), rtol=0, atol=0)
    np.testing.assert_allclose(list(info.scene_hi), cen.max(0), rtol=0, atol=0)
    assert info.max_abs == float(sc["vertices"].abs().max())
    assert info.agglomerated == int(hierarchy == "agglomerated" and P >= 64)
    depth = check_tree(info, *arrs, sc["vertices"].numpy())
    assert info.depth == (depth + 1 if info.agglomerated else 0)       # nodes above the deepest leaf
    moved = S.perturb_means(sc, 1, frac=0.5, sigma=0.2)
    tracer.build_acceleration_structure(moved["vertices"].cuda(), f, False)
    info2, *arrs2 = download(tracer)
    np.testing.assert_array_equal(arrs2[1]["g"], arrs[1]["g"])           # refit keeps the leaf order and topology
    np.testing.assert_array_equal(arrs2[0]["c0"], arrs[0]["c0"])
    check_tree(info2, *arrs2, moved["vertices"].numpy())
    assert info2.refits >= 1


@pytest.mark.parametrize("hierarchy", ["agglomerated", "morton"])
def test_duplicate_positions_give_a_bounded_tree(hierarchy):
    """All centroids in one Morton cell: the Morton hierarchy falls back to index bits and stays balanced; the
    agglomeration pairs the quads by their boxes whatever their order."""
    tracer = own_tracer(hierarchy)
    P = 4096
    sc = S.scene_cube(P=P, seed=2)
    sc["means3D"] = torch.zeros(P, 3)
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    tracer.build_acceleration_structure(sc["vertices"].cuda(), sc["faces"].cuda(), True)
    info, *arrs = download(tracer)
    depth = check_tree(info, *arrs, sc["vertices"].numpy())
    assert depth <= 44   # 30 key bits + 12 index bits


def test_identical_quads_pair_up(tracer):
    """20000 copies of one surfel (and a few others): every union has the same surface, and the agglomeration's order
    on equal pairs must still merge half of them per round and end in a hierarchy a dozen or so levels deep."""
    P = 20000
    sc = S.scene_cube(P=P, seed=3)
    for k in ("means3D", "scales", "rotations"):
        sc[k][:P - 50] = sc[k][0]
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    own = own_tracer("agglomerated")
    own.build_acceleration_structure(sc["vertices"].cuda(), sc["faces"].cuda(), True)
    info, *arrs = download(own)
    assert info.agglomerated == 1
    assert check_tree(info, *arrs, sc["vertices"].numpy()) <= 24


def _with_far_surfels(sc, factor, k=5, seed=4):
    """`k` surfels of the scene moved `factor` scene radii away (and grown by as much)."""
    out = {n: t.clone() for n, t in sc.items()}
    gen = torch.Generator().manual_seed(seed)
    dirs = torch.nn.functional.normalize(torch.randn(k, 3, generator=gen), dim=-1)
    out["means3D"][:k] = dirs * factor * float(sc["means3D"].abs().max())
    out["scales"][:k] = sc["scales"][:k] * factor
    out["vertices"], out["faces"] = S.get_triangles(out["means3D"], out["scales"], out["rotations"])
    return out


@pytest.mark.parametrize("hierarchy", ["agglomerated", "morton"])
def test_surfels_far_outside_a_compact_scene_switch_the_builds_to_two_level_keys(hierarchy):
    """A few surfels 2000 scene radii away stretch the 1024^3 Morton grid until the scene itself fills one cell: the
    build notices (nearly all neighbours in Morton order share their cell), builds again with 60-bit keys in two
    levels and keeps them for the context's later builds.  The structure obeys the same invariants either way."""
    own = own_tracer(hierarchy)
    sc = S.scene_cube(P=20000, seed=8)
    own.build_acceleration_structure(sc["vertices"].cuda(), sc["faces"].cuda(), True)
    info, *arrs = download(own)
    assert info.key_levels == 1 and info.builds == 1
    flat_depth = check_tree(info, *arrs, sc["vertices"].numpy())
    far = _with_far_surfels(sc, 2000.0)
    own.build_acceleration_structure(far["vertices"].cuda(), far["faces"].cuda(), True)
    info, *arrs = download(own)
    assert info.key_levels == 2 and info.builds == 2     # the abandoned one-level build is not counted
    depth = check_tree(info, *arrs, far["vertices"].numpy())
    assert depth <= flat_depth + 12                       # the scene's own levels, and a few for the far surfels
    # refit on the two-level structure, then a rebuild of the compact scene: still two levels
    moved = S.perturb_means(far, 1, frac=0.5, sigma=0.2)
    own.build_acceleration_structure(moved["vertices"].cuda(), far["faces"].cuda(), False)
    info, *arrs = download(own)
    check_tree(info, *arrs, moved["vertices"].numpy())
    own.build_acceleration_structure(sc["vertices"].cuda(), sc["faces"].cuda(), True)
    info, *arrs = download(own)
    assert info.key_levels == 2
    assert check_tree(info, *arrs, sc["vertices"].numpy()) <= flat_depth + 2


def test_two_level_keys_are_given_up_when_the_hierarchy_gets_too_deep():
    """Sixty surfels that each peel one bit off the 60-bit key (one per axis and scale, down to a millionth of the
    extent) in front of 16384 surfels at one point, and a uniform cloud that keeps the box of the keys at full
    size: with two-level keys the deepest leaf lies 74 nodes down, more than the walks' stacks are sized for.  The
    build measures that and returns to one-level keys for good.  (Hierarchies read off the Morton codes: an agglomerated
    one does not follow the key bits down.)"""
    own = own_tracer("morton")
    pts = [[0.0, 0.0, 0.0]] * 16384
    pts += (torch.rand(4096, 3, generator=torch.Generator().manual_seed(3)) * 1.2).tolist()
    for k in range(20):
        for a in range(3):
            p = [0.0, 0.0, 0.0]
            p[a] = 1.2 * 2.0 ** -k
            pts.append(p)
    P = len(pts)
    sc = S.scene_cube(P=P, seed=5)
    sc["means3D"] = torch.tensor(pts, dtype=torch.float32)
    sc["scales"] = torch.full((P, 2), 1e-8)
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    own.build_acceleration_structure(sc["vertices"].cuda(), sc["faces"].cuda(), True)
    info, *arrs = download(own)
    assert info.key_levels == 1 and info.builds == 1
    depth = check_tree(info, *arrs, sc["vertices"].numpy())
    assert 40 <= depth < 62        # thirty peeled bits, then the 16384 + 30 surfels of the last cell
    # the refusal holds: a scene that asks for two levels again is built with one
    far = _with_far_surfels(S.scene_cube(P=3000, seed=8), 2000.0)
    own.build_acceleration_structure(far["vertices"].cuda(), far["faces"].cuda(), True)
    assert own.optix_context.accel_info().key_levels == 1
    # ... but not for ever: the sixteenth build after it tries the finer keys again (and keeps them for this scene)
    for _ in range(15):
        own.build_acceleration_structure(far["vertices"].cuda(), far["faces"].cuda(), True)
    assert own.optix_context.accel_info().key_levels == 2


def test_boundary_errors(tracer):
    import diff_surfel_tracing as dst
    sc = S.scene_cube(P=100, seed=0)
    v, f = sc["vertices"].cuda(), sc["faces"].cuda()
    fresh = dst.SurfelTracer()
    with pytest.raises(RuntimeError, match="before any build"):
        fresh.build_acceleration_structure(v, f, False)
    bad = f.clone()
    bad[3, 0] = 0                                                        # second triangle no longer shares the edge
    with pytest.raises(RuntimeError, match="pairs"):
        fresh.build_acceleration_structure(v, bad, True)
    bad = f.clone()
    bad[0, 2] = 4 * 100 + 7                                              # vertex id out of range
    with pytest.raises(RuntimeError, match="pairs"):
        fresh.build_acceleration_structure(v, bad, True)
    with pytest.raises(RuntimeError, match="2 \\* num_surfels"):
        fresh.build_acceleration_structure(v, f[:-1], True)
    fresh.build_acceleration_structure(v, f, True)
    with pytest.raises(RuntimeError, match="different number of surfels"):
        fresh.build_acceleration_structure(v[:-4], f[:-2], False)
    # tracing with another surfel count than the structure holds
    from helpers import gpu_trace
    o, d = S.rays_cube(8, 8)
    other = S.scene_cube(P=50, seed=0)
    with pytest.raises(RuntimeError, match="differs from the acceleration structure"):
        gpu_trace(fresh, other, o, d, build=False)
    with pytest.raises(RuntimeError, match="mtd_alloc|max_trace_depth"):
        gpu_trace(fresh, sc, o, d, build=False, max_trace_depth=4)
    wide = S.scene_cube(P=100, seed=0, aux=9)
    with pytest.raises(RuntimeError, match="aux channels"):
        gpu_trace(fresh, wide, o, d, build=False)
    # a failed call leaves the context usable
    out, _ = gpu_trace(fresh, sc, o, d, build=False)
    assert np.isfinite(out["rgb"]).all()
