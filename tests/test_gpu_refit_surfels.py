"""Refit straight from the surfel parameters (dst_refit_from_surfels): the corners it generates are the 2DGS quads
in a stated fp32 operation order (bit-equal to that statement, a few ulps from dst_scenes.get_triangles, whose
quaternion norm is a library reduction), the refitted structure equals one built from those corners, and traces
on it equal the oracle's."""
import numpy as np
import pytest
import torch

import dst_scenes as S
from helpers import assert_forward_exact, gpu_trace, oracle_scene
from test_gpu_lbvh import check_tree, download

pytestmark = pytest.mark.gpu


def corners_as_stated(means, scales, quats):
    """include/dst_api.h, dst_refit_from_surfels: every operation in fp32, rounded once, in this order."""
    f = np.float32
    m, s, q = (np.ascontiguousarray(a, dtype=f) for a in (means, scales, quats))
    q0, q1, q2, q3 = q[:, 0], q[:, 1], q[:, 2], q[:, 3]
    nrm = np.sqrt(((q0 * q0 + q1 * q1) + q2 * q2) + q3 * q3)
    w, x, y, z = q0 / nrm, q1 / nrm, q2 / nrm, q3 / nrm
    one, two = f(1), f(2)
    u = np.stack([(one - two * (y * y + z * z)), (two * (x * y + w * z)), (two * (x * z - w * y))], -1) * s[:, 0:1]
    v = np.stack([(two * (x * y - w * z)), (one - two * (x * x + z * z)), (two * (y * z + w * x))], -1) * s[:, 1:2]
    out = np.empty((m.shape[0], 4, 3), f)
    for k, (a, b) in enumerate(((-3, 3), (-3, -3), (3, 3), (3, -3))):
        out[:, k] = (m + f(a) * u) + f(b) * v
    assert out.dtype == f
    return out.reshape(-1, 3)


def test_refit_from_surfels_equals_the_stated_quads_a_rebuild_and_the_oracle(oracle, tracer):
    sc = S.scene_lidar(P=30000, seed=5, aux=4)
    o, d = S.rays_lidar(beams=16, azimuths=128)
    gpu_trace(tracer, sc, o, d)                                   # build from get_triangles quads
    for frame in (1, 2):
        moved = S.perturb_means(sc, frame)
        moved["scales"] = moved["scales"] * (1.0 + 0.1 * frame)    # scales and rotations change too
        moved["rotations"] = moved["rotations"] + 0.05 * frame * torch.roll(moved["rotations"], 1, dims=1)
        dev = {k: moved[k].cuda() for k in ("means3D", "scales", "rotations")}
        v_out = tracer.refit_from_surfels(dev["means3D"], dev["scales"], dev["rotations"])
        torch.cuda.synchronize()
        want = corners_as_stated(moved["means3D"].numpy(), moved["scales"].numpy(), moved["rotations"].numpy())
        np.testing.assert_array_equal(v_out.cpu().numpy().view(np.uint32), want.view(np.uint32))
        ref_v, ref_f = S.get_triangles(moved["means3D"], moved["scales"], moved["rotations"])
        np.testing.assert_allclose(want, ref_v.numpy(), rtol=2e-6, atol=1e-6)
        # the refitted structure: leaves hold exactly these corners, boxes are exact unions
        tree = download(tracer)
        check_tree(*tree, want)
        snap_refit = (tree[1].copy(), tree[2].copy())
        # traces on it equal the oracle's on the same quads
        geo = dict(moved)
        geo["vertices"], geo["faces"] = torch.from_numpy(want.copy()), ref_f
        out, _ = gpu_trace(tracer, geo, o, d, build=False)
        ref = oracle.forward(oracle_scene(oracle, geo, o, d), oracle.HITS_BVH_LEXI)
        assert_forward_exact(out, ref)
        # and a refit from those vertices gives the same structure bit for bit
        tracer.build_acceleration_structure(geo["vertices"].cuda(), geo["faces"].cuda(), False)
        tree2 = download(tracer)
        for a, b in zip(snap_refit, (tree2[1], tree2[2])):
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    info = tracer.optix_context.accel_info()
    assert info.builds >= 1 and info.refits >= 4


def test_refit_from_surfels_needs_canonical_quads_and_matching_sizes(tracer):
    sc = S.scene_cube(P=500, seed=3)
    v, f = sc["vertices"].cuda(), sc["faces"].cuda()
    P = 500
    tracer.build_acceleration_structure(v, f, True)
    args = [sc[k].cuda() for k in ("means3D", "scales", "rotations")]
    with pytest.raises(RuntimeError, match="different number of surfels"):
        tracer.refit_from_surfels(args[0][:-1], args[1][:-1], args[2][:-1])
    # the same quads listed in another order are a valid build, but not one this refit can keep in step with
    perm = torch.arange(P - 1, -1, -1)
    f_rev = f.reshape(P, 2, 3)[perm.cuda()].reshape(-1, 3).contiguous()
    tracer.build_acceleration_structure(v, f_rev, True)
    with pytest.raises(RuntimeError, match="rows 4g"):
        tracer.refit_from_surfels(*args)
    tracer.build_acceleration_structure(v, f, True)
    out = tracer.refit_from_surfels(*args)
    assert out.shape == (4 * P, 3)
