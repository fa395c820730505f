"""The BASELINE configurations at their real sizes, forward AND backward, against the CPU oracle on the same
seeded inputs: per-ray outputs bit-identical, every gradient tensor element-wise within 1e-3 relative
(helpers.assert_gradients: assert_close_sum / assert_close_rays with their floor and rounding-noise allowance).  The oracle runs on the host cores of the GPU box
(OpenMP); each test prints how long it took."""
import time

import numpy as np
import pytest
import torch

import dst_scenes as S
from helpers import (GRAD_REL, assert_close_sum, assert_forward_exact, assert_gradients, assert_same_sums, gpu_trace,
                     oracle_scene, upstream)

pytestmark = pytest.mark.gpu


def compare_all(oracle, tracer, scene, o, d, ug, wet_rel=1e-4, tag="", **kw):
    """Forward + backward on both sides, everything compared; returns (ref, out)."""
    t0 = time.time()
    out, g = gpu_trace(tracer, scene, o, d, upstream=ug, **kw)
    t1 = time.time()
    trace_kw = {k: v for k, v in kw.items() if k not in ("rebuild", "build")}
    s = oracle_scene(oracle, scene, o, d, **trace_kw)
    ref = oracle.forward(s, oracle.HITS_BVH_LEXI)
    ugn = {k: v.numpy() for k, v in ug.items()}
    refg = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI)
    refg64 = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI, noise=True)
    t2 = time.time()
    print("%s gpu %.1f s, oracle %.1f s, %.1f composited hits per ray" % (tag, t1 - t0, t2 - t1, ref["n_con"].mean()),
          flush=True)
    assert_forward_exact(out, ref)
    assert_close_sum(out["wet"], ref["wet"], wet_rel, "wet")
    assert_gradients(g, refg, refg64, GRAD_REL, tag)
    return ref, out


def test_config3_room_1M_surfels_1080p_forward_and_backward(oracle, tracer):
    """BASELINE config 3, the configuration the headline number is quoted on: 1M surfels, 1920x1080, SH degree 3,
    depth 0.  The whole image, every output and every gradient tensor."""
    sc = S.scene_room(P=1000000, seed=0)
    o, d = S.rays_room(1080, 1920)
    ref, _ = compare_all(oracle, tracer, sc, o, d, upstream(1080, 1920, 2), tag="config3 ")
    assert ref["n_con"].mean() > 20 and ref["n_proc"].max() > 64


def test_config2_sphere_100k_800x800_build_once_then_refit(oracle, tracer):
    """BASELINE config 2: 100k surfels on a sphere, 800x800 orbit views, SH3, forward + backward; the structure
    is built for the first view and refitted (rebuild=False) for the others."""
    sc = S.scene_sphere(P=100000, seed=0)
    ug = upstream(800, 800, 2)
    for view in range(5):
        o, d = S.rays_sphere(800, 800, view=view)
        ref, _ = compare_all(oracle, tracer, sc, o, d, ug, rebuild=(view == 0), tag="config2 view %d " % view)
        assert ref["acc"].mean() > 0.2
    info = tracer.optix_context.accel_info()
    assert info.n_surfels == 100000


def test_config5_lidar_refit_loop_20_frames(oracle, tracer):
    """BASELINE config 5's sequence of 20 refits at a tenth of its size (200k surfels, 64 beams x 256 azimuths as a (1,N,3) ray list, 4 aux
    channels): 20 frames of perturb 10 % of the means -> refit -> forward + backward, each frame against the oracle
    (which builds its own BVH from the frame's quads)."""
    sc = S.scene_lidar(P=200000, seed=0, aux=4)
    o, d = S.rays_lidar(beams=64, azimuths=256)
    ug = upstream(o.shape[0], o.shape[1], 4)
    gpu_trace(tracer, sc, o, d)                     # build on the unperturbed scene
    builds = tracer.optix_context.accel_info().builds
    frame_sc = sc
    for frame in range(1, 21):
        frame_sc = S.perturb_means(frame_sc, frame)   # the perturbations accumulate, as in a running sequence
        compare_all(oracle, tracer, frame_sc, o, d, ug, rebuild=False, tag="config5 frame %d " % frame)
    info = tracer.optix_context.accel_info()
    assert info.builds == builds and info.refits >= 20


def test_config5_lidar_full_size_perturb_and_refit(oracle, tracer):
    """BASELINE config 5 at its real size: 2,000,000 surfels, 64 beams x 2048 azimuths as a (1,131072,3) ray list,
    4 aux channels; build, then three frames of perturb 10 % of the means -> refit -> forward + backward, each frame
    against the oracle (about 9 composited hits per ray here; the tenth-size loop above has less than one)."""
    sc = S.scene_lidar(P=2000000, seed=0, aux=4)
    o, d = S.rays_lidar()
    assert o.shape == (1, 131072, 3)
    ug = upstream(o.shape[0], o.shape[1], 4)
    ref, _ = compare_all(oracle, tracer, sc, o, d, ug, rebuild=True, tag="config5 full, built ")
    assert ref["n_con"].mean() > 5
    builds = tracer.optix_context.accel_info().builds
    frame_sc = sc
    for frame in range(1, 4):
        frame_sc = S.perturb_means(frame_sc, frame)
        compare_all(oracle, tracer, frame_sc, o, d, ug, rebuild=False, tag="config5 full, frame %d " % frame)
    info = tracer.optix_context.accel_info()
    assert info.builds == builds and info.refits >= 3 and info.n_surfels == 2000000


def test_config4_room_500k_720p_depth2_forward_and_backward(oracle, tracer):
    """BASELINE config 4: 500k surfels, 1280x720, 8 aux channels, max_trace_depth 2, specular_threshold 0.1,
    forward + backward through all bounces, whole image."""
    sc = S.scene_room(P=500000, seed=0, aux=8)
    o, d = S.rays_room(720, 1280)
    ref, out = compare_all(oracle, tracer, sc, o, d, upstream(720, 1280, 8), tag="config4 ", max_trace_depth=2,
                           specular_threshold=0.1)
    slots = ref["mid"].reshape(720, 1280, 3, 22)
    assert (np.abs(slots[:, :, 2, 3:6]).sum(-1) > 0).mean() > 0.3     # the third bounce is traced for many rays
    acc = out["acc"].astype(np.float64)
    assert (acc >= 0).all() and (acc <= 1).all()


@pytest.mark.parametrize("P,H,W,depth,aux", [(1000000, 2160, 3840, 0, 0), (300000, 1080, 1920, 2, 8)])
def test_a_larger_image_equals_its_quadrants_traced_on_their_own(tracer, P, H, W, depth, aux):
    """A size the oracle cannot reach in seconds (8.3M rays), held against a property that does not depend on size:
    no per-ray result depends on which rays share a wave, an image or a launch, so the image and its four quadrants
    must agree bit for bit in every per-ray output, and the quadrants' per-surfel gradients must add up to the image's."""
    sc = S.scene_room(P=P, seed=3, aux=aux)
    kw = {}
    if depth:
        sc["others_precomp"][:, 0] = sc["others_precomp"][:, 0] * 0.8 + 0.1
        kw = dict(max_trace_depth=depth, specular_threshold=0.1)
    o, d = S.rays_room(H, W)
    ug = upstream(H, W, max(aux, 2))
    full, gfull = gpu_trace(tracer, sc, o, d, upstream=ug, **kw)
    assert np.isfinite(full["rgb"]).all() and full["acc"].mean() > 0.5
    hh, hw = H // 2, W // 2
    total = None
    for r0, c0 in ((0, 0), (0, hw), (hh, 0), (hh, hw)):
        sl = (slice(r0, r0 + hh), slice(c0, c0 + hw))
        part, gpart = gpu_trace(tracer, sc, o[sl].contiguous(), d[sl].contiguous(),
                                upstream={k: v[sl].contiguous() for k, v in ug.items()}, build=False, **kw)
        for k in ("rgb", "dpt", "acc", "norm", "aux", "mid"):
            a = np.ascontiguousarray(full[k].reshape(H, W, -1)[sl])
            assert np.array_equal(a.view(np.uint32), part[k].reshape(hh, hw, -1).view(np.uint32)), (k, r0, c0)
        for k in ("ray_o", "ray_d"):
            a, b = gfull[k][sl], gpart[k]
            assert np.abs(a - b).max() <= 1e-5 * np.abs(b).max(), k
        rest = {k: v.astype(np.float64) for k, v in gpart.items() if v is not None and k not in ("ray_o", "ray_d")}
        total = rest if total is None else {k: total[k] + rest[k] for k in total}
    for k, v in total.items():
        assert_same_sums(gfull[k], v, GRAD_REL, k)
