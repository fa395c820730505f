"""Parity of the HIP path (through the public API and the C ABI underneath) with the CPU oracle on the
same seeded inputs.  Bar: per-ray forward outputs bit-identical (both sides run the same sequence of
unfused fp32 operations; the north star asks for 1e-4 absolute); atomically accumulated sums and all
gradients element-wise within 1e-3 relative (north star: 1e-3 relative) plus a floor for sums that cancel
(helpers.assert_close_sum / assert_close_rays)."""
import numpy as np
import pytest
import torch

import dst_scenes as S
from helpers import (GRAD_REL, assert_close_sum, assert_forward_exact, assert_gradients, gpu_trace, oracle_scene,
                     to_numpy, upstream)

pytestmark = pytest.mark.gpu


def check_case(oracle, tracer, scene, ray_o, ray_d, acc_grad=True, grads=True, skip=(), **kw):
    """Forward + backward on both sides and compare everything (but the gradient tensors named in `skip`)."""
    H, W = ray_o.shape[:2]
    s = oracle_scene(oracle, scene, ray_o, ray_d, **kw)
    ref = oracle.forward(s, oracle.HITS_BVH_LEXI)
    ug = upstream(H, W, s.aux, acc=acc_grad) if grads else None
    out, g = gpu_trace(tracer, scene, ray_o, ray_d, upstream=ug, **kw)
    assert_forward_exact(out, ref)
    assert_close_sum(out["wet"], ref["wet"], 1e-5, "wet")
    if grads:
        ugn = {k: v.numpy() for k, v in ug.items()}
        refg = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI)
        refg64 = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI, noise=True)
        assert_gradients(g, {k: v for k, v in refg.items() if k not in skip}, refg64, GRAD_REL)
        ref["grads_gpu"], ref["grads_ref"], ref["grads_noise"] = g, refg, refg64["noise"]
    return ref, out


def test_config1_cube_sh3(oracle, tracer):
    """BASELINE config 1: 10k surfels in [-1,1]^3, 128x128 pinhole at distance 3, SH degree 3, depth 0."""
    sc = S.scene_cube(P=10000, seed=0)
    ref, _ = check_case(oracle, tracer, sc, *S.rays_cube(128, 128))
    assert ref["n_con"].max() > 16 and ref["n_proc"].mean() > 10  # several chunks per ray are exercised


def test_config1_background_one(oracle, tracer):
    sc = S.scene_cube(P=10000, seed=0)
    check_case(oracle, tracer, sc, *S.rays_cube(128, 128, view=1), bg=(1.0, 1.0, 1.0))


@pytest.mark.parametrize("aux", [2, 4, 8])
def test_precomputed_colours_and_aux_channels(oracle, tracer, aux):
    sc = S.scene_cube(P=4000, seed=10 + aux, colors=True, aux=aux)
    check_case(oracle, tracer, sc, *S.rays_cube(48, 56, view=2), bg=(0.2, 0.4, 0.6), start_from_first=False)


@pytest.mark.parametrize("deg", [0, 1, 2])
def test_lower_sh_degrees(oracle, tracer, deg):
    sc = S.scene_cube(P=3000, seed=20 + deg)
    check_case(oracle, tracer, sc, *S.rays_cube(40, 40), sh_degree=deg)


def test_evaluation_mode_returns_zero_weights(oracle, tracer):
    sc = S.scene_cube(P=1000, seed=3)
    o, d = S.rays_cube(16, 16)
    out, _ = gpu_trace(tracer, sc, o, d, training=False)
    assert out["wet"].shape == (1000,) and (out["wet"] == 0).all()
    ref = oracle.forward(oracle_scene(oracle, sc, o, d), oracle.HITS_BVH_LEXI)
    assert_forward_exact(out, ref)


@pytest.mark.parametrize("depth,thr", [(1, 0.1), (2, 0.1), (2, 0.45), (3, 0.0)])
def test_multi_bounce(oracle, tracer, depth, thr):
    """Config-4 style: reflection rays above specular_threshold, forward and backward through all bounces."""
    sc = S.scene_room(P=30000, seed=depth, aux=8, half=1.5)
    sc["others_precomp"][:, 0] = sc["others_precomp"][:, 0] * 0.8 + 0.1   # specular away from 0 (reference divides by it)
    o, d = S.pinhole_rays(40, 64, 70.0, (-0.6, -0.3, 0.15), (0.9, 0.45, -0.15))
    ref, _ = check_case(oracle, tracer, sc, o, d, max_trace_depth=depth, specular_threshold=thr)
    slots = ref["mid"].reshape(40, 64, -1, 22)
    assert slots.shape[2] == max(depth, 1) + 1
    reached = (np.abs(slots[:, :, depth, 3:6]).sum(-1) > 0).mean()
    assert 0.05 < reached  # the deepest bounce is really traced for a good share of the rays


def test_thin_ray_lists(oracle, tracer):
    """(B,P,3) layout with B=1 (config 5's LiDAR rays) and with B=3."""
    sc = S.scene_lidar(P=20000, seed=1, aux=4)
    o, d = S.rays_lidar(beams=8, azimuths=256)
    check_case(oracle, tracer, sc, o, d)
    o3, d3 = o.reshape(8, 256, 3)[:3].contiguous(), d.reshape(8, 256, 3)[:3].contiguous()
    check_case(oracle, tracer, sc, o3, d3, grads=False)


def test_unrelated_rays_as_image_and_as_list(oracle, tracer):
    """Random origins and directions (nothing for a packet to share): as an image-shaped grid the packet kernels
    walk one direction-sign class at a time, as a ray list the per-lane walk takes over; both must equal the oracle
    bit for bit, and hence each other."""
    sc = S.scene_cube(P=6000, seed=77)
    gen = torch.Generator().manual_seed(78)
    n = 24 * 40
    o = (torch.rand(n, 3, generator=gen) * 2 - 1) * 1.5
    d = torch.nn.functional.normalize(torch.randn(n, 3, generator=gen), dim=-1)
    _, a = check_case(oracle, tracer, sc, o.reshape(24, 40, 3).contiguous(), d.reshape(24, 40, 3).contiguous())
    _, b = check_case(oracle, tracer, sc, o.reshape(1, n, 3).contiguous(), d.reshape(1, n, 3).contiguous())
    for k in ("rgb", "dpt", "acc", "norm"):
        assert np.array_equal(a[k].reshape(n, -1).view(np.uint32), b[k].reshape(n, -1).view(np.uint32)), k


def test_ragged_image_sizes(oracle, tracer):
    sc = S.scene_cube(P=2000, seed=5)
    for H, W in ((37, 53), (1, 1), (9, 7), (64, 1)):
        check_case(oracle, tracer, sc, *S.rays_cube(H, W))


def test_many_image_sizes_through_one_context(oracle):
    """Training at changing resolutions: every backward call hands its hit record back to the context's pool, which
    then holds storages of many sizes and drops the smallest ones."""
    import diff_surfel_tracing as dst
    own = dst.SurfelTracer()
    sc = S.scene_cube(P=1500, seed=6)
    for H, W in ((8, 8), (40, 24), (16, 16), (72, 64), (24, 8), (56, 56), (8, 16), (32, 32), (64, 72)):
        check_case(oracle, own, sc, *S.rays_cube(H, W, view=H % 3))
    assert 1 <= len(own.optix_context._record_pool) <= own.optix_context.RECORD_POOL_SIZE


def test_surfels_far_outside_the_scene(oracle):
    """Far surfels (some of them large and in view behind the scene) make the build go over to two-level Morton keys
    and widen the padding of the box tests (it scales with the largest coordinate): results stay the oracle's."""
    import diff_surfel_tracing as dst
    from test_gpu_lbvh import _with_far_surfels
    own = dst.SurfelTracer()
    sc = _with_far_surfels(S.scene_cube(P=8000, seed=12, aux=2), 1500.0, k=6)
    o, d = S.rays_cube(40, 48, view=1)
    # two more far surfels straight behind the scene, facing the camera, so that rays reach them
    back = -o[0, 0] / o[0, 0].norm()
    for k, dist in ((6, 40.0), (7, 900.0)):
        sc["means3D"][k] = back * dist
        sc["scales"][k] = torch.tensor([0.1, 0.1]) * dist
    nrm = (-back).expand(2, 3).clone()
    from dst_scenes import _quat_from_normal
    sc["rotations"][6:8] = _quat_from_normal(nrm, torch.Generator().manual_seed(0))
    sc["opacities"][6:8] = 0.9
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    ref, _ = check_case(oracle, own, sc, o, d, bg=(0.1, 0.2, 0.3))
    assert own.optix_context.accel_info().key_levels == 2
    assert ref["wet"][6] > 0 and ref["wet"][7] > 0     # both far surfels are seen


def test_surfels_with_nan_and_infinite_parameters(oracle, tracer):
    """A diverged optimisation leaves NaN and infinite means, scales and zero quaternions behind: such surfels are hit
    by nothing, take no part in the grid's extent or the coordinate bound, and the others render as the oracle's."""
    sc = S.scene_cube(P=6000, seed=31, aux=2)
    r = torch.rand(6000, generator=torch.Generator().manual_seed(32))
    sc["means3D"][r < 0.02, 0] = float("nan")
    sc["means3D"][(r >= 0.02) & (r < 0.04), 1] = float("inf")
    sc["means3D"][(r >= 0.04) & (r < 0.05), 2] = -float("inf")
    sc["scales"][(r >= 0.05) & (r < 0.06), 0] = float("inf")
    sc["scales"][(r >= 0.06) & (r < 0.07), 1] = float("nan")
    sc["rotations"][(r >= 0.07) & (r < 0.08)] = 0.0
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    assert not torch.isfinite(sc["vertices"]).all()
    ref, out = check_case(oracle, tracer, sc, *S.rays_cube(48, 48, view=2))
    assert ref["n_con"].mean() > 3 and np.isfinite(out["rgb"]).all()
    info = tracer.optix_context.accel_info()
    assert np.isfinite(info.max_abs) and np.isfinite(list(info.scene_lo)).all() and np.isfinite(list(info.scene_hi)).all()
    assert info.max_abs < 3.0 and max(info.scene_hi) < 2.0


@pytest.mark.parametrize("P", [1, 2, 3, 5])
def test_tiny_scenes(oracle, tracer, P):
    sc = S.scene_cube(P=P, seed=P)
    sc["scales"] = sc["scales"] * 8
    sc["means3D"] = sc["means3D"] * 0.3
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    ref, _ = check_case(oracle, tracer, sc, *S.rays_cube(16, 16))
    assert ref["n_con"].sum() > 0


def test_all_rays_miss(oracle, tracer):
    sc = S.scene_cube(P=500, seed=2)
    o, d = S.rays_cube(16, 16)
    ref, out = check_case(oracle, tracer, sc, o + 10.0, -d, bg=(0.3, 0.2, 0.1))
    assert (out["acc"] == 0).all() and np.allclose(out["rgb"], [0.3, 0.2, 0.1])


def test_coplanar_ties_and_dense_stacks(oracle, tracer):
    """Exactly equal depths (axis-aligned coplanar quads on a binary grid) and >16 hits per ray: the order must be
    the oracle's (ascending surfel index), whatever order the BVH delivers them in."""
    from test_oracle_scalar import _tie_scene
    sc = _tie_scene(600, seed=3)
    o = torch.stack(torch.meshgrid(torch.linspace(-0.4, 0.4, 24), torch.linspace(-0.4, 0.4, 24), indexing="ij"), -1)
    o = torch.cat([o, torch.full((24, 24, 1), 3.0)], -1).contiguous()
    d = torch.tensor([0.0, 0.0, -1.0]).expand(24, 24, 3).contiguous()
    # The quads are axis-aligned with the rays along -z: some quaternion components' gradients are zero by
    # symmetry (the oracle returns zeros or 1e-8), and what the GPU returns there is the rounding left over from cancelling
    # terms of the size of the other components.  That column is held against that size, the others element-wise.
    ref, _ = check_case(oracle, tracer, sc, o, d, skip=("rotations",))
    assert ref["n_proc"].max() >= 16
    want, got = ref["grads_ref"]["rotations"], ref["grads_gpu"]["rotations"]
    zero_cols = [k for k in range(4) if np.abs(want[:, k]).max() <= 1e-6 * np.abs(want).max()]
    live_cols = [k for k in range(4) if k not in zero_cols]
    assert zero_cols and live_cols
    assert np.abs(got[:, zero_cols]).max() <= 1e-6 * np.abs(want).max()
    assert_close_sum(got[:, live_cols], want[:, live_cols], GRAD_REL, "rotations",
                     noise=ref["grads_noise"]["rotations"][:, live_cols])


def _with_scales(sc, factor):
    """The scene with every surfel `factor` times larger (quads rebuilt)."""
    out = dict(sc)
    out["scales"] = sc["scales"] * factor
    out["vertices"], out["faces"] = S.get_triangles(sc["means3D"], out["scales"], sc["rotations"])
    return out


def test_later_chunks_where_a_work_list_cannot_help(oracle, tracer):
    """The forward walk of a ray's second and later chunks starts from the list the walk before left (nodes and leaf
    groups still ahead of some ray).  Cases that leave that path: more leaf groups ahead of one wave than a list holds
    (the walk falls back to the root), rays that graze their quads (no usable plane distance: a quad stays on the list
    until the sphere around it is behind the origin), and waves whose rays differ in direction signs (no list at all).
    Outputs must be the oracle's bits in each."""
    from test_oracle_scalar import _tie_scene
    # (a) 2400 coplanar quads, 1200 leaf groups, nearly all of them ahead of every ray of the wave at once
    sc = _tie_scene(2400, seed=5)
    o = torch.stack(torch.meshgrid(torch.linspace(-0.2, 0.2, 16), torch.linspace(-0.2, 0.2, 16), indexing="ij"), -1)
    o = torch.cat([o, torch.full((16, 16, 1), 3.0)], -1).contiguous()
    d = torch.tensor([0.0, 0.0, -1.0]).expand(16, 16, 3).contiguous()
    ref, _ = check_case(oracle, tracer, sc, o, d, grads=False)
    assert ref["n_proc"].max() > 16
    # (b) sixty large parallel quads 4 mm apart, met at 1.1 to 2.6 degrees: dozens of hits per ray, all of them grazing
    P = 60
    gen = torch.Generator().manual_seed(11)
    means = torch.cat([0.2 * torch.rand(P, 2, generator=gen), (0.4 - 0.004 * torch.arange(1, P + 1)).reshape(P, 1)], -1)
    scales = torch.ones(P, 2)
    rot = torch.tensor([1.0, 0.0, 0.0, 0.0]).repeat(P, 1)
    v, f = S.get_triangles(means, scales, rot)
    sc = {"means3D": means, "scales": scales, "rotations": rot, "opacities": torch.full((P, 1), 0.1),
          "colors_precomp": torch.rand(P, 3, generator=gen), "vertices": v, "faces": f}
    ys, slopes = torch.meshgrid(torch.linspace(-1.0, 1.0, 16), torch.linspace(0.02, 0.045, 16), indexing="ij")
    o = torch.stack([torch.full_like(ys, -2.5), ys, torch.full_like(ys, 0.4)], -1).contiguous()
    d = torch.stack([torch.ones_like(ys), torch.zeros_like(ys), -slopes], -1).contiguous()
    ref, _ = check_case(oracle, tracer, sc, o, d, grads=False)
    assert ref["n_proc"].max() > 32
    # (c) the image centre of a pinhole camera: the four tiles around it hold rays of four sign classes; surfels
    # enlarged until those rays need several chunks
    sc = _with_scales(S.scene_cube(P=6000, seed=7, colors=True), 4.0)
    o, d = S.rays_cube(32, 32)
    ref, _ = check_case(oracle, tracer, sc, o, d, grads=False)
    centre = ref["n_proc"].reshape(32, 32)[8:24, 8:24]
    assert centre.max() > 32


def test_refit_equals_rebuild(oracle, tracer):
    sc = S.scene_lidar(P=30000, seed=2, aux=4)
    o, d = S.rays_lidar(beams=16, azimuths=128)
    gpu_trace(tracer, sc, o, d)                       # build on the first frame
    for frame in (1, 2):
        moved = S.perturb_means(sc, frame)
        out_refit, _ = gpu_trace(tracer, moved, o, d, rebuild=False)
        out_build, _ = gpu_trace(tracer, moved, o, d, rebuild=True)
        ref = oracle.forward(oracle_scene(oracle, moved, o, d), oracle.HITS_BVH_LEXI)
        assert_forward_exact(out_refit, ref)
        assert_forward_exact(out_build, ref)


def test_config2_sphere_build_once_then_refit(oracle, tracer):
    sc = S.scene_sphere(P=100000, seed=0)
    for view in range(3):
        o, d = S.rays_sphere(96, 96, view=view)
        s = oracle_scene(oracle, sc, o, d)
        ref = oracle.forward(s, oracle.HITS_BVH_LEXI)
        out, _ = gpu_trace(tracer, sc, o, d, rebuild=(view == 0))
        assert_forward_exact(out, ref)
        assert ref["acc"].mean() > 0.2


def test_debug_flag_and_saved_tensor_reuse(oracle, tracer):
    sc = S.scene_cube(P=800, seed=9)
    o, d = S.rays_cube(16, 16)
    out, _ = gpu_trace(tracer, sc, o, d, debug=True, upstream=upstream(16, 16, 2))
    ref = oracle.forward(oracle_scene(oracle, sc, o, d), oracle.HITS_BVH_LEXI)
    assert_forward_exact(out, ref)


def test_config3_full_size_properties_and_sampled_parity(oracle, tracer):
    """BASELINE config 3 at its real size (1M surfels, 1920x1080): size-independent invariants on the whole
    image, run-to-run determinism, and bit parity with the oracle on a sample of 4096 pixels."""
    dev = "cuda"
    sc = S.scene_room(P=1000000, seed=0)
    o, d = S.rays_room(1080, 1920)
    out, _ = gpu_trace(tracer, sc, o, d)
    acc = out["acc"].astype(np.float64)
    assert np.isfinite(out["rgb"]).all() and (acc >= 0).all() and (acc <= 1).all()
    np.testing.assert_allclose(acc.sum(), out["wet"].astype(np.float64).sum(), rtol=1e-4)   # checksum of checksums
    np.testing.assert_array_equal(out["mid"][..., 13:16], out["rgb"])                       # bg = 0, depth 0
    np.testing.assert_array_equal(out["mid"][..., 16:], 0)
    out2, _ = gpu_trace(tracer, sc, o, d, build=False)
    for k in ("rgb", "dpt", "acc", "norm", "mid"):
        np.testing.assert_array_equal(out[k], out2[k])
    gen = torch.Generator().manual_seed(5)
    pick = torch.randperm(1080 * 1920, generator=gen)[:4096]
    so, sd = o.reshape(-1, 3)[pick].reshape(64, 64, 3).contiguous(), d.reshape(-1, 3)[pick].reshape(64, 64, 3).contiguous()
    ref = oracle.forward(oracle_scene(oracle, sc, so, sd), oracle.HITS_BVH_LEXI)
    for k in ("rgb", "dpt", "acc", "norm"):
        got = out[k].reshape(1080 * 1920, -1)[pick.numpy()].reshape(ref[k].shape)
        np.testing.assert_array_equal(got.view(np.uint32), ref[k].view(np.uint32), err_msg=k)
    assert ref["n_con"].mean() > 10
    del dev


def test_backward_replays_the_forward_hit_record_or_retraces(oracle, tracer):
    """The autograd path records the forward hit buffers and replays them in backward; a record that is too small
    makes backward walk the BVH again.  Both must give the oracle's gradients, and an overflow raises the estimate."""
    sc = S.scene_cube(P=6000, seed=4)
    o, d = S.rays_cube(64, 64)
    s = oracle_scene(oracle, sc, o, d)
    ref = oracle.forward(s, oracle.HITS_BVH_LEXI)
    ug = upstream(64, 64, 2)
    refg = oracle.backward(s, ref, {k: v.numpy() for k, v in ug.items()}, oracle.HITS_BVH_LEXI)
    refg64 = oracle.backward(s, ref, {k: v.numpy() for k, v in ug.items()}, oracle.HITS_BVH_LEXI, noise=True)
    ctx = tracer.optix_context
    saved = ctx.record_blocks_per_wave
    try:
        for estimate in (8.0, 0.01):
            ctx.record_blocks_per_wave = estimate
            out, g = gpu_trace(tracer, sc, o, d, upstream=ug)
            assert_forward_exact(out, ref)
            assert_gradients(g, refg, refg64, GRAD_REL)
        torch.cuda.synchronize()
        ctx.update_record_estimate()
        assert ctx.record_blocks_per_wave > 1.0   # learnt from the overflow, without the backward call waiting for it
    finally:
        ctx.record_blocks_per_wave = max(saved or 0.0, ctx.record_blocks_per_wave)


@pytest.mark.parametrize("case", ["cube_sh3", "room_aux8_depth2"])
def test_gradients_summed_straight_into_the_tensors(oracle, tracer, case):
    """The binding hands the backward trace one row of gradient columns per surfel by default (DstParams.grad_rows);
    a C caller may leave it out, and the kernels then add to the dL_d* tensors directly: same gradients."""
    ctx = tracer.optix_context
    assert ctx.gradient_rows
    ctx.gradient_rows = False
    try:
        if case == "cube_sh3":
            sc = S.scene_cube(P=10000, seed=0)
            check_case(oracle, tracer, sc, *S.rays_cube(96, 96))
        else:
            sc = S.scene_room(P=30000, seed=2, aux=8, half=1.5)
            sc["others_precomp"][:, 0] = sc["others_precomp"][:, 0] * 0.8 + 0.1
            o, d = S.pinhole_rays(40, 64, 70.0, (-0.6, -0.3, 0.15), (0.9, 0.45, -0.15))
            check_case(oracle, tracer, sc, o, d, max_trace_depth=2, specular_threshold=0.1)
    finally:
        ctx.gradient_rows = True


def test_raw_launcher_calls_without_a_record(oracle, tracer):
    """The four `_C` callables with exactly the reference's positional arguments (24 and 36)."""
    import diff_surfel_tracing._C as binding
    sc = S.scene_cube(P=3000, seed=6)
    o, d = S.rays_cube(32, 40)
    dev = "cuda"
    g = {k: v.to(dev) for k, v in sc.items()}
    ctx = tracer.optix_context
    binding.build_acceleration_structure(ctx, g["vertices"], g["faces"], True)
    e, eye, z3 = torch.empty(0, device=dev), torch.eye(4, device=dev), torch.zeros(3, device=dev)
    common = (g["vertices"], z3, g["means3D"], g["shs"], 3, e, e, g["opacities"], g["scales"], 1.0, g["rotations"], e,
              eye, eye, z3, False, False, 0, 0.0)
    fwd = binding.trace_surfels(ctx, True, True, o.to(dev), d.to(dev), *common)
    assert len(fwd) == 8
    ug = upstream(32, 40, 2)
    ups = [ug[k].to(dev) for k in ("rgb", "dpt", "acc", "norm")] + [torch.zeros(32, 40, 1, device=dev), ug["aux"].to(dev)]
    bwd = binding.trace_surfels_backward(ctx, True, o.to(dev), d.to(dev), *common, *fwd[:7], *ups)
    assert len(bwd) == 12
    s = oracle_scene(oracle, sc, o, d)
    ref = oracle.forward(s, oracle.HITS_BVH_LEXI)
    refg = oracle.backward(s, ref, {k: v.numpy() for k, v in ug.items()}, oracle.HITS_BVH_LEXI)
    refg64 = oracle.backward(s, ref, {k: v.numpy() for k, v in ug.items()}, oracle.HITS_BVH_LEXI, noise=True)
    np.testing.assert_array_equal(fwd[0].cpu().numpy(), ref["rgb"])
    # hit counts: entries evaluated and hits composited, summed over the rays, are the oracle's exactly
    counters = torch.zeros(2, dtype=torch.int64, device=dev)
    binding.trace_surfels(ctx, True, True, o.to(dev), d.to(dev), *common, counters=counters)
    assert counters.tolist() == [int(ref["n_proc"].sum()), int(ref["n_con"].sum())]
    names = ("ray_o", "ray_d", "means3D", "grads3D", None, "shs", "colors_precomp", None, "opacities", "scales",
             "rotations", None)
    got = {k: t.cpu().numpy() for t, k in zip(bwd, names) if k is not None}
    assert_gradients(got, {k: refg[k] for k in got}, refg64, GRAD_REL)
    assert bwd[4].abs().max() == 0 and bwd[11].shape == (3000, 9) and bwd[11].abs().max() == 0


def test_raw_launcher_calls_with_an_overflowed_and_with_a_damaged_record(oracle, tracer):
    """Through the launchers directly, with records made by hand.  A record too small for the forward trace is seen
    on the device: backward walks the BVH again and gives the oracle's gradients (not zeros).  A complete record whose
    directory was wiped afterwards cannot be replayed: the call still returns, and word 1 of the record counts the
    broken chains, which is how a caller can tell."""
    import diff_surfel_tracing._C as binding
    sc = S.scene_cube(P=3000, seed=6)
    o, d = S.rays_cube(32, 40)
    dev = "cuda"
    g = {k: v.to(dev) for k, v in sc.items()}
    ctx = tracer.optix_context
    binding.build_acceleration_structure(ctx, g["vertices"], g["faces"], True)
    e, eye, z3 = torch.empty(0, device=dev), torch.eye(4, device=dev), torch.zeros(3, device=dev)
    common = (g["vertices"], z3, g["means3D"], g["shs"], 3, e, e, g["opacities"], g["scales"], 1.0, g["rotations"], e,
              eye, eye, z3, False, False, 0, 0.0)
    ug = upstream(32, 40, 2)
    ups = [ug[k].to(dev) for k in ("rgb", "dpt", "acc", "norm")] + [torch.zeros(32, 40, 1, device=dev), ug["aux"].to(dev)]
    s = oracle_scene(oracle, sc, o, d)
    ref = oracle.forward(s, oracle.HITS_BVH_LEXI)
    refg = oracle.backward(s, ref, {k: v.numpy() for k, v in ug.items()}, oracle.HITS_BVH_LEXI)
    refg64 = oracle.backward(s, ref, {k: v.numpy() for k, v in ug.items()}, oracle.HITS_BVH_LEXI, noise=True)
    names = ("ray_o", "ray_d", "means3D", "grads3D", None, "shs", "colors_precomp", None, "opacities", "scales",
             "rotations", None)

    small = binding.HitRecord(32, 40, 1, 0.3, dev)          # room for a third of a block per wave
    fwd = binding.trace_surfels(ctx, True, True, o.to(dev), d.to(dev), *common, hit_record=small)
    bwd = binding.trace_surfels_backward(ctx, True, o.to(dev), d.to(dev), *common, *fwd[:7], *ups, hit_record=small)
    torch.cuda.synchronize()
    assert not small.complete() and small.broken_chains() == 0
    np.testing.assert_array_equal(fwd[0].cpu().numpy(), ref["rgb"])
    got = {k: t.cpu().numpy() for t, k in zip(bwd, names) if k is not None}
    assert_gradients(got, {k: refg[k] for k in got}, refg64, GRAD_REL)

    full = binding.HitRecord(32, 40, 1, 12.0, dev)
    fwd = binding.trace_surfels(ctx, True, True, o.to(dev), d.to(dev), *common, hit_record=full)
    torch.cuda.synchronize()
    assert full.complete()
    header = binding.HitRecord.layout(32, 40, 1, 12.0)[1]
    full.words[2:header].zero_()                             # the directory: every chain now starts nowhere
    binding.trace_surfels_backward(ctx, True, o.to(dev), d.to(dev), *common, *fwd[:7], *ups, hit_record=full)
    torch.cuda.synchronize()
    assert full.broken_chains() > 0


def test_distortion_output_is_opt_in_and_equals_the_oracle(oracle, tracer):
    """`dist` is zero as in the reference unless SurfelTracer.distortion is set; then it is the 2DGS depth distortion
    of the primary ray, bit-equal to the oracle's, and nothing else changes."""
    sc = S.scene_cube(P=6000, seed=12)
    o, d = S.rays_cube(56, 72)
    s = oracle_scene(oracle, sc, o, d)
    ref = oracle.forward(s, oracle.HITS_BVH_LEXI, compute_dist=True)
    plain, _ = gpu_trace(tracer, sc, o, d)
    assert (plain["dist"] == 0).all()
    tracer.distortion = True
    try:
        out, g = gpu_trace(tracer, sc, o, d, upstream=upstream(56, 72, 2))
    finally:
        tracer.distortion = False
    assert_forward_exact({**out, "dist": plain["dist"]}, {**ref, "dist": np.zeros_like(ref["dist"])})
    np.testing.assert_array_equal(out["dist"].view(np.uint32), ref["dist"][..., :1].view(np.uint32))
    assert out["dist"].max() > 1e-6 and g["means3D"] is not None
