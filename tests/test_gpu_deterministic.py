"""Deterministic mode (SurfelTracer.deterministic / DST_FLAG_DETERMINISTIC): the accumulated blending weights and
every per-surfel gradient are summed in 64-bit fixed point, so two runs on the same inputs are bit-identical, and
the sums still match the oracle's double-accumulated ones to the usual bar.  The default mode (float atomics) is
only required to match the oracle."""
import numpy as np
import pytest
import torch

import dst_scenes as S
from helpers import GRAD_REL, assert_close_sum, assert_forward_exact, assert_gradients, gpu_trace, oracle_scene, upstream

pytestmark = pytest.mark.gpu


def _run(tracer, sc, o, d, ug, **kw):
    out, g = gpu_trace(tracer, sc, o, d, upstream=ug, **kw)
    return out, g


@pytest.mark.parametrize("case", ["cube_sh3", "room_aux8_depth2", "record_too_small"])
def test_two_runs_are_bit_identical_and_match_the_oracle(oracle, tracer, case):
    kw = {}
    if case == "room_aux8_depth2":
        sc = S.scene_room(P=30000, seed=2, aux=8, half=1.5)
        sc["others_precomp"][:, 0] = sc["others_precomp"][:, 0] * 0.8 + 0.1
        o, d = S.pinhole_rays(40, 64, 70.0, (-0.6, -0.3, 0.15), (0.9, 0.45, -0.15))
        kw = dict(max_trace_depth=2, specular_threshold=0.1)
        aux = 8
    else:
        sc = S.scene_cube(P=10000, seed=0)
        o, d = S.rays_cube(128, 128)
        aux = 2
    ug = upstream(o.shape[0], o.shape[1], aux)
    ctx = tracer.optix_context
    saved = ctx.record_blocks_per_wave
    tracer.deterministic = True
    saved_cap = ctx.record_max_bytes
    try:
        # Runs are compared like with like: all three replay a complete record, or all three walk the BVH again
        # (the two backward kernels agree to rounding, not to the bit: their gradient algebra may be contracted
        # differently).
        if case == "record_too_small":
            ctx.record_max_bytes = 0                   # no record at all: backward walks the BVH again
        else:
            _run(tracer, sc, o, d, ug, **kw)           # sizes the record, so that the runs below replay
        runs = []
        for k in range(3):
            runs.append(_run(tracer, sc, o, d, ug, **kw))
            torch.cuda.synchronize()
        for out, g in runs[1:]:
            assert np.array_equal(out["wet"].view(np.uint32), runs[0][0]["wet"].view(np.uint32))
            for k, v in g.items():
                if v is not None:
                    assert np.array_equal(v.view(np.uint32), runs[0][1][k].view(np.uint32)), k
    finally:
        tracer.deterministic = False
        ctx.record_max_bytes = saved_cap
        ctx.record_blocks_per_wave = max(saved or 0.0, 6.0)
    out, g = runs[0]
    s = oracle_scene(oracle, sc, o, d, **kw)
    ref = oracle.forward(s, oracle.HITS_BVH_LEXI)
    assert_forward_exact(out, ref)
    assert_close_sum(out["wet"], ref["wet"], 1e-5, "wet")
    ugn = {k: v.numpy() for k, v in ug.items()}
    refg = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI)
    refg64 = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI, noise=True)
    assert_gradients(g, refg, refg64, GRAD_REL)
    # and the default mode gives the same values up to the order of its float additions
    out2, g2 = _run(tracer, sc, o, d, ug, **kw)
    assert_gradients(g2, refg, refg64, GRAD_REL)


def test_the_c_abi_rejects_the_flag_without_a_workspace(tracer):
    import ctypes as C
    import diff_surfel_tracing._C as binding
    lib = binding.load_library()
    assert lib.dst_det_workspace_words(1000, 2, 0) == 1000
    assert lib.dst_det_workspace_words(1000, 2, 1) == 1000 * 66
    assert lib.dst_det_workspace_words(1000, 8, 1) == 1000 * 72
    sc = S.scene_cube(P=100, seed=1)
    tracer.build_acceleration_structure(sc["vertices"].cuda(), sc["faces"].cuda(), True)
    p = binding.DstParams()
    p.P, p.H, p.W, p.D, p.M, p.aux, p.mtd_alloc = 100, 0, 0, 3, 16, 2, 1
    keep = {k: sc[k].cuda() for k in ("vertices", "means3D", "shs", "opacities", "scales", "rotations")}
    bg = torch.zeros(3, device="cuda")
    for k, v in keep.items():
        setattr(p, k, v.data_ptr())
    p.background = bg.data_ptr()
    p.flags = binding.FLAG_DETERMINISTIC
    rc = lib.dst_trace_forward(tracer.optix_context.handle, C.byref(p), None)
    assert rc == 1 and b"det_workspace" in lib.dst_last_error(tracer.optix_context.handle)


def test_sums_beyond_the_fixed_point_range_are_counted_and_warned_about(tracer):
    """Per-surfel gradients beyond about 6.7e7 (4.2e6 for colours and opacity) do not fit the mode's 64-bit fixed
    point: the closing kernel counts them and the binding warns after the backward trace; gradients of ordinary
    size are not counted."""
    import warnings
    sc = S.scene_cube(P=2000, seed=3)
    o, d = S.rays_cube(64, 64)
    ug = upstream(o.shape[0], o.shape[1], 2)
    huge = {k: v * 1e12 for k, v in ug.items()}
    ctx = tracer.optix_context
    tracer.deterministic = True
    try:
        ctx.check_deterministic_range()                # (whatever earlier tests left)
        with warnings.catch_warnings():
            warnings.simplefilter("error")
            _run(tracer, sc, o, d, ug)
        assert ctx.check_deterministic_range() == 0
        with pytest.warns(RuntimeWarning, match="left the fixed-point range"):
            _run(tracer, sc, o, d, huge)
        before = ctx.trace_info().det_out_of_range
        assert before > 0
        ctx.deterministic_check = False                # the count goes on, the warning does not
        with warnings.catch_warnings():
            warnings.simplefilter("error")
            _run(tracer, sc, o, d, huge)
        assert ctx.trace_info().det_out_of_range > before
    finally:
        ctx.deterministic_check = True
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            ctx.check_deterministic_range()
        tracer.deterministic = False
