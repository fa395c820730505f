"""Committed fixture (tests/golden/cube_p400.npz, written by tests/golden/make_golden.py): the oracle must keep
reproducing it bit for bit, and the HIP path must match it like it matches the oracle."""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden  # noqa: E402

from helpers import GRAD_REL, assert_close_sum, assert_gradients, assert_forward_exact, gpu_trace, oracle_scene  # noqa: E402


@pytest.fixture(scope="module")
def golden():
    z = np.load(os.path.join(HERE, "golden", "cube_p400.npz"))
    return {k: z[k] for k in z.files}


def test_oracle_reproduces_the_fixture(oracle, golden):
    sc, o, d, ug = make_golden.load_inputs()
    s = oracle_scene(oracle, sc, o, d, bg=make_golden.SPEC["bg"])
    for mode in (oracle.HITS_BRUTE_LITERAL, oracle.HITS_BVH_LEXI):
        fwd = oracle.forward(s, mode)
        for k in ("rgb", "dpt", "acc", "norm", "aux", "mid", "n_proc", "n_con"):
            np.testing.assert_array_equal(fwd[k], golden["fwd_" + k], err_msg=k)
        np.testing.assert_allclose(fwd["wet"], golden["fwd_wet"], rtol=1e-6)
    bwd = oracle.backward(s, fwd, {k: v.numpy() for k, v in ug.items()}, oracle.HITS_BVH_LEXI)
    for k, v in bwd.items():
        np.testing.assert_allclose(v, golden["bwd_" + k], rtol=1e-6, atol=1e-30, err_msg=k)
    assert golden["fwd_n_con"].max() > 16


@pytest.mark.gpu
def test_gpu_matches_the_fixture(tracer, golden, oracle):
    sc, o, d, ug = make_golden.load_inputs()
    out, g = gpu_trace(tracer, sc, o, d, upstream=ug, bg=make_golden.SPEC["bg"])
    fwd = {k[4:]: v for k, v in golden.items() if k.startswith("fwd_")}
    assert_forward_exact(out, fwd)
    assert_close_sum(out["wet"], golden["fwd_wet"], 1e-5, "wet")
    # the rounding-noise allowance of the comparison comes from the oracle's double-precision gradient algebra
    s = oracle_scene(oracle, sc, o, d, bg=make_golden.SPEC["bg"])
    ref64 = oracle.backward(s, fwd, {k: v.numpy() for k, v in ug.items()}, oracle.HITS_BVH_LEXI, noise=True)
    names = ("ray_o", "ray_d", "means3D", "grads3D", "shs", "others_precomp", "opacities", "scales", "rotations")
    assert_gradients({k: g[k] for k in names}, {k: golden["bwd_" + k] for k in names}, ref64, GRAD_REL)
