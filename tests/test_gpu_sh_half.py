"""DST_FLAG_SH_HALF: the traces read a binary16 copy of the SH coefficients.  The bar is the usual one - per-ray outputs
bit-identical, gradients within 1e-3 - against the oracle fed the coefficients the kernels see: shs.half().float()."""
import numpy as np
import pytest
import torch

import dst_scenes as S
from helpers import GRAD_REL, assert_close_sum, assert_forward_exact, assert_gradients, gpu_trace, oracle_scene, upstream

pytestmark = pytest.mark.gpu


def test_packing_rounds_like_ieee_binary16():
    from diff_surfel_tracing import _C
    gen = torch.Generator().manual_seed(1)
    x = torch.cat([0.3 * torch.randn(100000, generator=gen), torch.tensor([0.0, -0.0, 1e-8, -1e-8, 6e-8, 6.1e-5, 65504.0,
                  65519.9, 65520.0, 1e9, -1e9, float("inf"), float("-inf"), 1.00048828125, 1.0009765625, 1.00146484375]),
                   torch.randn(5000, generator=gen) * 1e-6, torch.randn(5000, generator=gen) * 3e4]).cuda()
    got = _C.pack_sh_half(x)
    assert got.dtype == torch.float16 and got.shape == x.shape
    assert torch.equal(got.view(torch.int16), x.half().view(torch.int16))
    nan = _C.pack_sh_half(torch.tensor([float("nan")]).cuda())
    assert torch.isnan(nan).all()


@pytest.mark.parametrize("case", ["cube_sh3", "cube_sh1", "room_aux8_depth2", "list_sh2"])
def test_half_coefficients_give_the_results_of_their_fp32_values(oracle, case):
    import diff_surfel_tracing as dst
    tracer = dst.SurfelTracer()
    tracer.sh_half = True
    kw, aux = {}, 2
    if case == "room_aux8_depth2":
        sc = S.scene_room(P=20000, seed=2, aux=8, half=1.5)
        sc["others_precomp"][:, 0] = sc["others_precomp"][:, 0] * 0.8 + 0.1
        o, d = S.pinhole_rays(40, 64, 70.0, (-0.6, -0.3, 0.15), (0.9, 0.45, -0.15))
        kw, aux = dict(max_trace_depth=2, specular_threshold=0.1), 8
    elif case == "list_sh2":
        sc = S.scene_cube(P=6000, seed=3)
        sc["shs"] = sc["shs"][:, :9].contiguous()      # rows of 27 coefficients: no 16-byte rows, the scalar path
        o, d = S.rays_cube(48, 64)
        o, d = o.reshape(1, -1, 3).contiguous(), d.reshape(1, -1, 3).contiguous()
        kw = dict(sh_degree=2)
    else:
        sc = S.scene_cube(P=8000, seed=1)
        o, d = S.rays_cube(64, 64)
        kw = dict(sh_degree=1) if case == "cube_sh1" else {}
    seen = dict(sc)
    seen["shs"] = sc["shs"].half().float()               # what the kernels read
    assert (seen["shs"] != sc["shs"]).float().mean() > 0.5
    ug = upstream(o.shape[0], o.shape[1], aux)
    s = oracle_scene(oracle, seen, o, d, **kw)
    ref = oracle.forward(s, oracle.HITS_BVH_LEXI)
    ugn = {k: v.numpy() for k, v in ug.items()}
    refg = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI)
    refg64 = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI, noise=True)
    ctx = tracer.optix_context
    for record_bytes in (ctx.record_max_bytes, 0):       # backward replays the record / walks the BVH again
        ctx.record_max_bytes = record_bytes
        out, g = gpu_trace(tracer, sc, o, d, upstream=ug, **kw)
        assert_forward_exact(out, ref)
        assert_close_sum(out["wet"], ref["wet"], 1e-4, "wet")
        assert_gradients(g, refg, refg64, GRAD_REL, case + " ")
    # and the fp32 coefficients give something else: the flag is not a no-op
    tracer.sh_half = False
    plain, _ = gpu_trace(tracer, sc, o, d, **kw)
    assert not np.array_equal(plain["rgb"], out["rgb"])
    assert np.abs(plain["rgb"] - out["rgb"]).max() < 5e-3
