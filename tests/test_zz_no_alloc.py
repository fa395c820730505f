"""dst_refit_accel_static (the refit that allocates nothing: its scratch is a fixed array inside the library)
against dst_build_accel(rebuild=0), through the C ABI: bit-identical hierarchy and leaves, and bit-identical
forward outputs, on two calls in a row, the second on a smaller structure."""
import ctypes as C

import numpy as np
import pytest
import torch

import dst_scenes as S
from helpers import assert_forward_exact, gpu_trace
from test_gpu_lbvh import check_tree, download

pytestmark = pytest.mark.gpu


def _refit(tracer, vertices, static):
    import diff_surfel_tracing._C as binding
    lib, ctx = binding.load_library(), tracer.optix_context
    v = vertices.to("cuda").contiguous()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    if static:
        rc = lib.dst_refit_accel_static(ctx.handle, v.data_ptr(), v.size(0), stream)
    else:
        rc = lib.dst_build_accel(ctx.handle, v.data_ptr(), v.size(0), None, v.size(0) // 2, 0, stream)
    assert rc == 0, lib.dst_last_error(ctx.handle)
    torch.cuda.synchronize()


def _snapshot(tracer, scene, o, d):
    info, nodes, leaves, npar, lpar, keys = download(tracer)
    out, _ = gpu_trace(tracer, scene, o, d, build=False)
    return (nodes.copy(), leaves.copy()), out, (info, nodes, leaves, npar, lpar, keys)


def _same(a, b):
    return all(np.array_equal(x.view(np.uint8), y.view(np.uint8)) for x, y in zip(a, b))


def test_static_refit_equals_refit_on_two_calls_the_second_smaller(tracer):
    import diff_surfel_tracing._C as binding
    lib, ctx = binding.load_library(), tracer.optix_context
    o, d = S.rays_lidar(beams=16, azimuths=128)
    for P, seed in ((40000, 11), (7000, 12)):          # the second structure is smaller than the first
        sc = S.scene_lidar(P=P, seed=seed, aux=4)
        gpu_trace(tracer, sc, o, d)                    # build
        f1, f2 = S.perturb_means(sc, 1), S.perturb_means(sc, 2)
        _refit(tracer, f1["vertices"], static=False)
        ref1, out1, _ = _snapshot(tracer, f1, o, d)
        _refit(tracer, f2["vertices"], static=False)
        ref2, out2, _ = _snapshot(tracer, f2, o, d)
        assert not _same(ref1, ref2)                   # the two frames really differ
        _refit(tracer, f1["vertices"], static=True)
        got1, gout1, tree = _snapshot(tracer, f1, o, d)
        assert _same(got1, ref1)
        check_tree(*tree, f1["vertices"].numpy())
        for k in ("rgb", "dpt", "acc", "norm", "aux", "mid"):
            assert np.array_equal(gout1[k].view(np.uint32), out1[k].view(np.uint32)), k
        _refit(tracer, f2["vertices"], static=True)
        got2, gout2, _ = _snapshot(tracer, f2, o, d)
        assert _same(got2, ref2)
        for k in ("rgb", "dpt", "acc", "norm", "aux", "mid"):
            assert np.array_equal(gout2[k].view(np.uint32), out2[k].view(np.uint32)), k
    # errors: fewer vertices than the build indexed; no launch happens
    v = f1["vertices"].to("cuda")
    rc = lib.dst_refit_accel_static(ctx.handle, v.data_ptr(), v.size(0) - 4,
                                    C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 3 and b"fewer vertices" in lib.dst_last_error(ctx.handle)
