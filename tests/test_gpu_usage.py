"""Ways of calling the autograd wrapper beyond one forward and one backward: several graphs alive at once, backward
passes in any order, a second backward through a kept graph, inputs of which only some ask for gradients,
non-contiguous views, a side stream, two contexts, gradient modes.  The reference is one call of each kind on
its own (those are held against the oracle in test_gpu_parity.py): per-ray outputs must repeat bit for bit,
atomically summed gradients within 1e-3 of the value plus 1e-3 of the channel's root mean square (two orders of
float atomics)."""
import numpy as np
import pytest
import torch

import dst_scenes as S
from helpers import GRAD_REL, PARAM_NAMES, assert_same_sums, settings

pytestmark = pytest.mark.gpu
H, W, DEV = 48, 64, "cuda"


class _Bench:
    def __init__(self):
        import diff_surfel_tracing as dst
        self.dst = dst
        self.tracer = dst.SurfelTracer()
        sc = S.scene_cube(P=6000, seed=1, aux=2)
        self.g = {k: v.to(DEV) for k, v in sc.items()}
        self.tracer.build_acceleration_structure(self.g["vertices"], self.g["faces"], True)
        self.views = [tuple(t.to(DEV) for t in S.rays_cube(H, W, view=v)) for v in range(3)]
        self.ups = [{k: t.to(DEV) for k, t in S.upstream_grads(H, W, 2, seed=v).items()} for v in range(3)]
        self.st = settings(dst, H, W, DEV)
        self.single, self.outs = [], []
        for (o, d), ug in zip(self.views, self.ups):
            lf = self.leaves()
            out = self.run(lf, o, d)
            self.loss(out, ug).backward()
            self.single.append(self.grads(lf))
            self.outs.append([t.detach().cpu().numpy() for t in out])
        self.total = {k: sum(s[k] for s in self.single) for k in self.single[0]}

    def leaves(self, req=PARAM_NAMES):
        return {k: self.g[k].clone().requires_grad_(k in req) for k in PARAM_NAMES if k in self.g}

    def run(self, leaf, o, d, tracer=None, g=None):
        g = self.g if g is None else g
        return (tracer or self.tracer)(o, d, g["vertices"], leaf["means3D"], torch.zeros_like(leaf["means3D"]),
                                       shs=leaf.get("shs"), others_precomp=leaf.get("others_precomp"),
                                       opacities=leaf["opacities"], scales=leaf["scales"], rotations=leaf["rotations"],
                                       tracer_settings=self.st)

    @staticmethod
    def loss(out, ug):
        idx = {"rgb": 0, "dpt": 1, "acc": 2, "norm": 3, "aux": 5}
        return sum((out[idx[k]] * v).sum() for k, v in ug.items() if k in idx)

    @staticmethod
    def grads(leaf):
        return {k: (None if v.grad is None else v.grad.cpu().numpy().copy()) for k, v in leaf.items()}

    def same_rays(self, out, view):
        """The per-ray outputs (everything but the atomically summed blending weights) repeat bit for bit."""
        for x, y in list(zip(out, self.outs[view]))[:7]:
            assert np.array_equal(x.detach().cpu().numpy().view(np.uint32), y.view(np.uint32))


def close(a, b, tag):
    for k in a:
        if a[k] is None or b[k] is None:
            assert a[k] is None and b[k] is None, (tag, k)
        else:
            assert_same_sums(a[k], b[k], GRAD_REL, tag + " " + k)


@pytest.fixture(scope="module")
def B():
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return _Bench()


def test_three_graphs_alive_and_one_backward(B):
    lf = B.leaves()
    outs = [B.run(lf, o, d) for o, d in B.views]
    for v, out in enumerate(outs):
        B.same_rays(out, v)
    sum(B.loss(o_, u_) for o_, u_ in zip(outs, B.ups)).backward()
    close(B.grads(lf), B.total, "three graphs")


def test_backward_passes_in_another_order_than_the_forward_passes(B):
    lf = B.leaves()
    outs = [B.run(lf, o, d) for o, d in B.views]
    for k in (2, 0, 1):
        B.loss(outs[k], B.ups[k]).backward()
    close(B.grads(lf), B.total, "reversed")


def test_second_backward_through_a_kept_graph(B):
    """The first backward hands the hit record back; the second walks the BVH again."""
    lf = B.leaves()
    L = B.loss(B.run(lf, *B.views[0]), B.ups[0])
    L.backward(retain_graph=True)
    L.backward()
    close(B.grads(lf), {k: 2 * v for k, v in B.single[0].items()}, "kept graph")


@pytest.mark.parametrize("req", [("means3D",), ("shs", "opacities"), ("scales", "rotations"), ("others_precomp",)])
def test_only_some_inputs_ask_for_gradients(B, req):
    lf = B.leaves(req)
    B.loss(B.run(lf, *B.views[1]), B.ups[1]).backward()
    got = B.grads(lf)
    for k in got:
        if k in req:
            assert_same_sums(got[k], B.single[1][k], GRAD_REL, "subset " + k)
        else:
            assert got[k] is None, k


def test_non_contiguous_views_as_inputs(B):
    lf = B.leaves()
    o, d = B.views[2]
    o_nc = torch.zeros(H, W, 6, device=DEV)[..., ::2]
    o_nc.copy_(o)
    d_nc = d.permute(1, 0, 2).contiguous().permute(1, 0, 2)
    wide = torch.zeros(B.g["means3D"].shape[0], 5, device=DEV)
    wide[:, 1:4] = B.g["means3D"]
    lf["means3D"] = wide[:, 1:4].detach().requires_grad_(True)
    lf["shs"] = B.g["shs"].permute(1, 0, 2).contiguous().permute(1, 0, 2).detach().requires_grad_(True)
    assert not any(t.is_contiguous() for t in (o_nc, d_nc, lf["means3D"], lf["shs"]))
    out = B.run(lf, o_nc, d_nc)
    B.same_rays(out, 2)
    B.loss(out, B.ups[2]).backward()
    close(B.grads(lf), B.single[2], "views")


def test_side_stream(B):
    side = torch.cuda.Stream()
    lf = B.leaves()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        out = B.run(lf, *B.views[0])
        B.loss(out, B.ups[0]).backward()
    side.synchronize()
    torch.cuda.synchronize()
    B.same_rays(out, 0)
    close(B.grads(lf), B.single[0], "side stream")


def test_two_contexts_in_one_graph(B):
    other = B.dst.SurfelTracer()
    sc2 = S.scene_cube(P=900, seed=9, aux=2)
    g2 = {k: v.to(DEV) for k, v in sc2.items()}
    other.build_acceleration_structure(g2["vertices"], g2["faces"], True)
    lf = B.leaves()
    lf2 = {k: g2[k].clone().requires_grad_(True) for k in PARAM_NAMES if k in g2}
    out_a = B.run(lf, *B.views[0])
    out_b = B.run(lf2, *B.views[0], tracer=other, g=g2)
    (B.loss(out_a, B.ups[0]) + B.loss(out_b, B.ups[0])).backward()
    close(B.grads(lf), B.single[0], "two contexts")
    alone = {k: g2[k].clone().requires_grad_(True) for k in PARAM_NAMES if k in g2}
    B.loss(B.run(alone, *B.views[0], tracer=other, g=g2), B.ups[0]).backward()
    close(B.grads(lf2), B.grads(alone), "second context")


def test_upstream_gradient_for_one_output_only(B):
    """Autograd hands zeros (or nothing) for the outputs the loss does not use."""
    lf = B.leaves()
    (B.run(lf, *B.views[0])[0] * B.ups[0]["rgb"]).sum().backward()
    a = B.grads(lf)
    lf = B.leaves()
    z = {k: torch.zeros_like(v) for k, v in B.ups[0].items()}
    z["rgb"] = B.ups[0]["rgb"]
    B.loss(B.run(lf, *B.views[0]), z).backward()
    close(a, B.grads(lf), "rgb only")


def test_no_grad_and_inference_mode(B):
    with torch.no_grad():
        B.same_rays(B.run(B.leaves(), *B.views[0]), 0)
    with torch.inference_mode():
        B.same_rays(B.run(B.leaves(()), *B.views[0]), 0)
