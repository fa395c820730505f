"""Tile hand-over of the forward trace: a tile whose first packet walk runs into the step limit is put on a list and
traced by a second launch in which every ray walks on its own.  Which walk finds the hits must not show anywhere:
per-ray outputs bit-identical to the oracle, gradients within the usual bar, with the limit forced low enough that
ordinary scenes hand over every tile, with the list overflowing, and on the kind of scene the hand-over is for (a
dense ball of quads far smaller than a pixel), where the context has to switch it on by itself."""
import numpy as np
import pytest
import torch

import dst_scenes as S
from helpers import GRAD_REL, assert_close_sum, assert_forward_exact, assert_gradients, gpu_trace, oracle_scene, upstream

pytestmark = pytest.mark.gpu


def own_tracer(mode, steps=0):
    import diff_surfel_tracing as dst
    from diff_surfel_tracing import _C
    tracer = dst.SurfelTracer()
    tracer.optix_context.set_handover({"off": _C.HANDOVER_OFF, "auto": _C.HANDOVER_AUTO, "always": _C.HANDOVER_ALWAYS}[mode],
                                      steps)
    return tracer


def handed(tracer):
    return tracer.optix_context.trace_info().tiles_handed_over


def ball_scene(P=170000, n_ball=150000, radius=0.06, centre=(1.0, 0.5, 0.0), shrink=0.018, seed=0):
    """The 10 m room with most of its surfels moved into a ball of 12 cm and shrunk to 2 mm quads: seen from half a
    metre away at 64x64 pixels, an 8x8 tile's frustum holds some ten thousand quads, each wanted by one ray at best.
    (Smaller quads seen from farther away: test_submillimetre_quads_seen_from_metres_away.)"""
    sc = S.scene_room(P=P, seed=seed)
    gen = torch.Generator().manual_seed(seed + 1)
    idx = torch.randperm(P, generator=gen)[:n_ball]
    u = torch.randn(n_ball, 3, generator=gen)
    u = u / u.norm(dim=1, keepdim=True)
    r = radius * torch.rand(n_ball, 1, generator=gen) ** (1.0 / 3.0)
    sc["means3D"][idx] = torch.tensor(centre) + r * u
    sc["scales"][idx] *= shrink
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    return sc


def forward_ms(tracer, sc, o, d, n=3):
    from diff_surfel_tracing import _C
    g = {k: v.cuda() for k, v in sc.items()}
    e, bg, eye = torch.empty(0, device="cuda"), torch.zeros(3, device="cuda"), torch.eye(4, device="cuda")
    og, dg = o.cuda(), d.cuda()
    best = 1e9
    for _ in range(n):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        _C.trace_surfels(tracer.optix_context, False, True, og, dg, g["vertices"], bg, g["means3D"], g["shs"], 3, e, e,
                         g["opacities"], g["scales"], 1.0, g["rotations"], e, eye, eye, bg, False, False, 0, 0.0)
        b.record()
        torch.cuda.synchronize()
        best = min(best, a.elapsed_time(b))
    return best


def test_dense_ball_of_subpixel_quads_is_handed_over_by_default(oracle):
    sc = ball_scene()
    o, d = S.pinhole_rays(64, 64, 22.0, (0.6, 0.2, 0.1), (1.0, 0.5, 0.0))
    ug = upstream(64, 64, 2)
    s = oracle_scene(oracle, sc, o, d)
    ref = oracle.forward(s, oracle.HITS_BVH_LEXI)
    # the oracle's own BVH agrees with testing every quad (the middle of the image, where the ball is)
    mid = slice(20, 44)
    brute = oracle.forward(oracle_scene(oracle, sc, o[mid, mid].contiguous(), d[mid, mid].contiguous()),
                           oracle.HITS_BRUTE_LEXI)
    assert np.array_equal(brute["acc"].view(np.uint32), ref["acc"][mid, mid].view(np.uint32))
    assert ref["n_proc"].max() > 48 and ref["acc"][mid, mid].mean() > 0.9
    ugn = {k: v.numpy() for k, v in ug.items()}
    refg = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI)
    refg64 = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI, noise=True)
    times = {}
    for mode in ("auto", "off"):
        tracer = own_tracer(mode)
        before = handed(tracer)
        out, g = gpu_trace(tracer, sc, o, d, upstream=ug)
        info = tracer.optix_context.trace_info()
        assert info.small_quads >= 2048 and info.handover_steps == 2048
        assert info.handover_active == (1 if mode == "auto" else 0)
        n = handed(tracer) - before
        assert (n >= 4) if mode == "auto" else (n == 0), n
        assert_forward_exact(out, ref)
        assert_close_sum(out["wet"], ref["wet"], 1e-4, "wet")
        assert_gradients(g, refg, refg64, GRAD_REL, "ball " + mode)
        times[mode] = forward_ms(tracer, sc, o, d)
    print("dense ball, forward: %.2f ms handed over, %.2f ms without" % (times["auto"], times["off"]), flush=True)
    assert times["auto"] < 0.75 * times["off"]


def test_submillimetre_quads_seen_from_metres_away(oracle):
    """Quads of about 1 mm, 3.4 m from the camera: the quad test has to decide them to a small fraction of their size,
    or a walk that tests every quad and walks that cull by boxes see different hits.  Brute force, the oracle's BVH
    and both GPU walks agree bit for bit."""
    P, n_ball = 200000, 180000
    sc = S.scene_room(P=P, seed=0)
    gen = torch.Generator().manual_seed(1)
    idx = torch.randperm(P, generator=gen)[:n_ball]
    centre = torch.tensor([1.0, 0.5, 0.0])
    sc["means3D"][idx] = sc["means3D"][idx] * 0.01 + centre
    sc["scales"][idx] *= 0.01
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    o, d = S.rays_room(540, 960)
    r, c = divmod(int((d * torch.nn.functional.normalize(centre - o[0, 0], dim=0)).sum(-1).argmax()), 960)
    r0, c0 = r - r % 8 - 16, c - c % 8 - 16
    o, d = o[r0:r0 + 32, c0:c0 + 32].contiguous(), d[r0:r0 + 32, c0:c0 + 32].contiguous()
    assert float((centre - o[0, 0]).norm()) > 3.0 and float(6 * sc["scales"][idx].median()) < 1.5e-3
    ref = oracle.forward(oracle_scene(oracle, sc, o, d), oracle.HITS_BVH_LEXI)
    mid = slice(8, 24)
    brute = oracle.forward(oracle_scene(oracle, sc, o[mid, mid].contiguous(), d[mid, mid].contiguous()),
                           oracle.HITS_BRUTE_LEXI)
    for k in ("rgb", "dpt", "acc", "norm"):
        assert np.array_equal(brute[k].view(np.uint32), ref[k][mid, mid].view(np.uint32)), k
    assert ref["n_con"][mid, mid].mean() > 8
    for mode, steps in (("off", 0), ("always", 256)):
        tracer = own_tracer(mode, steps)
        before = handed(tracer)
        out, _ = gpu_trace(tracer, sc, o, d, training=False)
        assert_forward_exact(out, ref)
        assert (handed(tracer) > before) == (mode == "always")


def test_ordinary_scenes_leave_the_hand_over_off(tracer):
    sc = S.scene_cube(P=10000, seed=0)
    o, d = S.rays_cube(64, 64)
    before = handed(tracer)
    gpu_trace(tracer, sc, o, d, training=False)
    info = tracer.optix_context.trace_info()
    assert info.handover_mode == 1 and info.small_quads == 0 and info.handover_active == 0
    assert handed(tracer) == before


@pytest.mark.parametrize("case", ["cube", "cube_eval", "room_aux8_depth2", "list"])
@pytest.mark.parametrize("steps", [1, 40])
def test_forced_hand_over_changes_nothing(oracle, case, steps):
    """A limit of 1 step hands every tile over whose first walk gets past the root; 40 steps splits the tiles of
    these scenes between the two walks."""
    tracer = own_tracer("always", steps)
    kw, aux = {}, 2
    if case == "room_aux8_depth2":
        sc = S.scene_room(P=20000, seed=2, aux=8, half=1.5)
        sc["others_precomp"][:, 0] = sc["others_precomp"][:, 0] * 0.8 + 0.1
        # (a narrow view: the kernels of reflection traces walk a tile as a packet only if its rays run side by side)
        o, d = S.pinhole_rays(40, 64, 5.0, (-0.6, -0.3, 0.15), (0.9, 0.45, -0.15))
        kw, aux = dict(max_trace_depth=2, specular_threshold=0.1), 8
    elif case == "list":
        sc = S.scene_cube(P=6000, seed=3)
        o, d = S.pinhole_rays(96, 128, 6.0, (3.0, 0.4, 0.2), (0.0, 0.0, 0.0))    # narrow, for the same reason
        o, d = o.reshape(1, -1, 3).contiguous(), d.reshape(1, -1, 3).contiguous()
    else:
        sc = S.scene_cube(P=8000, seed=1)
        o, d = S.rays_cube(61, 75)
        if case == "cube_eval":
            kw = dict(training=False)
    s = oracle_scene(oracle, sc, o, d, **{k: v for k, v in kw.items() if k != "training"})
    ref = oracle.forward(s, oracle.HITS_BVH_LEXI)
    before = handed(tracer)
    if case == "cube_eval":
        out, _ = gpu_trace(tracer, sc, o, d, **kw)
        assert_forward_exact(out, ref)
    else:
        ug = upstream(o.shape[0], o.shape[1], aux)
        ugn = {k: v.numpy() for k, v in ug.items()}
        refg = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI)
        refg64 = oracle.backward(s, ref, ugn, oracle.HITS_BVH_LEXI, noise=True)
        ctx = tracer.optix_context
        for record_bytes in (ctx.record_max_bytes, 0):       # backward replays the record / walks the BVH again
            ctx.record_max_bytes = record_bytes
            out, g = gpu_trace(tracer, sc, o, d, upstream=ug, **kw)
            assert_forward_exact(out, ref)
            assert_close_sum(out["wet"], ref["wet"], 1e-4, "wet")
            assert_gradients(g, refg, refg64, GRAD_REL, "%s steps %d" % (case, steps))
    n = handed(tracer) - before
    tiles = ((o.shape[0] + 7) // 8) * ((o.shape[1] + 7) // 8) if o.shape[0] >= 8 else (o.shape[1] + 63) // 64
    assert 0 < n <= 2 * tiles, (n, tiles)
    if steps == 1 and case == "cube":
        assert n >= tiles // 2    # (both traces of the loop above; tiles that look past the cube end at the root)


def test_a_full_list_leaves_the_other_tiles_to_their_own_waves():
    """1024 x 776 pixels = 12416 tiles against a list of 8192: the waves that find no place trace their tile after
    all, and the next trace starts with an empty list again."""
    sc = S.scene_cube(P=10000, seed=0)
    o, d = S.pinhole_rays(776, 1024, 40.0, (2.2, 1.4, 1.0), (0.0, 0.0, 0.0))
    off = own_tracer("off")
    ref, _ = gpu_trace(off, sc, o, d, training=False)
    assert (ref["acc"] > 0.5).mean() > 0.7    # the cube fills the image: more tiles with work than the list holds
    tracer = own_tracer("always", 1)
    cap = tracer.optix_context.trace_info().handover_capacity
    for k in range(3):
        before = handed(tracer)
        out, _ = gpu_trace(tracer, sc, o, d, training=False, build=(k == 0))
        assert handed(tracer) - before == cap
        for name in ("rgb", "dpt", "acc", "norm", "mid"):
            assert np.array_equal(out[name].view(np.uint32), ref[name].view(np.uint32)), name


def test_a_captured_forward_with_hand_over_can_be_replayed():
    """Nothing on the host changes from one forward call to the next (the takers empty the list themselves), so the
    launch pair can be recorded into a graph once and replayed: every replay hands the same tiles over and gives the
    eager result, with eager work of the program between the replays."""
    from diff_surfel_tracing import _C
    sc = S.scene_cube(P=8000, seed=1)
    o, d = S.rays_cube(64, 80)
    g = {k: v.cuda() for k, v in sc.items()}
    e, bg, eye = torch.empty(0, device="cuda"), torch.zeros(3, device="cuda"), torch.eye(4, device="cuda")
    og, dg = o.cuda(), d.cuda()
    tracer = own_tracer("off")
    ctx = tracer.optix_context
    tracer.build_acceleration_structure(g["vertices"], g["faces"], True)

    def trace():
        return _C.trace_surfels(ctx, False, True, og, dg, g["vertices"], bg, g["means3D"], g["shs"], 3, e, e,
                                g["opacities"], g["scales"], 1.0, g["rotations"], e, eye, eye, bg, False, False, 0, 0.0)
    ref = [t.clone() for t in trace()[:4]]
    ctx.set_handover(_C.HANDOVER_ALWAYS, 40)
    before = handed(tracer)
    trace()
    per_trace = handed(tracer) - before
    assert per_trace > 10
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        trace()                                   # warm-up on a side stream, as torch asks before a capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = trace()
    for k in range(4):
        for t in out[:4]:
            t.fill_(-7.0)
        assert torch.isfinite(torch.randn(1000, device="cuda").sum()).item()   # eager work between the replays
        before = handed(tracer)
        graph.replay()
        torch.cuda.synchronize()
        assert handed(tracer) - before == per_trace, k
        for a, b in zip(out[:4], ref):
            assert torch.equal(a, b), k


def test_refits_recount_the_small_quads():
    """A structure built over ordinary quads and refitted to quads a thousand times smaller (and back): the count
    made by the refit arrives behind the first forward trace after it and switches the hand-over for the next ones."""
    tracer = own_tracer("auto")
    ctx = tracer.optix_context
    sc = S.scene_cube(P=9000, seed=2)
    o, d = S.rays_cube(32, 32)
    gpu_trace(tracer, sc, o, d, training=False)
    assert (ctx.trace_info().small_quads, ctx.trace_info().handover_active) == (0, 0)
    for shrink, want in ((1e-3, 8000), (1.0, 0)):
        moved = dict(sc)
        moved["scales"] = (sc["scales"] * shrink).contiguous()
        if shrink < 1.0:     # from the surfel parameters
            moved["vertices"] = tracer.refit_from_surfels(moved["means3D"].cuda(), moved["scales"].cuda(),
                                                          moved["rotations"].cuda()).cpu()
        else:                # from a vertex buffer
            moved["vertices"], _ = S.get_triangles(moved["means3D"], moved["scales"], moved["rotations"])
            tracer.build_acceleration_structure(moved["vertices"].cuda(), sc["faces"].cuda(), False)
        gpu_trace(tracer, moved, o, d, training=False, build=False)
        info = ctx.trace_info()
        assert (info.small_quads >= want if want else info.small_quads == 0), (shrink, info.small_quads)
        assert info.handover_active == (1 if want else 0)


def test_set_handover_rejects_unknown_modes():
    tracer = own_tracer("auto")
    with pytest.raises(RuntimeError):
        tracer.optix_context.set_handover(7)
    tracer.optix_context.set_handover(2, 123)
    info = tracer.optix_context.trace_info()
    assert (info.handover_mode, info.handover_steps) == (2, 123)
    tracer.optix_context.set_handover(1)
    assert tracer.optix_context.trace_info().handover_steps == 123
