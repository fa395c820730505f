"""Host-side checks that need no GPU: the C ABI library loads and exports every symbol the header declares,
the Python mirror of the parameter block has the compiled layout, and argument validation behaves like the
reference's (same exception types and messages: reference diff_surfel_tracing/__init__.py:256-261,
trace_surfels.cpp:23-24,44-49,193-195)."""
import ctypes as C
import os
import re
import subprocess

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dst_api.h")


@pytest.fixture(scope="module")
def binding():
    import diff_surfel_tracing._C as binding
    if not os.path.exists(binding.LIB_PATH):  # built by __graft_entry__.build(); only compile if nothing is there
        subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "diff-surfel-tracing_amd", "csrc")])
    return binding


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(dst_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(binding):
    lib = binding.load_library()
    names = declared_functions()
    assert {"dst_create", "dst_destroy", "dst_build_accel", "dst_trace_forward", "dst_trace_backward",
            "dst_last_error"} <= set(names)
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(binding.EXPORTS) == names
    assert lib.dst_version().startswith(b"dst-")


def test_parameter_block_layout_matches_the_header(binding):
    lib = binding.load_library()
    assert lib.dst_sizeof_params() == C.sizeof(binding.DstParams)
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    body = re.search(r"typedef struct DstParams \{(.*?)\} DstParams;", text, flags=re.S).group(1)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        fields += [re.findall(r"\w+", part)[-1] for part in decl.split(",")]
    assert fields == [f[0] for f in binding.DstParams._fields_]


def test_null_context_is_rejected_without_touching_a_device(binding):
    lib = binding.load_library()
    assert lib.dst_build_accel(None, None, 0, None, 0, 1, None) == 1
    assert lib.dst_trace_forward(None, None, None) == 1
    assert lib.dst_trace_backward(None, None, None) == 1
    assert lib.dst_last_error(None) == b"null context"
    lib.dst_destroy(None)


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-GPU failure mode")
def test_no_gpu_fails_loudly(binding):
    import diff_surfel_tracing as dst
    with pytest.raises(RuntimeError, match="GPU"):
        dst.SurfelTracer()


def test_settings_fields_and_defaults():
    import diff_surfel_tracing as dst
    assert dst.SurfelTracingSettings._fields == (
        "image_height", "image_width", "tanfovx", "tanfovy", "bg", "scale_modifier", "viewmatrix", "projmatrix",
        "sh_degree", "campos", "prefiltered", "debug", "max_trace_depth", "specular_threshold")
    s = dst.SurfelTracingSettings(1, 1, 1.0, 1.0, None, 1.0, None, None, 3, None, False, False)
    assert s.max_trace_depth == 0 and s.specular_threshold == 0.0


def test_forward_argument_checks_raise_like_the_reference():
    import diff_surfel_tracing as dst
    t = torch.zeros(4, 3)
    fwd = dst.SurfelTracer.forward
    with pytest.raises(Exception, match="Please provide excatly one of either SHs or precomputed colors!"):
        fwd(None, t, t, t, t, t, scales=t, rotations=t)
    with pytest.raises(Exception, match="Please provide excatly one of either SHs or precomputed colors!"):
        fwd(None, t, t, t, t, t, shs=t, colors_precomp=t, scales=t, rotations=t)
    msg = "Please provide exactly one of either scale/rotation pair or precomputed 3D covariance!"
    with pytest.raises(Exception, match=msg):
        fwd(None, t, t, t, t, t, shs=t, scales=t)
    with pytest.raises(Exception, match=msg):
        fwd(None, t, t, t, t, t, shs=t, scales=t, rotations=t, cov3D_precomp=t)


def test_launcher_tensor_contract(binding):
    e = torch.empty(0)
    ray = torch.zeros(2, 2, 3)
    v, m = torch.zeros(8, 3), torch.zeros(2, 3)
    args = [None, True, True, ray, ray, v, torch.zeros(3), m, e, 3, torch.zeros(2, 3), e, torch.zeros(2, 1),
            torch.zeros(2, 2), 1.0, torch.zeros(2, 4), e, e, e, e, False, False, 0, 0.0]
    with pytest.raises(RuntimeError, match="ray_o must be a CUDA tensor"):
        binding.trace_surfels(*args)
    bad = list(args)
    bad[7] = torch.zeros(2, 4)
    with pytest.raises(RuntimeError, match=r"means3D must have dimensions \(num_points, 3\)"):
        binding.trace_surfels(*bad)
    with pytest.raises(RuntimeError, match=r"vertices must have dimensions \(num_vertices, 3\)"):
        binding.build_acceleration_structure(None, torch.zeros(8, 2), torch.zeros(4, 3, dtype=torch.int32), True)
    with pytest.raises(RuntimeError, match=r"triangles must have dimensions \(num_triangles, 3\)"):
        binding.build_acceleration_structure(None, torch.zeros(8, 3), torch.zeros(4, dtype=torch.int32), True)


def test_scene_generators_have_the_documented_shapes():
    import dst_scenes as S
    for sc, P in ((S.scene_cube(P=64), 64), (S.scene_sphere(P=64), 64), (S.scene_room(P=200, aux=8), 200),
                  (S.scene_lidar(P=100, aux=4), 100)):
        assert sc["means3D"].shape == (P, 3) and sc["scales"].shape == (P, 2) and sc["rotations"].shape == (P, 4)
        assert sc["opacities"].shape == (P, 1) and sc["shs"].shape == (P, 16, 3)
        assert sc["vertices"].shape == (4 * P, 3) and sc["faces"].shape == (2 * P, 3)
        assert sc["faces"].dtype == torch.int32 and all(v.is_contiguous() for v in sc.values())
        assert torch.allclose(sc["rotations"].norm(dim=-1), torch.ones(P), atol=1e-5)
    o, d = S.rays_room(27, 48)
    assert o.shape == d.shape == (27, 48, 3) and torch.allclose(d.norm(dim=-1), torch.ones(27, 48), atol=1e-6)
    o, d = S.rays_lidar(4, 32)
    assert o.shape == d.shape == (1, 128, 3)
    a, b = S.scene_cube(P=32, seed=7), S.scene_cube(P=32, seed=7)
    assert all(torch.equal(a[k], b[k]) for k in a)   # seeded: identical on every machine


def test_bench_byte_formula_reproduces_the_documented_constants():
    """bench.py's general byte formula at the reference constants (aux 2, two mid slots, SH3, training) is
    204 + 40 n_proc + 208 n_con forward, 272 + 40 n_proc + 764 n_con backward, 316 per surfel."""
    import importlib.util
    import os
    spec = importlib.util.spec_from_file_location("bench", os.path.join(os.path.dirname(__file__), "..", "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    assert bench.algorithmic_bytes(2, 2) == ((204, 40, 208), (272, 40, 764), 316)
    fwd8, bwd8, per8 = bench.algorithmic_bytes(8, 3)            # config 4: aux 8, three mid slots
    assert fwd8[0] == 24 + 4 * (11 + 8 + 22 * 3) and fwd8[2] == 192 + 32 + 8 and per8 == 316 + 4 * 6
    assert sorted(bench.workloads()) == ["config1", "config2", "config3", "config4", "config5"]


class _FakeContext:
    """Stands in for OptiXStateWrapper in host tests: remembers whether a hit record was asked for."""

    def __init__(self):
        self.record_wanted = True
        self.acquired = 0
        self.released = 0

    def acquire_record(self, H, W, mtd_alloc, device, max_trace_depth=None):
        self.acquired += 1
        return None   # "too large": the backward pass would walk the BVH again

    def release_record(self, rec):
        self.released += 1


def test_no_hit_record_is_made_when_no_backward_can_follow(monkeypatch):
    """Evaluation loops render nn.Parameter tensors under torch.no_grad(): `needs_input_grad` is still set inside
    the autograd function then, so the wrapper must look at the gradient mode before the call."""
    import diff_surfel_tracing as dst
    from diff_surfel_tracing import _C

    def fake_trace(ctx, training, sff, ray_o, *rest, hit_record=None):
        H, W = ray_o.shape[:2]
        z = lambda c: torch.zeros(H, W, c)  # noqa: E731
        return z(3), z(1), z(1), z(3), z(3), z(2), z(32), None

    monkeypatch.setattr(_C, "trace_surfels", fake_trace)
    eye = torch.eye(4)
    st = dst.SurfelTracingSettings(4, 4, 1.0, 1.0, torch.zeros(3), 1.0, eye, eye, 3, torch.zeros(3), False, False)
    P = 5
    means = torch.nn.Parameter(torch.zeros(P, 3))
    args = lambda ctx: (ctx, True, True, torch.zeros(4, 4, 3), torch.zeros(4, 4, 3), torch.zeros(4 * P, 3), means,  # noqa: E731
                        torch.zeros(P, 3), torch.zeros(P, 16, 3), torch.empty(0), torch.empty(0),
                        torch.zeros(P, 1), torch.ones(P, 2), torch.zeros(P, 4), torch.empty(0), st)
    ctx = _FakeContext()
    with torch.no_grad():
        dst.trace_surfels(*args(ctx))
    assert ctx.acquired == 0
    dst.trace_surfels(*args(ctx))
    assert ctx.acquired == 1
    ctx2 = _FakeContext()
    plain = list(args(ctx2))
    plain[6] = torch.zeros(P, 3)       # no input asks for a gradient
    dst.trace_surfels(*plain)
    assert ctx2.acquired == 0


def test_record_pool_takes_back_records_of_any_size():
    """The pool of hit-record storages keeps the largest RECORD_POOL_SIZE tensors; returning one more, of any size
    (training at several resolutions does that), drops the smallest and must not compare tensors by value."""
    from diff_surfel_tracing import _C

    class _Rec:
        def __init__(self, n):
            self.words = torch.zeros(n, dtype=torch.int64)

    pool = _C.OptiXStateWrapper.__new__(_C.OptiXStateWrapper)   # no device: only the pool's bookkeeping is used
    pool._record_pool, pool._record_fixed, pool._record_events = [], False, {}
    pool.record_pool_max_bytes = 1 << 40
    sizes = [7, 3, 9, 3, 5, 11, 2, 9]
    recs = [_Rec(n) for n in sizes]
    for r in recs:
        pool.release_record(r)
        assert r.words is None
    kept = sorted(t.numel() for t in pool._record_pool)
    assert kept == sorted(sizes)[-_C.OptiXStateWrapper.RECORD_POOL_SIZE:]
    pool.release_record(recs[0])    # a record already handed back is ignored
    pool.release_record(None)
    assert len(pool._record_pool) == _C.OptiXStateWrapper.RECORD_POOL_SIZE
    # the free storages are also bounded in bytes, whatever their number: the smallest go first, one always stays
    pool.record_pool_max_bytes = 8 * 21
    pool.release_record(_Rec(1))
    assert sorted(t.numel() for t in pool._record_pool) == [9, 11]
    pool.record_pool_max_bytes = 8
    pool.release_record(_Rec(4))
    assert [t.numel() for t in pool._record_pool] == [11]
