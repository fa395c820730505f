"""ctypes binding of libdst.so, shaped like the compiled `_C` module of the reference package
(reference ext.cpp:7-12): `OptiXStateWrapper`, `build_acceleration_structure`, `trace_surfels`,
`trace_surfels_backward` with the same positional arguments and return tuples
(reference trace_surfels.h:10-83).  There is no fallback: a missing library raises.
"""
import ctypes as C
import os
import warnings

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libdst.so")

NUM_CHANNELS = 3          # reference optix_tracer/config.h:5
DEFAULT_AUX_CHANNELS = 2  # reference optix_tracer/config.h:6
DEFAULT_MAX_TRACE_DEPTH = 1  # reference optix_tracer/config.h:27: mid_val always holds at least two slots
MAX_AUX_CHANNELS = 8
MAX_TRACE_DEPTH = 3
FLAG_DETERMINISTIC = 1
FLAG_DISTORTION = 2
FLAG_SH_HALF = 4

_FP = C.c_void_p


class DstParams(C.Structure):
    """Field-for-field mirror of `DstParams` in include/dst_api.h."""
    _fields_ = (
        [(n, C.c_int32) for n in ("P", "H", "W", "D", "M", "aux", "mtd_alloc", "max_trace_depth", "training",
                                  "start_from_first")]
        + [("specular_threshold", C.c_float), ("scale_modifier", C.c_float)]
        + [(n, _FP) for n in ("ray_o", "ray_d", "vertices", "background", "means3D", "shs", "colors_precomp",
                              "others_precomp", "opacities", "scales", "rotations")]
        + [(n, _FP) for n in ("out_rgb", "out_dpt", "out_acc", "out_norm", "out_dist", "out_aux", "mid_val",
                              "a_weights", "counters", "hit_record")]
        + [("hit_record_blocks", C.c_uint32), ("flags", C.c_uint32), ("det_workspace", _FP), ("grad_rows", _FP)]
        + [(n, _FP) for n in ("dL_drgb", "dL_ddpt", "dL_dacc", "dL_ddist", "dL_dnorm", "dL_daux")]
        + [(n, _FP) for n in ("dL_dray_o", "dL_dray_d", "dL_dmeans3D", "dL_dgrads3D", "dL_dshs", "dL_dcolors",
                              "dL_dothers", "dL_dopacities", "dL_dscales", "dL_drotations")]
        + [("shs_half", _FP)]
    )


class DstAccelInfo(C.Structure):
    _fields_ = [("n_surfels", C.c_uint32), ("n_internal", C.c_uint32), ("root", C.c_uint32),
                ("node_bytes", C.c_uint32), ("leaf_bytes", C.c_uint32), ("scene_lo", C.c_float * 3),
                ("scene_hi", C.c_float * 3), ("max_abs", C.c_float), ("builds", C.c_uint32), ("refits", C.c_uint32),
                ("key_levels", C.c_uint32), ("agglomerated", C.c_uint32), ("depth", C.c_uint32)]


class DstTraceInfo(C.Structure):
    _fields_ = [("handover_mode", C.c_uint32), ("handover_steps", C.c_uint32), ("handover_capacity", C.c_uint32),
                ("small_quads", C.c_uint32), ("handover_active", C.c_uint32), ("det_out_of_range", C.c_uint32),
                ("tiles_handed_over", C.c_uint64)]


HANDOVER_OFF, HANDOVER_AUTO, HANDOVER_ALWAYS = 0, 1, 2


EXPORTS = ("dst_create", "dst_destroy", "dst_build_accel", "dst_trace_forward", "dst_trace_backward",
           "dst_last_error", "dst_accel_info", "dst_accel_download", "dst_version", "dst_sizeof_params",
           "dst_hit_record_layout", "dst_refit_accel_static", "dst_refit_from_surfels",
           "dst_det_workspace_words", "dst_pack_sh_half", "dst_trace_info", "dst_set_handover")

_lib = None


def load_library():
    """Load libdst.so (once) and declare its prototypes.  Raises if the library is absent or stale."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("diff_surfel_tracing: %s is missing; build it with `make -C csrc` (hipcc, gfx950). "
                          "There is no CPU or PyTorch fallback." % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    L.dst_create.restype = C.c_void_p
    L.dst_create.argtypes = []
    L.dst_destroy.restype = None
    L.dst_destroy.argtypes = [C.c_void_p]
    L.dst_build_accel.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint32, C.c_int, C.c_void_p]
    L.dst_refit_accel_static.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p]
    L.dst_refit_from_surfels.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p,
                                         C.c_void_p]
    L.dst_trace_forward.argtypes = [C.c_void_p, C.POINTER(DstParams), C.c_void_p]
    L.dst_trace_backward.argtypes = [C.c_void_p, C.POINTER(DstParams), C.c_void_p]
    L.dst_last_error.restype = C.c_char_p
    L.dst_last_error.argtypes = [C.c_void_p]
    L.dst_accel_info.argtypes = [C.c_void_p, C.POINTER(DstAccelInfo)]
    L.dst_accel_download.argtypes = [C.c_void_p] * 7
    L.dst_trace_info.argtypes = [C.c_void_p, C.POINTER(DstTraceInfo)]
    L.dst_set_handover.argtypes = [C.c_void_p, C.c_int, C.c_uint32]
    L.dst_det_workspace_words.restype = C.c_uint64
    L.dst_det_workspace_words.argtypes = [C.c_int32, C.c_int32, C.c_int]
    L.dst_pack_sh_half.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p]
    L.dst_version.restype = C.c_char_p
    L.dst_sizeof_params.restype = C.c_size_t
    L.dst_hit_record_layout.restype = C.c_uint64
    L.dst_hit_record_layout.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_uint32, C.POINTER(C.c_uint64),
                                        C.POINTER(C.c_uint32)]
    if L.dst_sizeof_params() != C.sizeof(DstParams):
        raise ImportError("diff_surfel_tracing: DstParams layout mismatch between _C.py and libdst.so")
    _lib = L
    return L


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(ctx, rc):
    if rc != 0:
        msg = load_library().dst_last_error(ctx.handle)
        raise RuntimeError((msg or b"unknown error").decode() + " (status %d)" % rc)


def _cuda_f32(t, name):
    """The launcher's tensor contract: CUDA, fp32, contiguous (reference trace_surfels.cpp:23-24,252-277)."""
    if not isinstance(t, torch.Tensor):
        raise RuntimeError("%s must be a tensor" % name)
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if t.dtype != torch.float32:
        t = t.float()
    return t.contiguous()


def _ptr(t):
    return None if t is None or t.numel() == 0 else t.data_ptr()


class HitRecord:
    """Device buffer in which a forward trace stores its per-chunk hit buffers so that the backward trace can
    replay them instead of walking the BVH again (see `hit_record` in include/dst_api.h).  `storage` is a
    caller- or pool-owned int64 tensor that is at least `words_needed(...)` long."""

    @staticmethod
    def layout(H, W, mtd_alloc, blocks_per_wave):
        """(words of the whole buffer, header words, blocks, waves) for an (H,W) ray grid."""
        header, waves = C.c_uint64(0), C.c_uint32(0)
        lib = load_library()
        lib.dst_hit_record_layout(H, W, mtd_alloc, 0, C.byref(header), C.byref(waves))
        n_waves = max(1, waves.value)
        blocks = max(1, int(n_waves * blocks_per_wave) + 1)
        words = lib.dst_hit_record_layout(H, W, mtd_alloc, blocks, None, None)
        return int(words), int(header.value), blocks, n_waves

    def __init__(self, H, W, mtd_alloc, blocks_per_wave, device, storage=None):
        words, header, self.blocks, self.n_waves = self.layout(H, W, mtd_alloc, blocks_per_wave)
        if storage is None:
            storage = torch.empty(words, dtype=torch.int64, device=device)
        elif storage.numel() < words or storage.dtype != torch.int64 or not storage.is_cuda:
            raise RuntimeError("hit record storage must be a CUDA int64 tensor of at least %d elements" % words)
        self.words = storage
        self.words[:header].zero_()
        self._asked_host = None
        self._asked_event = None

    def note_request(self):
        """Stream-ordered, non-blocking copy of word 0 (blocks the forward trace asked for) to pinned host
        memory; `asked()` reads it once the copy has happened."""
        self._asked_host = torch.empty(1, dtype=torch.int64, pin_memory=True)
        self._asked_host.copy_(self.words[:1], non_blocking=True)
        self._asked_event = torch.cuda.Event()
        self._asked_event.record()

    def asked(self, wait=False):
        """Blocks requested by the forward trace, or None while that is not known yet (never waits unless told to)."""
        if self._asked_event is None:
            return int(self.words[0].item()) if wait else None
        if wait:
            self._asked_event.synchronize()
        elif not self._asked_event.query():
            return None
        return int(self._asked_host[0])

    def requested_blocks(self):
        """Blocks the forward trace asked for (waits for it to finish)."""
        return self.asked(wait=True)

    def complete(self):
        return self.requested_blocks() <= self.blocks

    def broken_chains(self):
        """Chains a replaying backward trace found broken (waits); 0 for every record a forward trace wrote."""
        return int(self.words[1].item())


class OptiXStateWrapper:
    """Owner of the acceleration structure; keeps the reference's class name (ext.cpp:8) so callers need not
    change.  `pkg_dir` was where the reference looked for its PTX files and is ignored.

    Also owns the hit-record buffers of the autograd path: a small pool that forward calls draw from and
    backward calls return to (no allocation per call once warm), bounded by `record_max_bytes` per record and
    `record_pool_max_bytes` for the free storages together; a record that would be larger, or whose allocation
    fails, is not made and the backward pass walks the BVH again (`records_skipped` counts those calls, the first
    one warns)."""

    RECORD_POOL_SIZE = 4
    RECORD_FIRST_BLOCKS = 5.0   # blocks per wave and bounce before a forward trace has said what it needs
    RECORD_HEADROOM = 1.08      # a record is sized this much above the largest request seen so far

    def __init__(self, pkg_dir=None):
        lib = load_library()
        if not torch.cuda.is_available():
            raise RuntimeError("diff_surfel_tracing needs a GPU: no HIP device is visible")
        self.handle = lib.dst_create()
        if not self.handle:
            raise RuntimeError("dst_create failed: no usable HIP device")
        self.device = torch.cuda.current_device()
        self.num_surfels = 0
        self.record_blocks_per_wave = None  # sizing estimate for hit records: largest request seen, with headroom
        self.record_max_bytes = 32 << 30    # no record larger than this is made (backward then re-traces); a 4K image
                                            # of the 1M-surfel room scene needs 13 GB, of the card's 288
        self.record_pool_max_bytes = 48 << 30   # free storages kept for reuse, all together
        self.records_skipped = 0            # forward calls that made no record because of the two limits above
        self.record_wanted = True           # set by the autograd wrapper for the call that follows
        self.deterministic = False          # True: a_weights and per-surfel gradients are bitwise reproducible
        self.deterministic_check = True     # with `deterministic`: warn after a backward trace whose sums left the range
        self._det_out_of_range = 0          # the library's count when last looked at
        self.gradient_rows = True           # backward sums per-surfel gradients in one row per surfel first (faster)
        self.distortion = False             # True: the dist output carries the 2DGS depth distortion (else zeros)
        self.sh_half = False                # True: the traces read the SH coefficients from a binary16 copy
        self._record_pool = []              # free storages (int64 tensors)
        self._record_events = {}            # id(storage) -> event recorded when the storage came back
        self._record_fixed = False          # True: only caller-provided storage is used, nothing is allocated
        self._record_watch = []             # records whose request count has not been read yet

    # ---- hit-record storage ---------------------------------------------------------------------------
    def use_record_storage(self, storage):
        """Use this caller-owned int64 CUDA tensor (and nothing else) for hit records; None returns to the
        pool.  One record is live at a time with a fixed storage: a forward call that finds it taken, or too
        small (HitRecord.layout gives the size), makes no record."""
        self._record_pool = [] if storage is None else [storage]
        self._record_fixed = storage is not None

    def update_record_estimate(self):
        """Raise the sizing estimate from records whose forward trace has finished.  Never waits, except in the
        deterministic mode: whether a backward trace replays a complete record or walks the BVH again changes its
        gradients in the last bit (the two kernels contract their gradient algebra differently), so there the
        sequence of record sizes must not depend on timing."""
        still = []
        for rec in self._record_watch:
            asked = rec.asked(wait=self.deterministic)
            if asked is None:
                still.append(rec)
            else:
                self.record_blocks_per_wave = max(self.record_blocks_per_wave or 0.0,
                                                  self.RECORD_HEADROOM * asked / rec.n_waves)
        self._record_watch = still[-8:]

    def acquire_record(self, H, W, mtd_alloc, device, max_trace_depth=None):
        """A record for an (H,W) grid traced with `mtd_alloc` mid_val slots - 1, or None.  Sized from what earlier
        forward traces asked for (with a little headroom); before any has finished, for RECORD_FIRST_BLOCKS blocks
        per wave and bounce actually traced (`max_trace_depth` + 1; `mtd_alloc` + 1 if that is not given): every bounce
        of a path opens at least one block per wave, so a multi-bounce run can replay from its first step."""
        self.update_record_estimate()
        per_wave = self.record_blocks_per_wave
        if per_wave is None:
            bounces = (mtd_alloc if max_trace_depth is None else max_trace_depth) + 1
            per_wave = self.RECORD_FIRST_BLOCKS * bounces
        words = HitRecord.layout(H, W, mtd_alloc, per_wave)[0]
        if 8 * words > self.record_max_bytes:
            self.records_skipped += 1
            if self.records_skipped == 1:
                warnings.warn("diff_surfel_tracing: a hit record for this %dx%d trace would take %.1f GiB (limit "
                              "record_max_bytes = %.1f GiB); backward passes walk the BVH again instead of replaying"
                              % (H, W, 8 * words / 2 ** 30, self.record_max_bytes / 2 ** 30))
            return None
        device = torch.device(device)
        if device.index is None:
            device = torch.device(device.type, torch.cuda.current_device())
        fit = [t for t in self._record_pool if t.numel() >= words and t.device == device]
        storage = None
        if fit:
            storage = min(fit, key=lambda t: t.numel())
            self._record_pool = [t for t in self._record_pool if t is not storage]
            # the backward trace that last read this storage may still be running on another stream
            done = self._record_events.pop(id(storage), None)
            if done is not None:
                torch.cuda.current_stream().wait_event(done)
        elif self._record_fixed:
            return None
        else:
            try:
                storage = torch.empty(words, dtype=torch.int64, device=device)
            except torch.OutOfMemoryError:
                self.records_skipped += 1
                return None
        return HitRecord(H, W, mtd_alloc, per_wave, device, storage=storage)

    def release_record(self, rec):
        """Back to the pool.  The storage's last reader (a backward trace just enqueued on the current stream) is
        marked with an event that the next user waits for, whatever stream that user runs on."""
        if rec is None or rec.words is None:
            return
        if rec.words.is_cuda:
            done = torch.cuda.Event()
            done.record()
            self._record_events[id(rec.words)] = done
        self._record_pool.append(rec.words)
        rec.words = None
        if self._record_fixed:
            return
        # by identity: list.remove() would compare tensors element-wise
        while len(self._record_pool) > 1 and (len(self._record_pool) > self.RECORD_POOL_SIZE or
                                              8 * sum(t.numel() for t in self._record_pool) > self.record_pool_max_bytes):
            smallest = min(self._record_pool, key=lambda t: t.numel())
            self._record_pool = [t for t in self._record_pool if t is not smallest]
            self._record_events.pop(id(smallest), None)

    def accel_info(self):
        info = DstAccelInfo()
        _check(self, load_library().dst_accel_info(self.handle, C.byref(info)))
        return info

    def trace_info(self):
        """Tile hand-over of the forward trace (include/dst_api.h): mode, step limit, list capacity, the small quads the
        last build counted, whether the next forward trace can hand over, tiles handed over so far; and the number of
        sums the deterministic mode has found out of its fixed-point range.  Waits."""
        info = DstTraceInfo()
        _check(self, load_library().dst_trace_info(self.handle, C.byref(info)))
        return info

    def check_deterministic_range(self):
        """Warn if sums of the deterministic mode have left their fixed-point range since the last look (gradients
        beyond about 6.7e7 for scales, rotations and means, 4.2e6 for the rest: they come out clamped or wrapped).
        Waits for the device.  Returns the number of such sums."""
        seen = int(self.trace_info().det_out_of_range)
        new, self._det_out_of_range = (seen - self._det_out_of_range) & 0xFFFFFFFF, seen
        if new:
            warnings.warn("deterministic mode: %d per-surfel sums left the fixed-point range and are wrong; scale the "
                          "loss down or trace without the mode" % new, RuntimeWarning, stacklevel=3)
        return new

    def set_handover(self, mode, steps=0):
        """HANDOVER_OFF / HANDOVER_AUTO (only for scenes with many quads far smaller than the scene) / HANDOVER_ALWAYS;
        `steps`: what a tile's first packet walk may take before its rays are walked one by one (0: unchanged)."""
        _check(self, load_library().dst_set_handover(self.handle, int(mode), int(steps)))

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h and _lib is not None:
            _lib.dst_destroy(h)


def build_acceleration_structure(ctx, vertices, triangles, rebuild):
    """Reference BuildAccelerationStructure (trace_surfels.cpp:36-159)."""
    if vertices.dim() != 2 or vertices.size(1) != 3:
        raise RuntimeError("vertices must have dimensions (num_vertices, 3)")
    if triangles.dim() != 2 or triangles.size(1) != 3:
        raise RuntimeError("triangles must have dimensions (num_triangles, 3)")
    v = _cuda_f32(vertices, "vertices")
    if not triangles.is_cuda:
        raise RuntimeError("triangles must be a CUDA tensor")
    f = triangles.to(torch.int32).contiguous()
    rc = load_library().dst_build_accel(ctx.handle, v.data_ptr(), v.size(0), f.data_ptr(), f.size(0),
                                        int(bool(rebuild)), _stream())
    _check(ctx, rc)
    ctx.num_surfels = f.size(0) // 2


def refit_from_surfels(ctx, means3D, scales, rotations, vertices_out=None):
    """Refit the structure straight from the surfel parameters (dst_refit_from_surfels in include/dst_api.h) and
    return the quad corners (4P,3) the trace calls take as `vertices`, written by the same kernel.  No counterpart
    in the reference, whose callers regenerate the quads with tensor operations and then call
    build_acceleration_structure(v, f, rebuild=False)."""
    m, s, q = _cuda_f32(means3D, "means3D"), _cuda_f32(scales, "scales"), _cuda_f32(rotations, "rotations")
    P = m.size(0)
    if m.dim() != 2 or m.size(1) != 3 or tuple(s.shape) != (P, 2) or tuple(q.shape) != (P, 4):
        raise RuntimeError("means3D (P,3), scales (P,2) and rotations (P,4) are required")
    if vertices_out is None:
        vertices_out = torch.empty((4 * P, 3), dtype=torch.float32, device=m.device)
    elif (not vertices_out.is_cuda or vertices_out.dtype != torch.float32 or not vertices_out.is_contiguous()
          or vertices_out.numel() != 12 * P):
        raise RuntimeError("vertices_out must be a contiguous CUDA float32 tensor of shape (4P,3)")
    rc = load_library().dst_refit_from_surfels(ctx.handle, m.data_ptr(), s.data_ptr(), q.data_ptr(), P,
                                               vertices_out.data_ptr(), _stream())
    _check(ctx, rc)
    return vertices_out


def pack_sh_half(shs):
    """binary16 copy of an fp32 CUDA tensor of SH coefficients (dst_pack_sh_half: round to nearest even)."""
    shs = _cuda_f32(shs, "shs")
    out = torch.empty(shs.shape, dtype=torch.float16, device=shs.device)
    rc = load_library().dst_pack_sh_half(shs.data_ptr(), out.data_ptr(), shs.numel(), _stream())
    if rc != 0:
        raise RuntimeError("dst_pack_sh_half failed (status %d)" % rc)
    return out


def _use_sh_half(ctx, p, keep):
    """With `ctx.sh_half` set and SH coefficients given: pack them and point the launch parameters at the copy."""
    if getattr(ctx, "sh_half", False) and keep["shs"].numel() != 0:
        keep["shs_half"] = pack_sh_half(keep["shs"])
        p.shs_half = keep["shs_half"].data_ptr()
        p.flags |= FLAG_SH_HALF


def _common_params(ray_o, ray_d, vertices, background, means3D, shs, degree, colors_precomp, others_precomp,
                   opacities, scales, scale_modifier, rotations, max_trace_depth, specular_threshold,
                   start_from_first):
    if means3D.dim() != 2 or means3D.size(1) != 3:
        raise RuntimeError("means3D must have dimensions (num_points, 3)")
    t = {
        "ray_o": _cuda_f32(ray_o, "ray_o"), "ray_d": _cuda_f32(ray_d, "ray_d"),
        "vertices": _cuda_f32(vertices, "vertices"), "background": _cuda_f32(background, "background"),
        "means3D": _cuda_f32(means3D, "means3D"), "shs": _cuda_f32(shs, "shs"),
        "colors_precomp": _cuda_f32(colors_precomp, "colors_precomp"),
        "others_precomp": _cuda_f32(others_precomp, "others_precomp"),
        "opacities": _cuda_f32(opacities, "opacities"), "scales": _cuda_f32(scales, "scales"),
        "rotations": _cuda_f32(rotations, "rotations"),
    }
    if t["ray_o"].dim() != 3 or t["ray_o"].size(2) != 3 or t["ray_d"].shape != t["ray_o"].shape:
        raise RuntimeError("ray_o and ray_d must have the same dimensions (H, W, 3) or (B, P, 3)")
    if t["scales"].numel() == 0 or t["rotations"].numel() == 0:
        raise RuntimeError("scales and rotations are required (a precomputed 3D covariance is not consumed by "
                           "the tracer)")
    p = DstParams()
    p.P, p.H, p.W = means3D.size(0), t["ray_o"].size(0), t["ray_o"].size(1)
    p.D = int(degree)
    p.M = t["shs"].size(1) if t["shs"].numel() != 0 else 0
    p.aux = t["others_precomp"].size(1) if t["others_precomp"].numel() != 0 else DEFAULT_AUX_CHANNELS
    p.max_trace_depth = int(max_trace_depth)
    p.mtd_alloc = max(DEFAULT_MAX_TRACE_DEPTH, p.max_trace_depth)
    p.start_from_first = int(bool(start_from_first))
    p.specular_threshold = float(specular_threshold)
    p.scale_modifier = float(scale_modifier)
    for name, ten in t.items():
        setattr(p, name, _ptr(ten))
    return p, t


def trace_surfels(ctx, training, start_from_first, ray_o, ray_d, vertices, background, means3D, shs, degree,
                  colors_precomp, others_precomp, opacities, scales, scale_modifier, rotations, transMat_precomp,
                  viewmatrix, projmatrix, campos, prefiltered, debug, max_trace_depth, specular_threshold,
                  counters=None, events=None, hit_record=None):
    """Reference TraceSurfelsCUDA (trace_surfels.cpp:162-304): returns
    (out_rgb, out_dpt, out_acc, out_norm, out_dist, out_aux, mid_val, a_weights or None).
    Extras for measurement: `counters` (2 int64 on the device) receives the evaluated / composited hit totals;
    `events` (two torch.cuda.Event) are recorded on the launch stream right around the kernel launch;
    `hit_record` (a HitRecord) receives the hit buffers for a later replay by trace_surfels_backward."""
    p, keep = _common_params(ray_o, ray_d, vertices, background, means3D, shs, degree, colors_precomp,
                             others_precomp, opacities, scales, scale_modifier, rotations, max_trace_depth,
                             specular_threshold, start_from_first)
    H, W, P, dev = p.H, p.W, p.P, means3D.device
    mid_ch = (14 + p.aux) * (p.mtd_alloc + 1)
    new = lambda *shape: torch.empty(shape, dtype=torch.float32, device=dev)  # noqa: E731 (kernel writes every element)
    out_rgb, out_dpt, out_acc = new(H, W, NUM_CHANNELS), new(H, W, 1), new(H, W, 1)
    out_norm, out_dist, out_aux, mid_val = new(H, W, 3), new(H, W, 3), new(H, W, p.aux), new(H, W, mid_ch)
    a_weights = torch.zeros((P, 1), dtype=torch.float32, device=dev) if training else None
    p.training = int(bool(training))
    p.out_rgb, p.out_dpt, p.out_acc = out_rgb.data_ptr(), out_dpt.data_ptr(), out_acc.data_ptr()
    p.out_norm, p.out_dist, p.out_aux = out_norm.data_ptr(), out_dist.data_ptr(), out_aux.data_ptr()
    p.mid_val = mid_val.data_ptr()
    p.a_weights = _ptr(a_weights)
    p.counters = _ptr(counters)
    if hit_record is not None:
        p.hit_record, p.hit_record_blocks = hit_record.words.data_ptr(), hit_record.blocks
    det_ws = None
    if getattr(ctx, "deterministic", False) and training:
        det_ws = torch.zeros(load_library().dst_det_workspace_words(P, p.aux, 0), dtype=torch.int64, device=dev)
        p.flags, p.det_workspace = FLAG_DETERMINISTIC, det_ws.data_ptr()
    if getattr(ctx, "distortion", False):
        p.flags |= FLAG_DISTORTION
    _use_sh_half(ctx, p, keep)
    if events is not None:
        events[0].record()
    _check(ctx, load_library().dst_trace_forward(ctx.handle, C.byref(p), _stream()))
    if events is not None:
        events[1].record()
    if hit_record is not None:
        hit_record.note_request()
        ctx._record_watch.append(hit_record)
    del keep
    return out_rgb, out_dpt, out_acc, out_norm, out_dist, out_aux, mid_val, a_weights


def trace_surfels_backward(ctx, start_from_first, ray_o, ray_d, vertices, background, means3D, shs, degree,
                           colors_precomp, others_precomp, opacities, scales, scale_modifier, rotations,
                           transMat_precomp, viewmatrix, projmatrix, campos, prefiltered, debug, max_trace_depth,
                           specular_threshold, out_rgb, out_dpt, out_acc, out_norm, out_dist, out_aux, mid_val,
                           dL_dout_rgb, dL_dout_dpt, dL_dout_acc, dL_dout_norm, dL_dout_dist, dL_dout_aux,
                           events=None, hit_record=None, counters=None):
    """Reference TraceSurfelsBackwardCUDA (trace_surfels.cpp:307-464): returns (dL_dray_o, dL_dray_d, dL_dmeans3D,
    dL_dgrads3D, dL_dgrads3D_abs, dL_dshs, dL_dcolors, dL_dothers, dL_dopacities, dL_dscales, dL_drotations,
    dL_dtransMat_precomp)."""
    p, keep = _common_params(ray_o, ray_d, vertices, background, means3D, shs, degree, colors_precomp,
                             others_precomp, opacities, scales, scale_modifier, rotations, max_trace_depth,
                             specular_threshold, start_from_first)
    H, W, P, dev = p.H, p.W, p.P, means3D.device
    saved = [_cuda_f32(x, n) for x, n in ((out_rgb, "out_rgb"), (out_dpt, "out_dpt"), (out_acc, "out_acc"),
                                          (out_norm, "out_norm"), (out_dist, "out_dist"), (out_aux, "out_aux"),
                                          (mid_val, "mid_val"))]
    mid_ch = (14 + p.aux) * (p.mtd_alloc + 1)
    if saved[6].numel() != H * W * mid_ch or saved[5].numel() != H * W * p.aux:
        raise RuntimeError("mid_val / out_aux do not match the settings they were traced with")
    p.out_rgb, p.out_dpt, p.out_acc, p.out_norm, p.out_dist, p.out_aux, p.mid_val = [x.data_ptr() for x in saved]
    ups = [_cuda_f32(x, n) for x, n in ((dL_dout_rgb, "dL_dout_rgb"), (dL_dout_dpt, "dL_dout_dpt"),
                                        (dL_dout_acc, "dL_dout_acc"), (dL_dout_norm, "dL_dout_norm"),
                                        (dL_dout_dist, "dL_dout_dist"), (dL_dout_aux, "dL_dout_aux"))]
    want = (3, 1, 1, 3, None, p.aux)
    for x, ch, n in zip(ups, want, ("rgb", "dpt", "acc", "norm", "dist", "aux")):
        if ch is not None and x.numel() != H * W * ch:
            raise RuntimeError("upstream gradient of %s has the wrong size" % n)
    p.dL_drgb, p.dL_ddpt, p.dL_dacc, p.dL_dnorm, p.dL_ddist, p.dL_daux = (
        ups[0].data_ptr(), ups[1].data_ptr(), ups[2].data_ptr(), ups[3].data_ptr(), _ptr(ups[4]), ups[5].data_ptr())
    zeros = lambda *shape: torch.zeros(shape, dtype=torch.float32, device=dev)  # noqa: E731 (atomically accumulated)
    dL_dray_o = torch.empty((H, W, 3), dtype=torch.float32, device=dev)
    dL_dray_d = torch.empty((H, W, 3), dtype=torch.float32, device=dev)
    dL_dmeans3D, dL_dgrads3D, dL_dgrads3D_abs = zeros(P, 3), zeros(P, 3), zeros(P, 3)
    dL_dshs, dL_dcolors, dL_dothers = zeros(P, p.M, 3), zeros(P, NUM_CHANNELS), zeros(P, p.aux)
    dL_dopacities, dL_dscales, dL_drotations = zeros(P, 1), zeros(P, 2), zeros(P, 4)
    dL_dtransMat = zeros(P, 9)
    p.dL_dray_o, p.dL_dray_d = dL_dray_o.data_ptr(), dL_dray_d.data_ptr()
    p.dL_dmeans3D, p.dL_dgrads3D, p.dL_dshs = dL_dmeans3D.data_ptr(), dL_dgrads3D.data_ptr(), _ptr(dL_dshs)
    p.dL_dcolors, p.dL_dothers = dL_dcolors.data_ptr(), dL_dothers.data_ptr()
    p.dL_dopacities, p.dL_dscales, p.dL_drotations = (dL_dopacities.data_ptr(), dL_dscales.data_ptr(),
                                                      dL_drotations.data_ptr())
    if hit_record is not None:
        # the kernels decide on the device whether the record is complete (replay) or not (walk the BVH again):
        # nothing here waits for the forward trace
        p.hit_record, p.hit_record_blocks = hit_record.words.data_ptr(), hit_record.blocks
    p.counters = _ptr(counters)
    det_ws = None
    if getattr(ctx, "deterministic", False):
        det_ws = torch.zeros(load_library().dst_det_workspace_words(P, p.aux, 1), dtype=torch.int64, device=dev)
        p.flags, p.det_workspace = FLAG_DETERMINISTIC, det_ws.data_ptr()
    elif getattr(ctx, "gradient_rows", True):
        # the per-surfel gradients are summed in rows of one buffer first (a surfel's columns side by side)
        det_ws = torch.zeros(load_library().dst_det_workspace_words(P, p.aux, 1), dtype=torch.float32, device=dev)
        p.grad_rows = det_ws.data_ptr()
    if getattr(ctx, "sh_half", False) and keep["shs"].numel() != 0:
        # the backward trace reads fp32 coefficients: the values the forward trace used
        keep["shs"] = pack_sh_half(keep["shs"]).float()
        p.shs = keep["shs"].data_ptr()
    if events is not None:
        events[0].record()
    _check(ctx, load_library().dst_trace_backward(ctx.handle, C.byref(p), _stream()))
    if events is not None:
        events[1].record()
    if p.flags & FLAG_DETERMINISTIC and getattr(ctx, "deterministic_check", False):
        ctx.check_deterministic_range()   # (the mode waits for the device elsewhere too: record sizes)
    del keep
    return (dL_dray_o, dL_dray_d, dL_dmeans3D, dL_dgrads3D, dL_dgrads3D_abs, dL_dshs, dL_dcolors, dL_dothers,
            dL_dopacities, dL_dscales, dL_drotations, dL_dtransMat)
