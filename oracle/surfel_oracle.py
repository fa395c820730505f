"""ctypes front end of the CPU oracle (test infrastructure only).

Only tests, the smoke check and the benchmark's cpu_baseline leg import this
module; the shipped package never does.  Arrays are numpy, fp32 / int32,
C-contiguous.  Field names follow surfel_oracle.h.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsurfel_oracle.so")

HITS_BRUTE_LITERAL, HITS_BRUTE_LEXI, HITS_BVH_LEXI = 0, 1, 2

_FP = C.POINTER(C.c_float)
_IP = C.POINTER(C.c_int32)


class OracleParams(C.Structure):
    _fields_ = (
        [(n, C.c_int32) for n in ("P", "H", "W", "D", "M", "aux", "mtd_alloc", "training", "start_from_first",
                                  "max_trace_depth")]
        + [("specular_threshold", C.c_float)]
        + [(n, C.c_int32) for n in ("hit_mode", "literal_stale", "n_threads", "compute_dist", "grad_f64")]
        + [("ray_o", _FP), ("ray_d", _FP), ("vertices", _FP), ("faces", _IP)]
        + [(n, _FP) for n in ("background", "means3D", "shs", "colors_precomp", "others_precomp", "opacities",
                              "scales", "rotations")]
        + [(n, _FP) for n in ("out_rgb", "out_dpt", "out_acc", "out_norm", "out_dist", "out_aux", "mid_val",
                              "a_weights")]
        + [("n_proc", _IP), ("n_con", _IP), ("trace_seconds", C.POINTER(C.c_double))]
        + [(n, _FP) for n in ("dL_drgb", "dL_ddpt", "dL_dacc", "dL_ddist", "dL_dnorm", "dL_daux")]
        + [(n, _FP) for n in ("dL_dray_o", "dL_dray_d", "dL_dmeans3D", "dL_dgrads3D", "dL_dshs", "dL_dcolors",
                              "dL_dothers", "dL_dopacities", "dL_dscales", "dL_drotations")]
        + [(n, _FP) for n in ("noise_ray_o", "noise_ray_d", "noise_means3D", "noise_grads3D", "noise_scales",
                              "noise_rotations")]
    )


def build(force=False):
    """Compile the oracle with the committed Makefile (g++, no GPU involved)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.oracle_trace_forward.argtypes = [C.POINTER(OracleParams)]
        L.oracle_trace_backward.argtypes = [C.POINTER(OracleParams)]
        L.oracle_expf.argtypes = [C.c_float]
        L.oracle_expf.restype = C.c_float
        L.oracle_sh_color.argtypes = [C.c_int, _FP, _FP, _FP, _FP]
        L.oracle_sh_color.restype = None
        L.oracle_quat_to_rows.argtypes = [_FP, _FP]
        L.oracle_quat_to_rows.restype = None
        L.oracle_ray_quad.argtypes = [_FP] * 6 + [_FP, _IP]
        L.oracle_reflection_vjp.argtypes = [C.c_int, _FP, _FP, _FP, _FP]
        L.oracle_reflection_vjp.restype = None
        L.oracle_k_nearest.argtypes = [C.POINTER(OracleParams), _FP, _FP, _FP, C.POINTER(C.c_uint32)]
        _lib = L
    return _lib


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _fp(a):
    return None if a is None else a.ctypes.data_as(_FP)


def _ip(a):
    return None if a is None else a.ctypes.data_as(_IP)


class Scene:
    """Inputs of one trace call, held as contiguous numpy arrays."""

    def __init__(self, ray_o, ray_d, vertices, faces, means3D, opacities, scales, rotations, shs=None,
                 colors_precomp=None, others_precomp=None, bg=(0.0, 0.0, 0.0), sh_degree=3, max_trace_depth=0,
                 specular_threshold=0.0, start_from_first=True, training=True, aux=None, mtd_alloc=None):
        self.ray_o, self.ray_d = _f32(ray_o), _f32(ray_d)
        self.H, self.W = self.ray_o.shape[0], self.ray_o.shape[1]
        self.vertices = _f32(vertices)
        self.faces = np.ascontiguousarray(faces, dtype=np.int32)
        self.means3D, self.opacities = _f32(means3D), _f32(opacities)
        self.scales, self.rotations = _f32(scales), _f32(rotations)
        self.shs, self.colors_precomp, self.others_precomp = _f32(shs), _f32(colors_precomp), _f32(others_precomp)
        self.bg = _f32(bg)
        self.P = self.means3D.shape[0]
        self.D = int(sh_degree)
        self.M = 0 if self.shs is None else self.shs.shape[1]
        self.aux = int(aux) if aux is not None else (2 if self.others_precomp is None else self.others_precomp.shape[1])
        self.max_trace_depth = int(max_trace_depth)
        self.mtd_alloc = int(mtd_alloc) if mtd_alloc is not None else max(1, self.max_trace_depth)
        self.specular_threshold = float(specular_threshold)
        self.start_from_first, self.training = bool(start_from_first), bool(training)

    def params(self, hit_mode, literal_stale=False, n_threads=0):
        p = OracleParams()
        p.P, p.H, p.W, p.D, p.M, p.aux, p.mtd_alloc = self.P, self.H, self.W, self.D, self.M, self.aux, self.mtd_alloc
        p.training, p.start_from_first = int(self.training), int(self.start_from_first)
        p.max_trace_depth, p.specular_threshold = self.max_trace_depth, self.specular_threshold
        p.hit_mode, p.literal_stale, p.n_threads = hit_mode, int(literal_stale), n_threads
        p.ray_o, p.ray_d, p.vertices, p.faces = _fp(self.ray_o), _fp(self.ray_d), _fp(self.vertices), _ip(self.faces)
        p.background, p.means3D, p.shs = _fp(self.bg), _fp(self.means3D), _fp(self.shs)
        p.colors_precomp, p.others_precomp = _fp(self.colors_precomp), _fp(self.others_precomp)
        p.opacities, p.scales, p.rotations = _fp(self.opacities), _fp(self.scales), _fp(self.rotations)
        return p


def forward(sc, hit_mode=HITS_BRUTE_LEXI, literal_stale=False, n_threads=0, counters=True, compute_dist=False):
    """Run the oracle forward.  Returns a dict of numpy arrays shaped like the reference outputs.  `compute_dist`:
    fill "dist" with the 2DGS depth distortion and its two moments instead of the reference's zeros."""
    H, W, P = sc.H, sc.W, sc.P
    MID = 14 + sc.aux
    out = {
        "rgb": np.zeros((H, W, 3), np.float32), "dpt": np.zeros((H, W, 1), np.float32),
        "acc": np.zeros((H, W, 1), np.float32), "norm": np.zeros((H, W, 3), np.float32),
        "dist": np.zeros((H, W, 3), np.float32), "aux": np.zeros((H, W, sc.aux), np.float32),
        "mid": np.zeros((H, W, MID * (sc.mtd_alloc + 1)), np.float32),
        "wet": np.zeros((P, 1), np.float32),
    }
    if counters:
        out["n_proc"] = np.zeros((H, W), np.int32)
        out["n_con"] = np.zeros((H, W), np.int32)
    p = sc.params(hit_mode, literal_stale, n_threads)
    p.compute_dist = int(bool(compute_dist))
    p.out_rgb, p.out_dpt, p.out_acc = _fp(out["rgb"]), _fp(out["dpt"]), _fp(out["acc"])
    p.out_norm, p.out_dist, p.out_aux = _fp(out["norm"]), _fp(out["dist"]), _fp(out["aux"])
    p.mid_val = _fp(out["mid"])
    p.a_weights = _fp(out["wet"]) if sc.training else None
    if counters:
        p.n_proc, p.n_con = _ip(out["n_proc"]), _ip(out["n_con"])
    secs = C.c_double(0.0)
    p.trace_seconds = C.pointer(secs)
    rc = lib().oracle_trace_forward(C.byref(p))
    if rc:
        raise RuntimeError("oracle_trace_forward failed with status %d" % rc)
    sc.trace_seconds = secs.value  # wall time of the ray loop of this call
    return out


def backward(sc, fwd, grads, hit_mode=HITS_BRUTE_LEXI, literal_stale=False, n_threads=0, grad_f64=False, noise=False):
    """Run the oracle backward.  `fwd` is forward()'s dict; `grads` maps rgb/dpt/acc/norm/aux (dist optional)
    to upstream gradients.  Returns the gradient dict.  `grad_f64`: evaluate the gradient algebra in double on
    the same fp32 inputs and decisions; `noise` (implies grad_f64): also return, under "noise", a dict with the
    rounding sensitivity of ray_o, ray_d, means3D, grads3D, scales, rotations (see surfel_oracle.h)."""
    grad_f64 = grad_f64 or noise
    H, W, P = sc.H, sc.W, sc.P
    g = {k: _f32(v) for k, v in grads.items()}
    for k, ch in (("rgb", 3), ("dpt", 1), ("acc", 1), ("norm", 3), ("dist", 1), ("aux", sc.aux)):
        if g.get(k) is None:
            g[k] = np.zeros((H, W, ch), np.float32)
    out = {
        "ray_o": np.zeros((H, W, 3), np.float32), "ray_d": np.zeros((H, W, 3), np.float32),
        "means3D": np.zeros((P, 3), np.float32), "grads3D": np.zeros((P, 3), np.float32),
        "shs": np.zeros((P, sc.M, 3), np.float32), "colors_precomp": np.zeros((P, 3), np.float32),
        "others_precomp": np.zeros((P, sc.aux), np.float32), "opacities": np.zeros((P, 1), np.float32),
        "scales": np.zeros((P, 2), np.float32), "rotations": np.zeros((P, 4), np.float32),
    }
    p = sc.params(hit_mode, literal_stale, n_threads)
    p.grad_f64 = int(bool(grad_f64))
    keep = [_f32(fwd[k]) for k in ("rgb", "dpt", "acc", "norm", "dist", "aux", "mid")]
    p.out_rgb, p.out_dpt, p.out_acc, p.out_norm, p.out_dist, p.out_aux, p.mid_val = [_fp(a) for a in keep]
    p.dL_drgb, p.dL_ddpt, p.dL_dacc = _fp(g["rgb"]), _fp(g["dpt"]), _fp(g["acc"])
    p.dL_ddist, p.dL_dnorm, p.dL_daux = _fp(g["dist"]), _fp(g["norm"]), _fp(g["aux"])
    p.dL_dray_o, p.dL_dray_d = _fp(out["ray_o"]), _fp(out["ray_d"])
    p.dL_dmeans3D, p.dL_dgrads3D, p.dL_dshs = _fp(out["means3D"]), _fp(out["grads3D"]), _fp(out["shs"])
    p.dL_dcolors, p.dL_dothers = _fp(out["colors_precomp"]), _fp(out["others_precomp"])
    p.dL_dopacities, p.dL_dscales, p.dL_drotations = _fp(out["opacities"]), _fp(out["scales"]), _fp(out["rotations"])
    if noise:
        nz = {k: np.zeros_like(out[k]) for k in ("ray_o", "ray_d", "means3D", "grads3D", "scales", "rotations")}
        p.noise_ray_o, p.noise_ray_d = _fp(nz["ray_o"]), _fp(nz["ray_d"])
        p.noise_means3D, p.noise_grads3D = _fp(nz["means3D"]), _fp(nz["grads3D"])
        p.noise_scales, p.noise_rotations = _fp(nz["scales"]), _fp(nz["rotations"])
        out["noise"] = nz
    secs = C.c_double(0.0)
    p.trace_seconds = C.pointer(secs)
    rc = lib().oracle_trace_backward(C.byref(p))
    if rc:
        raise RuntimeError("oracle_trace_backward failed with status %d" % rc)
    sc.trace_seconds = secs.value  # wall time of the ray loop of this call
    return out


def k_nearest(sc, o, d, hit_mode=HITS_BRUTE_LEXI):
    t = np.zeros(16, np.float32)
    idx = np.zeros(16, np.uint32)
    o, d = _f32(o), _f32(d)
    p = sc.params(hit_mode)
    cnt = lib().oracle_k_nearest(C.byref(p), _fp(o), _fp(d), _fp(t), idx.ctypes.data_as(C.POINTER(C.c_uint32)))
    if cnt < 0:
        raise RuntimeError("oracle_k_nearest failed with status %d" % -cnt)
    return cnt, t, idx


def expf(x):
    return np.array([lib().oracle_expf(float(v)) for v in np.asarray(x, np.float32).ravel()], np.float32)


def sh_color(deg, sh, d):
    sh, d = _f32(sh), _f32(d)
    rgb, cl = np.zeros(3, np.float32), np.zeros(3, np.float32)
    lib().oracle_sh_color(int(deg), _fp(sh), _fp(d), _fp(rgb), _fp(cl))
    return rgb, cl


def quat_to_rows(q):
    q = _f32(q)
    R = np.zeros(9, np.float32)
    lib().oracle_quat_to_rows(_fp(q), _fp(R))
    return R.reshape(3, 3)


def ray_quad(o, d, A, B, Cv, Dv):
    arrs = [_f32(a) for a in (o, d, A, B, Cv, Dv)]
    t = C.c_float(0)
    tri = C.c_int32(0)
    hit = lib().oracle_ray_quad(*[_fp(a) for a in arrs], C.byref(t), C.byref(tri))
    return bool(hit), t.value, tri.value


def reflection_vjp(which, a, b, g):
    """which: 'dnormvdv' (a = v), 'ddotndndn' (a = n, b = d), 'ddotndndd' (a = n, b = d); g = incoming gradient."""
    a, b, g = _f32(a), _f32(b), _f32(g)
    out = np.zeros(3, np.float32)
    lib().oracle_reflection_vjp({"dnormvdv": 0, "ddotndndn": 1, "ddotndndd": 2}[which], _fp(a), _fp(b), _fp(g), _fp(out))
    return out


def num_threads():
    return lib().oracle_num_threads()
