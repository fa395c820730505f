#!/usr/bin/env python3
"""Camera-path renderer over a surfel model: the counterpart of the reference harness (reference
example/render.py:48-155) on top of the MI355X tracer.

    python render.py --model_path model.ply --camera_dir path.json --result_dir out     # a trained 2DGS model
    python render.py --scene room --surfels 200000 --frames 8 --result_dir out          # a synthetic scene, orbit path

For every camera it traces rgb / depth / normal and writes RENDER/, DEPTH/ and NORMAL/ images with the reference's
post-processing (`normalize_depth`, `visualize_normal`: reference example/utils/data_utils.py:52-70).  What it
does not need: plyfile (the .ply reader below parses the binary little-endian layout 3DGS / 2DGS trainers write),
cv2 (PNG through zlib) and ffmpeg (no video; the frames are numbered for it).
"""
import argparse
import json
import math
import os
import struct
import sys
import zlib

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)

import dst_scenes as S  # noqa: E402

_PLY_TYPES = {"float": "<f4", "float32": "<f4", "double": "<f8", "float64": "<f8", "uchar": "u1", "uint8": "u1",
              "char": "i1", "int8": "i1", "short": "<i2", "int16": "<i2", "ushort": "<u2", "uint16": "<u2",
              "int": "<i4", "int32": "<i4", "uint": "<u4", "uint32": "<u4"}


def read_ply_vertices(path):
    """The `vertex` element of a binary little-endian .ply as a numpy structured array."""
    with open(path, "rb") as fh:
        if fh.readline().strip() != b"ply":
            raise ValueError("%s is not a .ply file" % path)
        fmt, count, props, in_vertex = None, None, [], False
        while True:
            line = fh.readline()
            if not line:
                raise ValueError("unterminated .ply header")
            tok = line.decode("ascii", "replace").split()
            if not tok:
                continue
            if tok[0] == "format":
                fmt = tok[1]
            elif tok[0] == "element":
                if count is not None and not in_vertex:
                    pass
                in_vertex = tok[1] == "vertex"
                if in_vertex:
                    count = int(tok[2])
                elif count is None:
                    raise ValueError("the vertex element must come first")
            elif tok[0] == "property" and in_vertex:
                if tok[1] == "list":
                    raise ValueError("list properties in the vertex element are not supported")
                props.append((tok[2], _PLY_TYPES[tok[1]]))
            elif tok[0] == "end_header":
                break
        if fmt != "binary_little_endian":
            raise ValueError("only binary_little_endian .ply files are supported (got %s)" % fmt)
        if count is None:
            raise ValueError("no vertex element")
        return np.fromfile(fh, dtype=np.dtype(props), count=count)


def load_surfel_model(path, max_sh_degree=3):
    """A trained 2DGS model -> the tracer's inputs, with the reference's activations
    (reference example/utils/gaussian_utils.py:60-90,97-170): scales = exp, rotations normalised, opacities =
    sigmoid, SH features (P, (D+1)^2, 3) with the DC term first."""
    v = read_ply_vertices(path)
    names = v.dtype.names
    f32 = lambda n: torch.from_numpy(np.ascontiguousarray(v[n], dtype=np.float32))  # noqa: E731
    numbered = lambda pre: sorted([n for n in names if n.startswith(pre)], key=lambda n: int(n.split("_")[-1]))  # noqa: E731
    xyz = torch.stack([f32("x"), f32("y"), f32("z")], 1)
    dc = torch.stack([f32("f_dc_0"), f32("f_dc_1"), f32("f_dc_2")], 1)[:, :, None]          # (P,3,1)
    rest_names = numbered("f_rest_")
    n_rest = (max_sh_degree + 1) ** 2 - 1
    if len(rest_names) != 3 * n_rest:
        raise ValueError("expected %d f_rest_* properties for SH degree %d, found %d"
                         % (3 * n_rest, max_sh_degree, len(rest_names)))
    rest = torch.stack([f32(n) for n in rest_names], 1).reshape(-1, 3, n_rest) if n_rest else torch.zeros(len(v), 3, 0)
    shs = torch.cat([dc, rest], 2).transpose(1, 2).contiguous()                               # (P,M,3)
    scales = torch.exp(torch.stack([f32(n) for n in numbered("scale_")], 1))[:, :2].contiguous()
    rot = torch.stack([f32(n) for n in numbered("rot")], 1)
    rot = rot / rot.norm(dim=-1, keepdim=True)
    model = {"means3D": xyz.contiguous(), "shs": shs, "opacities": torch.sigmoid(f32("opacity"))[:, None].contiguous(),
             "scales": scales, "rotations": rot.contiguous()}
    model["vertices"], model["faces"] = S.get_triangles(model["means3D"], model["scales"], model["rotations"])
    return model


def load_nerf_camera(cam):
    """One frame of a NeRF-style path.json -> (H, W, K, R, T) with the reference's axis flip and world-to-camera
    inversion (reference example/render.py:33-45)."""
    H, W = int(cam["h"]), int(cam["w"])
    K = torch.tensor([[cam["fl_x"], 0.0, cam["cx"]], [0.0, cam["fl_y"], cam["cy"]], [0.0, 0.0, 1.0]], dtype=torch.float32)
    c2w = torch.tensor(cam["transform_matrix"], dtype=torch.float32)
    c2w[:3, [1, 2]] *= -1
    w2c = torch.inverse(c2w)
    return H, W, K, w2c[:3, :3].contiguous(), w2c[:3, 3:].contiguous()


def get_rays(H, W, K, R, T):
    """World-space rays through the pixel centres, unit directions (reference example/utils/ray_utils.py:80-136)."""
    i, j = torch.meshgrid(torch.arange(H, dtype=torch.float32), torch.arange(W, dtype=torch.float32), indexing="ij")
    xy1 = torch.stack([j + 0.5, i + 0.5, torch.ones_like(i)], dim=-1)[..., None]
    world = R.mT @ (torch.linalg.inv(K) @ xy1 - T)
    o = (-(R.mT @ T))[:, 0]
    d = world[..., 0] - o
    d = d / torch.linalg.norm(d, dim=-1, keepdim=True)
    return o.expand(H, W, 3).contiguous(), d.contiguous()


def orbit_cameras(frames, H, W, fov_x_deg, radius, height, target=(0.0, 0.0, 0.0)):
    """A synthetic camera path in the same (H, W, K, R, T) form."""
    out = []
    fx = 0.5 * W / math.tan(0.5 * math.radians(fov_x_deg))
    K = torch.tensor([[fx, 0.0, 0.5 * W], [0.0, fx, 0.5 * H], [0.0, 0.0, 1.0]])
    for k in range(frames):
        a = 2.0 * math.pi * k / max(frames, 1)
        R, T = S.look_at((radius * math.cos(a), radius * math.sin(a), height), target)
        out.append((H, W, K, R.float(), T.float()))
    return out


def normalize_depth(depth, p=0.01):
    """Reference example/utils/data_utils.py:52-59."""
    n = max(1, int(depth.numel() * p))
    near = depth.ravel().topk(n, largest=False)[0].max()
    far = depth.ravel().topk(n, largest=True)[0].min()
    return (1 - (depth - near) / (far - near)).clip(0, 1)


def visualize_normal(n, R, eps=1e-8):
    """Reference example/utils/data_utils.py:62-70."""
    n = n / (torch.norm(n, dim=-1, keepdim=True) + eps)
    n = n @ R.mT
    n = n * torch.tensor([1.0, -1.0, -1.0], device=n.device)
    return n * 0.5 + 0.5


def save_png(path, img):
    """(H,W,1|3) floats in [0,1] (tensor or array) -> 8-bit PNG."""
    if isinstance(img, torch.Tensor):
        img = img.detach().cpu().numpy()
    img = np.asarray(img, dtype=np.float32)
    if img.ndim == 2:
        img = img[..., None]
    if img.shape[-1] == 1:
        img = np.repeat(img, 3, -1)
    data = (img[..., :3] * 255.0).clip(0, 255).astype(np.uint8)
    H, W = data.shape[:2]
    raw = b"".join(b"\x00" + data[y].tobytes() for y in range(H))
    chunk = lambda tag, body: struct.pack(">I", len(body)) + tag + body + struct.pack(">I", zlib.crc32(tag + body) & 0xFFFFFFFF)  # noqa: E731
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, "wb") as fh:
        fh.write(b"\x89PNG\r\n\x1a\n" + chunk(b"IHDR", struct.pack(">IIBBBBB", W, H, 8, 2, 0, 0, 0))
                 + chunk(b"IDAT", zlib.compress(raw, 6)) + chunk(b"IEND", b""))


def render_path(tracer, model, cameras, result_dir=None, white_bg=True, sh_degree=3, max_trace_depth=0,
                specular_threshold=0.0, scale_modifier=1.0, dev="cuda"):
    """Trace every camera of the path; returns the list of (rgb, dpt, acc, norm) tensors and writes the three image
    folders when `result_dir` is given.  Follows reference example/render.py:60-145 call for call."""
    import diff_surfel_tracing as dst
    g = {k: v.to(dev).contiguous() for k, v in model.items()}
    tracer.build_acceleration_structure(g["vertices"].detach().clone(), g["faces"].detach().clone(), rebuild=True)
    bg = torch.tensor([1.0, 1.0, 1.0] if white_bg else [0.0, 0.0, 0.0], dtype=torch.float32, device=dev)
    grads3D = torch.zeros_like(g["means3D"])
    eye = torch.eye(4, device=dev)
    outs = []
    for i, (H, W, K, R, T) in enumerate(cameras):
        ray_o, ray_d = get_rays(H, W, K, R, T)
        fovx, fovy = 2 * math.atan(W / (2 * float(K[0, 0]))), 2 * math.atan(H / (2 * float(K[1, 1])))
        settings = dst.SurfelTracingSettings(
            image_height=H, image_width=W, tanfovx=math.tan(fovx * 0.5), tanfovy=math.tan(fovy * 0.5), bg=bg,
            scale_modifier=scale_modifier, viewmatrix=eye, projmatrix=eye, sh_degree=sh_degree,
            campos=(-(R.mT @ T))[:, 0].to(dev), prefiltered=False, debug=False, max_trace_depth=max_trace_depth,
            specular_threshold=specular_threshold)
        with torch.no_grad():
            rgb, dpt, acc, norm, dist, aux, mid, wet = tracer(
                ray_o.to(dev), ray_d.to(dev), g["vertices"], means3D=g["means3D"], grads3D=grads3D, shs=g.get("shs"),
                colors_precomp=g.get("colors_precomp"), others_precomp=g.get("others_precomp"),
                opacities=g["opacities"], scales=g["scales"], rotations=g["rotations"], cov3D_precomp=None,
                tracer_settings=settings, start_from_first=True)
        outs.append((rgb, dpt, acc, norm))
        if result_dir:
            save_png(os.path.join(result_dir, "RENDER", "%04d.png" % i), rgb)
            save_png(os.path.join(result_dir, "DEPTH", "%04d.png" % i), normalize_depth(dpt))
            save_png(os.path.join(result_dir, "NORMAL", "%04d.png" % i), visualize_normal(norm, R.to(dev)))
    return outs


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model_path", type=str, default=None, help="trained 2DGS model (.ply); omit to use --scene")
    ap.add_argument("--camera_dir", type=str, default=None, help="NeRF-style path.json; omit for an orbit")
    ap.add_argument("--result_dir", type=str, default="result")
    ap.add_argument("--max_sh_degree", type=int, default=3)
    ap.add_argument("--white_bg", action="store_true")
    ap.add_argument("--scale_modifier", type=float, default=1.0)
    ap.add_argument("--max_trace_depth", type=int, default=0)
    ap.add_argument("--specular_threshold", type=float, default=0.0)
    ap.add_argument("--scene", choices=["cube", "sphere", "room"], default="cube")
    ap.add_argument("--surfels", type=int, default=100000)
    ap.add_argument("--frames", type=int, default=8)
    ap.add_argument("--height", type=int, default=540)
    ap.add_argument("--width", type=int, default=960)
    a = ap.parse_args()
    import diff_surfel_tracing as dst
    if a.model_path:
        model = load_surfel_model(a.model_path, a.max_sh_degree)
    else:
        model = {"cube": S.scene_cube, "sphere": S.scene_sphere, "room": S.scene_room}[a.scene](a.surfels)
    print("[INFO] Loaded number of Gaussians: %d." % model["means3D"].shape[0])
    if a.camera_dir:
        cameras = [load_nerf_camera(c) for c in json.load(open(a.camera_dir))["frames"]]
    else:
        radius = {"cube": 3.0, "sphere": 4.0, "room": 3.0}[a.scene]
        cameras = orbit_cameras(a.frames, a.height, a.width, 60.0, radius, 0.6)
    tracer = dst.SurfelTracer()
    render_path(tracer, model, cameras, a.result_dir, a.white_bg, a.max_sh_degree, a.max_trace_depth,
                a.specular_threshold, a.scale_modifier)
    print("[INFO] Rendering finished: %d frames in %s." % (len(cameras), a.result_dir))


if __name__ == "__main__":
    main()
