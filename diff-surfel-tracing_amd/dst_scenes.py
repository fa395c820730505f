"""Seeded synthetic scenes and ray bundles for the benchmark configurations.

Everything is generated with a CPU `torch.Generator`, so the same seed gives the same
tensors on any machine; callers move them to the GPU.  `get_triangles` and `pinhole_rays`
restate the conventions of the reference example code that the tracer hard-codes:
  - surfel -> quad: vertices mean + a*sx*Ru + b*sy*Rv for (a,b) in (-3,3),(-3,-3),(3,3),(3,-3),
    faces [4g,4g+1,4g+2] and [4g+1,4g+2,4g+3]   (reference example/utils/gaussian_utils.py:176-210)
  - quaternion (w,x,y,z) -> rotation columns Ru,Rv,Rn (reference example/utils/gaussian_utils.py:213-249)
  - pinhole rays through pixel centres (+0.5), unit directions (reference example/utils/ray_utils.py:80-136)
"""
import math

import torch

_SIGMA3 = torch.tensor([[-3.0, 3.0], [-3.0, -3.0], [3.0, 3.0], [3.0, -3.0]])


def build_rotation(q):
    """(..,4) quaternion (w,x,y,z), any norm -> (..,3,3) rotation matrix."""
    q = q / torch.linalg.norm(q, dim=-1, keepdim=True)
    r, x, y, z = q.unbind(-1)
    R = torch.stack([
        1 - 2 * (y * y + z * z), 2 * (x * y - r * z), 2 * (x * z + r * y),
        2 * (x * y + r * z), 1 - 2 * (x * x + z * z), 2 * (y * z - r * x),
        2 * (x * z - r * y), 2 * (y * z + r * x), 1 - 2 * (x * x + y * y)], dim=-1)
    return R.reshape(q.shape[:-1] + (3, 3))


def get_triangles(means3D, scales, rotations):
    """(P,3),(P,2),(P,4) -> vertices (4P,3) float32, faces (2P,3) int32."""
    R = build_rotation(rotations)
    sig = _SIGMA3.to(means3D)
    tu = R[:, :, 0] * scales[:, 0:1]
    tv = R[:, :, 1] * scales[:, 1:2]
    v = means3D[:, None, :] + sig[None, :, 0:1] * tu[:, None, :] + sig[None, :, 1:2] * tv[:, None, :]
    v = v.reshape(-1, 3).contiguous()
    idx = torch.arange(v.shape[0], device=v.device).reshape(-1, 4)
    f = torch.stack([idx[:, :3], idx[:, 1:]], dim=1).reshape(-1, 3).int().contiguous()
    return v, f


def look_at(eye, target, up=(0.0, 0.0, 1.0)):
    """World-to-camera rotation R (rows = camera right, down, forward) and translation T, OpenCV convention."""
    eye = torch.tensor(eye, dtype=torch.float64)
    fwd = torch.tensor(target, dtype=torch.float64) - eye
    fwd = fwd / fwd.norm()
    upv = torch.tensor(up, dtype=torch.float64)
    right = torch.linalg.cross(fwd, upv)
    right = right / right.norm()
    down = torch.linalg.cross(fwd, right)
    R = torch.stack([right, down, fwd], dim=0)
    T = -(R @ eye)[:, None]
    return R.float(), T.float()


def pinhole_rays(H, W, fov_x_deg, eye, target, up=(0.0, 0.0, 1.0)):
    """Rays through pixel centres: ray_o (H,W,3) constant, ray_d (H,W,3) unit length."""
    R, T = look_at(eye, target, up)
    fx = 0.5 * W / math.tan(0.5 * math.radians(fov_x_deg))
    K = torch.tensor([[fx, 0.0, 0.5 * W], [0.0, fx, 0.5 * H], [0.0, 0.0, 1.0]])
    i, j = torch.meshgrid(torch.arange(H, dtype=torch.float32), torch.arange(W, dtype=torch.float32), indexing="ij")
    xy1 = torch.stack([j + 0.5, i + 0.5, torch.ones_like(i)], dim=-1)[..., None]
    cam = torch.linalg.inv(K) @ xy1
    world = R.mT @ (cam - T)
    o = (-(R.mT @ T))[:, 0]
    d = world[..., 0] - o
    d = d / torch.linalg.norm(d, dim=-1, keepdim=True)
    return o.expand(H, W, 3).contiguous(), d.contiguous()


def _randn(gen, *shape):
    return torch.randn(*shape, generator=gen)


def _rand(gen, *shape):
    return torch.rand(*shape, generator=gen)


def _quat_from_normal(normal, gen):
    """Quaternions (w,x,y,z) whose rotation maps z to `normal`, with a random spin about it."""
    n = normal / torch.linalg.norm(normal, dim=-1, keepdim=True)
    helper = torch.where(n[:, 2:3].abs() < 0.9, torch.tensor([0.0, 0.0, 1.0]).expand_as(n),
                         torch.tensor([1.0, 0.0, 0.0]).expand_as(n))
    u = torch.linalg.cross(helper, n)
    u = u / torch.linalg.norm(u, dim=-1, keepdim=True)
    v = torch.linalg.cross(n, u)
    ang = _rand(gen, n.shape[0]) * (2 * math.pi)
    c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
    u2, v2 = c * u + s * v, -s * u + c * v
    R = torch.stack([u2, v2, n], dim=-1)  # columns
    # rotation matrix -> quaternion, numerically safe branch on the largest diagonal term
    m00, m11, m22 = R[:, 0, 0], R[:, 1, 1], R[:, 2, 2]
    qw = torch.sqrt(torch.clamp(1 + m00 + m11 + m22, min=0)) / 2
    qx = torch.sqrt(torch.clamp(1 + m00 - m11 - m22, min=0)) / 2
    qy = torch.sqrt(torch.clamp(1 - m00 + m11 - m22, min=0)) / 2
    qz = torch.sqrt(torch.clamp(1 - m00 - m11 + m22, min=0)) / 2
    big = torch.stack([qw, qx, qy, qz], dim=-1).argmax(dim=-1)
    q = torch.zeros(n.shape[0], 4)
    r = R
    for k in range(4):
        m = big == k
        if not m.any():
            continue
        rm = r[m]
        if k == 0:
            w = qw[m]
            q[m] = torch.stack([w, (rm[:, 2, 1] - rm[:, 1, 2]) / (4 * w), (rm[:, 0, 2] - rm[:, 2, 0]) / (4 * w),
                                (rm[:, 1, 0] - rm[:, 0, 1]) / (4 * w)], dim=-1)
        elif k == 1:
            x = qx[m]
            q[m] = torch.stack([(rm[:, 2, 1] - rm[:, 1, 2]) / (4 * x), x, (rm[:, 0, 1] + rm[:, 1, 0]) / (4 * x),
                                (rm[:, 0, 2] + rm[:, 2, 0]) / (4 * x)], dim=-1)
        elif k == 2:
            y = qy[m]
            q[m] = torch.stack([(rm[:, 0, 2] - rm[:, 2, 0]) / (4 * y), (rm[:, 0, 1] + rm[:, 1, 0]) / (4 * y), y,
                                (rm[:, 1, 2] + rm[:, 2, 1]) / (4 * y)], dim=-1)
        else:
            z = qz[m]
            q[m] = torch.stack([(rm[:, 1, 0] - rm[:, 0, 1]) / (4 * z), (rm[:, 0, 2] + rm[:, 2, 0]) / (4 * z),
                                (rm[:, 1, 2] + rm[:, 2, 1]) / (4 * z), z], dim=-1)
    return q


def _finish(gen, means, log_s, quats, op_mu, op_sigma, sh_degree=3, aux=0, colors=False):
    P = means.shape[0]
    s = {
        "means3D": means.float().contiguous(),
        "scales": torch.exp(log_s).float().contiguous(),
        "rotations": quats.float().contiguous(),
        "opacities": torch.sigmoid(op_mu + op_sigma * _randn(gen, P, 1)).float().contiguous(),
    }
    if colors:
        s["colors_precomp"] = _rand(gen, P, 3).contiguous()
    else:
        s["shs"] = (0.3 * _randn(gen, P, (sh_degree + 1) ** 2 if sh_degree < 3 else 16, 3)).contiguous()
    if aux:
        s["others_precomp"] = _rand(gen, P, aux).contiguous()
    s["vertices"], s["faces"] = get_triangles(s["means3D"], s["scales"], s["rotations"])
    return s


def scene_cube(P=10000, seed=0, colors=False, aux=0):
    """Config 1: means uniform in [-1,1]^3, log-scales N(-3.5,0.5), random orientations."""
    gen = torch.Generator().manual_seed(seed)
    means = _rand(gen, P, 3) * 2 - 1
    log_s = -3.5 + 0.5 * _randn(gen, P, 2)
    q = _randn(gen, P, 4)
    q = q / torch.linalg.norm(q, dim=-1, keepdim=True)
    return _finish(gen, means, log_s, q, 0.0, 1.0, colors=colors, aux=aux)


def rays_cube(H=128, W=128, view=0):
    ang = 0.7 * view
    eye = (3.0 * math.cos(ang), 3.0 * math.sin(ang), 0.0)
    return pinhole_rays(H, W, 60.0, eye, (0.0, 0.0, 0.0))


def scene_sphere(P=100000, seed=0):
    """Config 2: surfels on the unit sphere, normals radial, log-scales N(-4.5,0.3)."""
    gen = torch.Generator().manual_seed(seed)
    n = _randn(gen, P, 3)
    n = n / torch.linalg.norm(n, dim=-1, keepdim=True)
    log_s = -4.5 + 0.3 * _randn(gen, P, 2)
    q = _quat_from_normal(n, gen)
    return _finish(gen, n.clone(), log_s, q, 1.0, 1.0)


def rays_sphere(H=800, W=800, view=0, seed=0):
    gen = torch.Generator().manual_seed(1000 + seed)
    ang = _rand(gen, 30, 2)
    az, el = float(ang[view % 30, 0]) * 2 * math.pi, (float(ang[view % 30, 1]) - 0.5) * 1.2
    eye = (4.0 * math.cos(az) * math.cos(el), 4.0 * math.sin(az) * math.cos(el), 4.0 * math.sin(el))
    return pinhole_rays(H, W, 35.0, eye, (0.0, 0.0, 0.0))


def _room_points(gen, P, half, n_clusters, sigma):
    """70 % on 5 seeded faces of the box [-half,half]^3, 30 % in Gaussian clusters inside it."""
    n_plane = int(round(0.7 * P))
    faces = torch.randperm(6, generator=gen)[:5]
    which = faces[torch.randint(0, 5, (n_plane,), generator=gen)]
    axis, sign = which // 2, (which % 2).float() * 2 - 1
    pts = (_rand(gen, n_plane, 3) * 2 - 1) * half
    pts[torch.arange(n_plane), axis] = sign * half
    normals = torch.zeros(n_plane, 3)
    normals[torch.arange(n_plane), axis] = -sign
    n_cl = P - n_plane
    centres = (_rand(gen, n_clusters, 3) * 2 - 1) * (half - 1.0)
    cid = torch.randint(0, n_clusters, (n_cl,), generator=gen)
    cpts = centres[cid] + sigma * _randn(gen, n_cl, 3)
    cn = _randn(gen, n_cl, 3)
    return torch.cat([pts, cpts]), torch.cat([normals, cn])


def scene_room(P=1000000, seed=0, aux=0, half=5.0):
    """Configs 3/4: 10 m box, 5 planes + 200 clusters (sigma 0.3 m), log-scales N(-4,0.6)."""
    gen = torch.Generator().manual_seed(seed)
    pts, nrm = _room_points(gen, P, half, 200, 0.3)
    log_s = -4.0 + 0.6 * _randn(gen, P, 2)
    q = _quat_from_normal(nrm, gen)
    return _finish(gen, pts, log_s, q, 0.5, 1.5, aux=aux)


def rays_room(H=1080, W=1920):
    return pinhole_rays(H, W, 70.0, (-2.0, -1.0, 0.5), (3.0, 1.5, -0.5))


def scene_lidar(P=2000000, seed=0, aux=4):
    """Config 5: 60 % on a 200x200 m ground plane z=0, 40 % on the faces of 500 boxes."""
    gen = torch.Generator().manual_seed(seed)
    n_g = int(round(0.6 * P))
    ground = torch.cat([(_rand(gen, n_g, 2) * 2 - 1) * 100.0, torch.zeros(n_g, 1)], dim=-1)
    gn = torch.tensor([0.0, 0.0, 1.0]).expand(n_g, 3)
    n_b = P - n_g
    centres = torch.cat([(_rand(gen, 500, 2) * 2 - 1) * 95.0, torch.zeros(500, 1)], dim=-1)
    size = torch.cat([1.0 + 4.0 * _rand(gen, 500, 2), 1.0 + 3.0 * _rand(gen, 500, 1)], dim=-1)
    centres[:, 2] = 0.5 * size[:, 2]
    bid = torch.randint(0, 500, (n_b,), generator=gen)
    face = torch.randint(0, 5, (n_b,), generator=gen)  # +-x, +-y, +z (no floor)
    axis = torch.where(face < 4, face // 2, torch.full_like(face, 2))
    sign = torch.where(face < 4, (face % 2).float() * 2 - 1, torch.ones(n_b))
    local = (_rand(gen, n_b, 3) * 2 - 1) * 0.5
    local[torch.arange(n_b), axis] = 0.5 * sign
    bpts = centres[bid] + local * size[bid]
    bn = torch.zeros(n_b, 3)
    bn[torch.arange(n_b), axis] = sign
    log_s = -3.0 + 0.4 * _randn(gen, P, 2)
    q = _quat_from_normal(torch.cat([gn, bn]), gen)
    return _finish(gen, torch.cat([ground, bpts]), log_s, q, 1.0, 1.0, aux=aux)


def rays_lidar(beams=64, azimuths=2048, seed=0):
    """(1, beams*azimuths, 3) rays from a sensor 1.8 m above the ground, elevations U(-25,+3) deg per beam."""
    gen = torch.Generator().manual_seed(2000 + seed)
    el = torch.deg2rad(torch.sort(_rand(gen, beams) * 28.0 - 25.0).values)
    az = torch.arange(azimuths, dtype=torch.float32) * (2 * math.pi / azimuths)
    d = torch.stack([torch.cos(el)[:, None] * torch.cos(az)[None], torch.cos(el)[:, None] * torch.sin(az)[None],
                     torch.sin(el)[:, None].expand(beams, azimuths)], dim=-1).reshape(1, -1, 3)
    o = torch.tensor([0.0, 0.0, 1.8]).expand(1, beams * azimuths, 3).contiguous()
    return o, d.contiguous()


def perturb_means(scene, frame, frac=0.1, sigma=0.05, seed=0):
    """Config 5 dynamics: move `frac` of the means by N(0,sigma) and regenerate the quads (same topology)."""
    gen = torch.Generator().manual_seed(3000 + seed + frame)
    P = scene["means3D"].shape[0]
    pick = torch.randperm(P, generator=gen)[: int(frac * P)]
    means = scene["means3D"].clone()
    means[pick] += sigma * _randn(gen, pick.shape[0], 3)
    out = dict(scene)
    out["means3D"] = means
    out["vertices"], out["faces"] = get_triangles(means, scene["scales"], scene["rotations"])
    return out


def upstream_grads(H, W, aux, seed=0):
    """Fixed seeded upstream gradients for rgb, dpt, acc, norm, aux (the backward benchmark's loss)."""
    gen = torch.Generator().manual_seed(4000 + seed)
    return {
        "rgb": _randn(gen, H, W, 3), "dpt": _randn(gen, H, W, 1), "acc": _randn(gen, H, W, 1),
        "norm": _randn(gen, H, W, 3), "aux": _randn(gen, H, W, aux),
    }
