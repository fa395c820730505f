"""Writes tests/golden/cube_p400.npz: the inputs (generated from seeds here; stored, because vectorised exp / sin
differ in the last bit between CPUs) and the expected outputs from the CPU oracle (brute-force hit
enumeration, reference any-hit rule).  The reference ships no golden vectors and cannot be
run here (it needs nvcc + OptiX), so this fixture pins the oracle against later drift, not against the reference.

    python tests/golden/make_golden.py            (keeps the stored inputs of an existing fixture, renews the outputs)
    python tests/golden/make_golden.py --new-inputs
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "diff-surfel-tracing_amd"), os.path.join(ROOT, "tests")):
    sys.path.insert(0, p)

SPEC = dict(P=400, seed=11, H=24, W=24, view=1, aux=2, bg=(0.1, 0.2, 0.3), grad_seed=3)


def load_inputs():
    """The stored inputs of the fixture as torch tensors: (scene dict, ray_o, ray_d, upstream gradients)."""
    import torch
    z = np.load(os.path.join(HERE, "cube_p400.npz"))
    sc = {k[3:]: torch.from_numpy(z[k]) for k in z.files if k.startswith("in_")}
    o, d = sc.pop("ray_o"), sc.pop("ray_d")
    ug = {k[3:]: torch.from_numpy(z[k]) for k in z.files if k.startswith("up_")}
    return sc, o, d, ug


def inputs():
    import dst_scenes as S
    sc = S.scene_cube(P=SPEC["P"], seed=SPEC["seed"], aux=SPEC["aux"])
    sc["scales"] = sc["scales"] * 3.0   # enough overlap for multi-chunk rays at this small P
    sc["vertices"], sc["faces"] = S.get_triangles(sc["means3D"], sc["scales"], sc["rotations"])
    o, d = S.rays_cube(SPEC["H"], SPEC["W"], view=SPEC["view"])
    ug = S.upstream_grads(SPEC["H"], SPEC["W"], SPEC["aux"], seed=SPEC["grad_seed"])
    return sc, o, d, ug


def main():
    from helpers import oracle_scene
    from oracle import surfel_oracle as O
    keep = os.path.exists(os.path.join(HERE, "cube_p400.npz")) and "--new-inputs" not in sys.argv
    sc, o, d, ug = load_inputs() if keep else inputs()
    s = oracle_scene(O, sc, o, d, bg=SPEC["bg"])
    fwd = O.forward(s, O.HITS_BRUTE_LITERAL)
    bwd = O.backward(s, fwd, {k: v.numpy() for k, v in ug.items()}, O.HITS_BRUTE_LEXI)
    out = {"in_" + k: v.numpy() for k, v in sc.items()}
    out.update({"in_ray_o": o.numpy(), "in_ray_d": d.numpy()})
    out.update({"up_" + k: v.numpy() for k, v in ug.items()})
    out.update({"fwd_" + k: v for k, v in fwd.items()})
    out.update({"bwd_" + k: v for k, v in bwd.items()})
    np.savez_compressed(os.path.join(HERE, "cube_p400.npz"), **out)
    print("wrote", len(out), "arrays; composited hits per ray: mean %.1f max %d"
          % (fwd["n_con"].mean(), fwd["n_con"].max()))


if __name__ == "__main__":
    main()
