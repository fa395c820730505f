"""Differentiable surfel ray tracing on MI355X: drop-in for the `diff_surfel_tracing` Python API.

Public names, argument order, defaults and return tuples follow the reference package
(reference diff_surfel_tracing/__init__.py:14-290):
`SurfelTracer`, `SurfelTracingSettings`, `trace_surfels`, `_TraceSurfels`.  The work happens in
hand-written HIP kernels behind the C ABI of libdst.so (see `_C.py`); there is no fallback path.
"""
from typing import NamedTuple

import torch
import torch.nn as nn

from . import _C

__all__ = ["SurfelTracer", "SurfelTracingSettings", "trace_surfels"]


def cpu_deep_copy_tuple(input_tuple):
    """CPU snapshot of an argument tuple, for the debug dumps."""
    return tuple(x.detach().cpu().clone() if isinstance(x, torch.Tensor) else x for x in input_tuple)


class SurfelTracingSettings(NamedTuple):
    image_height: int      # unused by the tracer, kept for rasteriser compatibility
    image_width: int       # unused
    tanfovx: float         # unused
    tanfovy: float         # unused
    bg: torch.Tensor       # (3,) background colour
    scale_modifier: float  # accepted, ignored by the device math (as in the reference)
    viewmatrix: torch.Tensor  # unused
    projmatrix: torch.Tensor  # unused
    sh_degree: int
    campos: torch.Tensor   # unused
    prefiltered: bool      # unused
    debug: bool            # dump the arguments to snapshot_fw.dump / snapshot_bw.dump if a call raises
    max_trace_depth: int = 0
    specular_threshold: float = 0.0


def _settings_args(s):
    """The settings fields in the order the launcher takes them after `rotations, cov3Ds_precomp`."""
    return (s.viewmatrix, s.projmatrix, s.campos, s.prefiltered, s.debug, s.max_trace_depth, s.specular_threshold)


def _guarded(fn, args, debug, dump_name, what):
    if not debug:
        return fn(*args)
    snapshot = cpu_deep_copy_tuple(args[1:])  # everything but the context handle
    try:
        return fn(*args)
    except Exception:
        torch.save(snapshot, dump_name)
        print("\nAn error occured in %s. Please forward %s for debugging." % (what, dump_name))
        raise


class _TraceSurfels(torch.autograd.Function):
    @staticmethod
    def forward(ctx, optix_context, training, start_from_first, ray_o, ray_d, vertices, means3D, grads3D, shs,
                colors_precomp, others_precomp, opacities, scales, rotations, cov3Ds_precomp, tracer_settings):
        s = tracer_settings
        args = (optix_context, training, start_from_first, ray_o, ray_d, vertices, s.bg, means3D, shs, s.sh_degree,
                colors_precomp, others_precomp, opacities, scales, s.scale_modifier, rotations,
                cov3Ds_precomp) + _settings_args(s)
        # when a backward pass will follow, the forward trace records its hit buffers for it; the wrapper below
        # says whether one can follow (gradient mode is always off in here, and needs_input_grad stays set
        # under torch.no_grad())
        record = None
        if optix_context.record_wanted and any(ctx.needs_input_grad) and ray_o.dim() == 3 and ray_o.numel() > 0:
            record = optix_context.acquire_record(ray_o.size(0), ray_o.size(1),
                                                  max(_C.DEFAULT_MAX_TRACE_DEPTH, s.max_trace_depth), ray_o.device,
                                                  max_trace_depth=s.max_trace_depth)
        try:
            out_rgb, out_dpt, out_acc, out_norm, out_dist, out_aux, mid_val, a_weights = _guarded(
                lambda *a: _C.trace_surfels(*a, hit_record=record), args, s.debug, "snapshot_fw.dump", "forward")
        except Exception:
            optix_context.release_record(record)
            raise
        ctx.hit_record = record

        ctx.tracer_settings = s
        ctx.optix_context = optix_context
        ctx.start_from_first = start_from_first
        ctx.save_for_backward(ray_o, ray_d, vertices, means3D, shs, colors_precomp, others_precomp, opacities, scales,
                              rotations, cov3Ds_precomp, out_rgb, out_dpt, out_acc, out_norm, out_dist, out_aux,
                              mid_val)
        # per-surfel accumulated blending weight (training) or zeros of shape (P,) (evaluation)
        acc_wet = a_weights if a_weights is not None else torch.zeros_like(means3D[:, 0])
        return out_rgb, out_dpt, out_acc, out_norm, out_dist[..., :1].clone(), out_aux, mid_val, acc_wet

    @staticmethod
    def backward(ctx, grad_out_rgb, grad_out_dpt, grad_out_acc, grad_out_norm, grad_out_dist, grad_out_aux,
                 grad_mid_val, grad_acc_wet):
        s = ctx.tracer_settings
        (ray_o, ray_d, vertices, means3D, shs, colors_precomp, others_precomp, opacities, scales, rotations,
         cov3Ds_precomp, out_rgb, out_dpt, out_acc, out_norm, out_dist, out_aux, mid_val) = ctx.saved_tensors
        args = (ctx.optix_context, ctx.start_from_first, ray_o, ray_d, vertices, s.bg, means3D, shs, s.sh_degree,
                colors_precomp, others_precomp, opacities, scales, s.scale_modifier, rotations,
                cov3Ds_precomp) + _settings_args(s) + (
                    out_rgb, out_dpt, out_acc, out_norm, out_dist, out_aux, mid_val,
                    grad_out_rgb, grad_out_dpt, grad_out_acc, grad_out_norm, grad_out_dist, grad_out_aux)
        record = ctx.hit_record if (ctx.hit_record is not None and ctx.hit_record.words is not None) else None
        try:
            (g_ray_o, g_ray_d, g_means3D, g_grads3D, _g_grads3D_abs, g_shs, g_colors, g_others, g_opacities,
             g_scales, g_rotations, g_cov3Ds) = _guarded(
                 lambda *a: _C.trace_surfels_backward(*a, hit_record=record), args, s.debug, "snapshot_bw.dump",
                 "backward")
        finally:
            # the storage goes back to the pool (stream-ordered reuse); a second backward through the same graph
            # (retain_graph) walks the BVH again
            ctx.optix_context.release_record(record)

        def like(grad, inp):  # an absent optional input (empty placeholder tensor) gets no gradient
            return grad if inp.numel() != 0 else None

        # one entry per forward() argument after ctx
        return (None, None, None, g_ray_o, g_ray_d, None, g_means3D, g_grads3D, like(g_shs, shs),
                like(g_colors, colors_precomp), like(g_others, others_precomp), g_opacities, g_scales, g_rotations,
                like(g_cov3Ds, cov3Ds_precomp), None)


def trace_surfels(optix_context, training, start_from_first, ray_o, ray_d, vertices, means3D, grads3D, shs,
                  colors_precomp, others_precomp, opacities, scales, rotations, cov3Ds_precomp, tracer_settings):
    # a hit record only pays off when a backward pass can follow: not under torch.no_grad(), not for inputs
    # without gradients (the usual evaluation loop renders nn.Parameter tensors under no_grad)
    optix_context.record_wanted = torch.is_grad_enabled() and any(
        isinstance(t, torch.Tensor) and t.requires_grad
        for t in (ray_o, ray_d, means3D, grads3D, shs, colors_precomp, others_precomp, opacities, scales, rotations))
    return _TraceSurfels.apply(optix_context, training, start_from_first, ray_o, ray_d, vertices, means3D, grads3D,
                               shs, colors_precomp, others_precomp, opacities, scales, rotations, cov3Ds_precomp,
                               tracer_settings)


class SurfelTracer(nn.Module):
    def __init__(self) -> None:
        super().__init__()
        self.pkg_dir = _C._PKG_DIR
        # keeps the reference's attribute name; owns the BVH instead of an OptiX pipeline
        self.optix_context = _C.OptiXStateWrapper(self.pkg_dir)

    @property
    def deterministic(self) -> bool:
        """Extension (not in the reference): when set, the accumulated blending weights and all per-surfel
        gradients are summed in 64-bit fixed point (exact, order-independent) instead of with float atomics: the
        same inputs give the same bits on every run.  Costs time and a workspace of 8 bytes per sum."""
        return self.optix_context.deterministic

    @deterministic.setter
    def deterministic(self, value: bool) -> None:
        self.optix_context.deterministic = bool(value)

    @property
    def distortion(self) -> bool:
        """Extension (not in the reference, which returns zeros: forward.cu:286): when set, the `dist` output is the
        depth distortion of the primary ray as 2DGS defines it, sum_i sum_{j<i} w_i w_j (m_i - m_j)^2 with
        m = far/(far-near) (1 - near/depth), near 0.2, far 100.  Forward only: no gradient flows from it."""
        return self.optix_context.distortion

    @distortion.setter
    def distortion(self, value: bool) -> None:
        self.optix_context.distortion = bool(value)

    @property
    def sh_half(self) -> bool:
        """Extension (not in the reference): when set, every trace packs the SH coefficients to binary16 (round to
        nearest even) and the kernels read that copy, widening to fp32 as they go - half the bytes of the largest
        per-hit gather.  Results are exactly those of `shs.half().float()`; the gradient of `shs` is that of the fp32
        coefficients (the rounding is not differentiated)."""
        return self.optix_context.sh_half

    @sh_half.setter
    def sh_half(self, value: bool) -> None:
        self.optix_context.sh_half = bool(value)

    def build_acceleration_structure(self, vertices: torch.Tensor, triangles: torch.Tensor, rebuild: bool = 1):
        """Build (`rebuild` true) or refit in place the BVH over the surfel quads `vertices` (4P,3), `triangles` (2P,3)."""
        return _C.build_acceleration_structure(self.optix_context, vertices, triangles, rebuild)

    def refit_from_surfels(self, means3D: torch.Tensor, scales: torch.Tensor, rotations: torch.Tensor,
                           vertices_out: torch.Tensor = None) -> torch.Tensor:
        """Extension (not in the reference): refit the BVH in place from the surfel parameters and return the quad
        corners (4P,3) to pass to forward() as `vertices`: what `get_triangles` + `build_acceleration_structure(v, f,
        rebuild=False)` do, in one kernel.  Needs a structure built from `get_triangles`-style quads."""
        return _C.refit_from_surfels(self.optix_context, means3D.detach(), scales.detach(), rotations.detach(),
                                     vertices_out)

    def forward(self, ray_o: torch.Tensor, ray_d: torch.Tensor, vertices: torch.Tensor, means3D: torch.Tensor,
                grads3D: torch.Tensor, shs: torch.Tensor = None, colors_precomp: torch.Tensor = None,
                others_precomp: torch.Tensor = None, opacities: torch.Tensor = None, scales: torch.Tensor = None,
                rotations: torch.Tensor = None, cov3D_precomp: torch.Tensor = None,
                tracer_settings: SurfelTracingSettings = None, start_from_first: bool = True):
        if (shs is None) == (colors_precomp is None):
            raise Exception('Please provide excatly one of either SHs or precomputed colors!')
        has_sr, has_cov = (scales is not None or rotations is not None), cov3D_precomp is not None
        if ((scales is None or rotations is None) and not has_cov) or (has_sr and has_cov):
            raise Exception('Please provide exactly one of either scale/rotation pair or precomputed 3D covariance!')

        dev = means3D.device
        empty = lambda: torch.empty(0, dtype=torch.float32, device=dev)  # noqa: E731 placeholder for an absent input
        shs = empty() if shs is None else shs
        colors_precomp = empty() if colors_precomp is None else colors_precomp
        others_precomp = empty() if others_precomp is None else others_precomp
        scales = empty() if scales is None else scales
        rotations = empty() if rotations is None else rotations
        cov3D_precomp = empty() if cov3D_precomp is None else cov3D_precomp
        vertices = empty() if vertices is None else vertices

        return trace_surfels(self.optix_context, self.training, start_from_first, ray_o, ray_d, vertices, means3D,
                             grads3D, shs, colors_precomp, others_precomp, opacities, scales, rotations,
                             cov3D_precomp, tracer_settings)
