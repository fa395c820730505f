// C ABI of libdst.so: context management, argument validation, launches.
// Replaces the pybind module and host launcher of the reference (ext.cpp, trace_surfels.cpp).
#include "dst_internal.h"

#include <cstdlib>
#include <cstring>
#include <new>

namespace {

const char *kNoCtx = "null context";

int check_common(dst_ctx *ctx, const DstParams *p) {
    if (!p) return dst_fail(ctx, DST_E_INVALID, "params is null");
    if (!ctx->built) return dst_fail(ctx, DST_E_NO_ACCEL, "build_acceleration_structure has not been called");
    if (p->P <= 0) return dst_fail(ctx, DST_E_INVALID, "means3D must have dimensions (num_points, 3)");
    if ((uint32_t)p->P != ctx->n_leaves)
        return dst_fail(ctx, DST_E_INVALID, "number of surfels differs from the acceleration structure (" +
                                                std::to_string(p->P) + " vs " + std::to_string(ctx->n_leaves) + ")");
    if (p->H < 0 || p->W < 0) return dst_fail(ctx, DST_E_INVALID, "negative ray grid size");
    if (p->aux < 1 || p->aux > DST_MAX_AUX)
        return dst_fail(ctx, DST_E_UNSUPPORTED, "aux channels must be in 1.." + std::to_string(DST_MAX_AUX));
    if (p->mtd_alloc < 0 || p->mtd_alloc > DST_MAX_TRACE_DEPTH)
        return dst_fail(ctx, DST_E_UNSUPPORTED, "mtd_alloc must be in 0.." + std::to_string(DST_MAX_TRACE_DEPTH));
    if (p->max_trace_depth < 0 || p->max_trace_depth > p->mtd_alloc)
        return dst_fail(ctx, DST_E_INVALID, "max_trace_depth exceeds the depth mid_val was allocated for");
    if ((p->shs == nullptr) == (p->colors_precomp == nullptr))
        return dst_fail(ctx, DST_E_INVALID, "exactly one of shs / colors_precomp must be given");
    if (p->shs && (p->D < 0 || p->D > 3 || (p->D + 1) * (p->D + 1) > p->M))
        return dst_fail(ctx, DST_E_INVALID, "sh_degree must be 0..3 and fit the coefficients in shs");
    if (p->H > 0 && p->W > 0 && (!p->ray_o || !p->ray_d))
        return dst_fail(ctx, DST_E_INVALID, "ray_o / ray_d missing");
    if (!p->vertices || !p->background || !p->means3D || !p->opacities || !p->scales || !p->rotations)
        return dst_fail(ctx, DST_E_INVALID,
                        "vertices, background, means3D, opacities, scales and rotations are required");
    if ((p->flags & DST_FLAG_DETERMINISTIC) && !p->det_workspace)
        return dst_fail(ctx, DST_E_INVALID, "the deterministic mode needs det_workspace");
    if (p->flags & ~(DST_FLAG_DETERMINISTIC | DST_FLAG_DISTORTION | DST_FLAG_SH_HALF))
        return dst_fail(ctx, DST_E_INVALID, "unknown bits in flags");

    if (p->hit_record && (reinterpret_cast<uintptr_t>(p->hit_record) & 7u))
        return dst_fail(ctx, DST_E_INVALID, "hit_record must be 8-byte aligned");
    if (p->H > 0 && p->W > 0 &&
        (!p->out_rgb || !p->out_dpt || !p->out_acc || !p->out_norm || !p->out_dist || !p->out_aux || !p->mid_val))
        return dst_fail(ctx, DST_E_INVALID, "forward output buffers missing");
    return DST_OK;
}

}  // namespace

extern "C" {

const char *dst_version(void) { return "dst-mi355x 0.1"; }
size_t dst_sizeof_params(void) { return sizeof(DstParams); }

dst_ctx *dst_create(void) {
    dst_ctx *ctx = new (std::nothrow) dst_ctx();
    if (!ctx) return nullptr;
    if (hipGetDevice(&ctx->device) != hipSuccess) {
        delete ctx;
        return nullptr;
    }
    if (const char *h = std::getenv("DST_HIERARCHY")) ctx->use_ploc = std::strcmp(h, "morton") != 0;
    if (const char *h = std::getenv("DST_HANDOVER_STEPS")) {
        const unsigned long v = std::strtoul(h, nullptr, 10);
        if (v != 0ul) ctx->handover_steps = (uint32_t)std::min<unsigned long>(v, 1ul << 30);
    }
    if (const char *h = std::getenv("DST_HANDOVER"))
        ctx->handover_mode = std::strcmp(h, "off") == 0 ? DST_HANDOVER_OFF
                                                        : (std::strcmp(h, "always") == 0 ? DST_HANDOVER_ALWAYS : DST_HANDOVER_AUTO);
    if (dst_static_scratch_init(ctx) != DST_OK) {   // once per device, with that device current
        delete ctx;
        return nullptr;
    }
    const size_t bytes = kDstHandoverOffset + sizeof(uint32_t) * (kDstHandoverHeader + kDstHandoverCap);
    if (hipMalloc((void **)&ctx->bounds, bytes) != hipSuccess || hipMemset(ctx->bounds, 0, bytes) != hipSuccess ||
        hipDeviceSynchronize() != hipSuccess) {
        dst_destroy(ctx);
        return nullptr;
    }
    ctx->handover = dst_handover_list(ctx->bounds);
    return ctx;
}

void dst_destroy(dst_ctx *ctx) {
    if (!ctx) return;
    dst_lbvh_free(ctx);
    if (ctx->bounds) (void)hipFree(ctx->bounds);
    if (ctx->core_box) (void)hipFree(ctx->core_box);
    if (ctx->bounds_host) (void)hipHostFree(ctx->bounds_host);
    if (ctx->ploc_host) (void)hipHostFree(ctx->ploc_host);
    delete ctx;
}

const char *dst_last_error(dst_ctx *ctx) { return ctx ? ctx->err.c_str() : kNoCtx; }

int dst_build_accel(dst_ctx *ctx, const float *vertices, uint32_t n_vertices, const int32_t *triangles,
                    uint32_t n_triangles, int rebuild, void *stream) {
    if (!ctx) return DST_E_INVALID;
    if (!vertices) return dst_fail(ctx, DST_E_INVALID, "vertices must have dimensions (num_vertices, 3)");
    if (n_triangles == 0 || (n_triangles & 1u))
        return dst_fail(ctx, DST_E_TOPOLOGY, "triangles must have dimensions (2 * num_surfels, 3)");
    const uint32_t P = n_triangles / 2;
    if ((uint64_t)n_vertices < 4ull * P)
        return dst_fail(ctx, DST_E_TOPOLOGY, "vertices must hold four corners per surfel (4 * num_surfels, 3)");
    if (P > DST_MAX_SURFELS) return dst_fail(ctx, DST_E_UNSUPPORTED, "too many surfels");
    if (rebuild) {
        if (!triangles) return dst_fail(ctx, DST_E_INVALID, "triangles must have dimensions (num_triangles, 3)");
    } else {
        if (!ctx->built) return dst_fail(ctx, DST_E_NO_ACCEL, "refit (rebuild=False) before any build");
        if (P != ctx->n_leaves)
            return dst_fail(ctx, DST_E_TOPOLOGY, "refit (rebuild=False) with a different number of surfels");
        if (n_vertices < ctx->built_vertices)
            return dst_fail(ctx, DST_E_TOPOLOGY, "refit (rebuild=False) with fewer vertices than the build indexed");
    }
    if (rebuild && (ctx->fine_keys_refused || ctx->ploc_refused) && ++ctx->refused_builds >= 16u) {
        // a refusal (two-level keys or an agglomerated hierarchy came out too deep for one scene) is not for ever:
        // every sixteenth build tries again
        ctx->fine_keys_refused = ctx->ploc_refused = false;
        ctx->refused_builds = 0u;
    }
    return dst_lbvh_build(ctx, vertices, n_vertices, triangles, P, rebuild != 0, (hipStream_t)stream);
}

int dst_refit_accel_static(dst_ctx *ctx, const float *vertices, uint32_t n_vertices, void *stream) {
    if (!ctx) return DST_E_INVALID;
    if (!vertices) return dst_fail(ctx, DST_E_INVALID, "vertices must have dimensions (num_vertices, 3)");
    if (!ctx->built) return dst_fail(ctx, DST_E_NO_ACCEL, "refit before any build");
    if (ctx->n_leaves > DST_STATIC_REFIT_MAX_SURFELS)
        return dst_fail(ctx, DST_E_UNSUPPORTED, "dst_refit_accel_static holds scratch for at most " +
                                                    std::to_string(DST_STATIC_REFIT_MAX_SURFELS) + " surfels (" +
                                                    std::to_string(ctx->n_leaves) + " in the structure)");
    if (n_vertices < ctx->built_vertices)
        return dst_fail(ctx, DST_E_TOPOLOGY, "refit with fewer vertices than the build indexed");
    int dev = -1;
    DST_HIP(ctx, hipGetDevice(&dev));
    if (dev != ctx->device) return dst_fail(ctx, DST_E_INVALID, "the context belongs to another device");
    uint32_t *scratch = dst_static_scratch(ctx);
    if (!scratch) return dst_fail(ctx, DST_E_DEVICE, "static scratch was not set up on this device");
    return dst_lbvh_build(ctx, vertices, n_vertices, nullptr, ctx->n_leaves, false, (hipStream_t)stream, scratch);
}

int dst_refit_from_surfels(dst_ctx *ctx, const float *means3D, const float *scales, const float *rotations,
                           uint32_t n_surfels, float *vertices_out, void *stream) {
    if (!ctx) return DST_E_INVALID;
    if (!means3D || !scales || !rotations)
        return dst_fail(ctx, DST_E_INVALID, "means3D, scales and rotations are required");
    if (!ctx->built) return dst_fail(ctx, DST_E_NO_ACCEL, "refit before any build");
    if (n_surfels != ctx->n_leaves)
        return dst_fail(ctx, DST_E_TOPOLOGY, "refit with a different number of surfels");
    if (!ctx->canonical)
        return dst_fail(ctx, DST_E_TOPOLOGY,
                        "refit from surfel parameters needs a structure built from quads in rows 4g..4g+3 of the "
                        "vertex buffer (triangles [4g,4g+1,4g+2],[4g+1,4g+2,4g+3])");
    const DstSurfelSource src = {means3D, scales, rotations, vertices_out};
    return dst_lbvh_build(ctx, nullptr, 0, nullptr, n_surfels, false, (hipStream_t)stream, nullptr, &src);
}

int dst_trace_forward(dst_ctx *ctx, const DstParams *p, void *stream) {
    if (!ctx) return DST_E_INVALID;
    int rc = check_common(ctx, p);
    if (rc) return rc;
    if (p->training && !p->a_weights) return dst_fail(ctx, DST_E_INVALID, "training needs a_weights");
    if ((p->flags & DST_FLAG_SH_HALF) && (!p->shs || !p->shs_half))
        return dst_fail(ctx, DST_E_INVALID, "DST_FLAG_SH_HALF needs shs and its binary16 copy shs_half");
    return dst_launch_trace(ctx, *p, false, (hipStream_t)stream);
}

int dst_trace_backward(dst_ctx *ctx, const DstParams *p, void *stream) {
    if (!ctx) return DST_E_INVALID;
    int rc = check_common(ctx, p);
    if (rc) return rc;
    if (p->H > 0 && p->W > 0 &&
        (!p->dL_drgb || !p->dL_ddpt || !p->dL_dacc || !p->dL_dnorm || !p->dL_daux || !p->dL_dray_o || !p->dL_dray_d))
        return dst_fail(ctx, DST_E_INVALID, "upstream gradients or ray gradient buffers missing");
    if (!p->dL_dmeans3D || !p->dL_dgrads3D || !p->dL_dcolors || !p->dL_dopacities || !p->dL_dscales ||
        !p->dL_drotations)
        return dst_fail(ctx, DST_E_INVALID, "per-surfel gradient buffers missing");
    if (p->shs && !p->dL_dshs) return dst_fail(ctx, DST_E_INVALID, "dL_dshs missing");
    if (p->others_precomp && !p->dL_dothers) return dst_fail(ctx, DST_E_INVALID, "dL_dothers missing");
    return dst_launch_trace(ctx, *p, true, (hipStream_t)stream);
}

int dst_trace_info(dst_ctx *ctx, DstTraceInfo *info) {
    if (!ctx || !info) return DST_E_INVALID;
    uint32_t words[kDstHandoverHeader] = {};
    DST_HIP(ctx, hipDeviceSynchronize());
    DST_HIP(ctx, hipMemcpy(words, ctx->handover, sizeof(words), hipMemcpyDeviceToHost));
    info->handover_mode = (uint32_t)ctx->handover_mode;
    info->handover_steps = ctx->handover_steps;
    info->handover_capacity = kDstHandoverCap;
    if (ctx->small_quads_asked && ctx->bounds_host) ctx->small_quads = ctx->bounds_host->small_quads;   // (the device is idle)
    info->small_quads = ctx->small_quads;
    info->handover_active = dst_handover_active(ctx) ? 1u : 0u;
    info->det_out_of_range = words[kDstHandoverOutOfRange];
    info->tiles_handed_over = words[2];
    return DST_OK;
}

int dst_set_handover(dst_ctx *ctx, int mode, uint32_t steps) {
    if (!ctx) return DST_E_INVALID;
    if (mode != DST_HANDOVER_OFF && mode != DST_HANDOVER_AUTO && mode != DST_HANDOVER_ALWAYS)
        return dst_fail(ctx, DST_E_INVALID, "hand-over mode must be DST_HANDOVER_OFF, _AUTO or _ALWAYS");
    ctx->handover_mode = mode;
    if (steps != 0u) ctx->handover_steps = std::min<uint32_t>(steps, 1u << 30);
    return DST_OK;
}

int dst_pack_sh_half(const float *shs, uint16_t *out, uint64_t n_values, void *stream) {
    if (n_values == 0) return DST_OK;
    if (!shs || !out) return DST_E_INVALID;
    return dst_launch_pack_half(shs, out, n_values, (hipStream_t)stream);
}

int dst_accel_info(dst_ctx *ctx, DstAccelInfo *info) {
    if (!ctx || !info) return DST_E_INVALID;
    if (!ctx->built) return dst_fail(ctx, DST_E_NO_ACCEL, "no acceleration structure");
    info->n_surfels = ctx->n_leaves;
    info->n_internal = ctx->n_leaves - 1;
    info->root = dst_root_ref(ctx->n_leaves);
    info->node_bytes = sizeof(DstNode);
    info->leaf_bytes = sizeof(DstLeaf);
    for (int a = 0; a < 3; ++a) {
        info->scene_lo[a] = ctx->scene_lo[a];
        info->scene_hi[a] = ctx->scene_hi[a];
    }
    info->max_abs = ctx->max_abs;
    if (ctx->bounds != nullptr && ctx->bounds_host != nullptr) {
        // what refits and traces have left on the device since the build (waits for the device)
        DST_HIP(ctx, hipMemcpy(ctx->bounds_host, ctx->bounds, sizeof(DstBounds), hipMemcpyDeviceToHost));
        std::memcpy(&info->max_abs, &ctx->bounds_host->max_abs, 4);
    }
    info->builds = ctx->builds;
    info->refits = ctx->refits;
    info->key_levels = ctx->fine_keys ? 2u : 1u;
    info->agglomerated = ctx->agglomerated ? 1u : 0u;
    info->depth = ctx->hierarchy_depth;
    return DST_OK;
}

int dst_accel_download(dst_ctx *ctx, void *nodes, void *leaves, uint32_t *node_parent, uint32_t *leaf_parent,
                       uint32_t *sorted_keys, void *stream) {
    if (!ctx) return DST_E_INVALID;
    if (!ctx->built) return dst_fail(ctx, DST_E_NO_ACCEL, "no acceleration structure");
    hipStream_t s = (hipStream_t)stream;
    DST_HIP(ctx, hipStreamSynchronize(s));
    const size_t n = ctx->n_leaves;
    if (nodes && n > 1) DST_HIP(ctx, hipMemcpy(nodes, ctx->nodes, sizeof(DstNode) * (n - 1), hipMemcpyDeviceToHost));
    if (leaves) DST_HIP(ctx, hipMemcpy(leaves, ctx->leaves, sizeof(DstLeaf) * n, hipMemcpyDeviceToHost));
    if (node_parent && n > 1)
        DST_HIP(ctx, hipMemcpy(node_parent, ctx->node_parent, sizeof(uint32_t) * (n - 1), hipMemcpyDeviceToHost));
    if (leaf_parent) DST_HIP(ctx, hipMemcpy(leaf_parent, ctx->leaf_parent, sizeof(uint32_t) * n, hipMemcpyDeviceToHost));
    if (sorted_keys) DST_HIP(ctx, hipMemcpy(sorted_keys, ctx->keys[0], sizeof(uint32_t) * n, hipMemcpyDeviceToHost));
    return DST_OK;
}

}  // extern "C"
