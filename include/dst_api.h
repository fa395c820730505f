/*
 * C ABI of the MI355X surfel ray tracer (libdst.so).
 *
 * Plain pointers and sizes only: every pointer in DstParams is a DEVICE pointer
 * to fp32 data (int32 for the triangle indices), laid out exactly like the
 * tensors of the reference launcher.  `stream` is a hipStream_t passed as
 * void*; all work is enqueued on it and, except where noted, not waited for.
 * Every entry point returns 0 on success and a nonzero DST_E_* status
 * otherwise; dst_last_error() then describes the failure.
 *
 * Reference interfaces replaced (paths relative to the reference tree):
 *   ext.cpp:7-12                      pybind module with the four symbols below
 *   optix_tracer/optix_wrapper.cpp:166-222   OptiXStateWrapper ctor / dtor
 *   trace_surfels.cpp:36-159          BuildAccelerationStructure
 *   trace_surfels.cpp:162-304         TraceSurfelsCUDA
 *   trace_surfels.cpp:307-464         TraceSurfelsBackwardCUDA
 *   optix_tracer/params.h:21-84       struct Params (launch parameter block)
 */
#ifndef DST_API_H
#define DST_API_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    DST_OK = 0,
    DST_E_INVALID = 1,     /* malformed argument (shape, null pointer, out-of-range setting) */
    DST_E_NO_ACCEL = 2,    /* trace or refit before a successful build */
    DST_E_TOPOLOGY = 3,    /* triangles are not the two-triangles-per-surfel quads, or refit with another size */
    DST_E_DEVICE = 4,      /* a HIP runtime call failed */
    DST_E_UNSUPPORTED = 5  /* setting outside what the kernels are instantiated for */
};

#define DST_FLAG_DETERMINISTIC 1u /* bitwise reproducible a_weights (forward) and per-surfel gradients (backward) */
#define DST_FLAG_DISTORTION 2u    /* forward: out_dist = (depth distortion, M1, M2) of the primary ray as 2DGS defines
                                   * them; the reference leaves it at zero (forward.cu:286) and so does this library
                                   * without the flag.  No gradient flows from it (the reference's backward never reads
                                   * dL_ddist either). */

#define DST_FLAG_SH_HALF 4u       /* forward: the trace reads the SH coefficients from DstParams.shs_half, a binary16 copy
                                   * of shs (made with dst_pack_sh_half), and widens them to fp32 as they are read: half
                                   * the bytes of the largest per-hit gather; results are those of fp32 coefficients that
                                   * hold the rounded values, bit for bit.  A backward trace ignores the flag and reads
                                   * shs: give it the values the forward trace used (the binary16 values, widened); its
                                   * dL_dshs is then the gradient with respect to those.  No counterpart in the reference. */

#define DST_MAX_AUX 8        /* auxiliary channels per surfel (reference AUX_CHANNELS = 2) */
#define DST_MAX_TRACE_DEPTH 3 /* bounces after the primary ray (reference MAX_TRACE_DEPTH = 1) */
#define DST_STATIC_REFIT_MAX_SURFELS (1u << 21) /* largest structure dst_refit_accel_static serves */

/* Opaque tracer state: owns the acceleration structure and its scratch.
 * Replaces OptiXStateWrapper (optix_tracer/optix_wrapper.h:25-52). */
typedef struct dst_ctx dst_ctx;

/* Launch parameter block; mirrors struct Params (optix_tracer/params.h:21-84)
 * with the compile-time AUX_CHANNELS / MAX_TRACE_DEPTH made runtime fields.
 * Channel layout of one mid_val slot (optix_tracer/config.h:8-15):
 * ray_o 0..2, ray_d 3..5, dpt 6, acc 7, norm 8..10, aux 11..11+aux-1, rgb 11+aux..13+aux. */
typedef struct DstParams {
    /* sizes and settings */
    int32_t P, H, W;              /* surfels; ray grid (H,W) = first two dims of ray_o */
    int32_t D, M;                 /* active SH degree 0..3; coefficients per surfel in shs (0 when colours are given) */
    int32_t aux;                  /* auxiliary channels, 1..DST_MAX_AUX */
    int32_t mtd_alloc;            /* mid_val holds mtd_alloc+1 slots per ray */
    int32_t max_trace_depth;      /* 0..mtd_alloc */
    int32_t training;             /* accumulate a_weights */
    int32_t start_from_first;
    float specular_threshold;
    float scale_modifier;         /* accepted and ignored, as in the reference device code */
    /* inputs */
    const float *ray_o, *ray_d;   /* (H,W,3) */
    const float *vertices;        /* (4P,3) */
    const float *background;      /* (3) */
    const float *means3D;         /* (P,3) */
    const float *shs;             /* (P,M,3) or NULL */
    const float *colors_precomp;  /* (P,3) or NULL; exactly one of shs / colors_precomp */
    const float *others_precomp;  /* (P,aux) or NULL */
    const float *opacities;       /* (P,1) */
    const float *scales;          /* (P,2) */
    const float *rotations;       /* (P,4) quaternion (w,x,y,z) */
    /* forward outputs, fully written by the kernel (backward reads them) */
    float *out_rgb;               /* (H,W,3) */
    float *out_dpt, *out_acc;     /* (H,W,1) */
    float *out_norm, *out_dist;   /* (H,W,3) */
    float *out_aux;               /* (H,W,aux) */
    float *mid_val;               /* (H,W,(mtd_alloc+1)*(14+aux)) */
    float *a_weights;             /* (P,1), ACCUMULATED into: caller zero-fills; NULL when !training */
    /* optional forward statistics: counters[0] += entries evaluated, counters[1] += hits composited */
    unsigned long long *counters;
    /* optional hit record (no counterpart in the reference): when non-NULL the forward trace stores every
     * chunk's 16-entry hit buffer in it, together with the colour it evaluated for every composited hit, and a
     * backward trace given the same record replays the buffers instead of walking the BVH again and takes the
     * colours instead of evaluating the spherical harmonics again (same results up to rounding of the gradient
     * algebra, no traversal, no SH gather).  Device memory, 8-byte aligned, sized
     * with dst_hit_record_layout(); the caller zero-fills the first header_words words before the forward
     * call.  Word 0 then holds the number of blocks the forward trace asked for.  If that exceeds
     * hit_record_blocks the record is incomplete: the backward trace sees this ON THE DEVICE and walks the BVH
     * again instead (the host need not look at the record between the two calls; it may read word 0 later to
     * size the next record; at most 2^26 - 1 blocks of a record are used).  Word 1 counts chains a replay found broken: it stays 0 unless the buffer was
     * not written by a forward trace with the same grid, depth and a zeroed header. */
    uint64_t *hit_record;
    uint32_t hit_record_blocks;
    uint32_t flags;               /* DST_FLAG_* */
    /* workspace of the deterministic mode (DST_FLAG_DETERMINISTIC; no counterpart in the reference, whose float
     * atomics make a_weights and the per-surfel gradients depend on the order in which rays finish): every
     * atomically accumulated sum is formed in 64-bit fixed point, where addition is exact and hence independent of
     * order, in this buffer, and converted to fp32 into the caller's tensor by a closing kernel of the same call.
     * Range: the gradients of scales, rotations, means and the densification gradient are kept in units of 2^-36 and
     * hold sums up to about 6.7e7 in magnitude, everything else (colours, SH, opacity, aux, a_weights) in units of
     * 2^-40 up to about 4.2e6; an addend beyond the range is clamped to it and sums beyond it wrap.  Losses whose
     * per-surfel gradients can get there (coordinates in the tens of kilometres with upstream gradients of order
     * one) have to be scaled down by the caller, or traced without this flag.  The closing kernel counts the sums
     * it finds in the outer half of the range (one clamped addend puts a sum there; a sum that wrapped all the way
     * into the inner half escapes the count): DstTraceInfo.det_out_of_range, 0 as long as every sum was in range.
     * Device memory, dst_det_workspace_words() 8-byte words, zero-filled by the caller before each call. */
    unsigned long long *det_workspace;
    /* optional gradient rows (no counterpart in the reference): dst_det_workspace_words(P, aux, 1) floats of device
     * memory, zero-filled by the caller before each backward call.  When non-NULL (and not in the deterministic
     * mode) the backward trace sums the per-surfel gradients in this buffer, where the columns of one surfel lie
     * side by side in one row, and a closing kernel of the same call adds the rows to the dL_d* tensors below.
     * Same results up to the order of the float additions; faster, because a hit's 66-72 atomic additions then go
     * to a few consecutive cache lines instead of one line in each of seven tensors. */
    float *grad_rows;
    /* upstream gradients (backward) */
    const float *dL_drgb, *dL_ddpt, *dL_dacc, *dL_ddist, *dL_dnorm, *dL_daux;
    /* gradient outputs; the per-surfel ones are ACCUMULATED into: caller zero-fills */
    float *dL_dray_o, *dL_dray_d; /* (H,W,3), fully written */
    float *dL_dmeans3D, *dL_dgrads3D; /* (P,3) */
    float *dL_dshs;               /* (P,M,3) */
    float *dL_dcolors;            /* (P,3) */
    float *dL_dothers;            /* (P,aux) */
    float *dL_dopacities;         /* (P,1) */
    float *dL_dscales;            /* (P,2) */
    float *dL_drotations;         /* (P,4) */
    /* forward, DST_FLAG_SH_HALF: binary16 copy of shs, same shape (P,M,3); NULL otherwise (last in the block: the
     * kernels fetch their arguments in groups, and a field in the middle would move the others) */
    const uint16_t *shs_half;
} DstParams;

/* Shape of the current acceleration structure, for tests and tools. */
typedef struct DstAccelInfo {
    uint32_t n_surfels;    /* leaves */
    uint32_t n_internal;   /* internal nodes (n_surfels-1, 0 for a single surfel) */
    uint32_t root;         /* root reference (leaf bit set when n_surfels == 1) */
    uint32_t node_bytes, leaf_bytes;
    float scene_lo[3], scene_hi[3]; /* bounds of the quad centroids used for the Morton grid, as of the last build */
    float max_abs;         /* largest |coordinate| of any vertex, as of the last build or refit the device has finished */
    uint32_t builds, refits;
    uint32_t key_levels;   /* 1: the builds sort 30-bit Morton keys; 2: 60-bit keys in two levels, which a context goes
                              over to, for good, when a build finds more than three quarters of the surfels sharing
                              their cell of the 1024^3 grid with a neighbour (surfels far outside a compact scene) */
    uint32_t agglomerated; /* 1: the hierarchy was made by merging neighbouring clusters of quads by the surface of their
                              union, starting from the Morton order (what builds do by default); 0: read off the Morton
                              codes alone (scenes of fewer than 64 surfels, DST_HIERARCHY=morton in the environment when
                              the context was created, or a context whose agglomerated hierarchy came out deeper than
                              the walks' stacks allow) */
    uint32_t depth;        /* nodes above the deepest leaf of an agglomerated hierarchy (0: not measured) */
} DstAccelInfo;

/* Create / destroy the tracer state on the current HIP device.
 * Replaces OptiXStateWrapper::OptiXStateWrapper / ~OptiXStateWrapper
 * (optix_tracer/optix_wrapper.cpp:166-222).  dst_create returns NULL on failure. */
dst_ctx *dst_create(void);
void dst_destroy(dst_ctx *ctx);

/* Build (rebuild != 0) or refit in place (rebuild == 0) the BVH over the
 * surfel quads.  vertices: (n_vertices,3) fp32; triangles: (n_triangles,3)
 * int32 with rows 2g and 2g+1 forming surfel g's quad and sharing an edge
 * (rows [a,b,c] and [b,c,d]).  A refit reuses the topology of the last build:
 * n_triangles must be unchanged and `triangles` is not read.  A build waits
 * for the stream a few times (it reads back a validity flag and, while it merges
 * clusters into the hierarchy, how many are left); a refit does not.
 * Replaces BuildAccelerationStructure (trace_surfels.cpp:36-159). */
int dst_build_accel(dst_ctx *ctx, const float *vertices, uint32_t n_vertices, const int32_t *triangles,
                    uint32_t n_triangles, int rebuild, void *stream);

/* Refit straight from the surfel parameters (no counterpart in the reference, where the caller regenerates the
 * quads with tensor operations every frame: example/utils/gaussian_utils.py:176-210): the kernel that fills the
 * leaf records builds the four corners of every surfel itself,
 *     v_k = (mean + a_k * (sx * R[:,0])) + b_k * (sy * R[:,1]),   (a,b) = (-3,3), (-3,-3), (3,3), (3,-3),
 * R = rotation of the quaternion (w,x,y,z) divided by its norm sqrt(((w*w + x*x) + y*y) + z*z), every operation
 * in fp32, rounded once, in this order.  means3D (P,3), scales (P,2), rotations (P,4) are device pointers;
 * vertices_out, if not NULL, receives the corners as a (4P,3) buffer in the order the trace calls expect
 * (`vertices` of DstParams).  The structure must come from a build whose quads were rows 4g..4g+3 of its vertex
 * buffer (what get_triangles produces), else DST_E_TOPOLOGY.  Stream-ordered, no wait. */
int dst_refit_from_surfels(dst_ctx *ctx, const float *means3D, const float *scales, const float *rotations,
                           uint32_t n_surfels, float *vertices_out, void *stream);

/* Refit that allocates nothing: dst_build_accel with rebuild == 0, except that the scratch of the refit
 * kernels (one arrival counter per surfel for the bottom-up box fit) is a fixed array inside the library,
 * 4 bytes x DST_STATIC_REFIT_MAX_SURFELS = 8 MiB, which every GPU the library runs on holds until the process
 * ends.  No counterpart in the reference; it is for callers that cannot allocate device memory: code under
 * stream capture, tight per-frame serving loops, harnesses that forbid it.  Calls no hipMalloc / hipFree.
 * A structure of more than DST_STATIC_REFIT_MAX_SURFELS surfels is rejected with DST_E_UNSUPPORTED.  All
 * contexts on one GPU share the array: calls that overlap on one GPU (different streams or threads) race;
 * calls ordered on one stream do not (the counters are cleared by a fill kernel at the start of each call).
 * Stream-ordered, no wait; same results as dst_build_accel(..., rebuild = 0, ...). */
int dst_refit_accel_static(dst_ctx *ctx, const float *vertices, uint32_t n_vertices, void *stream);

/* Forward trace: fills out_* and mid_val, accumulates a_weights.
 * Replaces TraceSurfelsCUDA (trace_surfels.cpp:162-304); stream-ordered, no wait. */
int dst_trace_forward(dst_ctx *ctx, const DstParams *params, void *stream);

/* Backward re-trace: fills dL_dray_o/d, accumulates the per-surfel gradients.
 * Replaces TraceSurfelsBackwardCUDA (trace_surfels.cpp:307-464); stream-ordered, no wait. */
int dst_trace_backward(dst_ctx *ctx, const DstParams *params, void *stream);

/* Message of the last failure on this context (never NULL).  The reference
 * prints CUDA/OptiX failures and carries on (optix_tracer/common.h:38-50). */
const char *dst_last_error(dst_ctx *ctx);

/* Introspection for tests: shape of the BVH, and copies of its arrays to HOST
 * buffers (each may be NULL to skip).  nodes: n_internal*node_bytes, leaves:
 * n_surfels*leaf_bytes, node_parent: n_internal uint32, leaf_parent: n_surfels
 * uint32, sorted_keys: the n_surfels uint32 Morton codes in ascending order (the leaf order of a hierarchy read off
 * the codes; the order an agglomeration starts from).  Waits for the stream. */
int dst_accel_info(dst_ctx *ctx, DstAccelInfo *info);
int dst_accel_download(dst_ctx *ctx, void *nodes, void *leaves, uint32_t *node_parent, uint32_t *leaf_parent,
                       uint32_t *sorted_keys, void *stream);

/* Tile hand-over of the forward trace (no counterpart in the reference, whose rays are traversed one by one by the
 * hardware: optix_tracer/forward.cu:318).  The trace kernels walk the BVH once for the 64 rays of an 8x8 pixel tile.
 * Over geometry much finer than the ray spacing (a dense cloud of surfels far smaller than a pixel) that walk visits
 * everything inside the tile's frustum for the sake of one ray at a time, and one wave runs for milliseconds.  A tile
 * whose first walk takes more than `handover_steps` steps (nodes and leaf groups; default 2048, a few hundred on
 * ordinary scenes) is therefore put on a list and traced by a second launch in which every ray walks on its own: same
 * results bit for bit.  At most `handover_capacity` tiles per call are handed over; further ones are traced the usual
 * way.  The kernels that can hand over are 1 to 4 % slower than those that cannot, so by default (DST_HANDOVER_AUTO)
 * a context uses them only while its last build or refit counted at least 2048 quads with edges below 1/2048 of the scene's
 * size (`small_quads`; refits count too, and their count reaches the host behind the first forward trace that follows,
 * so it serves from the second one on); DST_HANDOVER_ALWAYS and DST_HANDOVER_OFF decide regardless of the
 * scene.  dst_set_handover: steps = 0 keeps the current limit.  DST_HANDOVER=off|auto|always and DST_HANDOVER_STEPS=n
 * in the environment of dst_create set the initial values.  The list is emptied on the device by the second launch, so
 * a forward call recorded into a graph can be replayed.  dst_trace_info waits for the device; tiles_handed_over
 * counts since the context was created (a 32-bit count). */
#define DST_HANDOVER_OFF 0
#define DST_HANDOVER_AUTO 1
#define DST_HANDOVER_ALWAYS 2
typedef struct DstTraceInfo {
    uint32_t handover_mode, handover_steps, handover_capacity;
    uint32_t small_quads;        /* as counted by the last build, or by a refit whose count has arrived */
    uint32_t handover_active;    /* 1: the next forward trace uses the kernels that can hand tiles over */
    uint32_t det_out_of_range;   /* DST_FLAG_DETERMINISTIC: sums found in the outer half of their range since dst_create */
    uint64_t tiles_handed_over;
} DstTraceInfo;
int dst_trace_info(dst_ctx *ctx, DstTraceInfo *info);
int dst_set_handover(dst_ctx *ctx, int mode, uint32_t steps);

/* Size in 8-byte words of a hit record with room for `blocks` chunk blocks, for an (H,W) ray grid traced with
 * `mtd_alloc`.  Also returns the words of the header the caller must zero-fill, and the number of waves the
 * grid is traced with (a forward trace at depth 0 asks for about 3-6 blocks per wave). */
uint64_t dst_hit_record_layout(int32_t H, int32_t W, int32_t mtd_alloc, uint32_t blocks, uint64_t *header_words,
                               uint32_t *n_waves);

/* Words (8 bytes each) of DstParams.det_workspace for a forward (backward = 0: one per surfel) or a backward
 * call (one per surfel and gradient column: 16 + aux table columns + 48 SH columns). */
uint64_t dst_det_workspace_words(int32_t P, int32_t aux, int backward);

/* fp32 -> binary16 (round to nearest even, overflow to infinity) of `n_values` SH coefficients: out[i] = half(shs[i]).
 * Device pointers; stream-ordered, no wait.  Makes DstParams.shs_half for DST_FLAG_SH_HALF.  No counterpart in the
 * reference, whose SH coefficients are fp32 (optix_tracer/forward.cu:265-268). */
int dst_pack_sh_half(const float *shs, uint16_t *out, uint64_t n_values, void *stream);

/* Library version string, and sizeof(DstParams) as compiled (lets a foreign-language binding
 * verify its own struct layout before the first launch). */
const char *dst_version(void);
size_t dst_sizeof_params(void);

#ifdef __cplusplus
}
#endif
#endif
