// Internal declarations shared by the BVH builder, the trace kernels and the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string>

#include "dst_api.h"

#define DST_LEAF_BIT 0x80000000u
#define DST_NO_PARENT 0xFFFFFFFFu
#define DST_WAVE 64

#ifndef DST_GROUP
#define DST_GROUP 2             // quads per leaf group (a subtree of at most this many leaves is tested as a unit)
#endif
#define DST_WIDE 4             // children per traversal node
#define DST_REF_FIRST_MASK 0x0FFFFFFFu   // leaf-group reference: DST_LEAF_BIT | (count-1) << 28 | first leaf position
#define DST_MAX_SURFELS 0x0FFFFFFFu

// Internal node of the binary hierarchy (Karras): the boxes of both children live in the parent.
// The builder and the refit work on these; the trace kernels read the 4-wide nodes derived from them.
struct alignas(64) DstNode {
    float lo0[3], hi0[3];
    float lo1[3], hi1[3];
    uint32_t c0, c1;      // child references: DST_LEAF_BIT | leaf position, or internal node index
    uint32_t first, last; // range of leaf positions below this node
};

// Traversal node, indexed like the binary node it was collapsed from: up to four children (the binary
// node's grandchildren, or a child itself where that child is a leaf group), boxes stored by coordinate.
// One 128-byte wave-uniform fetch decides four descents.
struct alignas(128) DstWideNode {
    float lox[DST_WIDE], loy[DST_WIDE], loz[DST_WIDE];
    float hix[DST_WIDE], hiy[DST_WIDE], hiz[DST_WIDE];
    uint32_t ref[DST_WIDE];   // wide node index, or leaf-group reference
    uint32_t count;           // children in use (2..4)
    uint32_t pad[3];
};

// Leaf = one surfel quad in leaf order (triangles ABC and BCD), as the hit test wants it: corner A, the edge vectors
// AB = B-A, AC = C-A, AD = D-A (fp32 differences of the corners), the plane normals n0 = AB x AC, n1 = (C-B)x(D-B),
// n2 = AC x AD, c1 = n1.AB (crosses and dots in the fused form the test is defined with), and the surfel id.
// 96 bytes, fetched once per wave.  The first 64 bytes hold what cannot be derived (n1 is formed from the corners B, C,
// D, which A + AB and so on need not give back); n0, n2 and c1 follow from them by the same fp32 operations, so the
// per-lane walk, whose every lane fetches its own quads, reads 64 bytes and computes them.
struct alignas(16) DstLeaf {
    float A[3], AB[3], AC[3], AD[3];
    float n1[3];
    uint32_t g;
    float n0[3], n2[3];
    float c1;
    uint32_t pad;
};
static_assert(sizeof(DstLeaf) == 96, "leaf records are 24 dwords");

// Cheap conservative stand-in for the exact ray/quad test, one per leaf (same order): the quad as a parallelogram
// on its mean plane.  A ray whose hit point on that plane has |s|, |r| beyond `lim0` (plus a margin for rounding)
// cannot pass the exact test; the walk fetches the 96-byte record and runs the exact test only if some lane
// survives.  c = centroid, n = unit normal, fu/fv = dual vectors of the averaged half edges (s = fu.(P-c),
// r = fv.(P-c): the corners sit at about (+-1, +-1)), mfu = max(|fu|, |fv|), lim0 = largest |s| or |r| of a
// corner, a little enlarged, tdev = how far the corners leave the mean plane, enlarged (0 for a planar quad),
// rad = radius of a sphere around c that holds the quad.  A degenerate quad gets mfu = rad = inf: every ray survives.
struct alignas(64) DstLeafPre {
    float c[3], n[3], fu[3], fv[3];
    float mfu, lim0, tdev, rad;
};
static_assert(sizeof(DstLeafPre) == 64, "one 16-dword scalar fetch");

struct DstBounds {          // device-resident reduction targets, order-preserving uint encoding
    uint32_t lo[3], hi[3];  // centroid bounds
    uint32_t max_abs;       // raw bits of a non-negative float: largest |coordinate| of any vertex
    uint32_t bad_topology;  // set by the quad set-up kernel
    uint32_t equal_keys;    // neighbours in Morton order with equal keys, counted while the hierarchy is made
    uint32_t max_depth;     // nodes above the deepest leaf (builds with two-level keys only)
    uint32_t scale;         // raw bits of a float: size of the scene's bulk (set by a build, kept by refits); what ray
                            // origins are compared with (packets, ray keys) - not a bound on anything
    uint32_t small_quads;   // quads with edges below kDstSmallQuad of that size, counted by every build and refit
};
// Quads this much smaller than the scene are smaller than a pixel at usual resolutions (a 1080p pixel at half the
// scene's size away is about 5e-4 of it wide); a context whose last build counted kDstSmallQuadsMin of them traces
// with the kernels that can hand a tile over (trace.hip), the others with kernels that do not carry that code.
constexpr float kDstSmallQuad = 1.0f / 2048.0f;
constexpr uint32_t kDstSmallQuadsMin = 2048;

// Device-side view of the acceleration structure handed to the trace kernels.
struct DstAccelView {
    const DstWideNode *wide;
    const DstLeaf *leaves;
    const DstLeafPre *pre;
    const DstBounds *bounds;  // max_abs sizes the conservative slab padding; read on the device so that a
                              // refit never needs a host round trip
    uint32_t root;
    uint32_t n_leaves;
};

// Tile hand-over list of the forward trace (layout: trace.hip).  Steps: walks of the benchmark scenes take a few
// hundred; DST_HANDOVER_STEPS in the environment of dst_create sets another limit.
constexpr uint32_t kDstHandoverHeader = 4, kDstHandoverCap = 8192, kDstHandoverSteps = 2048;
constexpr uint32_t kDstHandoverOutOfRange = 3;   // header word lent to the deterministic mode's out-of-range count
// The list shares its allocation with the bounds (made by dst_create).
constexpr size_t kDstHandoverOffset = 64;   // bytes from the bounds to the list
static_assert(sizeof(DstBounds) <= kDstHandoverOffset, "the hand-over list starts behind the bounds");
__host__ __device__ static inline uint32_t *dst_handover_list(const DstBounds *bounds) {
    return reinterpret_cast<uint32_t *>(reinterpret_cast<uintptr_t>(bounds) + kDstHandoverOffset);
}

struct dst_ctx;
// Whether the context's next forward trace uses the kernels that can hand tiles over.
static inline bool dst_handover_active(const dst_ctx *ctx);

struct dst_ctx {
    int device = 0;
    std::string err;
    // acceleration structure
    uint32_t n_leaves = 0;      // surfels in the current structure
    uint32_t capacity = 0;      // surfels the buffers can hold
    bool fine_keys = false;     // builds sort two-level Morton keys (set when a build finds the one-level grid too coarse)
    bool fine_keys_refused = false;   // a build with two-level keys came out too deep for the walks' stacks
    uint32_t refused_builds = 0;      // builds since a refusal (the sixteenth tries again)
    bool built = false;
    uint32_t built_vertices = 0;   // rows of the vertex buffer the stored quad ids were validated against
    bool canonical = false;        // the build's quads were rows 4g..4g+3 of the vertex buffer, in that order
    uint32_t builds = 0, refits = 0;
    bool use_ploc = true;          // builds make the hierarchy by agglomeration (DST_HIERARCHY=morton in the environment: Karras)
    bool ploc_refused = false;     // an agglomerated hierarchy came out too deep: Morton hierarchy for good
    bool agglomerated = false;     // how the current structure's hierarchy was made
    uint32_t hierarchy_depth = 0;  // nodes above its deepest leaf (agglomerated hierarchies; 0: not measured)
    uint32_t *ploc_state = nullptr, *ploc_host = nullptr;   // device / pinned host: counters of the agglomeration
    uint32_t ploc_blocks = 0;
    DstNode *nodes = nullptr;
    DstWideNode *wide = nullptr;
    DstLeaf *leaves = nullptr;
    DstLeafPre *pre = nullptr;
    uint32_t *node_parent = nullptr, *leaf_parent = nullptr;  // (parent << 1) | which child
    uint32_t *flags = nullptr;                                // arrival counters of the bottom-up fit
    int32_t *quad_ids = nullptr;                              // 4 vertex ids per surfel (int4)
    float *centroids = nullptr;                               // 4 floats per surfel
    // boxes of leaf ranges for the fit by look-up: per leaf its own box, the union of its 64-leaf block up to it and
    // from it on (6 floats each), and the unions of 2^l consecutive blocks for every l
    float *range_lbox = nullptr, *range_pbox = nullptr, *range_sbox = nullptr, *range_table = nullptr;
    uint32_t *keys[2] = {nullptr, nullptr}, *vals[2] = {nullptr, nullptr};
    uint32_t *tile_hist = nullptr;
    size_t tile_hist_elems = 0;
    // ordering of ray lists (thin ray grids): sort keys / ray numbers ping-pong and radix histograms, grow-only
    uint32_t *ray_keys[2] = {nullptr, nullptr}, *ray_vals[2] = {nullptr, nullptr}, *ray_hist = nullptr;
    uint32_t ray_capacity = 0;
    uint32_t *block_order = nullptr;   // dispatch order of a replaying backward trace (longest blocks first), grow-only
    uint32_t block_order_capacity = 0;
    // forward traces: tiles whose packet walk ran long, handed over to waves that walk every ray on its own (trace.hip)
    uint32_t *handover = nullptr;      // device, behind `bounds`: kDstHandoverHeader words + kDstHandoverCap entries, zeroed at creation
    uint32_t handover_steps = kDstHandoverSteps;   // limit of a tile's first walk
    int handover_mode = DST_HANDOVER_AUTO;         // auto: only for scenes with many small quads
    uint32_t small_quads = 0;          // as counted by the last build, or by a refit since (see dst_launch_trace)
    uint32_t small_quads_refits = 0;   // ctx->refits when the count was last asked for
    bool small_quads_asked = false;    // a copy of the device's count into bounds_host has been enqueued since the build
    DstBounds *bounds = nullptr;       // device (allocated by dst_create together with the hand-over list)
    DstBounds *bounds_host = nullptr;  // pinned host copy
    void *core_box = nullptr;          // device: the box the two-level Morton keys are laid over (lbvh.hip)
    float scene_lo[3] = {0, 0, 0}, scene_hi[3] = {0, 0, 0}, max_abs = 0;
};

static inline bool dst_handover_active(const dst_ctx *ctx) {
    if (ctx->handover_mode == DST_HANDOVER_OFF || ctx->handover_steps == 0u || ctx->handover == nullptr) return false;
    return ctx->handover_mode == DST_HANDOVER_ALWAYS || ctx->small_quads >= kDstSmallQuadsMin;
}

// Where a traversal starts: the wide node of the binary root, or one leaf group when the scene is that small.
static inline uint32_t dst_root_ref(uint32_t n_leaves) {
    return n_leaves <= DST_GROUP ? (DST_LEAF_BIT | ((n_leaves - 1u) << 28)) : 0u;
}

// lbvh.hip
// Refit source other than a vertex buffer: the surfel parameters themselves (device pointers).
struct DstSurfelSource {
    const float *means, *scales, *rotations;   // (P,3) (P,2) (P,4)
    float *vertices_out;                        // (4P,3) or nullptr
};
// `fit_flags`: arrival counters of the bottom-up fit (one per surfel); nullptr = the context's own.
// `surfels`: refit only; the quads are generated from the surfel parameters instead of read from `vertices`.
int dst_lbvh_build(dst_ctx *ctx, const float *vertices, uint32_t n_vertices, const int32_t *triangles,
                   uint32_t n_surfels, bool rebuild, hipStream_t stream, uint32_t *fit_flags = nullptr,
                   const DstSurfelSource *surfels = nullptr);
// Per-device address of the static scratch array (set up once per device by dst_create).
int dst_static_scratch_init(dst_ctx *ctx);
uint32_t *dst_static_scratch(const dst_ctx *ctx);
void dst_lbvh_free(dst_ctx *ctx);
void dst_sort_pairs(uint32_t *keys[2], uint32_t *vals[2], uint32_t *tile_hist, uint32_t n, hipStream_t stream);
size_t dst_sort_hist_elems(uint32_t n);
// trace.hip
int dst_launch_trace(dst_ctx *ctx, const DstParams &p, bool backward, hipStream_t stream);
int dst_launch_pack_half(const float *src, uint16_t *dst, uint64_t n, hipStream_t stream);

static inline int dst_fail(dst_ctx *ctx, int code, const std::string &msg) {
    if (ctx) ctx->err = msg;
    return code;
}
#define DST_HIP(ctx, call)                                                                       \
    do {                                                                                         \
        hipError_t e_ = (call);                                                                  \
        if (e_ != hipSuccess)                                                                    \
            return dst_fail(ctx, DST_E_DEVICE, std::string(#call) + ": " + hipGetErrorString(e_)); \
    } while (0)
