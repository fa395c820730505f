/*
 * CPU oracle for the differentiable surfel ray tracer -- TEST INFRASTRUCTURE ONLY.
 * Nothing in the shipped library calls, links or imports this file; it exists so
 * that tests, the smoke check and the benchmark's cpu_baseline leg have an
 * independent statement of the reference algorithm to compare the HIP path with.
 *
 * Follows (reference paths, relative to the reference tree):
 *   optix_tracer/forward.cu:18-58    SH colour               -> sh_color()
 *   optix_tracer/forward.cu:63-90    world->splat uv          -> splat_uv()
 *   optix_tracer/forward.cu:136-315  per-bounce compositing   -> bounce_forward()
 *   optix_tracer/forward.cu:318-424  bounce loop              -> path_forward()
 *   optix_tracer/forward.cu:428-477  per-ray IO shell         -> oracle_trace_forward()
 *   optix_tracer/forward.cu:481-525  any-hit sorted insert    -> insert_literal()
 *   optix_tracer/backward.cu:68-166  SH colour backward       -> sh_color_backward()
 *   optix_tracer/backward.cu:201-287 geometry backward        -> splat_uv_backward()
 *   optix_tracer/backward.cu:332-655 per-bounce backward      -> bounce_backward()
 *   optix_tracer/backward.cu:658-853 reverse bounce loop      -> path_backward()
 *   optix_tracer/backward.cu:857-928 per-ray IO shell         -> oracle_trace_backward()
 *   optix_tracer/auxiliary.h:20,26-43,111-121,234-252,403-477 constants, dnormvdv, ddotnd*, quaternion maps
 *   optix_tracer/config.h:5-30       channel layout and tracing constants
 *
 * Parts the reference delegates to NVIDIA OptiX (optix-dev headers + driver
 * runtime, version unpinned, absent from the reference tree) are DEFINED here,
 * because no source for them exists to follow -- parity of these against OptiX
 * itself is UNPINNED:
 *   - the set of hits of a ray: every surfel quad (two triangles sharing the
 *     edge B-C) is tested with signed-volume edge functions, formed from the
 *     cross product of the ray with corner A relative to the origin and the
 *     quad's edge vectors (cross and dot products with fused multiply-adds,
 *     written out in ray_quad()); at most one hit per quad; triangle 0 wins
 *     ties on the shared edge;
 *   - the hit parameter: t = n.(v1-o) / n.d with n = (v2-v1)x(v3-v1) of the hit
 *     triangle (the formula backward.cu:256-262 differentiates), accepted for
 *     0 < t < 1e16;
 *   - arrival order at the any-hit program: ascending primitive index (the
 *     reference's strict ">" then keeps the lower index first among equal t),
 *     which the lexicographic (t, idx) rule reproduces for any arrival order.
 * Two further definitions replace hardware-approximate CUDA intrinsics by
 * exactly-rounded IEEE sequences so that results are reproducible bit for bit
 * on any IEEE machine: rsqrtf(x) := 1/sqrtf(x), exp(x) := oracle_expf(x)
 * (Cody-Waite + degree-6 polynomial, <= 1 ulp from the true value on the range
 * used).  All arithmetic is fp32, evaluated left to right as written and never
 * contracted by the compiler (compile with -ffp-contract=off); the only fused
 * multiply-adds are the explicit std::fmaf calls of the ray/quad test.
 *
 * Deviations from the literal reference, all switchable or unreachable there:
 *   - a buffer entry skipped because its surfel equals the last contributing
 *     one is cleared like any consumed entry (the reference leaves it stale,
 *     forward.cu:207-216); literal_stale=1 restores the reference behaviour;
 *   - mid_val slots of bounces never reached are written as zeros (the
 *     reference copies uninitialised local memory, forward.cu:446,471-476);
 *   - max_trace_depth > mtd_alloc is rejected (overflow in the reference);
 *   - a chunk that neither advances the restart depth nor composites anything
 *     ends the bounce (the reference would loop forever on it);
 *   - per-surfel sums are accumulated in double and rounded once (the
 *     reference uses float atomics whose order is unspecified).
 */
#include "surfel_oracle.h"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <vector>
#include <algorithm>
#include <chrono>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

// ---- constants (config.h:5-30, auxiliary.h:20,26-43) ------------------------------------------
constexpr int kChunk = 16;
constexpr float kInfDepth = 1e16f;
constexpr double kStepEps = 0.00001;
constexpr int kMaxContrib = 256;
constexpr float kStartOffset = 0.06f;
constexpr float kNear = 0.2f;
constexpr float kFar = 100.0f;  // auxiliary.h:20-21
constexpr float kTmin = 0.0001f;
constexpr int kMaxAux = 8;
constexpr int kMaxSlots = 4;  // mtd_alloc + 1
constexpr float C0 = 0.28209479177387814f;
constexpr float C1 = 0.4886025119029199f;
constexpr float C2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                         -1.0925484305920792f, 0.5462742152960396f};
constexpr float C3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f, 0.3731763325901154f,
                         -0.4570457994644658f, 1.445305721320277f, -0.5900435899266435f};

// V3T<float> carries every decision; the gradient algebra is written once for float (the restatement of the
// reference, which is what the GPU path is compared with) and for double (same formulas, same fp32 inputs and
// decisions: shows how much of a float gradient value is rounding of an ill-conditioned formula).
template <typename T> struct V3T { T x, y, z; };
using V3 = V3T<float>;
template <typename T> inline V3T<T> v3t(T x, T y, T z) { return V3T<T>{x, y, z}; }
inline V3 v3(float x, float y, float z) { return V3{x, y, z}; }
inline V3 ld3(const float *p) { return V3{p[0], p[1], p[2]}; }
template <typename T> inline V3T<T> cast3(V3 a) { return V3T<T>{(T)a.x, (T)a.y, (T)a.z}; }
template <typename T> inline V3T<T> operator+(V3T<T> a, V3T<T> b) { return V3T<T>{a.x + b.x, a.y + b.y, a.z + b.z}; }
template <typename T> inline V3T<T> operator-(V3T<T> a, V3T<T> b) { return V3T<T>{a.x - b.x, a.y - b.y, a.z - b.z}; }
template <typename T> inline V3T<T> operator-(V3T<T> a) { return V3T<T>{-a.x, -a.y, -a.z}; }
template <typename T, typename S> inline V3T<T> operator*(V3T<T> a, S s) { return V3T<T>{a.x * (T)s, a.y * (T)s, a.z * (T)s}; }
template <typename T, typename S> inline V3T<T> operator*(S s, V3T<T> a) { return V3T<T>{(T)s * a.x, (T)s * a.y, (T)s * a.z}; }
template <typename T, typename S> inline V3T<T> operator/(V3T<T> a, S s) { return V3T<T>{a.x / (T)s, a.y / (T)s, a.z / (T)s}; }
template <typename T> inline T dot(V3T<T> a, V3T<T> b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
template <typename T> inline V3T<T> cross(V3T<T> a, V3T<T> b) {
    return V3T<T>{a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
}
template <typename T> inline T len(V3T<T> a) { return std::sqrt(dot(a, a)); }

struct Hit { float t; uint32_t idx; };

// ---- exp: Cody-Waite reduction + Cephes single-precision polynomial --------------------------
inline float exp_det(float x) {
    if (!(x >= -87.0f)) return 0.0f;  // also NaN
    if (x > 88.0f) x = 88.0f;
    float kf = std::nearbyint(x * 1.44269504088896341f);
    float r = (x - kf * 0.693359375f) - kf * -2.12194440e-4f;
    float z = r * r;
    float p = 1.9875691500e-4f;
    p = p * r + 1.3981999507e-3f;
    p = p * r + 8.3334519073e-3f;
    p = p * r + 4.1665795894e-2f;
    p = p * r + 1.6666665459e-1f;
    p = p * r + 5.0000001201e-1f;
    p = p * z + r;
    p = p + 1.0f;
    uint32_t bits;
    std::memcpy(&bits, &p, 4);
    bits += (uint32_t)((int32_t)kf << 23);
    std::memcpy(&p, &bits, 4);
    return p;
}

// ---- quaternion (w,x,y,z) -> rows (tangent u, tangent v, normal); auxiliary.h:403-429 ---------
inline void quat_rows(const float *q, V3 R[3]) {
    float s = 1.0f / std::sqrt(q[3] * q[3] + q[0] * q[0] + q[1] * q[1] + q[2] * q[2]);
    float w = q[0] * s, x = q[1] * s, y = q[2] * s, z = q[3] * s;
    R[0] = v3(1.f - 2.f * (y * y + z * z), 2.f * (x * y + w * z), 2.f * (x * z - w * y));
    R[1] = v3(2.f * (x * y - w * z), 1.f - 2.f * (x * x + z * z), 2.f * (y * z + w * x));
    R[2] = v3(2.f * (x * z + w * y), 2.f * (y * z - w * x), 1.f - 2.f * (x * x + y * y));
}

// auxiliary.h:433-477 (no Jacobian of the normalisation)
template <typename T> inline void quat_rows_vjp(const float *qf, const V3T<T> g[3], T out[4]) {
    const T q[4] = {(T)qf[0], (T)qf[1], (T)qf[2], (T)qf[3]};
    T s = (T)1.0f / std::sqrt(q[3] * q[3] + q[0] * q[0] + q[1] * q[1] + q[2] * q[2]);
    T w = q[0] * s, x = q[1] * s, y = q[2] * s, z = q[3] * s;
    out[0] = 2.f * (x * (g[1].z - g[2].y) + y * (g[2].x - g[0].z) + z * (g[0].y - g[1].x));
    out[1] = 2.f * (-2.f * x * (g[1].y + g[2].z) + y * (g[0].y + g[1].x) + z * (g[0].z + g[2].x) + w * (g[1].z - g[2].y));
    out[2] = 2.f * (x * (g[0].y + g[1].x) - 2.f * y * (g[0].x + g[2].z) + z * (g[1].z + g[2].y) + w * (g[2].x - g[0].z));
    out[3] = 2.f * (x * (g[0].z + g[2].x) + y * (g[1].z + g[2].y) - 2.f * z * (g[0].x + g[1].y) + w * (g[0].y - g[1].x));
}

// ---- SH colour; forward.cu:18-58 / backward.cu:18-63 ----------------------------------------------
inline V3 sh_color(int deg, const float *sh, V3 dir, float clamped[3]) {
    auto S = [&](int j) { return ld3(sh + 3 * j); };
    V3 r = C0 * S(0);
    if (deg > 0) {
        float x = dir.x, y = dir.y, z = dir.z;
        r = r - C1 * y * S(1) + C1 * z * S(2) - C1 * x * S(3);
        if (deg > 1) {
            float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
            r = r + C2[0] * xy * S(4) + C2[1] * yz * S(5) + C2[2] * (2.0f * zz - xx - yy) * S(6) +
                C2[3] * xz * S(7) + C2[4] * (xx - yy) * S(8);
            if (deg > 2) {
                r = r + C3[0] * y * (3.0f * xx - yy) * S(9) + C3[1] * xy * z * S(10) +
                    C3[2] * y * (4.0f * zz - xx - yy) * S(11) +
                    C3[3] * z * (2.0f * zz - 3.0f * xx - 3.0f * yy) * S(12) +
                    C3[4] * x * (4.0f * zz - xx - yy) * S(13) + C3[5] * z * (xx - yy) * S(14) +
                    C3[6] * x * (xx - 3.0f * yy) * S(15);
            }
        }
    }
    r = v3(r.x + 0.5f, r.y + 0.5f, r.z + 0.5f);
    clamped[0] = (r.x < 0) ? 1.f : 0.f;
    clamped[1] = (r.y < 0) ? 1.f : 0.f;
    clamped[2] = (r.z < 0) ? 1.f : 0.f;
    return v3(r.x > 0.f ? r.x : 0.f, r.y > 0.f ? r.y : 0.f, r.z > 0.f ? r.z : 0.f);
}

// backward.cu:68-166.  g_sh receives (deg+1)^2 float3; g_dir is ASSIGNED (backward.cu:165).
template <typename T>
inline void sh_color_backward(int deg, const float *sh, V3 dirf, const float clamped[3], const T g_col[3],
                              V3T<T> *g_sh, V3T<T> &g_dir) {
    using W3 = V3T<T>;
    auto S = [&](int j) { return cast3<T>(ld3(sh + 3 * j)); };
    W3 g = v3t<T>(g_col[0] * (clamped[0] != 0.f ? 0.f : 1.f), g_col[1] * (clamped[1] != 0.f ? 0.f : 1.f),
                  g_col[2] * (clamped[2] != 0.f ? 0.f : 1.f));
    W3 dx = v3t<T>(0, 0, 0), dy = v3t<T>(0, 0, 0), dz = v3t<T>(0, 0, 0);
    T x = dirf.x, y = dirf.y, z = dirf.z;
    g_sh[0] = C0 * g;
    if (deg > 0) {
        g_sh[1] = (-C1 * y) * g;
        g_sh[2] = (C1 * z) * g;
        g_sh[3] = (-C1 * x) * g;
        dx = -C1 * S(3);
        dy = -C1 * S(1);
        dz = C1 * S(2);
        if (deg > 1) {
            T xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
            g_sh[4] = (C2[0] * xy) * g;
            g_sh[5] = (C2[1] * yz) * g;
            g_sh[6] = (C2[2] * (2.f * zz - xx - yy)) * g;
            g_sh[7] = (C2[3] * xz) * g;
            g_sh[8] = (C2[4] * (xx - yy)) * g;
            dx = dx + C2[0] * y * S(4) + C2[2] * 2.f * -x * S(6) + C2[3] * z * S(7) + C2[4] * 2.f * x * S(8);
            dy = dy + C2[0] * x * S(4) + C2[1] * z * S(5) + C2[2] * 2.f * -y * S(6) + C2[4] * 2.f * -y * S(8);
            dz = dz + C2[1] * y * S(5) + C2[2] * 2.f * 2.f * z * S(6) + C2[3] * x * S(7);
            if (deg > 2) {
                g_sh[9] = (C3[0] * y * (3.f * xx - yy)) * g;
                g_sh[10] = (C3[1] * xy * z) * g;
                g_sh[11] = (C3[2] * y * (4.f * zz - xx - yy)) * g;
                g_sh[12] = (C3[3] * z * (2.f * zz - 3.f * xx - 3.f * yy)) * g;
                g_sh[13] = (C3[4] * x * (4.f * zz - xx - yy)) * g;
                g_sh[14] = (C3[5] * z * (xx - yy)) * g;
                g_sh[15] = (C3[6] * x * (xx - 3.f * yy)) * g;
                dx = dx + (C3[0] * S(9) * 3.f * 2.f * xy + C3[1] * S(10) * yz + C3[2] * S(11) * -2.f * xy +
                           C3[3] * S(12) * -3.f * 2.f * xz + C3[4] * S(13) * (-3.f * xx + 4.f * zz - yy) +
                           C3[5] * S(14) * 2.f * xz + C3[6] * S(15) * 3.f * (xx - yy));
                dy = dy + (C3[0] * S(9) * 3.f * (xx - yy) + C3[1] * S(10) * xz +
                           C3[2] * S(11) * (-3.f * yy + 4.f * zz - xx) + C3[3] * S(12) * -3.f * 2.f * yz +
                           C3[4] * S(13) * -2.f * xy + C3[5] * S(14) * -2.f * yz + C3[6] * S(15) * -3.f * 2.f * xy);
                dz = dz + (C3[1] * S(10) * xy + C3[2] * S(11) * 4.f * 2.f * yz +
                           C3[3] * S(12) * 3.f * (2.f * zz - xx - yy) + C3[4] * S(13) * 4.f * 2.f * xz +
                           C3[5] * S(14) * (xx - yy));
            }
        }
    }
    g_dir = v3t<T>(dot(dx, g), dot(dy, g), dot(dz, g));
}

// ---- world -> splat; forward.cu:63-90 ------------------------------------------------------------
struct Splat {
    V3 R[3];      // rows of world2splat (tangent u, tangent v, normal)
    float mT[3];  // fourth column: -(R mean)
    float u, v;   // uv / scale
};
inline void splat_uv(const float *mean, const float *scale, const float *rot, V3 xyz, Splat &s) {
    quat_rows(rot, s.R);
    V3 m = ld3(mean);
    V3 T = v3(dot(s.R[0], m), dot(s.R[1], m), dot(s.R[2], m));
    s.mT[0] = -T.x; s.mT[1] = -T.y; s.mT[2] = -T.z;
    // dot of a float4 row with (xyz, 1): ((a.x*b.x + a.y*b.y) + a.z*b.z) + a.w*b.w
    float ux = s.R[0].x * xyz.x + s.R[0].y * xyz.y + s.R[0].z * xyz.z + s.mT[0] * 1.0f;
    float uy = s.R[1].x * xyz.x + s.R[1].y * xyz.y + s.R[1].z * xyz.z + s.mT[1] * 1.0f;
    s.u = ux / scale[0];
    s.v = uy / scale[1];
}

// ---- ray / surfel-quad test (defined here, see the header comment) ---------------------------
// Products that feed a difference or a running sum are fused (std::fmaf, one rounding), exactly as written:
// the fused form is part of the definition, so any IEEE machine reproduces it bit for bit.
inline V3 cross_f(V3 x, V3 y) {
    return V3{std::fmaf(x.y, y.z, -(x.z * y.y)), std::fmaf(x.z, y.x, -(x.x * y.z)), std::fmaf(x.x, y.y, -(x.y * y.x))};
}
inline float dot_f(V3 a, V3 b) { return std::fmaf(a.z, b.z, std::fmaf(a.y, b.y, a.x * b.x)); }
inline bool same_sign(float a, float b, float c) {
    return (a >= 0.f && b >= 0.f && c >= 0.f) || (a <= 0.f && b <= 0.f && c <= 0.f);
}
// Quad = triangles ABC and BCD.  With a = A - o, m = d x a and the edge vectors AB, AC, AD from corner A, the signed
// volume of an edge test is  d.((A+P'-o) x (A+Q'-o)) = (Q'-P').m + d.(P' x Q'):  the only product of two vectors as
// long as the way from the origin to the quad is m itself, so the test decides to within about eps |a| of an edge.
// (Formed from the four corners relative to the origin, the volumes carry an error of eps |a|^2 / |edge|: half a quad's
// width for millimetre quads seen from a few metres.)  Everything that depends on the quad alone - the edge vectors,
// n0 = AB x AC, n1 = (C-B) x (D-B), n2 = AC x AD, c1 = n1.AB - is what the library keeps per quad.
inline bool ray_quad(V3 o, V3 d, V3 A, V3 B, V3 C, V3 Dv, float &t, int &tri) {
    const V3 AB = B - A, AC = C - A, AD = Dv - A;
    const V3 n0 = cross_f(AB, AC), n1 = cross_f(C - B, Dv - B), n2 = cross_f(AC, AD);
    const float c1 = dot_f(n1, AB);
    const V3 a = A - o;
    const V3 m = cross_f(d, a);
    const float X = dot_f(AB, m), Y = dot_f(AC, m), Z = dot_f(AD, m);
    const float q0 = dot_f(n0, d), q1 = dot_f(n1, d), q2 = dot_f(n2, d);
    const float u2 = X, u1 = -Y, u0 = (Y - X) + q0;   // edges AB, CA, BC
    float p, q;
    if (same_sign(u0, u1, u2)) {
        p = dot_f(n0, a);
        q = q0;
        tri = 0;
    } else {
        const float w0 = (Z - Y) + q2;                  // edge CD
        const float w1 = (X - Z) + ((q1 - q0) - q2);    // edge DB: AD x AB = n1 - n0 - n2
        if (!same_sign(w0, w1, u0)) return false;
        const float pa = dot_f(n1, a);
        p = pa + c1;                                    // n1.(B-o)
        q = q1;
        tri = 1;
    }
    t = p / q;
    return (t > 0.0f) && (t < kInfDepth);
}

// forward.cu:481-525 with the candidates arriving in the caller's order
inline void insert_literal(Hit buf[kChunk], uint32_t &cnt, float t, uint32_t idx) {
    if (t < buf[kChunk - 1].t) {
        cnt += 1;
        Hit cur{t, idx};
        for (int i = 0; i < kChunk; ++i) {
            if (buf[i].t > cur.t) std::swap(buf[i], cur);
        }
    }
}
// arrival-order independent variant: (t, idx) compared lexicographically
inline bool lex_less(const Hit &a, const Hit &b) { return a.t < b.t || (a.t == b.t && a.idx < b.idx); }
inline void insert_lexi(Hit buf[kChunk], uint32_t &cnt, float t, uint32_t idx) {
    Hit cur{t, idx};
    if (lex_less(cur, buf[kChunk - 1])) {
        cnt += 1;
        for (int i = 0; i < kChunk; ++i) {
            if (lex_less(cur, buf[i])) std::swap(buf[i], cur);
        }
    }
}

// ---- a plain median-split BVH over the quads (CPU only; speeds up the baseline) --------------------
struct CpuBvh {
    struct Node { float lo[3], hi[3]; int32_t left, right, first, count; };
    std::vector<Node> nodes;
    std::vector<int32_t> order;
    float max_abs = 0.f;
};

struct Scene {
    const OracleParams *p;
    std::vector<int32_t> quad_v;  // 4 vertex ids per surfel, through the face buffer
    CpuBvh bvh;
};

void quad_vertex_ids(const OracleParams *p, std::vector<int32_t> &ids) {
    ids.resize((size_t)p->P * 4);
    for (int g = 0; g < p->P; ++g) {
        const int32_t *f0 = p->faces + (size_t)(2 * g) * 3;
        const int32_t *f1 = f0 + 3;
        ids[4 * (size_t)g + 0] = f0[0];
        ids[4 * (size_t)g + 1] = f0[1];
        ids[4 * (size_t)g + 2] = f0[2];
        ids[4 * (size_t)g + 3] = f1[2];
    }
}

bool faces_are_quads(const OracleParams *p) {
    for (int g = 0; g < p->P; ++g) {
        const int32_t *f0 = p->faces + (size_t)(2 * g) * 3;
        const int32_t *f1 = f0 + 3;
        if (f1[0] != f0[1] || f1[1] != f0[2]) return false;
        for (int k = 0; k < 3; ++k)
            if (f0[k] < 0 || f0[k] >= 4 * p->P || f1[k] < 0 || f1[k] >= 4 * p->P) return false;
    }
    return true;
}

void build_cpu_bvh(Scene &sc) {
    const OracleParams *p = sc.p;
    const int P = p->P;
    CpuBvh &b = sc.bvh;
    b.order.resize(P);
    std::vector<float> lo((size_t)P * 3), hi((size_t)P * 3), ce((size_t)P * 3);
    for (int g = 0; g < P; ++g) {
        b.order[g] = g;
        for (int a = 0; a < 3; ++a) {
            float mn = INFINITY, mx = -INFINITY;
            for (int k = 0; k < 4; ++k) {
                float c = p->vertices[(size_t)sc.quad_v[4 * (size_t)g + k] * 3 + a];
                mn = std::min(mn, c);
                mx = std::max(mx, c);
            }
            lo[(size_t)g * 3 + a] = mn;
            hi[(size_t)g * 3 + a] = mx;
            ce[(size_t)g * 3 + a] = 0.5f * (mn + mx);
            b.max_abs = std::max(b.max_abs, std::max(std::fabs(mn), std::fabs(mx)));
        }
    }
    b.nodes.reserve((size_t)P);
    struct Task { int node, first, count; };
    std::vector<Task> todo;
    b.nodes.push_back({});
    todo.push_back({0, 0, P});
    while (!todo.empty()) {
        Task t = todo.back();
        todo.pop_back();
        CpuBvh::Node nd{};
        float cl[3] = {INFINITY, INFINITY, INFINITY}, ch[3] = {-INFINITY, -INFINITY, -INFINITY};
        for (int a = 0; a < 3; ++a) { nd.lo[a] = INFINITY; nd.hi[a] = -INFINITY; }
        for (int i = t.first; i < t.first + t.count; ++i) {
            int g = b.order[i];
            for (int a = 0; a < 3; ++a) {
                nd.lo[a] = std::min(nd.lo[a], lo[(size_t)g * 3 + a]);
                nd.hi[a] = std::max(nd.hi[a], hi[(size_t)g * 3 + a]);
                cl[a] = std::min(cl[a], ce[(size_t)g * 3 + a]);
                ch[a] = std::max(ch[a], ce[(size_t)g * 3 + a]);
            }
        }
        nd.first = t.first;
        nd.count = t.count;
        nd.left = nd.right = -1;
        if (t.count > 4) {
            int axis = 0;
            if (ch[1] - cl[1] > ch[axis] - cl[axis]) axis = 1;
            if (ch[2] - cl[2] > ch[axis] - cl[axis]) axis = 2;
            int mid = t.first + t.count / 2;
            std::nth_element(b.order.begin() + t.first, b.order.begin() + mid, b.order.begin() + t.first + t.count,
                             [&](int x, int y) { return ce[(size_t)x * 3 + axis] < ce[(size_t)y * 3 + axis]; });
            nd.left = (int)b.nodes.size();
            b.nodes.push_back({});
            nd.right = (int)b.nodes.size();
            b.nodes.push_back({});
            todo.push_back({nd.left, t.first, mid - t.first});
            todo.push_back({nd.right, mid, t.first + t.count - mid});
        }
        b.nodes[t.node] = nd;
    }
}

inline bool test_surfel(const Scene &sc, int g, V3 o, V3 d, float &t, int &tri) {
    const float *V = sc.p->vertices;
    const int32_t *q = &sc.quad_v[4 * (size_t)g];
    return ray_quad(o, d, ld3(V + 3 * (size_t)q[0]), ld3(V + 3 * (size_t)q[1]), ld3(V + 3 * (size_t)q[2]),
                    ld3(V + 3 * (size_t)q[3]), t, tri);
}

// One traversal: the (up to) 16 nearest hits of the ray (o, d), 0 < t < 1e16.
void k_nearest(const Scene &sc, V3 o, V3 d, Hit buf[kChunk], uint32_t &cnt) {
    const OracleParams *p = sc.p;
    if (p->hit_mode != ORACLE_HITS_BVH_LEXI) {
        for (int g = 0; g < p->P; ++g) {
            float t;
            int tri;
            if (!test_surfel(sc, g, o, d, t, tri)) continue;
            if (p->hit_mode == ORACLE_HITS_BRUTE_LITERAL) insert_literal(buf, cnt, t, 2u * (uint32_t)g + (uint32_t)tri);
            else insert_lexi(buf, cnt, t, 2u * (uint32_t)g + (uint32_t)tri);
        }
        return;
    }
    const CpuBvh &b = sc.bvh;
    // Slab test made conservative against the rounding of the quad test by widening every
    // interval by a tolerance proportional to the distances involved.
    float oa = std::max(std::fabs(o.x), std::max(std::fabs(o.y), std::fabs(o.z)));
    float pad = 4e-6f * (oa + b.max_abs);
    float dd[3] = {d.x, d.y, d.z}, oo[3] = {o.x, o.y, o.z}, inv[3];
    for (int a = 0; a < 3; ++a) {
        float v = dd[a];
        if (std::fabs(v) < 1e-20f) v = std::copysign(1e-20f, v);
        inv[a] = 1.0f / v;
    }
    int stack[128];
    int sp = 0;
    stack[sp++] = 0;
    while (sp > 0) {
        const CpuBvh::Node &nd = b.nodes[stack[--sp]];
        float tn = 0.f, tf = buf[kChunk - 1].t;
        bool ok = true;
        for (int a = 0; a < 3; ++a) {
            float t1 = (nd.lo[a] - oo[a]) * inv[a], t2 = (nd.hi[a] - oo[a]) * inv[a];
            float w = pad * std::fabs(inv[a]);
            float lo_t = std::min(t1, t2) - w, hi_t = std::max(t1, t2) + w;
            tn = std::max(tn, lo_t);
            tf = std::min(tf, hi_t);
            if (!(tn <= tf)) { ok = false; break; }
        }
        if (!ok) continue;
        if (nd.left < 0) {
            for (int i = nd.first; i < nd.first + nd.count; ++i) {
                int g = b.order[i];
                float t;
                int tri;
                if (test_surfel(sc, g, o, d, t, tri)) insert_lexi(buf, cnt, t, 2u * (uint32_t)g + (uint32_t)tri);
            }
        } else {
            stack[sp++] = nd.left;
            stack[sp++] = nd.right;
        }
    }
}

// ---- per-surfel accumulators (double, rounded once at the end) ----------------------------------------
struct Accum {
    std::vector<double> w, means, grads, shs, colors, others, opac, scales, rots;
    // optional (backward with grad_f64 and noise outputs): summed first-order sensitivity of the geometric
    // gradients to fp32 rounding of the plane-hit chain
    bool noise = false;
    std::vector<double> n_means, n_grads, n_scales, n_rots;
};
inline void aadd(std::vector<double> &v, size_t i, double x) {
    double *d = v.data();
#pragma omp atomic
    d[i] += x;
}
void flush(const std::vector<double> &a, float *out) {
    if (!out) return;
    for (size_t i = 0; i < a.size(); ++i) out[i] = (float)a[i];
}

struct BounceOut {
    float C[3], D, A, O[kMaxAux], T;
    V3 N, E;
    float DS, M1, M2;   // depth distortion and its running moments (only with compute_dist)
};

inline int mid_channels(const OracleParams *p) { return 11 + p->aux + 3; }

// forward.cu:136-315
void bounce_forward(const Scene &sc, V3 ray_o, V3 ray_d, float min_depth, float T_threshold, BounceOut &r,
                    Accum *acc, int &n_proc, int &n_con) {
    const OracleParams *p = sc.p;
    Hit buf[kChunk];
    for (int i = 0; i < kChunk; ++i) buf[i] = Hit{kInfDepth, 0u};
    float pay_dpt = 0.0f;
    uint32_t pay_cnt = 0;
    V3 ray_ot = ray_o;
    int last_g = -1, contributor = 0;
    float T_prev = 1.0f, T_next = 1.0f, dpt = 0.0f;
    for (int ch = 0; ch < 3; ++ch) r.C[ch] = 0.f;
    for (int ch = 0; ch < kMaxAux; ++ch) r.O[ch] = 0.f;
    r.D = 0.f;
    r.N = v3(0, 0, 0);
    r.DS = r.M1 = r.M2 = 0.f;
    for (;;) {
        k_nearest(sc, ray_ot, ray_d, buf, pay_cnt);
        int contributed_here = 0;
        for (int i = 0; i < kChunk; ++i) {
            if ((uint32_t)i >= pay_cnt) break;
            int pidx = (int)buf[i].idx;
            int g = pidx / 2;
            if (g == last_g) {
                if (!p->literal_stale) buf[i] = Hit{kInfDepth, 0u};
                continue;
            }
            dpt = buf[i].t + pay_dpt;
            V3 xyz = v3(ray_o.x + dpt * ray_d.x, ray_o.y + dpt * ray_d.y, ray_o.z + dpt * ray_d.z);
            buf[i] = Hit{kInfDepth, 0u};
            Splat s;
            splat_uv(p->means3D + 3 * (size_t)g, p->scales + 2 * (size_t)g, p->rotations + 4 * (size_t)g, xyz, s);
            n_proc++;
            float rho = s.u * s.u + s.v * s.v;
            V3 normal = s.R[2];
            float cosv = -(ray_d.x * normal.x + ray_d.y * normal.y + ray_d.z * normal.z);
            if (cosv == 0) continue;
            normal = cosv > 0 ? normal : -normal;
            if (dpt < min_depth) continue;
            float power = -0.5f * rho;
            if (power > 0.0f) continue;
            float alpha = p->opacities[g] * exp_det(power);
            alpha = (alpha < 0.99f) ? alpha : 0.99f;  // min(0.99f, .), NaN -> 0.99 like fminf
            if (alpha < 1.0f / 255.0f) continue;
            T_next = T_prev * (1 - alpha);
            if (T_next < T_threshold) break;
            contributor++;
            if (contributor > kMaxContrib) break;
            last_g = g;
            float w = alpha * T_prev;
            if (p->colors_precomp == nullptr) {
                float cl[3];
                V3 c = sh_color(p->D, p->shs + (size_t)g * p->M * 3, ray_d, cl);
                r.C[0] += w * c.x;
                r.C[1] += w * c.y;
                r.C[2] += w * c.z;
            } else {
                for (int ch = 0; ch < 3; ++ch) r.C[ch] += w * p->colors_precomp[ch + 3 * (size_t)g];
            }
            if (p->others_precomp != nullptr)
                for (int ch = 0; ch < p->aux; ++ch) r.O[ch] += w * p->others_precomp[ch + (size_t)p->aux * g];
            if (p->compute_dist) {
                // the distortion the reference declares and leaves open (forward.cu:147-152,286), as 2DGS defines it
                const float A_before = 1 - T_prev;
                const float m = kFar / (kFar - kNear) * (1 - kNear / dpt);
                r.DS += (m * m * A_before + r.M2 - 2 * m * r.M1) * w;
                r.M1 += m * w;
                r.M2 += m * m * w;
            }
            r.D += w * dpt;
            r.N = v3(r.N.x + w * normal.x, r.N.y + w * normal.y, r.N.z + w * normal.z);
            T_prev = T_next;
            n_con++;
            contributed_here++;
            if (p->training && acc) aadd(acc->w, (size_t)g, (double)w);
        }
        if (T_next < T_threshold || pay_cnt < (uint32_t)kChunk || contributor > kMaxContrib) break;
        float next_dpt = (float)((double)dpt + kStepEps);  // STEP_EPSILON is a double literal (config.h:21)
        if (!(next_dpt > pay_dpt) && contributed_here == 0) break;  // would never end
        pay_dpt = next_dpt;
        pay_cnt = 0;
        ray_ot = v3(ray_o.x + pay_dpt * ray_d.x, ray_o.y + pay_dpt * ray_d.y, ray_o.z + pay_dpt * ray_d.z);
    }
    for (int ch = 0; ch < 3; ++ch) r.C[ch] += T_prev * p->background[ch];
    r.A = 1 - T_prev;
    r.T = T_prev;
    r.E = v3(ray_o.x + r.D * ray_d.x, ray_o.y + r.D * ray_d.y, ray_o.z + r.D * ray_d.z);
}

// forward.cu:318-424
void path_forward(const Scene &sc, V3 ray_o, V3 ray_d, float *out_rgb, float &out_dpt, float &out_acc, V3 &out_norm,
                  V3 &out_dist, float *out_aux, float *mid, Accum *acc, int &n_proc, int &n_con) {
    const OracleParams *p = sc.p;
    const int MID = mid_channels(p), AUXO = 11, RGBO = 11 + p->aux;
    V3 ot = ray_o, dt = ray_d;
    float s_prod = 1.0f;
    for (int i = 0; i < p->max_trace_depth + 1; ++i) {
        float min_depth = (i == 0 && p->start_from_first) ? kNear : (i == 0 && !p->start_from_first) ? 0.0f : kStartOffset;
        BounceOut b;
        bounce_forward(sc, ot, dt, min_depth, kTmin, b, acc, n_proc, n_con);
        if (i == 0) {
            out_dpt = b.D;
            out_acc = b.A;
            out_norm = b.N;
            out_dist = v3(b.DS, b.M1, b.M2);   // forward.cu:384 (zeros in the reference: never accumulated)
            for (int ch = 0; ch < p->aux; ++ch) out_aux[ch] = b.O[ch];
        }
        float f_this = (i == p->max_trace_depth) ? 1.0f : 1 - b.O[0];
        for (int ch = 0; ch < 3; ++ch) out_rgb[ch] += b.C[ch] * f_this * s_prod;
        s_prod *= b.O[0];
        float *m = mid + (size_t)i * MID;
        m[0] = ot.x; m[1] = ot.y; m[2] = ot.z;
        m[3] = dt.x; m[4] = dt.y; m[5] = dt.z;
        for (int ch = 0; ch < 3; ++ch) m[RGBO + ch] = b.C[ch];
        m[6] = b.D;
        m[7] = b.A;
        m[8] = b.N.x; m[9] = b.N.y; m[10] = b.N.z;
        for (int ch = 0; ch < p->aux; ++ch) m[AUXO + ch] = b.O[ch];
        if (len(b.N) == 0.0f || b.O[0] <= p->specular_threshold) break;
        V3 n = b.N / len(b.N);
        dt = dt - 2 * dot(n, dt) * n;
        ot = b.E + kStartOffset * dt;
    }
}

// backward.cu:201-287
template <typename T> struct GeoGrad { T scale[2], rot[4]; V3T<T> mean; };
template <typename T>
void splat_uv_backward(const float *mean, const float *scale, const float *rot, V3 xyzf, const Splat &sf,
                       float normal_sign, V3 ray_of, V3 ray_df, float dptf, V3 v1f, V3 v2f, V3 v3f, V3 h1, V3 h2, V3 h3,
                       float Gf, float pclamp, V3T<T> g_N, T g_D, T g_G, V3T<T> &g_ray_o, V3T<T> &g_ray_d,
                       GeoGrad<T> &out, int perturb = 0) {
    using W3 = V3T<T>;
    const W3 pm = cast3<T>(ld3(mean)), xyz = cast3<T>(xyzf), ray_o = cast3<T>(ray_of), ray_d = cast3<T>(ray_df);
    const W3 v1 = cast3<T>(v1f), v2 = cast3<T>(v2f), v3_ = cast3<T>(v3f);
    const W3 R0 = cast3<T>(sf.R[0]), R1 = cast3<T>(sf.R[1]);
    const T sx = scale[0], sy = scale[1], G = Gf, su_ = sf.u, sv_ = sf.v, dpt = dptf;
    T gu = g_G * pclamp * -G * su_, gv = g_G * pclamp * -G * sv_;
    W3 gR[3];
    gR[0] = gu * (xyz - pm) / sx;
    gR[1] = gv * (xyz - pm) / sy;
    gR[2] = g_N * normal_sign;
    out.scale[0] = g_G * pclamp * (G * su_ * su_ / sx);
    out.scale[1] = g_G * pclamp * (G * sv_ * sv_ / sy);
    W3 dG_dmean = G * (R0 * su_ / sx + R1 * sv_ / sy);
    out.mean = g_G * pclamp * dG_dmean;
    W3 g_xyz = v3t<T>(gu / sx * R0.x + gv / sy * R1.x, gu / sx * R0.y + gv / sy * R1.y, gu / sx * R0.z + gv / sy * R1.z);
    T g_d = g_D + dot(g_xyz, ray_d);
    W3 n = cross(v2 - v1, v3_ - v1);
    W3 c = v1 - ray_o;
    // `perturb` (sensitivity estimate only): move one rounded intermediate of the plane-hit chain by one unit of
    // fp32 rounding of the operands it was computed from
    const T ulp = (T)1.1920929e-7f;
    if (perturb == 3) c = c + v3t<T>(ulp * (std::abs(v1.x) + std::abs(ray_o.x)), ulp * (std::abs(v1.y) + std::abs(ray_o.y)),
                                     ulp * (std::abs(v1.z) + std::abs(ray_o.z)));
    T pp = dot(n, c), q = dot(n, ray_d);
    if (perturb == 1) pp += ulp * (std::abs(n.x * c.x) + std::abs(n.y * c.y) + std::abs(n.z * c.z));
    if (perturb == 2) q += ulp * (std::abs(n.x * ray_d.x) + std::abs(n.y * ray_d.y) + std::abs(n.z * ray_d.z));
    W3 g_n = (c - pp / q * ray_d) / q;
    W3 g_v1 = g_d * cross(v2 - v3_, g_n) + g_d * n / q;
    W3 g_v2 = g_d * cross(v3_ - v1, g_n);
    W3 g_v3 = g_d * cross(v1 - v2, g_n);
    g_ray_o = g_ray_o + (g_xyz + g_d * -n / q);
    g_ray_d = g_ray_d + (g_xyz * dpt + g_d * -pp / (q * q) * n);
    gR[0].x += sx * (h1.x * g_v1.x + h2.x * g_v2.x + h3.x * g_v3.x);
    gR[0].y += sx * (h1.x * g_v1.y + h2.x * g_v2.y + h3.x * g_v3.y);
    gR[0].z += sx * (h1.x * g_v1.z + h2.x * g_v2.z + h3.x * g_v3.z);
    gR[1].x += sy * (h1.y * g_v1.x + h2.y * g_v2.x + h3.y * g_v3.x);
    gR[1].y += sy * (h1.y * g_v1.y + h2.y * g_v2.y + h3.y * g_v3.y);
    gR[1].z += sy * (h1.y * g_v1.z + h2.y * g_v2.z + h3.y * g_v3.z);
    quat_rows_vjp<T>(rot, gR, out.rot);
    out.scale[0] += dot(R0, h1.x * g_v1 + h2.x * g_v2 + h3.x * g_v3);
    out.scale[1] += dot(R1, h1.y * g_v1 + h2.y * g_v2 + h3.y * g_v3);
    out.mean = out.mean + (g_v1 + g_v2 + g_v3);
}

template <typename T>
struct BounceIn {  // saved results of this bounce and its upstream gradients
    float rgb[3], dpt, acc, aux[kMaxAux];
    V3 norm;
    T g_rgb[3], g_dpt, g_acc, g_aux[kMaxAux];
    V3T<T> g_norm;
};

// backward.cu:332-655
template <typename T>
void bounce_backward(const Scene &sc, V3 ray_o, V3 ray_d, float min_depth, float T_threshold, const BounceIn<T> &in,
                     V3T<T> &g_ray_o, V3T<T> &g_ray_d, Accum &acc, V3T<T> *n_ray_o = nullptr,
                     V3T<T> *n_ray_d = nullptr) {
    const OracleParams *p = sc.p;
    Hit buf[kChunk];
    for (int i = 0; i < kChunk; ++i) buf[i] = Hit{kInfDepth, 0u};
    float pay_dpt = 0.0f;
    uint32_t pay_cnt = 0;
    V3 ray_ot = ray_o;
    int last_g = -1, contributor = 0;
    float T_prev = 1.0f, T_next = 1.0f, dpt = 0.0f;
    float C[3] = {0, 0, 0}, c[3] = {0, 0, 0}, O[kMaxAux] = {0}, D = 0.f, W = 0.f;
    V3 N = v3(0, 0, 0);
    float clamped[3] = {0, 0, 0};
    const float cutoff = 3.0f;
    const float T_final = 1.0f - in.acc;
    for (;;) {
        k_nearest(sc, ray_ot, ray_d, buf, pay_cnt);
        int contributed_here = 0;
        for (int i = 0; i < kChunk; ++i) {
            if ((uint32_t)i >= pay_cnt) break;
            int pidx = (int)buf[i].idx;
            int g = pidx / 2;
            if (g == last_g) {
                if (!p->literal_stale) buf[i] = Hit{kInfDepth, 0u};
                continue;
            }
            dpt = buf[i].t + pay_dpt;
            V3 xyz = v3(ray_o.x + dpt * ray_d.x, ray_o.y + dpt * ray_d.y, ray_o.z + dpt * ray_d.z);
            buf[i] = Hit{kInfDepth, 0u};
            Splat s;
            const float *mean = p->means3D + 3 * (size_t)g, *scale = p->scales + 2 * (size_t)g,
                        *rot = p->rotations + 4 * (size_t)g;
            splat_uv(mean, scale, rot, xyz, s);
            float rho = s.u * s.u + s.v * s.v;
            V3 normal = s.R[2];
            float cosv = -(ray_d.x * normal.x + ray_d.y * normal.y + ray_d.z * normal.z);
            if (cosv == 0) continue;
            float normal_sign = cosv > 0 ? 1.0f : -1.0f;
            normal = normal_sign * normal;
            if (dpt < min_depth) continue;
            float power = -0.5f * rho;
            if (power > 0.0f) continue;
            const float G = exp_det(power);
            float alpha = p->opacities[g] * G;
            alpha = (alpha < 0.99f) ? alpha : 0.99f;
            if (alpha < 1.0f / 255.0f) continue;
            T_next = T_prev * (1 - alpha);
            if (T_next < T_threshold) break;
            contributor++;
            if (contributor > kMaxContrib) break;
            last_g = g;
            contributed_here++;
            float w = alpha * T_prev;
            if (p->colors_precomp == nullptr) {
                V3 col = sh_color(p->D, p->shs + (size_t)g * p->M * 3, ray_d, clamped);
                c[0] = col.x; c[1] = col.y; c[2] = col.z;
            } else {
                for (int ch = 0; ch < 3; ++ch) c[ch] = p->colors_precomp[ch + 3 * (size_t)g];
            }
            for (int ch = 0; ch < 3; ++ch) C[ch] += w * c[ch];
            if (p->others_precomp != nullptr)
                for (int ch = 0; ch < p->aux; ++ch) O[ch] += w * p->others_precomp[ch + (size_t)p->aux * g];
            D += w * dpt;
            N = v3(N.x + w * normal.x, N.y + w * normal.y, N.z + w * normal.z);

            // gradient of this hit (backward.cu:528-640); T = float is the restatement, T = double the same
            // formulas on the same fp32 inputs and decisions
            T g_alpha = 0.0f;
            const T num = (T)1.0f - (T)alpha;
            const T Tp = T_prev, wT = w;
            T g_color[3];
            for (int ch = 0; ch < 3; ++ch) {
                g_color[ch] = in.g_rgb[ch] * wT;
                aadd(acc.colors, ch + 3 * (size_t)g, (double)(in.g_rgb[ch] * wT));
                g_alpha += in.g_rgb[ch] * (Tp * (T)c[ch] - ((T)in.rgb[ch] - (T)C[ch]) / num);
                g_alpha += in.g_rgb[ch] * (T)p->background[ch] * (-(T)T_final / num);
            }
            if (p->others_precomp != nullptr) {
                for (int ch = 0; ch < p->aux; ++ch) {
                    T o = p->others_precomp[ch + (size_t)p->aux * g];
                    aadd(acc.others, ch + (size_t)p->aux * g, (double)(in.g_aux[ch] * wT));
                    g_alpha += in.g_aux[ch] * (Tp * o - ((T)in.aux[ch] - (T)O[ch]) / num);
                }
            }
            T g_D = in.g_dpt * wT;
            g_alpha += in.g_dpt * (Tp * (T)dpt - ((T)in.dpt - (T)D) / num);
            V3T<T> g_N = in.g_norm * wT;
            {
                V3T<T> tn = Tp * cast3<T>(normal) - (cast3<T>(in.norm) - cast3<T>(N)) / num;
                g_alpha += in.g_norm.x * tn.x + in.g_norm.y * tn.y + in.g_norm.z * tn.z;
            }
            g_alpha += in.g_acc * (Tp * 1.f - ((T)in.acc - (T)W) / num);
            const float opac = p->opacities[g];
            const T g_G = g_alpha * (T)opac;
            float pclamp = (opac * G) > 0.99f ? 0.0f : 1.0f;
            aadd(acc.opac, (size_t)g, (double)(g_alpha * (T)G * pclamp));
            const float *V = p->vertices + (size_t)g * 12;
            V3 v1, v2, v3_, h1, h2, h3;
            if (pidx % 2 == 0) {
                v1 = ld3(V + 0); v2 = ld3(V + 3); v3_ = ld3(V + 6);
                h1 = v3(-1.f, 1.f, 1.f) * cutoff; h2 = v3(-1.f, -1.f, 1.f) * cutoff; h3 = v3(1.f, 1.f, 1.f) * cutoff;
            } else {
                v1 = ld3(V + 3); v2 = ld3(V + 6); v3_ = ld3(V + 9);
                h1 = v3(-1.f, -1.f, 1.f) * cutoff; h2 = v3(1.f, 1.f, 1.f) * cutoff; h3 = v3(1.f, -1.f, 1.f) * cutoff;
            }
            GeoGrad<T> gg;
            splat_uv_backward<T>(mean, scale, rot, xyz, s, normal_sign, ray_o, ray_d, dpt, v1, v2, v3_, h1, h2, h3, G,
                                 pclamp, g_N, g_D, g_G, g_ray_o, g_ray_d, gg);
            if (acc.noise) {
                GeoGrad<T> gb;
                V3T<T> bo = v3t<T>(0, 0, 0), bd = v3t<T>(0, 0, 0);
                splat_uv_backward<T>(mean, scale, rot, xyz, s, normal_sign, ray_o, ray_d, dpt, v1, v2, v3_, h1, h2, h3, G,
                                     pclamp, g_N, g_D, g_G, bo, bd, gb, 0);
                for (int pert = 1; pert <= 3; ++pert) {
                    GeoGrad<T> gq;
                    V3T<T> qo = v3t<T>(0, 0, 0), qd = v3t<T>(0, 0, 0);
                    splat_uv_backward<T>(mean, scale, rot, xyz, s, normal_sign, ray_o, ray_d, dpt, v1, v2, v3_, h1, h2, h3,
                                         G, pclamp, g_N, g_D, g_G, qo, qd, gq, pert);
                    for (int k = 0; k < 2; ++k) aadd(acc.n_scales, 2 * (size_t)g + k, std::abs((double)(gq.scale[k] - gb.scale[k])));
                    for (int k = 0; k < 4; ++k) aadd(acc.n_rots, 4 * (size_t)g + k, std::abs((double)(gq.rot[k] - gb.rot[k])));
                    const double dm[3] = {std::abs((double)(gq.mean.x - gb.mean.x)), std::abs((double)(gq.mean.y - gb.mean.y)),
                                          std::abs((double)(gq.mean.z - gb.mean.z))};
                    for (int k = 0; k < 3; ++k) {
                        aadd(acc.n_means, 3 * (size_t)g + k, dm[k]);
                        aadd(acc.n_grads, 3 * (size_t)g + k, dm[k] * 0.5 * (double)dpt);
                    }
                    if (n_ray_o && n_ray_d) {
                        *n_ray_o = *n_ray_o + v3t<T>(std::abs(qo.x - bo.x), std::abs(qo.y - bo.y), std::abs(qo.z - bo.z));
                        *n_ray_d = *n_ray_d + v3t<T>(std::abs(qd.x - bd.x), std::abs(qd.y - bd.y), std::abs(qd.z - bd.z));
                    }
                }
            }
            aadd(acc.scales, 2 * (size_t)g + 0, gg.scale[0]);
            aadd(acc.scales, 2 * (size_t)g + 1, gg.scale[1]);
            for (int k = 0; k < 4; ++k) aadd(acc.rots, 4 * (size_t)g + k, gg.rot[k]);
            aadd(acc.means, 3 * (size_t)g + 0, gg.mean.x);
            aadd(acc.means, 3 * (size_t)g + 1, gg.mean.y);
            aadd(acc.means, 3 * (size_t)g + 2, gg.mean.z);
            aadd(acc.grads, 3 * (size_t)g + 0, gg.mean.x * 0.5f * (T)dpt);
            aadd(acc.grads, 3 * (size_t)g + 1, gg.mean.y * 0.5f * (T)dpt);
            aadd(acc.grads, 3 * (size_t)g + 2, gg.mean.z * 0.5f * (T)dpt);
            if (p->colors_precomp == nullptr) {
                V3T<T> g_sh[16];
                sh_color_backward<T>(p->D, p->shs + (size_t)g * p->M * 3, ray_d, clamped, g_color, g_sh, g_ray_d);
                if (n_ray_d) *n_ray_d = v3t<T>(0, 0, 0);   // the direction gradient was just replaced (backward.cu:165)
                for (int j = 0; j < (p->D + 1) * (p->D + 1); ++j) {
                    aadd(acc.shs, ((size_t)g * p->M + j) * 3 + 0, g_sh[j].x);
                    aadd(acc.shs, ((size_t)g * p->M + j) * 3 + 1, g_sh[j].y);
                    aadd(acc.shs, ((size_t)g * p->M + j) * 3 + 2, g_sh[j].z);
                }
            }
            T_prev = T_next;
        }
        if (T_next < T_threshold || pay_cnt < (uint32_t)kChunk || contributor > kMaxContrib) break;
        float next_dpt = (float)((double)dpt + kStepEps);
        if (!(next_dpt > pay_dpt) && contributed_here == 0) break;
        pay_dpt = next_dpt;
        pay_cnt = 0;
        ray_ot = v3(ray_o.x + pay_dpt * ray_d.x, ray_o.y + pay_dpt * ray_d.y, ray_o.z + pay_dpt * ray_d.z);
    }
}

// auxiliary.h:111-121
template <typename T> inline V3T<T> dnormvdv(V3T<T> v, V3T<T> dv) {
    T sum2 = v.x * v.x + v.y * v.y + v.z * v.z;
    T inv = (T)1.0f / std::sqrt(sum2 * sum2 * sum2);
    return v3t<T>(((+sum2 - v.x * v.x) * dv.x - v.y * v.x * dv.y - v.z * v.x * dv.z) * inv,
                  (-v.x * v.y * dv.x + (sum2 - v.y * v.y) * dv.y - v.z * v.y * dv.z) * inv,
                  (-v.x * v.z * dv.x - v.y * v.z * dv.y + (sum2 - v.z * v.z) * dv.z) * inv);
}
// auxiliary.h:234-252
template <typename T> inline V3T<T> ddotndndn(V3T<T> n, V3T<T> d, V3T<T> g) {
    T nd = dot(n, d);
    return v3t<T>(g.x * (nd + d.x * n.x) + g.y * d.x * n.y + g.z * d.x * n.z,
                  g.x * d.y * n.x + g.y * (nd + d.y * n.y) + g.z * d.y * n.z,
                  g.x * d.z * n.x + g.y * d.z * n.y + g.z * (nd + d.z * n.z));
}
template <typename T> inline V3T<T> ddotndndd(V3T<T> n, V3T<T> /*d*/, V3T<T> g) {
    return v3t<T>(g.x * n.x * n.x + g.y * n.x * n.y + g.z * n.x * n.z, g.x * n.y * n.x + g.y * n.y * n.y + g.z * n.y * n.z,
                  g.x * n.z * n.x + g.y * n.z * n.y + g.z * n.z * n.z);
}

// backward.cu:658-853
template <typename T>
void path_backward(const Scene &sc, const float *out_rgb, const float *mid, const float *g_out_rgb, float g_out_dpt,
                   float g_out_acc, V3 g_out_norm, const float *g_out_aux, V3T<T> &g_ray_o, V3T<T> &g_ray_d, Accum &acc,
                   V3T<T> *n_ray_o = nullptr, V3T<T> *n_ray_d = nullptr) {
    const OracleParams *p = sc.p;
    const int MID = mid_channels(p), AUXO = 11, RGBO = 11 + p->aux, mtd = p->max_trace_depth;
    T C_prev[3], c_prev[3] = {0, 0, 0};
    for (int ch = 0; ch < 3; ++ch) C_prev[ch] = out_rgb[ch];
    T s_prod = 1.0f;
    for (int i = 0; i < mtd; ++i) {
        for (int ch = 0; ch < 3; ++ch) {
            T c_curr = mid[ch + RGBO + i * MID];
            C_prev[ch] = C_prev[ch] + s_prod * (c_prev[ch] - c_curr);
            c_prev[ch] = c_curr;
        }
        s_prod *= (T)mid[AUXO + i * MID];
    }
    for (int i = mtd; i >= 0; --i) {
        const float *m = mid + (size_t)i * MID;
        V3 ot = ld3(m + 0), dt = ld3(m + 3);
        float s_prev = (i > 0) ? mid[AUXO + (i - 1) * MID] : 1.0f;
        if (len(dt) == 0.0f || s_prev <= p->specular_threshold) continue;
        BounceIn<T> in;
        for (int ch = 0; ch < 3; ++ch) in.rgb[ch] = m[RGBO + ch];
        in.dpt = m[6];
        in.acc = m[7];
        in.norm = ld3(m + 8);
        for (int ch = 0; ch < kMaxAux; ++ch) in.aux[ch] = (ch < p->aux) ? m[AUXO + ch] : 0.f;
        in.g_dpt = 0.f;
        in.g_acc = 0.f;
        in.g_norm = v3t<T>(0, 0, 0);
        for (int ch = 0; ch < kMaxAux; ++ch) in.g_aux[ch] = 0.f;
        float f_this = (i == mtd) ? 1.0f : 1 - in.aux[0];
        for (int ch = 0; ch < 3; ++ch) in.g_rgb[ch] = (T)g_out_rgb[ch] * (T)f_this * s_prod;
        s_prod /= (T)s_prev;
        if (i != mtd) {
            for (int ch = 0; ch < 3; ++ch) {
                in.g_aux[0] += (T)g_out_rgb[ch] * (C_prev[ch] / (T)in.aux[0]);
                c_prev[ch] = (i > 0) ? mid[ch + RGBO + (i - 1) * MID] : 0.0f;
                C_prev[ch] = C_prev[ch] - s_prod * (c_prev[ch] - (T)in.rgb[ch]);
            }
            if (len(in.norm) != 0) {
                const V3T<T> normT = cast3<T>(in.norm), dtT = cast3<T>(dt);
                g_ray_d = g_ray_d + g_ray_o * (T)(float)kStepEps;
                V3T<T> n = normT / len(normT);
                in.g_dpt += g_ray_o.x * dtT.x + g_ray_o.y * dtT.y + g_ray_o.z * dtT.z;
                in.g_norm = in.g_norm + dnormvdv<T>(normT, ddotndndn<T>(n, dtT, g_ray_d * -2.0f));
                g_ray_d = g_ray_o * (T)in.dpt + g_ray_d + ddotndndd<T>(n, dtT, g_ray_d * -2.0f);
            }
        }
        if (i == 0) {
            in.g_dpt += g_out_dpt;
            in.g_acc += g_out_acc;
            in.g_norm = in.g_norm + cast3<T>(g_out_norm);
            for (int ch = 0; ch < p->aux; ++ch) in.g_aux[ch] += g_out_aux[ch];
        }
        float min_depth = (i == 0 && p->start_from_first) ? kNear : (i == 0 && !p->start_from_first) ? 0.0f : kStartOffset;
        bounce_backward<T>(sc, ot, dt, min_depth, kTmin, in, g_ray_o, g_ray_d, acc, n_ray_o, n_ray_d);
    }
}

int prepare(const OracleParams *p, Scene &sc) {
    if (!p || p->P <= 0 || p->H < 0 || p->W < 0) return 1;
    if (p->aux < 0 || p->aux > kMaxAux) return 2;
    if (p->mtd_alloc < 0 || p->mtd_alloc + 1 > kMaxSlots) return 3;
    if (p->max_trace_depth < 0 || p->max_trace_depth > p->mtd_alloc) return 4;
    if ((p->shs == nullptr) == (p->colors_precomp == nullptr)) return 5;
    if (p->shs && (p->D < 0 || p->D > 3 || (p->D + 1) * (p->D + 1) > p->M)) return 6;
    if (!faces_are_quads(p)) return 7;
    sc.p = p;
    quad_vertex_ids(p, sc.quad_v);
    if (p->hit_mode == ORACLE_HITS_BVH_LEXI) build_cpu_bvh(sc);
#ifdef _OPENMP
    if (p->n_threads > 0) omp_set_num_threads(p->n_threads);
#endif
    return 0;
}

}  // namespace

extern "C" {

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

float oracle_expf(float x) { return exp_det(x); }

void oracle_sh_color(int deg, const float *sh, const float *dir, float *rgb, float *clamped) {
    V3 c = sh_color(deg, sh, ld3(dir), clamped);
    rgb[0] = c.x; rgb[1] = c.y; rgb[2] = c.z;
}

void oracle_quat_to_rows(const float *rot, float *R) {
    V3 r[3];
    quat_rows(rot, r);
    for (int i = 0; i < 3; ++i) { R[3 * i] = r[i].x; R[3 * i + 1] = r[i].y; R[3 * i + 2] = r[i].z; }
}

int oracle_ray_quad(const float *o, const float *d, const float *A, const float *B, const float *C, const float *Dv,
                    float *t, int *tri) {
    float tt = 0.f;
    int k = 0;
    bool hit = ray_quad(ld3(o), ld3(d), ld3(A), ld3(B), ld3(C), ld3(Dv), tt, k);
    *t = tt;
    *tri = k;
    return hit ? 1 : 0;
}

void oracle_reflection_vjp(int which, const float *a, const float *b, const float *g, float *out) {
    V3 r = v3(0, 0, 0);
    if (which == 0) r = dnormvdv<float>(ld3(a), ld3(g));                 // a = v
    else if (which == 1) r = ddotndndn<float>(ld3(a), ld3(b), ld3(g));   // a = n, b = d
    else if (which == 2) r = ddotndndd<float>(ld3(a), ld3(b), ld3(g));
    out[0] = r.x; out[1] = r.y; out[2] = r.z;
}

int oracle_k_nearest(const OracleParams *p, const float *o, const float *d, float *t16, uint32_t *idx16) {
    Scene sc;
    OracleParams q = *p;
    if (!q.shs && !q.colors_precomp) q.colors_precomp = q.means3D;  // colour is irrelevant here
    int rc = prepare(&q, sc);
    if (rc) return -rc;
    Hit buf[kChunk];
    for (int i = 0; i < kChunk; ++i) buf[i] = Hit{kInfDepth, 0u};
    uint32_t cnt = 0;
    k_nearest(sc, ld3(o), ld3(d), buf, cnt);
    for (int i = 0; i < kChunk; ++i) { t16[i] = buf[i].t; idx16[i] = buf[i].idx; }
    return (int)cnt;
}

int oracle_trace_forward(const OracleParams *p) {
    Scene sc;
    int rc = prepare(p, sc);
    if (rc) return rc;
    const int MID = mid_channels(p), slots = p->mtd_alloc + 1;
    const long R = (long)p->H * p->W;
    Accum acc;
    if (p->training && p->a_weights) acc.w.assign((size_t)p->P, 0.0);
    Accum *accp = (p->training && p->a_weights) ? &acc : nullptr;
    const auto t_start = std::chrono::steady_clock::now();
#pragma omp parallel for schedule(dynamic, 64)
    for (long r = 0; r < R; ++r) {
        V3 o = ld3(p->ray_o + 3 * r), d = ld3(p->ray_d + 3 * r);
        float rgb[3] = {0, 0, 0}, dptv = 0.f, accv = 0.f, aux[kMaxAux] = {0};
        V3 nrm = v3(0, 0, 0), dist = v3(0, 0, 0);
        float mid[kMaxSlots * (14 + kMaxAux)];
        for (float &m : mid) m = 0.f;
        int n_proc = 0, n_con = 0;
        path_forward(sc, o, d, rgb, dptv, accv, nrm, dist, aux, mid, accp, n_proc, n_con);
        for (int ch = 0; ch < 3; ++ch) p->out_rgb[3 * r + ch] = rgb[ch];
        p->out_dpt[r] = dptv;
        p->out_acc[r] = accv;
        p->out_norm[3 * r + 0] = nrm.x; p->out_norm[3 * r + 1] = nrm.y; p->out_norm[3 * r + 2] = nrm.z;
        p->out_dist[3 * r + 0] = dist.x; p->out_dist[3 * r + 1] = dist.y; p->out_dist[3 * r + 2] = dist.z;
        for (int ch = 0; ch < p->aux; ++ch) p->out_aux[(size_t)p->aux * r + ch] = aux[ch];
        for (int i = 0; i < slots * MID; ++i)
            p->mid_val[(size_t)slots * MID * r + i] = (i < (p->max_trace_depth + 1) * MID) ? mid[i] : 0.f;
        if (p->n_proc) p->n_proc[r] = n_proc;
        if (p->n_con) p->n_con[r] = n_con;
    }
    if (p->trace_seconds)
        *p->trace_seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t_start).count();
    if (accp) flush(acc.w, p->a_weights);
    return 0;
}

int oracle_trace_backward(const OracleParams *p) {
    Scene sc;
    int rc = prepare(p, sc);
    if (rc) return rc;
    const int MID = mid_channels(p), slots = p->mtd_alloc + 1;
    const long R = (long)p->H * p->W;
    const size_t P = (size_t)p->P;
    Accum acc;
    acc.means.assign(P * 3, 0.0);
    acc.grads.assign(P * 3, 0.0);
    acc.shs.assign(P * (size_t)p->M * 3, 0.0);
    acc.colors.assign(P * 3, 0.0);
    acc.others.assign(P * (size_t)p->aux, 0.0);
    acc.opac.assign(P, 0.0);
    acc.scales.assign(P * 2, 0.0);
    acc.rots.assign(P * 4, 0.0);
    acc.noise = p->grad_f64 && p->noise_ray_o && p->noise_ray_d && p->noise_means3D && p->noise_grads3D &&
                p->noise_scales && p->noise_rotations;
    if (acc.noise) {
        acc.n_means.assign(P * 3, 0.0);
        acc.n_grads.assign(P * 3, 0.0);
        acc.n_scales.assign(P * 2, 0.0);
        acc.n_rots.assign(P * 4, 0.0);
    }
    const auto t_start = std::chrono::steady_clock::now();
#pragma omp parallel for schedule(dynamic, 64)
    for (long r = 0; r < R; ++r) {
        float g_aux[kMaxAux] = {0};
        for (int ch = 0; ch < p->aux; ++ch) g_aux[ch] = p->dL_daux[(size_t)p->aux * r + ch];
        const float *rgb = p->out_rgb + 3 * r, *mid = p->mid_val + (size_t)slots * MID * r, *g_rgb = p->dL_drgb + 3 * r;
        if (p->grad_f64) {
            V3T<double> g_o = v3t<double>(0, 0, 0), g_d = v3t<double>(0, 0, 0);
            V3T<double> n_o = v3t<double>(0, 0, 0), n_d = v3t<double>(0, 0, 0);
            path_backward<double>(sc, rgb, mid, g_rgb, p->dL_ddpt[r], p->dL_dacc[r], ld3(p->dL_dnorm + 3 * r), g_aux, g_o,
                                  g_d, acc, &n_o, &n_d);
            if (acc.noise) {
                p->noise_ray_o[3 * r + 0] = (float)n_o.x; p->noise_ray_o[3 * r + 1] = (float)n_o.y; p->noise_ray_o[3 * r + 2] = (float)n_o.z;
                p->noise_ray_d[3 * r + 0] = (float)n_d.x; p->noise_ray_d[3 * r + 1] = (float)n_d.y; p->noise_ray_d[3 * r + 2] = (float)n_d.z;
            }
            p->dL_dray_o[3 * r + 0] = (float)g_o.x; p->dL_dray_o[3 * r + 1] = (float)g_o.y; p->dL_dray_o[3 * r + 2] = (float)g_o.z;
            p->dL_dray_d[3 * r + 0] = (float)g_d.x; p->dL_dray_d[3 * r + 1] = (float)g_d.y; p->dL_dray_d[3 * r + 2] = (float)g_d.z;
        } else {
            V3 g_o = v3(0, 0, 0), g_d = v3(0, 0, 0);
            path_backward<float>(sc, rgb, mid, g_rgb, p->dL_ddpt[r], p->dL_dacc[r], ld3(p->dL_dnorm + 3 * r), g_aux, g_o,
                                 g_d, acc);
            p->dL_dray_o[3 * r + 0] = g_o.x; p->dL_dray_o[3 * r + 1] = g_o.y; p->dL_dray_o[3 * r + 2] = g_o.z;
            p->dL_dray_d[3 * r + 0] = g_d.x; p->dL_dray_d[3 * r + 1] = g_d.y; p->dL_dray_d[3 * r + 2] = g_d.z;
        }
    }
    if (p->trace_seconds)
        *p->trace_seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t_start).count();
    flush(acc.means, p->dL_dmeans3D);
    flush(acc.grads, p->dL_dgrads3D);
    flush(acc.shs, p->dL_dshs);
    flush(acc.colors, p->dL_dcolors);
    flush(acc.others, p->dL_dothers);
    flush(acc.opac, p->dL_dopacities);
    flush(acc.scales, p->dL_dscales);
    flush(acc.rots, p->dL_drotations);
    if (acc.noise) {
        flush(acc.n_means, p->noise_means3D);
        flush(acc.n_grads, p->noise_grads3D);
        flush(acc.n_scales, p->noise_scales);
        flush(acc.n_rots, p->noise_rotations);
    }
    return 0;
}

}  // extern "C"
