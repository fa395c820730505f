// Forward trace and backward re-trace kernels.
//
// One wavefront (64 lanes) carries an 8x8 tile of rays as a PACKET: the BVH walk is wave-uniform
// (node and leaf records are fetched once per wave through the scalar path, the traversal stack
// is two VGPRs indexed by lane), every lane tests its own ray against the shared node / quad,
// and each lane keeps its own 16-entry nearest-hit buffer in registers.  Replaces the raygen /
// any-hit programs of the reference (optix_tracer/forward.cu, optix_tracer/backward.cu).
//
// Arithmetic that feeds a decision (hit test, hit order, uv, alpha, transmittance, reflection)
// is plain fp32 evaluated as written: this file is compiled with -ffp-contract=off, rsqrt is
// 1/sqrt with IEEE division and square root, and exp is the fixed polynomial below.  Only the
// gradient algebra, which feeds no decision, allows fused multiply-adds.
#include "dst_internal.h"

#include <algorithm>

namespace {

constexpr int kChunk = 16;
constexpr float kInfDepth = 1e16f;
constexpr double kStepEps = 0.00001;
constexpr int kMaxContrib = 256;
constexpr float kStartOffset = 0.06f;
constexpr float kNear = 0.2f;
constexpr float kFar = 100.0f;   // reference auxiliary.h:20-21
constexpr float kTmin = 0.0001f;
constexpr int kWavesPerBlock = 4;
#ifndef DST_FWD_WPB
#define DST_FWD_WPB 1
#endif
constexpr int kFwdWavesPerBlock = DST_FWD_WPB;   // 1 or kWavesPerBlock
#ifndef DST_STRIP_FWD
#define DST_STRIP_FWD 8   // width of the column strips the blocks of an image grid are walked in (0: row-major)
#endif
#ifndef DST_STRIP_BWD
#define DST_STRIP_BWD 8
#endif
constexpr uint32_t kOrderMinBlocks = 1536;   // replay: blocks are taken longest first on grids of at least two rounds of blocks
                                             // (768 fit the chip at once; below that the order kernel costs more than it saves)
constexpr uint32_t kStripMinBlocks = 4096;   // forward: strips only for grids of at least this many blocks (see launch())

__device__ const float SH0 = 0.28209479177387814f;
__device__ const float SH1 = 0.4886025119029199f;
__device__ const float SH2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                                 -1.0925484305920792f, 0.5462742152960396f};
__device__ const float SH3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
                                 0.3731763325901154f, -0.4570457994644658f, 1.445305721320277f,
                                 -0.5900435899266435f};

struct F3 { float x, y, z; };
// Lanes for which `b` holds (the compare result itself becomes the mask: no 0/1 detour through a register).
__device__ __forceinline__ uint64_t wave_ballot(bool b) { return __builtin_amdgcn_ballot_w64(b); }
__device__ __forceinline__ F3 f3(float x, float y, float z) { return F3{x, y, z}; }
__device__ __forceinline__ F3 operator+(F3 a, F3 b) { return F3{a.x + b.x, a.y + b.y, a.z + b.z}; }
__device__ __forceinline__ F3 operator-(F3 a, F3 b) { return F3{a.x - b.x, a.y - b.y, a.z - b.z}; }
__device__ __forceinline__ F3 operator-(F3 a) { return F3{-a.x, -a.y, -a.z}; }
__device__ __forceinline__ F3 operator*(F3 a, float s) { return F3{a.x * s, a.y * s, a.z * s}; }
__device__ __forceinline__ F3 operator*(float s, F3 a) { return F3{s * a.x, s * a.y, s * a.z}; }
__device__ __forceinline__ F3 operator/(F3 a, float s) { return F3{a.x / s, a.y / s, a.z / s}; }
__device__ __forceinline__ float dot(F3 a, F3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
__device__ __forceinline__ F3 cross(F3 a, F3 b) {
    return F3{a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
}
__device__ __forceinline__ float length(F3 a) { return __builtin_sqrtf(dot(a, a)); }
__device__ __forceinline__ F3 ld3(const float *p) { return F3{p[0], p[1], p[2]}; }

// exp for x <= 0 (any x works): Cody-Waite reduction, degree-6 polynomial, exponent patched in.
__device__ __forceinline__ float exp_det(float x) {
    if (!(x >= -87.0f)) return 0.0f;
    if (x > 88.0f) x = 88.0f;
    float kf = __builtin_rintf(x * 1.44269504088896341f);
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
    return __uint_as_float(__float_as_uint(p) + ((uint32_t)((int32_t)kf << 23)));
}

// quaternion (w,x,y,z) -> rows: tangent u, tangent v, normal (reference auxiliary.h:403-429)
__device__ __forceinline__ void quat_rows(const float q0, const float q1, const float q2, const float q3, F3 (&R)[3]) {
    float s = 1.0f / __builtin_sqrtf(q3 * q3 + q0 * q0 + q1 * q1 + q2 * q2);
    float w = q0 * s, x = q1 * s, y = q2 * s, z = q3 * s;
    R[0] = f3(1.f - 2.f * (y * y + z * z), 2.f * (x * y + w * z), 2.f * (x * z - w * y));
    R[1] = f3(2.f * (x * y - w * z), 1.f - 2.f * (x * x + z * z), 2.f * (y * z + w * x));
    R[2] = f3(2.f * (x * z + w * y), 2.f * (y * z - w * x), 1.f - 2.f * (x * x + y * y));
}

// Where a surfel's SH coefficients come from: the caller's fp32 tensor, or (DST_FLAG_SH_HALF) its binary16 copy,
// widened to fp32 as it is read - the arithmetic after that is the same fp32 sequence either way.
struct ShF32 {
    const float *p;
    __device__ __forceinline__ float operator()(int k) const { return p[k]; }
};
struct ShF16 {
    const uint16_t *p;
    __device__ __forceinline__ float operator()(int k) const { return (float)__builtin_bit_cast(_Float16, p[k]); }
};
// The first `n_halves` binary16 coefficients of a surfel as 16-byte loads (rows of 16 coefficients x 3 channels are 96
// bytes, so every row starts on a 16-byte boundary when the tensor does), kept in registers.
struct ShF16Row {
    uint32_t w[24];
    __device__ __forceinline__ void load(const uint16_t *row, int n_halves) {
        const uint4 *src = reinterpret_cast<const uint4 *>(row);
#pragma unroll
        for (int k = 0; k < 6; ++k) {
            if (8 * k < n_halves) {
                const uint4 v = src[k];
                w[4 * k] = v.x; w[4 * k + 1] = v.y; w[4 * k + 2] = v.z; w[4 * k + 3] = v.w;
            } else {
                w[4 * k] = w[4 * k + 1] = w[4 * k + 2] = w[4 * k + 3] = 0u;
            }
        }
    }
    __device__ __forceinline__ float operator()(int k) const {
        const uint32_t word = w[k >> 1];
        return (float)__builtin_bit_cast(_Float16, (uint16_t)((k & 1) ? (word >> 16) : (word & 0xFFFFu)));
    }
};

// SH colour of one surfel in direction d (reference forward.cu:18-58); clamp flags for backward.
template <class SH>
__device__ __forceinline__ F3 sh_color(int deg, const SH &sh, F3 d, bool (&neg)[3]) {
#define SHC(j) f3(sh(3 * (j)), sh(3 * (j) + 1), sh(3 * (j) + 2))
    F3 r = SH0 * SHC(0);
    if (deg > 0) {
        float x = d.x, y = d.y, z = d.z;
        r = r - SH1 * y * SHC(1) + SH1 * z * SHC(2) - SH1 * x * SHC(3);
        if (deg > 1) {
            float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
            r = r + SH2[0] * xy * SHC(4) + SH2[1] * yz * SHC(5) + SH2[2] * (2.0f * zz - xx - yy) * SHC(6) +
                SH2[3] * xz * SHC(7) + SH2[4] * (xx - yy) * SHC(8);
            if (deg > 2) {
                r = r + SH3[0] * y * (3.0f * xx - yy) * SHC(9) + SH3[1] * xy * z * SHC(10) +
                    SH3[2] * y * (4.0f * zz - xx - yy) * SHC(11) +
                    SH3[3] * z * (2.0f * zz - 3.0f * xx - 3.0f * yy) * SHC(12) +
                    SH3[4] * x * (4.0f * zz - xx - yy) * SHC(13) + SH3[5] * z * (xx - yy) * SHC(14) +
                    SH3[6] * x * (xx - 3.0f * yy) * SHC(15);
            }
        }
    }
#undef SHC
    r = f3(r.x + 0.5f, r.y + 0.5f, r.z + 0.5f);
    neg[0] = r.x < 0.f;
    neg[1] = r.y < 0.f;
    neg[2] = r.z < 0.f;
    return f3(r.x > 0.f ? r.x : 0.f, r.y > 0.f ? r.y : 0.f, r.z > 0.f ? r.z : 0.f);
}
// The colour from the binary16 copy of the coefficients (DST_FLAG_SH_HALF).
__device__ __forceinline__ F3 sh_color_half(const DstParams &p, int g, F3 d, bool (&neg)[3]) {
    const uint16_t *row = p.shs_half + (size_t)g * p.M * 3;
    if ((p.M & 7) == 0 && p.M <= 16 && (reinterpret_cast<uintptr_t>(p.shs_half) & 15u) == 0u) {
        ShF16Row r;
        r.load(row, 3 * (p.D + 1) * (p.D + 1));
        return sh_color(p.D, r, d, neg);
    }
    return sh_color(p.D, ShF16{row}, d, neg);
}

// ---- ray / quad -----------------------------------------------------------------------------------------
// Products feeding a difference or a running sum are fused here BY DEFINITION (explicit fma, one rounding);
// the CPU statement of the same test uses the same calls, so both sides produce the same bits.
__device__ __forceinline__ F3 cross_f(F3 x, F3 y) {
    return F3{__builtin_fmaf(x.y, y.z, -(x.z * y.y)), __builtin_fmaf(x.z, y.x, -(x.x * y.z)),
              __builtin_fmaf(x.x, y.y, -(x.y * y.x))};
}
__device__ __forceinline__ float dot_f(F3 a, F3 b) {
    return __builtin_fmaf(a.z, b.z, __builtin_fmaf(a.y, b.y, a.x * b.x));
}
__device__ __forceinline__ bool same_sign(float a, float b, float c) {
    return (a >= 0.f && b >= 0.f && c >= 0.f) || (a <= 0.f && b <= 0.f && c <= 0.f);
}
// Quad = triangles ABC and BCD, given as the leaf record holds it: corner A, edge vectors AB, AC, AD, normals
// n0 = AB x AC, n1 = (C-B) x (D-B), n2 = AC x AD, c1 = n1.AB.  The signed volumes d.((P-o) x (Q-o)) of the edge tests
// are formed from one cross product with the ray, m = d x (A-o), and the edge vectors:
//     d.((A+P'-o) x (A+Q'-o)) = (Q'-P').m + d.(P' x Q'),
// so that nothing is multiplied that is as long as the way from the origin to the quad except in m itself (with the
// corners relative to the origin in every product, a ray passing half a millimetre-sized quad outside it counted as
// a hit from a few metres away).  Then t = n.(v1-o) / n.d on the plane of the triangle that was hit.
__device__ __forceinline__ bool ray_quad(F3 o, F3 d, F3 A, F3 AB, F3 AC, F3 AD, F3 n0, F3 n1, F3 n2, float c1, float &t,
                                         uint32_t &tri) {
    const F3 a = A - o;
    const F3 m = cross_f(d, a);
    const float X = dot_f(AB, m), Y = dot_f(AC, m), Z = dot_f(AD, m);
    const float q0 = dot_f(n0, d), q1 = dot_f(n1, d), q2 = dot_f(n2, d);
    const float u2 = X, u1 = -Y, u0 = (Y - X) + q0;          // edges AB, CA, BC
    const bool in0 = same_sign(u0, u1, u2);
    const float w0 = (Z - Y) + q2;                            // edge CD
    const float w1 = (X - Z) + ((q1 - q0) - q2);              // edge DB (AD x AB = n1 - n0 - n2)
    const bool in1 = same_sign(w0, w1, u0);
    if (!(in0 || in1)) return false;
    tri = in0 ? 0u : 1u;
    const float pa = dot_f(in0 ? n0 : n1, a);
    const float p = in0 ? pa : pa + c1;                       // n1.(B-o) = n1.(A-o) + n1.AB
    const float q = in0 ? q0 : q1;
    t = p / q;
    return (t > 0.0f) && (t < kInfDepth);
}

// v_writelane_b32: value (uniform) into lane `lane` (uniform) of `old`; the compiler offers no builtin for it.
__device__ int dst_writelane(int value, int lane, int old) __asm("llvm.amdgcn.writelane.i32");

// ---- wave-uniform fetches ---------------------------------------------------------------------------------
typedef const __attribute__((address_space(4))) uint32_t *const_u32_ptr;
typedef __attribute__((address_space(3))) uint32_t *lds_u32;
template <int N>
__device__ __forceinline__ void load_uniform(const void *p, uint32_t (&out)[N]) {
    const_u32_ptr c = (const_u32_ptr)(uintptr_t)p;
#pragma unroll
    for (int k = 0; k < N; ++k) out[k] = c[k];
}

// A whole traversal node in one trip: the six face arrays picked by byte offset (scalar-register offsets, so no
// address arithmetic per array), the child references and the child count, and one wait for all of them.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void load_node(const void *node, uint32_t onx, uint32_t ony, uint32_t onz, uint32_t ofx,
                                          uint32_t ofy, uint32_t ofz, u32x4 &NX, u32x4 &NY, u32x4 &NZ, u32x4 &FX,
                                          u32x4 &FY, u32x4 &FZ, u32x4 &refs, uint32_t &count) {
    asm volatile(
        "s_load_dwordx4 %0, %8, %9\n\t"
        "s_load_dwordx4 %1, %8, %10\n\t"
        "s_load_dwordx4 %2, %8, %11\n\t"
        "s_load_dwordx4 %3, %8, %12\n\t"
        "s_load_dwordx4 %4, %8, %13\n\t"
        "s_load_dwordx4 %5, %8, %14\n\t"
        "s_load_dwordx4 %6, %8, 0x60\n\t"
        "s_load_dword %7, %8, 0x70\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&s"(NX), "=&s"(NY), "=&s"(NZ), "=&s"(FX), "=&s"(FY), "=&s"(FZ), "=&s"(refs), "=&s"(count)
        : "s"(node), "s"(onx), "s"(ony), "s"(onz), "s"(ofx), "s"(ofy), "s"(ofz)
        : "memory");
}
// Two consecutive 64-byte records (the stand-ins of a leaf group's two quads), or one 96-byte quad record, in one
// trip: left to itself the compiler splits these fetches and waits for the first part before asking for the rest.
typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
__device__ __forceinline__ void load_record_pair(const void *p, u32x16 &a, u32x16 &b) {
    asm volatile("s_load_dwordx16 %0, %2, 0x0\n\ts_load_dwordx16 %1, %2, 0x40\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(a), "=&s"(b)
                 : "s"(p)
                 : "memory");
}
typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ void load_quad_record(const void *p, u32x16 &a, u32x8 &b) {
    asm volatile("s_load_dwordx16 %0, %2, 0x0\n\ts_load_dwordx8 %1, %2, 0x40\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(a), "=&s"(b)
                 : "s"(p)
                 : "memory");
}
// bits = 2 * bits + (mask != 0): one compare and one add-with-carry per lane mask.
__device__ __forceinline__ uint32_t shift_in_any(uint32_t bits, uint64_t mask) {
    asm("s_cmp_lg_u64 %1, 0\n\ts_addc_u32 %0, %0, %0" : "+s"(bits) : "s"(mask) : "scc");
    return bits;
}
// The same for two masks at once: hit takes (a & b) != 0, ahead takes b != 0 (the and sets the carry itself).
__device__ __forceinline__ void shift_in_near_far(uint32_t &hit, uint32_t &ahead, uint64_t a, uint64_t b) {
    uint64_t both;
    asm("s_and_b64 %2, %3, %4\n\ts_addc_u32 %0, %0, %0\n\ts_cmp_lg_u64 %4, 0\n\ts_addc_u32 %1, %1, %1"
        : "+s"(hit), "+s"(ahead), "=&s"(both)
        : "s"(a), "s"(b)
        : "scc");
}

struct RaySlab {   // per-lane precomputation for the conservative slab test
    float ix, iy, iz;     // 1/d, with tiny components pushed away from zero
    float nx, ny, nz;     // -o * (1/d)
    float wx, wy, wz;     // interval widening per axis
    float max_abs;        // largest vertex coordinate of the scene (uniform)
};

__device__ __forceinline__ float safe_inv(float d) {
    float a = __builtin_fabsf(d);
    float v = (a < 1e-20f) ? __builtin_copysignf(1e-20f, d) : d;   // NaN passes through
    return 1.0f / v;
}

__device__ __forceinline__ RaySlab make_slab(F3 o, F3 d, float max_abs) {
    RaySlab s;
    s.ix = safe_inv(d.x);
    s.iy = safe_inv(d.y);
    s.iz = safe_inv(d.z);
    s.nx = -o.x * s.ix;
    s.ny = -o.y * s.iy;
    s.nz = -o.z * s.iz;
    // The quad test works in origin-relative fp32 coordinates, so it can accept a ray that passes
    // a few ulps of (|o| + |vertex|) outside the quad; boxes are widened by well above that: by 4e-6 |o| here,
    // and by 4e-6 of the quad's own largest coordinate where the boxes are made (lbvh.hip, kBoxPad).
    float oa = __builtin_fmaxf(__builtin_fabsf(o.x), __builtin_fmaxf(__builtin_fabsf(o.y), __builtin_fabsf(o.z)));
    s.max_abs = max_abs;
    float pad = 4e-6f * oa;
    s.wx = pad * __builtin_fabsf(s.ix);
    s.wy = pad * __builtin_fabsf(s.iy);
    s.wz = pad * __builtin_fabsf(s.iz);
    return s;
}

// Conservative slab test for a packet whose lanes all have the same direction signs: the near and far plane of
// each axis are then the same box faces for all lanes, picked once per wave, and the widening folds into the
// offsets.  The box is hit iff the entry distance tn <= min(exit distance, tmax); tmax < 0 disables a lane.
struct RaySlabFast {
    float ix, iy, iz;
    float cnx, cny, cnz;   // -o/d - widening: added to (near face)/d
    float cfx, cfy, cfz;   // -o/d + widening: added to (far face)/d
};
// Returns the lanes that hit as a mask (the compare writes the wave mask directly).
__device__ __forceinline__ uint64_t slab_hit_fast(const RaySlabFast &s, float nx, float ny, float nz, float fx,
                                                  float fy, float fz, float tmax, float &tn) {
    const float a = __builtin_fmaf(nx, s.ix, s.cnx), b = __builtin_fmaf(ny, s.iy, s.cny),
                c = __builtin_fmaf(nz, s.iz, s.cnz);
    const float e = __builtin_fmaf(fx, s.ix, s.cfx), f = __builtin_fmaf(fy, s.iy, s.cfy),
                g = __builtin_fmaf(fz, s.iz, s.cfz);
    tn = __builtin_fmaxf(__builtin_fmaxf(a, b), __builtin_fmaxf(c, 0.0f));
    const float tf = __builtin_fminf(__builtin_fminf(e, f), __builtin_fminf(g, tmax));
    return __builtin_amdgcn_fcmpf(tn, tf, 5);   // 5 = ordered <=
}

// The same test as two masks: `far` = lanes whose ray meets the box at all (at a distance >= 0), result = those of
// them that meet it within tmax.  Lanes that are switched off carry slab constants that fail both (see packet_walk).
__device__ __forceinline__ uint64_t slab_hit_near_far(const RaySlabFast &s, float nx, float ny, float nz, float fx,
                                                      float fy, float fz, float tmax, uint64_t &far) {
    const float a = __builtin_fmaf(nx, s.ix, s.cnx), b = __builtin_fmaf(ny, s.iy, s.cny),
                c = __builtin_fmaf(nz, s.iz, s.cnz);
    const float e = __builtin_fmaf(fx, s.ix, s.cfx), f = __builtin_fmaf(fy, s.iy, s.cfy),
                g = __builtin_fmaf(fz, s.iz, s.cfz);
    const float tn = __builtin_fmaxf(__builtin_fmaxf(a, b), __builtin_fmaxf(c, 0.0f));
    const float tf = __builtin_fminf(__builtin_fminf(e, f), g);
    far = __builtin_amdgcn_fcmpf(tn, tf, 5);   // 5 = ordered <=
    return far & __builtin_amdgcn_fcmpf(tn, tmax, 5);
}

// The 16 nearest hits of a lane, ascending.  One entry = (bits of t) << 32 | idx: t is positive, so the
// unsigned 64-bit order is the (t, idx) lexicographic order and the content does not depend on the order in
// which the BVH delivers candidates (ties in t resolve to ascending primitive index).
struct KBuf {
    uint64_t e[kChunk];
};
__device__ __forceinline__ uint64_t kb_pack(float t, uint32_t idx) { return ((uint64_t)__float_as_uint(t) << 32) | idx; }
__device__ __forceinline__ float kb_t(uint64_t e) { return __uint_as_float((uint32_t)(e >> 32)); }
__device__ __forceinline__ uint32_t kb_idx(uint64_t e) { return (uint32_t)e; }

__device__ __forceinline__ void kbuf_reset(KBuf &b) {
#pragma unroll
    for (int k = 0; k < kChunk; ++k) b.e[k] = kb_pack(kInfDepth, 0u);
}

// Sorted insert in place: slot k keeps its entry if that is smaller than the new one, else takes the new one
// (if the slot above kept its entry) or the entry from the slot above.
__device__ __forceinline__ void kbuf_insert(KBuf &b, uint64_t x_in, bool on) {
    // a lane that inserts nothing offers the largest key: every slot keeps its entry (no per-slot gating)
    const uint64_t x = on ? x_in : ~0ull;
    bool keep_k = b.e[kChunk - 1] < x;
#pragma unroll
    for (int k = kChunk - 1; k >= 1; --k) {
        const bool keep_up = b.e[k - 1] < x;
        const uint64_t in = keep_up ? x : b.e[k - 1];
        b.e[k] = keep_k ? b.e[k] : in;
        keep_k = keep_up;
    }
    b.e[0] = keep_k ? b.e[0] : x;
}

#ifdef DST_STATS
struct WaveStats { unsigned long long nodes, leaves, t_trav, t_comp, chunks, leaf_any, t_plan, t_hb, steps; };
#define STAT(x) x
#define WSP , ws
#else
#define STAT(x)
#define WSP
#endif

// Per-lane constants of the conservative stand-in for the quad test (DstLeafPre).  With S = |o|_max + the largest
// coordinate of the quad: the stand-in's distance along the ray is off by at most about 3.4e-5 S/|d| + 1e-5 |t| when
// |n.d| >= 0.05 |d| (flatter rays skip the stand-in), its hit point by 7e-5 S; the margins below are twice that.
struct RayPre {
    float padw;     // in-plane slack, world units
    float tp;       // slack on the distance along the ray
    float graze;    // |n.d| below this: too flat for the stand-in
    float inv_dl;   // 1 / |d|
};
__device__ __forceinline__ RayPre make_pre(F3 o, F3 d, float max_abs) {
    RayPre r;
    const float oa = __builtin_fmaxf(__builtin_fabsf(o.x), __builtin_fmaxf(__builtin_fabsf(o.y), __builtin_fabsf(o.z)));
    const float S = oa;   // the ray's share; the quad's own coordinates are in its limits already (lbvh.hip, write_leaf)
    const float dl = __builtin_sqrtf(d.x * d.x + d.y * d.y + d.z * d.z);
    r.inv_dl = 1.0f / dl;
    r.padw = 1.5e-4f * S;
    r.tp = 1e-4f * S * r.inv_dl;
    r.graze = 0.05f * dl;
    return r;
}

// The stand-in test of one quad for all lanes (about 28 instructions), as a lane mask: bit clear = that lane's ray
// cannot pass the exact test (lanes that are switched off come back set or clear; the caller masks them).
// FAR: also `far`, the same without the limit tmax (lanes whose ray may hit the quad at any distance ahead); for a
// grazing ray, whose distance to the plane says nothing, the quad counts as ahead unless the sphere around it lies
// behind the origin.
template <bool FAR>
__device__ __forceinline__ uint64_t quad_may_hit(const u32x16 &Q, const RayPre &rp, F3 o, F3 d, float tmax,
                                                 uint64_t live, uint64_t &far) {
#define QF(k) __uint_as_float(Q[k])
    const float hx = QF(0) - o.x, hy = QF(1) - o.y, hz = QF(2) - o.z;
    const float qd = __builtin_fmaf(QF(5), d.z, __builtin_fmaf(QF(4), d.y, QF(3) * d.x));
    const float ph = __builtin_fmaf(QF(5), hz, __builtin_fmaf(QF(4), hy, QF(3) * hx));
    const float t = ph * __builtin_amdgcn_rcpf(qd);
    const float wx = __builtin_fmaf(t, d.x, -hx), wy = __builtin_fmaf(t, d.y, -hy), wz = __builtin_fmaf(t, d.z, -hz);
    const float s = __builtin_fmaf(QF(8), wz, __builtin_fmaf(QF(7), wy, QF(6) * wx));
    const float r = __builtin_fmaf(QF(11), wz, __builtin_fmaf(QF(10), wy, QF(9) * wx));
    const float m = __builtin_fmaxf(__builtin_fabsf(s), __builtin_fabsf(r));
    const float lim = __builtin_fmaf(rp.padw, QF(12), QF(13));
    const float tpq = __builtin_fmaf(QF(14), rp.inv_dl, rp.tp);
    // every comparison is written so that a NaN keeps the ray in; the lane masks are combined without branches
    uint64_t flat = wave_ballot(__builtin_fabsf(qd) < rp.graze);
    const uint64_t out_base = wave_ballot(m > lim) | wave_ballot(t < -tpq);
    const uint64_t out_t = wave_ballot(__builtin_fmaf(t, 0.9999f, -tpq) > tmax);
    if (FAR) {
        if ((flat & live) != 0ull) {
            // (centre - o).d < -(radius + slack) |d|: every point of the quad is behind the origin
            const float hd = __builtin_fmaf(hz, d.z, __builtin_fmaf(hy, d.y, hx * d.x));
            flat &= ~wave_ballot(hd < -(QF(15) + rp.padw) * (20.0f * rp.graze));
        }
        far = flat | ~out_base;
    }
#undef QF
    return flat | ~(out_base | out_t);
}

// The exact test of one quad record for all lanes; hits are admitted into the lanes' buffers.
__device__ __forceinline__ void quad_exact(const u32x16 &La, const u32x8 &Lb, F3 o, F3 d, bool active, KBuf &buf, uint32_t &cnt
#ifdef DST_STATS
                                           , WaveStats &ws
#endif
) {
    STAT(ws.t_plan++;)
#define LW(k) ((k) < 16 ? La[(k) & 15] : Lb[((k) - 16) & 7])
#define LF3(k) f3(__uint_as_float(LW(k)), __uint_as_float(LW((k) + 1)), __uint_as_float(LW((k) + 2)))
    float t = 0.f;
    uint32_t tri = 0u;
    const bool hit = active && ray_quad(o, d, LF3(0), LF3(3), LF3(6), LF3(9), LF3(16), LF3(12), LF3(19),
                                        __uint_as_float(LW(22)), t, tri);
#undef LF3
    const uint64_t x = kb_pack(t, 2u * LW(15) + tri);
#undef LW
    const bool adm = hit && (x < buf.e[kChunk - 1]);
    if (wave_ballot(adm) != 0ull) {
        STAT(ws.leaf_any++;)
        cnt += adm ? 1u : 0u;
        kbuf_insert(buf, x, adm);
    }
}

// A leaf group (up to DST_GROUP quads, consecutive records) against all lanes' rays.  The stand-in records of
// two quads are fetched together, then the exact records of those that some lane's ray may hit, again together:
// one trip to memory per stage instead of one per quad.  FAR: returns whether some live lane's ray may hit a quad
// of the group at any distance ahead (the group has to be looked at again when the ray's next chunk is traced).
template <bool FAR>
__device__ __forceinline__ bool test_group(const DstAccelView &acc, uint32_t first, uint32_t count, const RayPre &rp,
                                           F3 o, F3 d, bool active, KBuf &buf, uint32_t &cnt
#ifdef DST_STATS
                                           , WaveStats &ws
#endif
) {
    uint32_t q0 = 0;   // count >= 1
    bool again = false;
#pragma unroll 1
    do {
        const bool two = q0 + 1u < count;
        // the record after the last quad of the structure exists (the array has one spare record)
        u32x16 Q0, Q1;
        load_record_pair(&acc.pre[first + q0], Q0, Q1);
        STAT(ws.leaves += two ? 2 : 1;)
        const float tmax = kb_t(buf.e[kChunk - 1]);
        const uint64_t live = wave_ballot(active);
        uint64_t f0 = 0ull, f1 = 0ull;
        const uint64_t k0 = quad_may_hit<FAR>(Q0, rp, o, d, tmax, live, f0) & live;
        const uint64_t k1 = two ? (quad_may_hit<FAR>(Q1, rp, o, d, tmax, live, f1) & live) : 0ull;
        if (FAR) again = again || (((f0 | (two ? f1 : 0ull)) & live) != 0ull);
        uint32_t todo = (k0 != 0ull ? 1u : 0u) | (k1 != 0ull ? 2u : 0u);
#pragma unroll 1
        while (todo != 0u) {
            const uint32_t k = (todo & 1u) ? 0u : 1u;
            todo &= ~(1u << k);
            u32x16 La;
            u32x8 Lb;
            load_quad_record(&acc.leaves[first + q0 + k], La, Lb);
            quad_exact(La, Lb, o, d, active, buf, cnt WSP);
        }
        q0 += 2;
    } while (DST_GROUP > 2 && q0 < count);   // groups of at most two quads: one pass, no loop
    return again;
}

// Work list of a walk that can be resumed.  The rays of a wave are traced in chunks of 16 hits, each chunk from an
// origin moved up to the last hit of the one before.  Instead of walking down from the root again, a walk writes
// down what the next chunk can still need - the nodes it left with children that lie ahead of some ray but beyond
// its 16th hit so far (with the children concerned), and the leaf groups it tested that hold a quad ahead of some
// ray - and the next walk starts from that list.  What is ahead of a ray from the moved origin was ahead of it
// before, and both tests have margins far above the rounding of the moved origin, so the list is a superset of
// what a walk from the root would reach; the buffer's content does not depend on the order or on extra candidates.
// An item is a leaf-group reference, or a node index with the children NOT to look at in bits 27..30.
constexpr uint32_t kListCap = 512;            // items per list (a multiple of the wave size); a longer list is dropped
constexpr uint32_t kListFresh = 0xFFFFFFFFu;  // n_in: no list, walk from the root
constexpr uint32_t kListIndexBits = 27;       // node indices must fit below the excluded-children bits
struct WalkList {
    lds_u32 in, out;   // kListCap words each (LDS of this wave)
    uint32_t n_in;     // items in `in`, or kListFresh
    bool record;       // write `out` (false: plain walks from the root)
    uint32_t limit;    // steps this walk may take at most (0: as many as the hierarchy can need)
    bool spent;        // set by a walk that ran into its limit: its buffer is not to be used
};

// One traversal for the whole wave: every active lane ends with its own 16 nearest hits (t relative
// to its origin, 0 < t < 1e16) and the number of admissions.  Wave-uniform control flow: nodes and quads
// are fetched once per wave, the stack is two VGPRs addressed by lane.  128 entries are enough by construction:
// a step defers at most three children, and the builder only hands over hierarchies whose wide nodes are at most 42
// levels deep (grandchildren nodes over a binary hierarchy of at most 62 levels, whose depth the Morton keys bound or
// the build measures; nodes that open one level at a time only over hierarchies measured to be at most 42 deep).  A
// stack that is full all the same loses the entry (no fault; checked on the builder's side, not here).
// All active lanes share the direction signs `sgn` (bit a set = axis a negative), see slab_hit_fast.
template <bool RESUME, bool HAND>
__device__ __forceinline__ void packet_walk(const DstAccelView &acc, const RaySlab &slab, uint32_t sgn, F3 o, F3 d,
                                            bool active, int rep, KBuf &buf, uint32_t &cnt, WalkList &wl
#ifdef DST_STATS
                                            , WaveStats &ws
#endif
) {
    const uint32_t lane = __lane_id();
    const RayPre rp = make_pre(o, d, slab.max_abs);
    RaySlabFast fs;
    // byte offsets of the near / far face arrays inside a wide node (lox 0, loy 16, loz 32, hix 48, hiy 64, hiz 80)
    uint32_t onx = 0, ony = 16, onz = 32, ofx = 48, ofy = 64, ofz = 80;
    fs.ix = slab.ix; fs.iy = slab.iy; fs.iz = slab.iz;
    fs.cnx = slab.nx - slab.wx; fs.cny = slab.ny - slab.wy; fs.cnz = slab.nz - slab.wz;
    fs.cfx = slab.nx + slab.wx; fs.cfy = slab.ny + slab.wy; fs.cfz = slab.nz + slab.wz;
    const bool recording = RESUME && wl.record;
    if (RESUME && !active) {   // a lane that is switched off meets no box: exit distance -inf on every axis
        fs.ix = fs.iy = fs.iz = 0.f;
        fs.cfx = fs.cfy = fs.cfz = -INFINITY;
    }
    if (sgn & 1u) { onx = 48; ofx = 0; }
    if (sgn & 2u) { ony = 64; ofy = 16; }
    if (sgn & 4u) { onz = 80; ofz = 32; }
    uint32_t stack0 = 0u, stack1 = 0u;
    int sp = 0;
    // A well-formed hierarchy is walked in at most one step per node and per leaf group; the cap makes the
    // loops finite whatever the memory holds.  Two loops: the inner one goes down through nodes and never touches
    // the hit buffer, the outer one tests a leaf group and pops (with one loop around both, the compiler kept two
    // copies of the buffer's 32 registers and moved them back and forth at every leaf group).
    constexpr uint32_t kEnd = 0xFFFFFFFFu;   // not a reference: leaf bit set, impossible position
    uint32_t budget = 2u * acc.n_leaves + 8u;
    if constexpr (RESUME && HAND) {
        if (wl.limit != 0u) budget = min(budget, wl.limit);
    }
    // The work lists are read and written a page of 64 items at a time: lane k of a page register holds item k.
    uint32_t in_page = 0u, out_page = 0u, in_pos = 0u, n_out = 0u;
    const uint32_t n_in = (RESUME && wl.n_in != kListFresh) ? wl.n_in : 0u;
    auto next_input = [&]() -> uint32_t {
        if (!RESUME || in_pos >= n_in) return kEnd;
        if ((in_pos & 63u) == 0u) in_page = wl.in[in_pos + lane];
        const uint32_t v = __builtin_amdgcn_readlane(in_page, in_pos & 63u);
        ++in_pos;
        return v;
    };
    auto record = [&](uint32_t v) {
        if (n_out < kListCap) {
            out_page = (uint32_t)dst_writelane((int)v, n_out & 63u, (int)out_page);
            if ((n_out & 63u) == 63u) wl.out[(n_out & ~63u) + lane] = out_page;
        }
        n_out = min(n_out + 1u, kListCap + 1u);
    };
    auto pop = [&]() -> uint32_t {
        if (sp == 0) return next_input();
        --sp;
        const uint32_t a = __builtin_amdgcn_readlane(stack0, sp & 63), b = __builtin_amdgcn_readlane(stack1, sp & 63);
        return sp < 64 ? a : b;
    };
    // node items of a list carry the children to leave out; plain references (stack, root) leave out none
    const bool packed = RESUME && acc.n_leaves <= (1u << kListIndexBits);
    uint32_t ref = (RESUME && wl.n_in != kListFresh) ? next_input() : acc.root;
    for (;;) {
        while ((ref & DST_LEAF_BIT) == 0u) {
            const uint32_t excl = packed ? (ref >> kListIndexBits) : 0u;
            if (packed) ref &= (1u << kListIndexBits) - 1u;
            if (budget == 0u || ref + 1u >= acc.n_leaves) {   // spent, or not a node of this hierarchy
                ref = kEnd;
                break;
            }
            --budget;
            const char *node = reinterpret_cast<const char *>(&acc.wide[ref]);
            STAT(ws.nodes++;)
            const float tmax = active ? kb_t(buf.e[kChunk - 1]) : -1.0f;
            uint32_t tail[5];
            uint32_t hit = 0u;                     // bit k: some lane enters child k
            uint32_t ahead = 0u;                   // bit k: child k lies ahead of some lane's ray, at any distance
            {
                u32x4 NX, NY, NZ, FX, FY, FZ, refs;
                load_node(node, onx, ony, onz, ofx, ofy, ofz, NX, NY, NZ, FX, FY, FZ, refs, tail[4]);
                tail[0] = refs[0]; tail[1] = refs[1]; tail[2] = refs[2]; tail[3] = refs[3];
#pragma unroll
                for (int k = DST_WIDE - 1; k >= 0; --k) {   // last child first: its bit is shifted up the furthest
                    const float a = __builtin_fmaf(__uint_as_float(NX[k]), fs.ix, fs.cnx),
                                b = __builtin_fmaf(__uint_as_float(NY[k]), fs.iy, fs.cny),
                                c = __builtin_fmaf(__uint_as_float(NZ[k]), fs.iz, fs.cnz);
                    const float e = __builtin_fmaf(__uint_as_float(FX[k]), fs.ix, fs.cfx),
                                f = __builtin_fmaf(__uint_as_float(FY[k]), fs.iy, fs.cfy),
                                g = __builtin_fmaf(__uint_as_float(FZ[k]), fs.iz, fs.cfz);
                    const float tn = __builtin_fmaxf(__builtin_fmaxf(a, b), __builtin_fmaxf(c, 0.0f));
                    if (RESUME) {
                        // met at all (at a distance >= 0) / met within tmax; lanes that are switched off fail both
                        const float tf = __builtin_fminf(__builtin_fminf(e, f), g);
                        shift_in_near_far(hit, ahead, __builtin_amdgcn_fcmpf(tn, tmax, 5), __builtin_amdgcn_fcmpf(tn, tf, 5));
                    } else {
                        const float tf = __builtin_fminf(__builtin_fminf(e, f), __builtin_fminf(g, tmax));
                        hit = shift_in_any(hit, __builtin_amdgcn_fcmpf(tn, tf, 5));   // 5 = ordered <=
                    }
                }
                const uint32_t valid = ((1u << tail[4]) - 1u) & ~excl;   // unused slots are never entered
                hit &= valid;
                ahead &= valid;
            }
            if (recording) {
                const uint32_t later = ahead & ~hit;   // beyond every ray's 16th hit so far: the next chunk's business
                if (later != 0u) record(ref | ((~later & 15u) << kListIndexBits));
            }
            if (hit != 0u) {
                // Children are taken in stored order: the first one that is hit next, the others deferred (last
                // first).  Ordering them by entry distance was measured: 3 % fewer visits, but the scalar work of
                // the sort costs more than those visits.
                const uint32_t rest = hit & (hit - 1u);   // the hit children after the first one (never child 0)
                if (__builtin_expect(sp + 3 <= DST_WAVE, 1)) {
                    // Without branches: each candidate is written at the top of the stack and the top moves up only
                    // if the child was hit (an entry above the top is dead, so a write there does no harm).
                    stack0 = (uint32_t)dst_writelane((int)tail[3], sp, (int)stack0);
                    sp += (int)((rest >> 3) & 1u);
                    stack0 = (uint32_t)dst_writelane((int)tail[2], sp, (int)stack0);
                    sp += (int)((rest >> 2) & 1u);
                    stack0 = (uint32_t)dst_writelane((int)tail[1], sp, (int)stack0);
                    sp += (int)((rest >> 1) & 1u);
                } else {
#define DST_PUSH(v)                                                                                          \
    {                                                                                                        \
        if (sp < 64) stack0 = (uint32_t)dst_writelane((int)(v), sp, (int)stack0);               \
        else stack1 = (uint32_t)dst_writelane((int)(v), sp - 64, (int)stack1);                  \
        sp = min(sp + 1, 2 * DST_WAVE - 1);                                                                  \
    }
                    if (rest & 8u) DST_PUSH(tail[3])
                    if (rest & 4u) DST_PUSH(tail[2])
                    if (rest & 2u) DST_PUSH(tail[1])
#undef DST_PUSH
                }
                ref = (hit & 1u) ? tail[0] : ((hit & 2u) ? tail[1] : ((hit & 4u) ? tail[2] : tail[3]));
            } else {
                ref = pop();
            }
        }
        if (ref == kEnd || budget == 0u) break;
        --budget;
        const uint32_t first = ref & DST_REF_FIRST_MASK, count = ((ref >> 28) & 7u) + 1u;
        if (first + count > acc.n_leaves) break;   // not a leaf group of this hierarchy
        const bool again = test_group<RESUME>(acc, first, count, rp, o, d, active, buf, cnt WSP);
        if (recording && again) record(ref);
        ref = pop();
    }
    if (RESUME) {
        if constexpr (HAND) {
            if (wl.limit != 0u && budget == 0u) wl.spent = true;
        }
        if (recording) {
            // a walk that stopped early (budget, damaged structure) or a list that overflowed leaves no list
            const bool whole = n_out <= kListCap && budget != 0u && ref == kEnd;
            if (whole && (n_out & 63u) != 0u) wl.out[(n_out & ~63u) + lane] = out_page;
            wl.n_in = whole ? n_out : kListFresh;
            const lds_u32 t = wl.in;
            wl.in = wl.out;
            wl.out = t;
        } else {
            wl.n_in = kListFresh;
        }
    }
}

// ---- per-lane walk ------------------------------------------------------------------------------------------
// For rays that share neither origin nor direction (reflection rays off rough geometry, arbitrary ray lists) a
// packet visits the union of 64 unrelated paths with one useful lane each.  Here every lane walks the hierarchy
// on its own: own stack (private memory), own node and quad fetches through the vector path, same slab and
// quad tests, same buffer.  The buffer's content does not depend on the order of arrival, so both walks give
// the same result bit for bit; the choice between them only changes the time.
#ifndef DST_PACKET_DIR_SPREAD
#define DST_PACKET_DIR_SPREAD 0.02f   // measured: 0.06 makes packets of lidar rays that are metres apart at their hits
#endif
#ifndef DST_PACKET_ORG_SPREAD
#define DST_PACKET_ORG_SPREAD 0.02f
#endif
constexpr float kPacketDirSpread = DST_PACKET_DIR_SPREAD;   // largest direction difference (relative) inside a packet
constexpr float kPacketOrgSpread = DST_PACKET_ORG_SPREAD;   // largest origin difference, relative to the scene extent
constexpr int kLaneStack = 2 * 64;        // as deep as the packet's two lane-indexed registers
constexpr uint32_t kWalkDone = 0xFFFFFFFFu;   // not a reference: leaf bit set with an impossible position
// A real call on purpose: inlined, its register needs would spill the packet walk that nearly every wave takes.
// The walk is a real function, so the compiler cannot see where its pointers lead: say it (global memory, LDS).
typedef const __attribute__((address_space(1))) float *global_f32;
typedef const __attribute__((address_space(1))) uint32_t *global_u32;
#define LD3(p, k) f3((p)[(k)], (p)[(k) + 1], (p)[(k) + 2])
// `shelf`: optional LDS for the first kLaneShelf stack entries of every lane ([entry][lane], conflict-free);
// deeper entries, or all of them without a shelf, live in private memory.
constexpr int kLaneShelf = 32;
struct LaneWalkAccel { const DstLeaf *leaves; const DstWideNode *wide; uint32_t n_leaves, root; };   // by value: registers
static_assert(DST_GROUP <= 2, "the per-lane walk fetches a leaf group as at most two quad records");
static_assert(sizeof(DstWideNode) == 128 && sizeof(DstLeaf) == 96, "the per-lane walk reads both as 16-byte words");
// A value that is the same in every lane, moved to a scalar register (arguments of a real call arrive in vector ones).
template <class T>
__device__ __forceinline__ T *uniform_ptr(T *p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<T *>(((uint64_t)hi << 32) | lo);
}
__device__ __attribute__((noinline)) void lane_walk(const LaneWalkAccel acc_in, const RaySlab &slab, F3 o, F3 d,
                                                    bool active, KBuf &buf_mem, uint32_t &cnt_mem, uint32_t *shelf_in) {
    const LaneWalkAccel acc = {uniform_ptr(acc_in.leaves), uniform_ptr(acc_in.wide),
                               (uint32_t)__builtin_amdgcn_readfirstlane(acc_in.n_leaves),
                               (uint32_t)__builtin_amdgcn_readfirstlane(acc_in.root)};
    uint32_t *const shelf = uniform_ptr(shelf_in);
    // The caller's buffer is in memory (its address crosses the call): work on a register copy and store it once
    // at the end.  Left in memory, every leaf test re-read its 128 bytes per lane and every admission re-wrote them.
    KBuf buf = buf_mem;
    uint32_t cnt = cnt_mem;
    RaySlabFast fs;
    fs.ix = slab.ix; fs.iy = slab.iy; fs.iz = slab.iz;
    fs.cnx = slab.nx - slab.wx; fs.cny = slab.ny - slab.wy; fs.cnz = slab.nz - slab.wz;
    fs.cfx = slab.nx + slab.wx; fs.cfy = slab.ny + slab.wy; fs.cfz = slab.nz + slab.wz;
    const bool neg_x = slab.ix < 0.f, neg_y = slab.iy < 0.f, neg_z = slab.iz < 0.f;
    uint32_t stack[kLaneStack];
    int sp = 0;
    uint32_t ref = active ? acc.root : kWalkDone;
    uint32_t budget = 2u * acc.n_leaves + 8u;   // a well-formed hierarchy needs fewer steps; bounds the loop regardless
    // A step of a lane is one dependent trip to memory: the lane's node (128 bytes) or its leaf group (two quad
    // records of 96 bytes, consecutive, the first 64 of each) is requested whole - eight to ten 16-byte loads from one base address, whatever
    // the lane is at - before anything is tested, so that lanes at nodes and lanes at leaf groups wait together,
    // once.  (Left to the compiler, a quad came in three trips - the first words, then the rest behind the first edge
    // test, then the surfel id behind the hit - and the lanes at leaf groups took theirs after the lanes at nodes had
    // finished theirs.)
    typedef const __attribute__((address_space(1))) v4f *global_v4f;
#pragma unroll 1
    while (wave_ballot(ref != kWalkDone) != 0ull) {
        if (ref == kWalkDone) continue;
        uint32_t next = kWalkDone;
        bool have_next = false;
        const bool is_leaf = (ref & DST_LEAF_BIT) != 0u;
        const uint32_t first = ref & DST_REF_FIRST_MASK, count = ((ref >> 28) & 7u) + 1u;
        const bool good = is_leaf ? (first < acc.n_leaves) : (ref + 1u < acc.n_leaves);
        if (good) {
            const bool two = is_leaf && count > 1u && first + 1u < acc.n_leaves;
            const global_v4f src = is_leaf ? (global_v4f)reinterpret_cast<const v4f *>(&acc.leaves[first])
                                           : (global_v4f)reinterpret_cast<const v4f *>(&acc.wide[ref]);
            // a node is 8 x 16 bytes; of a quad's record the first 4 words of 16 bytes are read (a leaf group of one quad
            // asks for 8 as well: the array has spare records behind its last quad), the second quad's are words 6 to 9
            v4f r0 = src[0], r1 = src[1], r2 = src[2], r3 = src[3], r4 = src[4], r5 = src[5], r6 = src[6], r7 = src[7];
            v4f r8 = {0.f, 0.f, 0.f, 0.f}, r9 = {0.f, 0.f, 0.f, 0.f};
            if (two) {
                r8 = src[8];
                r9 = src[9];
            }
            // every value is in its registers here: nothing of the above may be requested later, behind a test
            asm volatile("" : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3), "+v"(r4));
            asm volatile("" : "+v"(r5), "+v"(r6), "+v"(r7), "+v"(r8), "+v"(r9));
            if (is_leaf) {
                // the first 64 bytes of a record: A, AB, AC, AD, n1 (three floats each), surfel id; n0, n2 and c1 are
                // formed as the builder forms them for the record's other 32 bytes
#define DST_LANE_QUAD(w0, w1, w2, w3)                                                                                  \
    {                                                                                                                  \
        float t = 0.f;                                                                                                 \
        uint32_t tri = 0u;                                                                                             \
        const F3 AB = f3(w0.w, w1.x, w1.y), AC = f3(w1.z, w1.w, w2.x), AD = f3(w2.y, w2.z, w2.w), n1 = f3(w3.x, w3.y, w3.z); \
        const bool hit = ray_quad(o, d, f3(w0.x, w0.y, w0.z), AB, AC, AD, cross_f(AB, AC), n1, cross_f(AC, AD),        \
                                  dot_f(n1, AB), t, tri);                                                              \
        const uint64_t x = kb_pack(t, 2u * __float_as_uint(w3.w) + tri);                                               \
        if (hit && (x < buf.e[kChunk - 1])) {                                                                          \
            cnt += 1u;                                                                                                 \
            kbuf_insert(buf, x, true);                                                                                 \
        }                                                                                                              \
    }
                DST_LANE_QUAD(r0, r1, r2, r3)
                if (two) DST_LANE_QUAD(r6, r7, r8, r9)
#undef DST_LANE_QUAD
                // (groups of more than two quads do not occur: DST_GROUP = 2; a longer one would lose its tail)
            } else {
                // lox r0, loy r1, loz r2, hix r3, hiy r4, hiz r5, child references r6, child count r7.x
                const uint32_t n_child = __float_as_uint(r7.x);
                const float tmax = kb_t(buf.e[kChunk - 1]);
                uint32_t key[DST_WIDE], cref[DST_WIDE];
#pragma unroll
                for (int k = 0; k < DST_WIDE; ++k) {
                    float tn;
                    const uint64_t h = slab_hit_fast(fs, neg_x ? r3[k] : r0[k], neg_y ? r4[k] : r1[k], neg_z ? r5[k] : r2[k],
                                                     neg_x ? r0[k] : r3[k], neg_y ? r1[k] : r4[k], neg_z ? r2[k] : r5[k],
                                                     tmax, tn);
                    const bool mine = ((h >> __lane_id()) & 1ull) != 0ull && (uint32_t)k < n_child;
                    key[k] = mine ? __float_as_uint(tn) : 0xFFFFFFFFu;   // entry distance (non-negative: bits order like the value)
                    cref[k] = __float_as_uint(r6[k]);
                }
#define CSWAP(a, b)                                                            \
    {                                                                          \
        const bool sw_ = key[b] < key[a];                                      \
        const uint32_t ka_ = sw_ ? key[b] : key[a], kb_ = sw_ ? key[a] : key[b]; \
        const uint32_t ra_ = sw_ ? cref[b] : cref[a], rb_ = sw_ ? cref[a] : cref[b]; \
        key[a] = ka_; key[b] = kb_; cref[a] = ra_; cref[b] = rb_;              \
    }
                CSWAP(0, 1) CSWAP(2, 3) CSWAP(0, 2) CSWAP(1, 3) CSWAP(1, 2)
#undef CSWAP
                // defer the farther children (farthest first), go on with the nearest
#pragma unroll
                for (int k = DST_WIDE - 1; k >= 1; --k) {
                    if (key[k] != 0xFFFFFFFFu && sp < kLaneStack) {
                        if (shelf != nullptr && sp < kLaneShelf) ((lds_u32)shelf)[sp * DST_WAVE + (int)__lane_id()] = cref[k];
                        else stack[sp] = cref[k];
                        ++sp;
                    }
                }
                if (key[0] != 0xFFFFFFFFu) {
                    next = cref[0];
                    have_next = true;
                }
            }
        }
        if (!have_next && sp > 0) {
            --sp;
            next = (shelf != nullptr && sp < kLaneShelf) ? ((lds_u32)shelf)[sp * DST_WAVE + (int)__lane_id()] : stack[sp];
        }
        ref = (--budget == 0u) ? kWalkDone : next;
    }
    buf_mem = buf;
    cnt_mem = cnt;
}

// Packet or per-lane walk for the rays of this wave?  A packet pays off when the rays run side by side: every
// live ray is compared with the first live one (origins as given by the caller, not advanced along the ray).
__device__ __forceinline__ bool rays_run_together(F3 o, F3 d, bool active, float max_abs) {
    const uint64_t live = wave_ballot(active);
    if (live == 0ull) return true;
    const int lead = __builtin_ctzll(live);
    const F3 o0 = f3(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(o.x), lead)),
                     __int_as_float(__builtin_amdgcn_readlane(__float_as_int(o.y), lead)),
                     __int_as_float(__builtin_amdgcn_readlane(__float_as_int(o.z), lead)));
    const F3 d0 = f3(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(d.x), lead)),
                     __int_as_float(__builtin_amdgcn_readlane(__float_as_int(d.y), lead)),
                     __int_as_float(__builtin_amdgcn_readlane(__float_as_int(d.z), lead)));
    const float dd = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(d.x - d0.x), __builtin_fabsf(d.y - d0.y)),
                                     __builtin_fabsf(d.z - d0.z));
    const float od = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(o.x - o0.x), __builtin_fabsf(o.y - o0.y)),
                                     __builtin_fabsf(o.z - o0.z));
    const float dl = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(d0.x), __builtin_fabsf(d0.y)),
                                     __builtin_fabsf(d0.z));
    const bool apart = active && (!(dd <= kPacketDirSpread * dl) || !(od <= kPacketOrgSpread * max_abs));
    return wave_ballot(apart) == 0ull;
}

template <bool MIXED, bool SHELF, bool RESUME, bool HAND>
__device__ __forceinline__ void packet_knn(const DstAccelView &acc, float max_abs, F3 o, F3 d, bool active, KBuf &buf,
                                           uint32_t &cnt, bool as_packet, WalkList &wl, uint32_t *shelf
#ifdef DST_STATS
                                           , WaveStats &ws
#endif
) {
    const uint64_t live = wave_ballot(active);
    if (live == 0ull) return;
    const RaySlab slab = make_slab(o, d, max_abs);
    if (MIXED && !as_packet) {
        KBuf mine = buf;   // a copy the call may keep in memory; the caller's buffer stays in registers
        uint32_t n = cnt;
        // forward kernels (one wave per workgroup, no other LDS) give the walk an LDS shelf for its stacks
        const LaneWalkAccel view = {acc.leaves, acc.wide, acc.n_leaves, acc.root};
        lane_walk(view, slab, o, d, active, mine, n, SHELF ? shelf : nullptr);
        buf = mine;
        cnt = n;
        return;
    }
    // The walk assumes one set of direction signs per packet (the near face of every box is then the same for
    // all lanes).  A wave whose rays straddle an axis plane (about 1 % of the tiles of a pinhole image) is
    // walked once per sign class present, each time with the lanes of that class only.
    const uint32_t my_sgn = (slab.ix < 0.f ? 1u : 0u) | (slab.iy < 0.f ? 2u : 0u) | (slab.iz < 0.f ? 4u : 0u);
    uint64_t todo = live;
    if (RESUME) {
        // a work list serves one walk per chunk: waves with several sign classes walk from the root every time
        const uint32_t sgn0 = __builtin_amdgcn_readlane(my_sgn, __builtin_ctzll(live));
        wl.record = wave_ballot(active && my_sgn != sgn0) == 0ull && acc.n_leaves <= (1u << kListIndexBits);
        if (!wl.record) wl.n_in = kListFresh;
    }
    while (todo != 0ull) {
        const int rep = __builtin_ctzll(todo);   // also the lane whose entry distances order the children
        const uint32_t sgn = __builtin_amdgcn_readlane(my_sgn, rep);
        const bool mine = active && my_sgn == sgn;
        todo &= ~wave_ballot(mine);
        packet_walk<RESUME, HAND>(acc, slab, sgn, o, d, mine, rep, buf, cnt, wl WSP);
    }
}

__device__ __forceinline__ void aadd(float *p, float v) { unsafeAtomicAdd(p, v); }

// ---- per-block gradient table (backward) ---------------------------------------------------------------
// The 16x16 pixel tile of a block keeps hitting the same few hundred surfels, so the per-surfel gradients
// are first summed in an LDS hash table (one row of columns per surfel, LDS atomics) and written to
// global memory once per surfel and block when the block ends.  A surfel that finds no free row within a
// few probes goes straight to global atomics, so the table can never be wrong, only less effective.
#ifndef DST_TABLE_FLUSH_NUM
#define DST_TABLE_FLUSH_NUM 3   // the table is emptied between rounds once this many eighths of its rows are in use
                                // (measured 1..6: a fuller table sends more hits past it, straight to memory)
#endif
#ifndef DST_TABLE_ROWS_LOG2
#define DST_TABLE_ROWS_LOG2 7
#endif
constexpr uint32_t kEmptyKey = 0xFFFFFFFFu;
constexpr int kMaxProbe = 8;
// row columns: colour 0-2, opacity 3, scales 4-5, rotation 6-9, mean 10-12, densification mean 13-15, SH coefficient
// j channel c at 16+3j+c (16..63), aux 64..64+AUXM-1.  The auxiliary channels come last so that a scene without
// them (the usual one) fills exactly four 16-column tiles of the group reduction and skips the fifth.
constexpr int kColColor = 0, kColOpac = 3, kColScale = 4, kColRot = 6, kColMean = 10, kColGrad = 13, kColSh = 16,
              kColAux = 64;
template <int AUXM> struct RowLayout {
    static constexpr int sh0 = kColSh;
    static constexpr int cols = kColAux + AUXM;
    static constexpr int stride = cols | 1;     // odd: rows spread over all LDS banks
    // rows of the block's table: with more auxiliary channels the rows are longer, and three blocks must fit a CU
    static constexpr int rows_log2 = AUXM <= 2 ? DST_TABLE_ROWS_LOG2 : DST_TABLE_ROWS_LOG2 - 1;
    static constexpr int rows = 1 << rows_log2;
};
// The deterministic mode keeps 64-bit fixed-point sums in the table: half as many rows in the same memory.
template <int AUXM, bool DET> struct TableRows {
    static constexpr int rows_log2 = RowLayout<AUXM>::rows_log2 - (DET ? 1 : 0);
    static constexpr int rows = 1 << rows_log2;
};

// ---- deterministic mode: sums in 64-bit fixed point ------------------------------------------------------
// Integer addition is exact, so a sum of fixed-point numbers does not depend on the order of its terms: every
// atomically accumulated value (LDS table, global memory) is converted first.  2^-36 units for the geometric
// columns (scale, rotation, mean, densification: range +-6.7e7), 2^-40 for the others and for the blending
// weights (+-4.2e6); a value outside the range saturates.  The closing kernels count the sums they find in the outer
// half of the range (one saturated term puts a sum there), so that a scene too large for the mode is noticed.
constexpr int kDetShiftGeo = 36, kDetShiftOther = 40;
__device__ __forceinline__ bool det_out_of_range(long long q) { return q >= (1LL << 61) || q <= -(1LL << 61); }
__device__ __forceinline__ int det_shift(int col) { return (col >= kColScale && col < kColSh) ? kDetShiftGeo : kDetShiftOther; }
__device__ __forceinline__ long long to_fixed(float v, int shift) {
    float x = __builtin_ldexpf(v, shift);                       // exact scaling
    x = __builtin_fminf(__builtin_fmaxf(x, -4.6e18f), 4.6e18f);   // |x| < 2^62; NaN becomes a bound
    return (long long)x;
}
__device__ __forceinline__ float from_fixed(long long q, int shift) { return (float)__builtin_ldexp((double)q, -shift); }

// Address in the caller's gradient tensors of column `col` of surfel g (nullptr: nothing to write).
template <int AUXM>
__device__ __forceinline__ float *tensor_address(const DstParams &p, uint32_t g, int col) {
    if (col < kColOpac) return p.dL_dcolors + 3 * (size_t)g + col;
    if (col < kColScale) return p.dL_dopacities + g;
    if (col < kColRot) return p.dL_dscales + 2 * (size_t)g + (col - kColScale);
    if (col < kColMean) return p.dL_drotations + 4 * (size_t)g + (col - kColRot);
    if (col < kColGrad) return p.dL_dmeans3D + 3 * (size_t)g + (col - kColMean);
    if (col < kColSh) return p.dL_dgrads3D + 3 * (size_t)g + (col - kColGrad);
    if (col >= kColAux) {
        const int ch = col - kColAux;
        return (p.others_precomp != nullptr && ch < p.aux) ? p.dL_dothers + (size_t)p.aux * g + ch : nullptr;
    }
    const int k = col - kColSh;   // 3j + c
    return (p.colors_precomp == nullptr && k < 3 * p.M) ? p.dL_dshs + (size_t)g * p.M * 3 + k : nullptr;
}
// Is column `col` in use?  (no auxiliary input: no aux columns; colours given: no SH columns; SH degree < 3: fewer)
template <int AUXM>
__device__ __forceinline__ bool column_live(const DstParams &p, int col) {
    if (col < kColSh) return true;
    if (col >= kColAux) return p.others_precomp != nullptr && col - kColAux < p.aux;
    return p.colors_precomp == nullptr && col - kColSh < 3 * p.M;
}
// Where the kernels add column `col` of surfel g: the row of g in the caller's gradient rows if there are any
// (all columns of a surfel side by side; a closing kernel adds the rows to the tensors), else the tensors.
template <int AUXM>
__device__ __forceinline__ float *grad_address(const DstParams &p, uint32_t g, int col) {
    if (p.grad_rows == nullptr) return tensor_address<AUXM>(p, g, col);
    return column_live<AUXM>(p, col) ? p.grad_rows + (size_t)g * RowLayout<AUXM>::cols + col : nullptr;
}

// Sum of v over the 64 lanes; every lane must be active.
__device__ __forceinline__ float wave_sum_f32(float v) {
#define DST_DPP_ADD(ctrl, rmask)                                                                              \
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, rmask, 0xf, true))
    DST_DPP_ADD(0x111, 0xf);   // row_shr:1
    DST_DPP_ADD(0x112, 0xf);   // row_shr:2
    DST_DPP_ADD(0x114, 0xf);   // row_shr:4
    DST_DPP_ADD(0x118, 0xf);   // row_shr:8   -> lane 15 of each row holds the row total
    DST_DPP_ADD(0x142, 0xa);   // row_bcast:15 into rows 1 and 3
    DST_DPP_ADD(0x143, 0xc);   // row_bcast:31 into rows 2 and 3 -> lane 63 holds the wave total
#undef DST_DPP_ADD
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));   // the builtin moves bits of an int
}

// base[key] += v for every lane with `on`, wave-uniform call.  Neighbouring rays mostly composite the same surfel
// in the same step, and atomics of one instruction to one address are served one after the other, so the lanes
// of the most frequent keys are summed across the wave and their first lane adds the total.
__device__ __forceinline__ void wave_add_grouped(float *base, unsigned long long *det, bool on, uint32_t key, float v) {
    auto add = [&](uint32_t k, float x) {
        if (det != nullptr) atomicAdd(det + k, (unsigned long long)to_fixed(x, kDetShiftOther));
        else aadd(base + k, x);
    };
    const uint32_t lane = __lane_id();
    uint64_t rem = wave_ballot(on);
#pragma unroll 1
    for (int tries = 0; tries < 6 && rem != 0ull; ++tries) {
        const int first = __builtin_ctzll(rem);
        const uint32_t k0 = __builtin_amdgcn_readlane(key, first);
        const bool same = on && key == k0;
        const uint64_t grp = wave_ballot(same);
        if (__popcll(grp) >= 3) {
            const float s = wave_sum_f32(same ? v : 0.f);
            if (lane == (uint32_t)first) add(k0, s);
            on = on && !same;
        }
        rem &= ~grp;
    }
    if (on) add(key, v);
}

// The blending weights of an image wave (forward, training): a wave composites the same two hundred or so surfels over
// and over (64 neighbouring rays, some 37 hits each), so their weights are first summed in a small hash table in LDS
// (surfel id -> running sum, LDS atomics) and go to memory once per surfel and wave when the wave ends - a sixteenth of
// the global atomics.  A surfel that finds no slot within a few probes adds straight to memory.
constexpr int kWetSlotsLog2 = 8, kWetSlots = 1 << kWetSlotsLog2, kWetProbes = 4;
__device__ __forceinline__ void wet_add(uint32_t *keys, float *vals, float *a_weights, bool on, uint32_t g, float w) {
    if (!on) return;
    uint32_t slot = (g * 2654435761u) >> (32 - kWetSlotsLog2);
#pragma unroll 1
    for (int probe = 0; probe < kWetProbes; ++probe) {
        uint32_t k = __hip_atomic_load(keys + slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (k == 0xFFFFFFFFu) {
            uint32_t expected = 0xFFFFFFFFu;
            __hip_atomic_compare_exchange_strong(keys + slot, &expected, g, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_WORKGROUP);
            k = expected == 0xFFFFFFFFu ? g : expected;
        }
        if (k == g) {
            __hip_atomic_fetch_add(vals + slot, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            return;
        }
        slot = (slot + 1u) & (uint32_t)(kWetSlots - 1);
    }
    aadd(a_weights + g, w);
}

// Find or claim the table row of surfel g; -1 if none is free within a few probes.  keys[rows] counts the
// rows claimed since the table was last emptied.
template <int ROWS_LOG2>
__device__ __forceinline__ int table_slot(uint32_t *keys, uint32_t g) {
    uint32_t slot = (g * 2654435761u) >> (32 - ROWS_LOG2);
#pragma unroll 1
    for (int probe = 0; probe < kMaxProbe; ++probe) {
        uint32_t k = __hip_atomic_load(keys + slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (k == kEmptyKey) {
            uint32_t expected = kEmptyKey;
            __hip_atomic_compare_exchange_strong(keys + slot, &expected, g, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_WORKGROUP);
            if (expected == kEmptyKey) {
                k = g;
                __hip_atomic_fetch_add(keys + (1u << ROWS_LOG2), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            } else {
                k = expected;
            }
        }
        if (k == g) return (int)slot;
        slot = (slot + 1) & ((1u << ROWS_LOG2) - 1u);
    }
    return -1;
}

// Where one step's per-surfel gradients go.  Neighbouring rays mostly composite the same few surfels in the
// same step, so the wave first sums the lanes of each surfel and only the sums go to the table.  That sum is
// a matrix product: (columns x rays) times (rays x surfel groups, entries 0 or 1).  The lanes stage their
// column values in LDS, sixteen columns at a time, and sixteen 16x16x4 fp32 MFMAs per tile produce the sums
// of up to sixteen groups at once; lanes of further groups (rare) add their values directly.
constexpr int kStageCols = 16;                 // columns per tile
constexpr int kStageStride = DST_WAVE + 1;     // floats per staged column: conflict-free writes and reads
constexpr int kStageWords = kStageCols * kStageStride;
template <int AUXM, bool DET>
struct GradSink {
    const DstParams *p;
    float *rows;         // the block's table
    float *stage;        // this wave's staging tile: [column in tile][lane]
    bool did;            // this lane composited a hit in this step
    uint32_t g;          // its surfel
    int own_slot;        // table row of g, -1: none
    bool stray;          // hit, but not in one of the sixteen groups
    bool any_stray;      // wave-uniform: some lane is a stray
    uint32_t members;    // bit m: the ray of lane 16*(lane/16)+m belongs to group lane%16
    bool out_on;         // lane%16 is a group of this step
    int out_slot;        // table row of group lane%16, -1: write through to global memory
    uint32_t out_g;      // surfel of group lane%16
    int limit;           // columns in use
    uint64_t wt;         // wave-uniform: lanes whose surfel has no table row (their values go to global memory)

    // Wave-uniform; every lane of the wave must be active.
    __device__ __forceinline__ void plan(uint32_t *keys) {
        const uint32_t lane = __lane_id();
        uint64_t rem = wave_ballot(did);
        int n_groups = 0;
        bool grouped = false;
        uint32_t leader = 0u;
        members = 0u;
#pragma unroll 1
        while (rem != 0ull && n_groups < kStageCols) {
            const int first = __builtin_ctzll(rem);
            const uint32_t k0 = __builtin_amdgcn_readlane(g, first);
            const bool same = did && g == k0;
            const uint64_t grp = wave_ballot(same);
            if ((lane & 15u) == (uint32_t)n_groups) {
                members = (uint32_t)(grp >> (lane & 48u)) & 0xFFFFu;
                leader = (uint32_t)first;
            }
            grouped = grouped || same;
            ++n_groups;
            rem &= ~grp;
        }
        stray = did && !grouped;
        any_stray = wave_ballot(stray) != 0ull;
        out_on = (lane & 15u) < (uint32_t)n_groups;
        own_slot = did ? table_slot<TableRows<AUXM, DET>::rows_log2>(keys, g) : -1;
        out_slot = __builtin_amdgcn_ds_bpermute((int)(leader << 2), own_slot);
        out_g = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(leader << 2), (int)g);
        // (deterministic mode: a group's sum must be rounded to fixed point as one number whether or not it finds
        // a table row, which depends on timing; so only the lanes outside the groups take this route there)
        wt = wave_ballot(did && own_slot < 0 && (!DET || stray));
    }

    __device__ __forceinline__ void put_global(uint32_t surfel, int col, float v) const {
        if (DET) {
            if (column_live<AUXM>(*p, col))
                atomicAdd(p->det_workspace + (size_t)surfel * RowLayout<AUXM>::cols + col,
                          (unsigned long long)to_fixed(v, det_shift(col)));
        } else {
            float *dst = grad_address<AUXM>(*p, surfel, col);
            if (dst != nullptr) aadd(dst, v);
        }
    }

    // Add v to column `col` of table row `slot` (>= 0).
    __device__ __forceinline__ void put(int slot, int col, float v) const {
        if (DET)
            __hip_atomic_fetch_add(reinterpret_cast<long long *>(rows) + (size_t)slot * RowLayout<AUXM>::stride + col,
                                   to_fixed(v, det_shift(col)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else
            __hip_atomic_fetch_add(rows + (size_t)slot * RowLayout<AUXM>::stride + col, v, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_WORKGROUP);
    }

    // The staged tile's values of the lanes in `wt`, added to global memory.  Sixteen lanes take the sixteen
    // columns of one such lane's hit, so that one instruction adds to four runs of consecutive addresses (four hits)
    // instead of to one address in each of up to 64 surfels' rows: the memory system works on whole cache lines.
    __device__ __forceinline__ void write_through(int tile) const {
        const uint32_t lane = __lane_id();
        const int c = (int)(lane & 15u), k = (int)(lane >> 4);
        const int col = tile * kStageCols + c;
        uint64_t m = wt;
#pragma unroll 1
        while (m != 0ull) {
            int h = -1;   // quarter k of the wave takes the k-th of the next four hits
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (m != 0ull) {
                    const int hq = __builtin_ctzll(m);
                    m &= m - 1ull;
                    if (k == q) h = hq;
                }
            }
            const int src = h < 0 ? 0 : h;
            const uint32_t gh = (uint32_t)__builtin_amdgcn_ds_bpermute(src << 2, (int)g);   // every lane is active here
            const float v = stage[c * kStageStride + src];
            if (h >= 0 && col < limit && v != 0.f) put_global(gh, col, v);
        }
    }

    // Sums of the staged tile per group, added to the groups' rows.  Wave-uniform.
    __device__ __forceinline__ void flush(int tile) const {
        const uint32_t lane = __lane_id();
        const float *a = stage + (lane & 15u) * kStageStride + (lane & 48u);
        v4f acc = {0.f, 0.f, 0.f, 0.f};
        // all sixteen operands are asked for before the first product: left alone, the compiler reads two, waits,
        // multiplies, reads the next two, ... - eight trips to LDS one after the other per tile
        float av[16];
#pragma unroll
        for (int m = 0; m < 16; ++m) av[m] = a[m];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < 16; ++m)
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[m], ((members >> m) & 1u) ? 1.0f : 0.0f, acc, 0, 0, 0);
        // acc[r] = column 16*tile + 4*(lane/16) + r summed over the rays of group lane%16
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int col = tile * kStageCols + 4 * (int)(lane >> 4) + r;
            if (out_on && col < limit && acc[r] != 0.f) {
                if (out_slot >= 0) put(out_slot, col, acc[r]);
                else if (DET) put_global(out_g, col, acc[r]);
            }
        }
        if (wt != 0ull) write_through(tile);   // groups and further lanes without a table row
    }

    // Wave-uniform calls in ascending column order (every lane reaches them); `col` is a constant after
    // inlining.  The tile is reduced when its last column arrives; finish() reduces a partly filled last tile.
    __device__ __forceinline__ void add(int col, float v) const {
        stage[(col & (kStageCols - 1)) * kStageStride + __lane_id()] = did ? v : 0.f;
        if (any_stray) {   // rare: more than sixteen surfels in one step
            if (stray && own_slot >= 0 && col < limit) put(own_slot, col, v);
        }
        if ((col & (kStageCols - 1)) == kStageCols - 1) flush(col / kStageCols);
    }
    __device__ __forceinline__ void finish(int next_col) const {
        if ((next_col & (kStageCols - 1)) != 0) flush(next_col / kStageCols);
    }
};

template <int AUXM>
struct BounceIn {  // backward: saved results of the bounce and the gradients flowing into them
    float rgb[3], dpt, acc, nrm[3], aux[AUXM];
    float g_rgb[3], g_dpt, g_acc, g_nrm[3], g_aux[AUXM];
};

template <int AUXM>
struct BounceAcc {
    float C[3], D, N[3], O[AUXM], T;
};

// The SH colour's derivative with respect to the direction it was evaluated for, contracted with the colour
// gradient gc (backward.cu:100-165).
struct LastShHit {
    int g; F3 gc; bool any;
#ifdef DST_STATS
    unsigned long long t0, t_alg, t_sh;
#endif
};
template <class SH>
__device__ __forceinline__ F3 sh_direction_gradient(int deg, const SH &sh, F3 rd, F3 gc) {
#pragma clang fp contract(fast)
    auto S = [&](int j) { return f3(sh(3 * j), sh(3 * j + 1), sh(3 * j + 2)); };
    F3 ddx = f3(0, 0, 0), ddy = f3(0, 0, 0), ddz = f3(0, 0, 0);
    const float x = rd.x, y = rd.y, z = rd.z;
    if (deg > 0) {
        ddx = -SH1 * S(3);
        ddy = -SH1 * S(1);
        ddz = SH1 * S(2);
        if (deg > 1) {
            const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
            ddx = ddx + SH2[0] * y * S(4) + SH2[2] * 2.f * -x * S(6) + SH2[3] * z * S(7) + SH2[4] * 2.f * x * S(8);
            ddy = ddy + SH2[0] * x * S(4) + SH2[1] * z * S(5) + SH2[2] * 2.f * -y * S(6) + SH2[4] * 2.f * -y * S(8);
            ddz = ddz + SH2[1] * y * S(5) + SH2[2] * 4.f * z * S(6) + SH2[3] * x * S(7);
            if (deg > 2) {
                ddx = ddx + (SH3[0] * 6.f * xy) * S(9) + (SH3[1] * yz) * S(10) + (SH3[2] * -2.f * xy) * S(11) +
                      (SH3[3] * -6.f * xz) * S(12) + (SH3[4] * (-3.f * xx + 4.f * zz - yy)) * S(13) +
                      (SH3[5] * 2.f * xz) * S(14) + (SH3[6] * 3.f * (xx - yy)) * S(15);
                ddy = ddy + (SH3[0] * 3.f * (xx - yy)) * S(9) + (SH3[1] * xz) * S(10) +
                      (SH3[2] * (-3.f * yy + 4.f * zz - xx)) * S(11) + (SH3[3] * -6.f * yz) * S(12) +
                      (SH3[4] * -2.f * xy) * S(13) + (SH3[5] * -2.f * yz) * S(14) + (SH3[6] * -6.f * xy) * S(15);
                ddz = ddz + (SH3[1] * xy) * S(10) + (SH3[2] * 8.f * yz) * S(11) +
                      (SH3[3] * 3.f * (2.f * zz - xx - yy)) * S(12) + (SH3[4] * 8.f * xz) * S(13) +
                      (SH3[5] * (xx - yy)) * S(14);
            }
        }
    }
    return f3(dot(ddx, gc), dot(ddy, gc), dot(ddz, gc));
}

// Gradient of one composited hit (reference backward.cu:528-640 and 201-287, 68-166).
// Pure gradient algebra: nothing here feeds a decision, so contraction is allowed.
template <int AUXM, bool DET>
__device__ __forceinline__ void hit_backward(const DstParams &p, const BounceIn<AUXM> &in, const BounceAcc<AUXM> &run,
                                             int g, uint32_t pidx, float Tp, float alpha, float G, float w, float dpt,
                                             F3 xyz, const F3 (&R)[3], float u, float v, float sx, float sy, F3 mean,
                                             float q0, float q1, float q2, float q3, float opac, float nsign,
                                             F3 normal, const float (&col)[3], const bool (&neg)[3], F3 ro, F3 rd,
                                             const float *__restrict__ sh, F3 &g_ro, F3 &g_rd,
                                             const GradSink<AUXM, DET> &sink, bool did, LastShHit &last) {
#pragma clang fp contract(fast)
    // gradient algebra only: divisions become multiplications by a hardware reciprocal (1 ulp)
    const float num = 1.0f - alpha, inv_num = __builtin_amdgcn_rcpf(num);
    const float T_final = 1.0f - in.acc;
    float g_alpha = 0.f;
    float g_col[3], g_aux_w[AUXM];
#pragma unroll
    for (int ch = 0; ch < 3; ++ch) {
        g_col[ch] = in.g_rgb[ch] * w;
        g_alpha += in.g_rgb[ch] * (Tp * col[ch] - (in.rgb[ch] - run.C[ch]) * inv_num);
        g_alpha += in.g_rgb[ch] * p.background[ch] * (-T_final * inv_num);
    }
#pragma unroll
    for (int ch = 0; ch < AUXM; ++ch) g_aux_w[ch] = 0.f;
    if (p.others_precomp != nullptr) {
#pragma unroll
        for (int ch = 0; ch < AUXM; ++ch) {
            if (ch < p.aux) {
                float o = p.others_precomp[(size_t)p.aux * g + ch];
                g_aux_w[ch] = in.g_aux[ch] * w;
                g_alpha += in.g_aux[ch] * (Tp * o - (in.aux[ch] - run.O[ch]) * inv_num);
            }
        }
    }
    const float g_D = in.g_dpt * w;
    g_alpha += in.g_dpt * (Tp * dpt - (in.dpt - run.D) * inv_num);
    const F3 g_N = f3(in.g_nrm[0] * w, in.g_nrm[1] * w, in.g_nrm[2] * w);
    g_alpha += in.g_nrm[0] * (Tp * normal.x - (in.nrm[0] - run.N[0]) * inv_num) +
               in.g_nrm[1] * (Tp * normal.y - (in.nrm[1] - run.N[1]) * inv_num) +
               in.g_nrm[2] * (Tp * normal.z - (in.nrm[2] - run.N[2]) * inv_num);
    g_alpha += in.g_acc * (Tp - in.acc * inv_num);   // the reference never accumulates W (backward.cu:568)
    const float g_G = g_alpha * opac;
    const float pc = (opac * G) > 0.99f ? 0.0f : 1.0f;

    // triangle that was hit, with its corner coordinates in splat units (backward.cu:583-602)
    const float *V = p.vertices + (size_t)g * 12;
    const bool second = (pidx & 1u) != 0u;
    const F3 v1 = ld3(second ? V + 3 : V), v2 = ld3(second ? V + 6 : V + 3), v3 = ld3(second ? V + 9 : V + 6);
    const float k = g_G * pc;
    const float gu = k * -G * u, gv = k * -G * v;
    F3 gR[3];
    const F3 rel = xyz - mean;
    const float inv_sx = __builtin_amdgcn_rcpf(sx), inv_sy = __builtin_amdgcn_rcpf(sy);
    gR[0] = (gu * inv_sx) * rel;
    gR[1] = (gv * inv_sy) * rel;
    gR[2] = g_N * nsign;
    float g_sx = k * (G * u * u * inv_sx), g_sy = k * (G * v * v * inv_sy);
    F3 g_mean = k * (G * (R[0] * (u * inv_sx) + R[1] * (v * inv_sy)));
    const F3 g_xyz = (gu * inv_sx) * R[0] + (gv * inv_sy) * R[1];
    const float g_d = g_D + dot(g_xyz, rd);
    const F3 n = cross(v2 - v1, v3 - v1);
    const F3 c = v1 - ro;
    const float pp = dot(n, c), q = dot(n, rd), inv_q = __builtin_amdgcn_rcpf(q);
    const F3 g_n = (c - (pp * inv_q) * rd) * inv_q;
    if (did) {
        g_ro = g_ro + (g_xyz + (-g_d * inv_q) * n);
        g_rd = g_rd + (g_xyz * dpt + ((g_d * -pp) * (inv_q * inv_q)) * n);
    }
    // The corner gradients (backward.cu:583-602) are g_v1 = g_d (v2-v3) x g_n + (g_d/q) n, g_v2 = g_d (v3-v1) x g_n,
    // g_v3 = g_d (v1-v2) x g_n, and the corners sit at (+-3, +-3) splat units.  Their sums with those weights are
    // taken on the edge vectors first, where they collapse to one edge each: the three cross products nearly
    // cancel for a long thin quad, and summed after the fact they leave mostly rounding.
    //   sum of the corners' gradients          = (g_d/q) n
    //   weighted by the corners' u coordinates = g_d 6 a x g_n + hu (g_d/q) n
    //   weighted by the corners' v coordinates = g_d 6 b x g_n + hv (g_d/q) n
    // with a = v1-v2, b = v1-v3, (hu,hv) = (-3,3) for the first triangle; a = v3-v2, b = v3-v1, (-3,-3) for the second.
    const F3 g_c = (g_d * inv_q) * n;
    const F3 ea = second ? v3 - v2 : v1 - v2, eb = second ? v3 - v1 : v1 - v3;
    const F3 su = (6.f * g_d) * cross(ea, g_n) - 3.f * g_c;
    const F3 sv = (6.f * g_d) * cross(eb, g_n) + (second ? -3.f : 3.f) * g_c;
    gR[0] = gR[0] + sx * su;
    gR[1] = gR[1] + sy * sv;
    g_sx += dot(R[0], su);
    g_sy += dot(R[1], sv);
    g_mean = g_mean + g_c;
    // rotation: vjp of quat_rows without the normalisation Jacobian (auxiliary.h:433-477)
    float g_rot[4];
    {
        float s = __builtin_amdgcn_rsqf(q3 * q3 + q0 * q0 + q1 * q1 + q2 * q2);
        float w_ = q0 * s, x = q1 * s, y = q2 * s, z = q3 * s;
        float r0 = 2.f * (x * (gR[1].z - gR[2].y) + y * (gR[2].x - gR[0].z) + z * (gR[0].y - gR[1].x));
        float r1 = 2.f * (-2.f * x * (gR[1].y + gR[2].z) + y * (gR[0].y + gR[1].x) + z * (gR[0].z + gR[2].x) +
                          w_ * (gR[1].z - gR[2].y));
        float r2 = 2.f * (x * (gR[0].y + gR[1].x) - 2.f * y * (gR[0].x + gR[2].z) + z * (gR[1].z + gR[2].y) +
                          w_ * (gR[2].x - gR[0].z));
        float r3 = 2.f * (x * (gR[0].z + gR[2].x) + y * (gR[1].z + gR[2].y) - 2.f * z * (gR[0].x + gR[1].y) +
                          w_ * (gR[0].y - gR[1].x));
        g_rot[0] = r0; g_rot[1] = r1; g_rot[2] = r2; g_rot[3] = r3;
    }
    STAT(last.t_alg += __builtin_readcyclecounter() - last.t0; last.t0 = __builtin_readcyclecounter();)
    // the table columns, in ascending order
    sink.add(kColColor + 0, g_col[0]); sink.add(kColColor + 1, g_col[1]); sink.add(kColColor + 2, g_col[2]);
    sink.add(kColOpac, g_alpha * G * pc);
    sink.add(kColScale + 0, g_sx);
    sink.add(kColScale + 1, g_sy);
    sink.add(kColRot + 0, g_rot[0]); sink.add(kColRot + 1, g_rot[1]); sink.add(kColRot + 2, g_rot[2]); sink.add(kColRot + 3, g_rot[3]);
    sink.add(kColMean + 0, g_mean.x); sink.add(kColMean + 1, g_mean.y); sink.add(kColMean + 2, g_mean.z);
    const float hd = 0.5f * dpt;
    sink.add(kColGrad + 0, g_mean.x * hd); sink.add(kColGrad + 1, g_mean.y * hd); sink.add(kColGrad + 2, g_mean.z * hd);
    // (the first tile, columns 0..15, has just been reduced: its last column triggers that)

    STAT(last.t_sh += __builtin_readcyclecounter() - last.t0;)   // first tile done
    if (p.colors_precomp == nullptr) {
        // SH backward (backward.cu:68-166); the direction gradient REPLACES the ray's (backward.cu:165)
        const int deg = p.D;
        F3 gc = f3(neg[0] ? 0.f : g_col[0], neg[1] ? 0.f : g_col[1], neg[2] ? 0.f : g_col[2]);
        auto put = [&](int j, float basis) {
            sink.add(RowLayout<AUXM>::sh0 + 3 * j + 0, basis * gc.x);
            sink.add(RowLayout<AUXM>::sh0 + 3 * j + 1, basis * gc.y);
            sink.add(RowLayout<AUXM>::sh0 + 3 * j + 2, basis * gc.z);
        };
        const float x = rd.x, y = rd.y, z = rd.z;
        float basis[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) basis[j] = 0.f;
        basis[0] = SH0;
        if (deg > 0) {
            basis[1] = -SH1 * y;
            basis[2] = SH1 * z;
            basis[3] = -SH1 * x;
            if (deg > 1) {
                const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
                basis[4] = SH2[0] * xy;
                basis[5] = SH2[1] * yz;
                basis[6] = SH2[2] * (2.f * zz - xx - yy);
                basis[7] = SH2[3] * xz;
                basis[8] = SH2[4] * (xx - yy);
                if (deg > 2) {
                    basis[9] = SH3[0] * y * (3.f * xx - yy);
                    basis[10] = SH3[1] * xy * z;
                    basis[11] = SH3[2] * y * (4.f * zz - xx - yy);
                    basis[12] = SH3[3] * z * (2.f * zz - 3.f * xx - 3.f * yy);
                    basis[13] = SH3[4] * x * (4.f * zz - xx - yy);
                    basis[14] = SH3[5] * z * (xx - yy);
                    basis[15] = SH3[6] * x * (xx - 3.f * yy);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) put(j, basis[j]);   // columns 16..63: three full tiles
        // The reference overwrites the ray-direction gradient with the SH term at every hit (backward.cu:165), so
        // only the last composited hit's term survives: remember it, walk_bounce computes it once per bounce.
        if (did) {
            last.g = g;
            last.gc = gc;
            last.any = true;
        }
    }
    if (p.others_precomp != nullptr) {   // the fifth tile only where there are auxiliary channels
#pragma unroll
        for (int ch = 0; ch < AUXM; ++ch) sink.add(kColAux + ch, g_aux_w[ch]);
        sink.finish(RowLayout<AUXM>::cols);
    }
}

// ---- hit record: the forward trace can store every chunk's hit buffer, the backward trace then replays
// them instead of walking the BVH again.  Layout of the caller's buffer, in 8-byte words:
//   [0] blocks requested so far (the forward kernel counts on past the capacity, which is how overflow shows)
//   [1] chains that a replay found broken (stays 0 for a record written by a forward trace with a zeroed header)
//   [2 ...) directory: one uint32 per (wave, bounce slot): low 26 bits = 1 + first block of that wave's bounce (0 =
//           none), high 6 bits = the number of chunks the wave stored for that bounce (what its replay will cost)
//   then `capacity` blocks of kRecBlockWords words: 16x64 entries ([slot][lane]), 64 uint32 counts, next+1, and
//   the colour of every composited hit as the forward evaluated it ([slot][channel][lane] floats; a channel clamped
//   at zero is stored as -0): the replay then neither gathers nor evaluates the 48 SH coefficients per hit again.
constexpr uint32_t kRecDirBlockBits = 26, kRecDirBlockMask = (1u << kRecDirBlockBits) - 1u;
constexpr uint32_t kRecColourWord = kChunk * DST_WAVE + DST_WAVE / 2 + 8;   // first word of the colours
constexpr uint32_t kRecBlockWords = kRecColourWord + kChunk * 3 * DST_WAVE / 2;
struct RecView {
    uint64_t *base;      // nullptr: not recording / not replaying
    uint64_t *blocks;    // first block
    uint32_t *dir;       // this wave's directory entries (one per bounce slot)
    uint32_t capacity;
};

// Forward: append one chunk of this wave to the record.  `prev` is the wave's previous block in this bounce.
// Returns where the chunk's colours go (nullptr: the record is full).
__device__ __forceinline__ float *rec_store(const RecView &rv, int bounce, uint32_t &prev, const KBuf &buf, uint32_t cnt) {
    const uint32_t lane = __lane_id();
    uint32_t blk = 0;
    if (lane == 0) blk = (uint32_t)atomicAdd((unsigned long long *)rv.base, 1ull);
    blk = __builtin_amdgcn_readfirstlane(blk);
    if (blk >= rv.capacity || blk >= kRecDirBlockMask) return nullptr;   // too small: the host sees the count and the backward pass re-traces
    uint64_t *b = rv.blocks + (size_t)blk * kRecBlockWords;
#pragma unroll
    for (int k = 0; k < kChunk; ++k) __builtin_nontemporal_store(buf.e[k], b + k * DST_WAVE + lane);
    uint32_t *cnts = reinterpret_cast<uint32_t *>(b + kChunk * DST_WAVE);
    cnts[lane] = cnt;
    if (lane == 0) {
        cnts[DST_WAVE] = 0u;   // next: none yet
        if (prev == 0xFFFFFFFFu) rv.dir[bounce] = blk + 1u;
        else reinterpret_cast<uint32_t *>(rv.blocks + (size_t)prev * kRecBlockWords + kChunk * DST_WAVE)[DST_WAVE] = blk + 1u;
    }
    prev = blk;
    return reinterpret_cast<float *>(b + kRecColourWord);
}

// Backward: locate the next chunk of this wave's bounce; its entries are then read one slot at a time.
// Returns nullptr when the chain ends early.
__device__ __forceinline__ const uint64_t *rec_open(const RecView &rv, uint32_t &cur, uint32_t &cnt) {
    if (cur == 0u || cur > rv.capacity) return nullptr;
    const uint32_t lane = __lane_id();
    const uint64_t *b = rv.blocks + (size_t)(cur - 1u) * kRecBlockWords;
    const uint32_t *cnts = reinterpret_cast<const uint32_t *>(b + kChunk * DST_WAVE);
    cnt = cnts[lane];
    cur = __builtin_amdgcn_readfirstlane(cnts[DST_WAVE]);
    return b;
}

// Block-wide: write the table to the caller's gradient tensors and empty it.  Consecutive threads take
// consecutive columns of a row, so the 48 SH columns of a surfel go out as contiguous atomics.  The caller
// puts barriers around it.
template <int AUXM, bool DET>
__device__ __forceinline__ void table_flush(const DstParams &p, uint32_t *keys, float *rows) {
    constexpr int stride = RowLayout<AUXM>::stride, n_rows = TableRows<AUXM, DET>::rows;
    for (int k = threadIdx.x; k < n_rows * stride; k += kWavesPerBlock * DST_WAVE) {
        const int row = k / stride, col = k - row * stride;
        const uint32_t g = keys[row];
        if (g == kEmptyKey || col >= RowLayout<AUXM>::cols) continue;
        if (DET) {
            long long *qrows = reinterpret_cast<long long *>(rows);
            const long long q = qrows[k];
            if (q == 0) continue;
            qrows[k] = 0;
            if (column_live<AUXM>(p, col))
                atomicAdd(p.det_workspace + (size_t)g * RowLayout<AUXM>::cols + col, (unsigned long long)q);
        } else {
            const float v = rows[k];
            if (v == 0.f) continue;
            rows[k] = 0.f;
            float *dst = grad_address<AUXM>(p, g, col);
            if (dst != nullptr) aadd(dst, v);
        }
    }
}
template <int AUXM, bool DET>
__device__ __forceinline__ void table_clear_keys(uint32_t *keys) {
    for (int k = threadIdx.x; k <= TableRows<AUXM, DET>::rows; k += kWavesPerBlock * DST_WAVE)
        keys[k] = (k < TableRows<AUXM, DET>::rows) ? kEmptyKey : 0u;
}

// One bounce: chunked 16-nearest traversal + front-to-back compositing (reference forward.cu:136-315),
// and for BWD the per-hit gradients of the re-trace (reference backward.cu:332-655).
// `first_walk` (forward): 0, or the number of steps the packet walk of the bounce's first chunk may take before the
// wave gives its tile up (returns true, nothing written yet: see the tile hand-over in trace_body), or kWalkPerLane:
// every ray of the wave walks on its own whatever the rays look like (the waves that take such tiles over).
// HAND: kernels without the hand-over do not contain its code at all (first_walk is ignored).
constexpr uint32_t kWalkPerLane = 0xFFFFFFFFu;
template <bool BWD, int AUXM, bool REC, bool MIXED, bool DET, bool HAND>
__device__ __forceinline__ bool walk_bounce(const DstParams &p, const DstAccelView &acc, float max_abs, bool lane_on,
                                            F3 ro, F3 rd, float min_depth, BounceAcc<AUXM> &run,
                                            const BounceIn<AUXM> &in, F3 &g_ro, F3 &g_rd, uint32_t &n_proc,
                                            uint32_t &n_con, uint32_t *tab_keys, float *tab_rows, float *stage,
                                            const RecView &rv, int bounce, F3 &dist_acc, uint32_t first_walk
#ifdef DST_STATS
                                            , WaveStats &ws
#endif
) {
    run.C[0] = run.C[1] = run.C[2] = 0.f;
    run.D = 0.f;
    run.N[0] = run.N[1] = run.N[2] = 0.f;
#pragma unroll
    for (int ch = 0; ch < AUXM; ++ch) run.O[ch] = 0.f;
    float pay_dpt = 0.f, dpt = 0.f, Tp = 1.f, Tn = 1.f;
    int last_g = -1, contrib = 0;
    F3 ot = ro;
    bool live = lane_on;
    KBuf buf;
    LastShHit last_sh = {0, f3(0, 0, 0), false};
    STAT(last_sh.t_alg = 0; last_sh.t_sh = 0;)
    // kernels built without the per-lane walk (MIXED false) take every wave as a packet
    const bool as_packet = (!MIXED || (REC && BWD)) ? true
                                                    : (HAND && first_walk == kWalkPerLane ? false : rays_run_together(ro, rd, lane_on, max_abs));
    // Forward: the walks of a bounce's later chunks resume from the list the walk before left (the backward
    // re-trace has its LDS taken by the gradient table and walks from the root).
    constexpr bool RESUME = !BWD;
    // One LDS area per wave serves the packet walk's two lists or the per-lane walk's stack shelf: all chunks of
    // a bounce use the same walk, and a bounce starts without a list.
    constexpr bool SHELF = MIXED && !BWD;
    constexpr uint32_t kListWords = 2u * kListCap;
    constexpr uint32_t kWaveLds = (SHELF && (uint32_t)(kLaneShelf * DST_WAVE) > kListWords) ? (uint32_t)(kLaneShelf * DST_WAVE)
                                                                                            : (RESUME ? kListWords : 1u);
    __shared__ uint32_t s_list[(RESUME || SHELF) ? kFwdWavesPerBlock * kWaveLds : 1];
    uint32_t *const wave_lds = s_list + ((RESUME || SHELF) ? (threadIdx.x / DST_WAVE) * kWaveLds : 0);
    WalkList wl;
    wl.in = (lds_u32)wave_lds;
    wl.out = wl.in + (RESUME ? kListCap : 0);
    wl.n_in = kListFresh;
    wl.record = false;
    wl.limit = (HAND && first_walk != kWalkPerLane) ? first_walk : 0u;
    wl.spent = false;
    uint32_t rec_pos = (REC && BWD) ? (rv.dir[bounce] & kRecDirBlockMask) : 0xFFFFFFFFu;   // replay: next block + 1; record: previous block
    uint32_t rec_chunks = 0u;   // forward with a record: chunks stored for this bounce
    for (;;) {
        // Backward: the four waves of the block take their chunks in step, so that between two rounds nobody
        // touches the gradient table and it can be emptied when it fills up.
        const bool wave_live = wave_ballot(live) != 0ull;
        if (BWD) {
            if (__syncthreads_or(wave_live ? 1 : 0) == 0) break;
        } else if (!wave_live) {
            break;
        }
        if (wave_live) do {
        uint32_t cnt = 0;
        STAT(ws.chunks++; unsigned long long c0 = __builtin_readcyclecounter();)
        // Where the compositing loop below takes its entries from: the recorded block, one slot at a time
        // (backward replay: no buffer registers at all), or the register buffer the traversal just filled.
        const uint64_t *rec_block = nullptr;
        float *rec_colours = nullptr;   // forward with a record: where this chunk's hit colours are kept
        const uint32_t lane_ = __lane_id();
        if (REC && BWD) {
            rec_block = rec_open(rv, rec_pos, cnt);
            if (rec_block == nullptr) {   // cannot happen with a complete record: count it where the caller can see it
                if (lane_ == 0) atomicAdd((unsigned long long *)(rv.base + 1), 1ull);
                live = false;
                break;
            }
        } else {
            kbuf_reset(buf);
            packet_knn<MIXED, SHELF, RESUME, HAND>(acc, max_abs, ot, rd, live, buf, cnt, as_packet, wl, wave_lds WSP);
            if constexpr (HAND) {
                if (wl.spent) return true;   // only a bounce's first walk has a limit: nothing has been written yet
                wl.limit = 0u;
            }
            if (REC && !BWD) {
                rec_colours = rec_store(rv, bounce, rec_pos, buf, cnt);
                rec_chunks += rec_colours != nullptr ? 1u : 0u;
            }
        }
        STAT(unsigned long long c1 = __builtin_readcyclecounter(); ws.t_trav += c1 - c0;)
        int here = 0;
        bool stop = false;
        // Replay runs one step ahead of itself: the entry of step it+1 is fetched while step it evaluates, and its
        // surfel's geometry while step it does its gradient algebra, so a step starts with its operands in registers
        // instead of two dependent trips to memory.
        struct Ahead { uint64_t e; float m[3], s[2], q[4], o, c[3]; } nx = {0ull, {0.f, 0.f, 0.f}, {1.f, 1.f}, {1.f, 0.f, 0.f, 0.f}, 0.f, {0.f, 0.f, 0.f}};
        auto fetch_geometry = [&](bool want) {
            if (!want) return;
            const size_t gn = (size_t)(kb_idx(nx.e) >> 1);
            nx.m[0] = p.means3D[3 * gn]; nx.m[1] = p.means3D[3 * gn + 1]; nx.m[2] = p.means3D[3 * gn + 2];
            nx.s[0] = p.scales[2 * gn]; nx.s[1] = p.scales[2 * gn + 1];
            nx.q[0] = p.rotations[4 * gn]; nx.q[1] = p.rotations[4 * gn + 1];
            nx.q[2] = p.rotations[4 * gn + 2]; nx.q[3] = p.rotations[4 * gn + 3];
            nx.o = p.opacities[gn];
        };
        if (REC && BWD) {
            const bool want = live && cnt > 0u;
            if (want) {
                nx.e = __builtin_nontemporal_load(rec_block + lane_);
                const float *cs = reinterpret_cast<const float *>(rec_block + kRecColourWord) + lane_;
                for (int ch = 0; ch < 3; ++ch) nx.c[ch] = __builtin_nontemporal_load(cs + ch * DST_WAVE);
            }
            fetch_geometry(want);
        }
#pragma unroll 1
        for (int it = 0; it < kChunk; ++it) {
            const bool on = live && !stop && (uint32_t)it < cnt;
            if (wave_ballot(on) == 0ull) break;
            STAT(if (!BWD) { ws.steps++; ws.t_hb += __popcll(wave_ballot(on)); })
            // next entry in depth order (consumed slots need no reset: the buffer is rebuilt for every chunk)
            uint64_t e;
            Ahead cur = nx;
            const bool want_next = (REC && BWD) && live && it + 1 < kChunk && (uint32_t)(it + 1) < cnt;
            if (REC && BWD) {
                e = cur.e;
                if (want_next) {
                    nx.e = __builtin_nontemporal_load(rec_block + (it + 1) * DST_WAVE + lane_);
                    // (the colour slot of an entry that was not composited holds whatever was there: never used)
                    const float *cs = reinterpret_cast<const float *>(rec_block + kRecColourWord) + (it + 1) * 3 * DST_WAVE + lane_;
                    for (int ch = 0; ch < 3; ++ch) nx.c[ch] = __builtin_nontemporal_load(cs + ch * DST_WAVE);
                }
            } else {
                e = buf.e[0];
#pragma unroll
                for (int k = 0; k < kChunk - 1; ++k) buf.e[k] = buf.e[k + 1];
            }
            const float e_t = kb_t(e);
            const uint32_t e_i = kb_idx(e);
            // ---- phase 1 (per lane): evaluate the entry, decide, composite ------------------------------
            bool did = false;          // this lane composited a hit in this iteration
            int g = 0;
            float Tp_hit = 1.f, alpha = 0.f, G = 0.f, w = 0.f, u = 0.f, v = 0.f, sx = 1.f, sy = 1.f, opac = 0.f;
            float nsign = 1.f, q0 = 1.f, q1 = 0.f, q2 = 0.f, q3 = 0.f, dpt_hit = 0.f;
            F3 xyz = f3(0, 0, 0), mean = f3(0, 0, 0), normal = f3(0, 0, 1);
            F3 R[3] = {f3(1, 0, 0), f3(0, 1, 0), f3(0, 0, 1)};
            float col[3] = {0.f, 0.f, 0.f};
            bool neg[3] = {false, false, false};
            const float *sh = p.shs;   // valid address for lanes that sit phase 2 out
            do {
                if (!on) break;
                g = (int)(e_i >> 1);
                if (g == last_g) break;
                dpt = e_t + pay_dpt;
                xyz = f3(ro.x + dpt * rd.x, ro.y + dpt * rd.y, ro.z + dpt * rd.z);
                if (REC && BWD) {
                    mean = f3(cur.m[0], cur.m[1], cur.m[2]);
                    sx = cur.s[0]; sy = cur.s[1];
                    q0 = cur.q[0]; q1 = cur.q[1]; q2 = cur.q[2]; q3 = cur.q[3];
                } else {
                    mean = ld3(p.means3D + 3 * (size_t)g);
                    sx = p.scales[2 * (size_t)g];
                    sy = p.scales[2 * (size_t)g + 1];
                    const float *qp = p.rotations + 4 * (size_t)g;
                    q0 = qp[0]; q1 = qp[1]; q2 = qp[2]; q3 = qp[3];
                }
                quat_rows(q0, q1, q2, q3, R);
                const float Tx = dot(R[0], mean), Ty = dot(R[1], mean);
                const float ux = R[0].x * xyz.x + R[0].y * xyz.y + R[0].z * xyz.z + (-Tx);
                const float uy = R[1].x * xyz.x + R[1].y * xyz.y + R[1].z * xyz.z + (-Ty);
                u = ux / sx;
                v = uy / sy;
                const float rho = u * u + v * v;
                n_proc++;
                normal = R[2];
                const float cosv = -(rd.x * normal.x + rd.y * normal.y + rd.z * normal.z);
                if (cosv == 0.f) break;
                nsign = cosv > 0.f ? 1.0f : -1.0f;
                normal = cosv > 0.f ? normal : -normal;
                if (dpt < min_depth) break;
                const float power = -0.5f * rho;
                if (power > 0.0f) break;
                opac = (REC && BWD) ? cur.o : p.opacities[g];
                G = exp_det(power);
                alpha = opac * G;
                alpha = (alpha < 0.99f) ? alpha : 0.99f;
                if (alpha < 1.0f / 255.0f) break;
                Tn = Tp * (1 - alpha);
                if (Tn < kTmin) { stop = true; break; }
                contrib++;
                if (contrib > kMaxContrib) { stop = true; break; }
                last_g = g;
                w = alpha * Tp;
                if (REC && BWD) {   // as the forward trace evaluated it
#pragma unroll
                    for (int ch = 0; ch < 3; ++ch) {
                        col[ch] = cur.c[ch];
                        // -0: clamped (a colour evaluated from SH is never negative; given colours may be)
                        neg[ch] = p.colors_precomp == nullptr && (__float_as_uint(col[ch]) >> 31) != 0u;
                    }
                } else if (p.colors_precomp == nullptr) {
                    sh = p.shs + (size_t)g * p.M * 3;
                    // (the binary16 source lives in the forward kernels that carry the rarely used options; a backward
                    // trace is given the widened values as shs)
                    const F3 c = (!BWD && DET && (p.flags & DST_FLAG_SH_HALF)) ? sh_color_half(p, g, rd, neg)
                                                                              : sh_color(p.D, ShF32{sh}, rd, neg);
                    col[0] = c.x; col[1] = c.y; col[2] = c.z;
                } else {
                    col[0] = p.colors_precomp[3 * (size_t)g];
                    col[1] = p.colors_precomp[3 * (size_t)g + 1];
                    col[2] = p.colors_precomp[3 * (size_t)g + 2];
                }
                if (REC && !BWD && rec_colours != nullptr) {
                    float *cs = rec_colours + it * 3 * DST_WAVE + lane_;
#pragma unroll
                    for (int ch = 0; ch < 3; ++ch) __builtin_nontemporal_store(neg[ch] ? -0.0f : col[ch], cs + ch * DST_WAVE);
                }
                run.C[0] += w * col[0];
                run.C[1] += w * col[1];
                run.C[2] += w * col[2];
                if (p.others_precomp != nullptr) {
#pragma unroll
                    for (int ch = 0; ch < AUXM; ++ch)
                        if (ch < p.aux) run.O[ch] += w * p.others_precomp[(size_t)p.aux * g + ch];
                }
                if (!BWD && DET && (p.flags & DST_FLAG_DISTORTION)) {
                    // depth distortion of 2DGS with its running moments (x = distortion, y = M1, z = M2); the
                    // reference declares the three and leaves the computation open (forward.cu:286)
                    const float A_before = 1 - Tp;
                    const float m = kFar / (kFar - kNear) * (1 - kNear / dpt);
                    dist_acc.x += (m * m * A_before + dist_acc.z - 2 * m * dist_acc.y) * w;
                    dist_acc.y += m * w;
                    dist_acc.z += m * m * w;
                }
                run.D += w * dpt;
                run.N[0] += w * normal.x;
                run.N[1] += w * normal.y;
                run.N[2] += w * normal.z;
                n_con++;
                here++;
                did = true;
                Tp_hit = Tp;
                dpt_hit = dpt;
                Tp = Tn;
            } while (false);
            if (REC && BWD) fetch_geometry(want_next);
            if (!BWD && p.training && p.a_weights != nullptr) {
                if (!MIXED && !DET) wet_add(tab_keys, tab_rows, p.a_weights, did, (uint32_t)g, w);   // the wave's LDS table
                else wave_add_grouped(p.a_weights, (DET && (p.flags & DST_FLAG_DETERMINISTIC)) ? p.det_workspace : nullptr, did,
                                      (uint32_t)g, w);
            }
            // ---- phase 2 (whole wave, backward only): gradients of the hits composited above -----------
            if (BWD && wave_ballot(did) != 0ull) {
                GradSink<AUXM, DET> sink;
                sink.p = &p;
                sink.rows = tab_rows;
                sink.stage = stage;
                sink.did = did;
                sink.g = (uint32_t)g;
                sink.limit = RowLayout<AUXM>::cols;   // dead columns (no SH, no aux) are never staged
                STAT(unsigned long long d0 = __builtin_readcyclecounter();)
                sink.plan(tab_keys);
                STAT(last_sh.t0 = __builtin_readcyclecounter();)
                STAT(unsigned long long d1 = __builtin_readcyclecounter(); ws.t_plan += d1 - d0; ws.steps++;
                     ws.leaf_any += __popcll(wave_ballot(did));)
                hit_backward<AUXM, DET>(p, in, run, did ? g : 0, e_i, Tp_hit, alpha, G, w, dpt_hit, xyz, R, u, v, sx, sy, mean,
                                   q0, q1, q2, q3, opac, nsign, normal, col, neg, ro, rd, sh, g_ro, g_rd, sink, did, last_sh);
                STAT(ws.t_hb += __builtin_readcyclecounter() - d1;)
            }
        }
        STAT(ws.t_comp += __builtin_readcyclecounter() - c1;)
        if (live) {
            bool fin = (Tn < kTmin) || (cnt < (uint32_t)kChunk) || (contrib > kMaxContrib);
            const float next_dpt = (float)((double)dpt + kStepEps);
            if (!(next_dpt > pay_dpt) && here == 0) fin = true;   // the reference would never leave this state
            if (fin) {
                live = false;
            } else {
                pay_dpt = next_dpt;
                ot = f3(ro.x + pay_dpt * rd.x, ro.y + pay_dpt * rd.y, ro.z + pay_dpt * rd.z);
            }
        }
        } while (false);
        if (BWD) {
            __syncthreads();   // every wave's additions of this round are in the table
            if (tab_keys[TableRows<AUXM, DET>::rows] > (uint32_t)(DST_TABLE_FLUSH_NUM * TableRows<AUXM, DET>::rows / 8)) {
                table_flush<AUXM, DET>(p, tab_keys, tab_rows);
                __syncthreads();
                table_clear_keys<AUXM, DET>(tab_keys);   // the barrier at the top of the next round publishes it
            }
        }
    }
    if (REC && !BWD && rec_chunks != 0u && __lane_id() == 0u)   // the replay's cost of this wave and bounce, for its launcher
        rv.dir[bounce] = (rv.dir[bounce] & kRecDirBlockMask) | (min(rec_chunks, 63u) << kRecDirBlockBits);
    STAT(if (BWD) { ws.nodes += last_sh.t_alg; ws.leaves += last_sh.t_sh; })
    if (BWD && p.colors_precomp == nullptr && last_sh.any)
        g_rd = sh_direction_gradient(p.D, ShF32{p.shs + (size_t)last_sh.g * p.M * 3}, rd, last_sh.gc);
    run.T = Tp;
    return false;
}

__device__ __forceinline__ F3 dnormvdv(F3 v, F3 dv) {
    float sum2 = v.x * v.x + v.y * v.y + v.z * v.z;
    float inv = 1.0f / __builtin_sqrtf(sum2 * sum2 * sum2);
    return f3(((+sum2 - v.x * v.x) * dv.x - v.y * v.x * dv.y - v.z * v.x * dv.z) * inv,
              (-v.x * v.y * dv.x + (sum2 - v.y * v.y) * dv.y - v.z * v.y * dv.z) * inv,
              (-v.x * v.z * dv.x - v.y * v.z * dv.y + (sum2 - v.z * v.z) * dv.z) * inv);
}
__device__ __forceinline__ F3 ddotndndn(F3 n, F3 d, F3 g) {
    float nd = dot(n, d);
    return f3(g.x * (nd + d.x * n.x) + g.y * d.x * n.y + g.z * d.x * n.z,
              g.x * d.y * n.x + g.y * (nd + d.y * n.y) + g.z * d.y * n.z,
              g.x * d.z * n.x + g.y * d.z * n.y + g.z * (nd + d.z * n.z));
}
__device__ __forceinline__ F3 ddotndndd(F3 n, F3 g) {
    return f3(g.x * n.x * n.x + g.y * n.x * n.y + g.z * n.x * n.z, g.x * n.y * n.x + g.y * n.y * n.y + g.z * n.y * n.z,
              g.x * n.z * n.x + g.y * n.z * n.y + g.z * n.z * n.z);
}

__device__ __forceinline__ uint32_t wave_sum(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// Position j in the dispatch order of an image grid -> block (bx, by): column strips `strip` blocks wide, row by row
// inside a strip (strip 0 or a ray list: row-major).  See trace_body for why.
__device__ __forceinline__ void block_of_position(uint32_t j, uint32_t btiles_x, uint32_t rows, uint32_t strip_width,
                                                  bool image, uint32_t &bx, uint32_t &by) {
    bx = j % btiles_x;
    by = j / btiles_x;
    if (strip_width != 0u && image) {
        const uint32_t per_strip = strip_width * rows, strip = j / per_strip, r = j % per_strip;
        if (strip * strip_width < btiles_x) {   // (positions past the grid keep the row-major numbers: their blocks leave)
            const uint32_t w = min(strip_width, btiles_x - strip * strip_width);
            bx = strip * strip_width + r % w;
            by = r / w;
        }
    }
}

// Order of the blocks of a replaying backward trace: longest first.  The forward trace left in the record's directory
// how many chunks every wave stored (what its replay costs); a block takes as long as the longest of its four waves
// (they take their chunks in step).  With the long blocks first, the chip runs out of work with short blocks, not
// with one long block per CU still going.  One workgroup: a counting sort over 64 cost classes, positions taken
// 1024 at a time so that blocks of equal cost keep their neighbourhood.
__global__ __launch_bounds__(1024) void k_block_order(const uint32_t *__restrict__ dir, uint32_t slots, uint32_t btiles_x,
                                                     uint32_t rows, uint32_t strip_width, int image, uint32_t n_blocks,
                                                     uint32_t *__restrict__ order) {
    __shared__ uint32_t s_count[64], s_base[64];
    auto cost_class = [&](uint32_t j) -> uint32_t {   // 0 = the most expensive
        uint32_t bx, by;
        block_of_position(j, btiles_x, rows, strip_width, image != 0, bx, by);
        if (by >= rows) return 63u;
        const uint32_t *d = dir + (size_t)(by * btiles_x + bx) * kWavesPerBlock * slots;
        uint32_t worst = 0u;
        for (uint32_t w = 0; w < (uint32_t)kWavesPerBlock; ++w) {
            uint32_t sum = 0u;
            for (uint32_t k = 0; k < slots; ++k) sum += d[w * slots + k] >> kRecDirBlockBits;
            worst = max(worst, sum);
        }
        return 63u - min(worst, 63u);
    };
    constexpr uint32_t kKept = 32768;   // classes of the first pass kept in LDS for the second (grids up to this size)
    __shared__ uint8_t s_class[kKept];
    if (threadIdx.x < 64) s_count[threadIdx.x] = 0u;
    __syncthreads();
    for (uint32_t j = threadIdx.x; j < n_blocks; j += blockDim.x) {
        const uint32_t c = cost_class(j);
        if (j < kKept) s_class[j] = (uint8_t)c;
        atomicAdd(&s_count[c], 1u);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t run = 0u;
        for (int c = 0; c < 64; ++c) {
            s_base[c] = run;
            run += s_count[c];
        }
    }
    __syncthreads();
    for (uint32_t base = 0; base < n_blocks; base += blockDim.x) {   // in order, 1024 positions at a time
        const uint32_t j = base + threadIdx.x;
        if (j < n_blocks) order[atomicAdd(&s_base[j < kKept ? (uint32_t)s_class[j] : cost_class(j)], 1u)] = j;
        __syncthreads();
    }
}

// Tile hand-over (forward).  A packet walk visits what any of its 64 rays needs, one dependent fetch after the other.
// Over geometry much finer than the ray spacing (a dense cloud of surfels far smaller than a pixel) that is the whole
// content of the tile's frustum, wanted by one ray at best, and a single wave walks for milliseconds while the chip
// idles.  So the first walk of a tile may take `hand_arg` steps and no more: a wave that runs into that limit has
// written nothing yet, puts its tile on the context's list and leaves, and a second, small launch right behind
// (kernels with the per-lane walk, hand_arg = 0: the takers) traces the listed tiles with every ray walking on its
// own - the same buffer content, so the same results bit for bit.  List: word 0 = tiles listed by this trace, word 1 =
// takers that have read their entry (the last one empties the list for the next trace: nothing on the host changes
// from call to call, so a captured launch pair can be replayed), word 2 = tiles handed over since the context was
// made, word 3 = not the list's: sums of the deterministic mode found out of range (its closing kernels count there),
// entries ((by * btiles_x + bx) * 4 + wave) from word 4.  A wave that finds the list full starts again without a limit.
constexpr uint32_t kHandHeader = kDstHandoverHeader, kHandCap = kDstHandoverCap;
template <bool BWD, int AUXM, bool REC, bool MIXED, bool DET, bool HAND>
__device__ __forceinline__ void trace_body(const DstParams &p, const DstAccelView &acc, int tw_log2, int th_log2,
                                           uint32_t tiles_x, uint32_t tiles_y, uint32_t btiles_x,
                                           const uint32_t *__restrict__ ray_order, uint32_t strip_width,
                                           const uint32_t *__restrict__ block_order, uint32_t *handover,
                                           uint32_t hand_arg) {
    // a block = 2x2 wave tiles (16x16 pixels for the usual 8x8 tile): neighbouring rays share surfels, which
    // is what the block's gradient table and the caches live on
    constexpr int kTableRows = RowLayout<AUXM>::rows;
    __shared__ uint32_t s_keys[BWD ? kTableRows + 1 : 1];   // + the count of claimed rows
    __shared__ __attribute__((aligned(8))) float s_rows[BWD ? kTableRows * RowLayout<AUXM>::stride : 1];   // DET: half the rows, 8 bytes each
    __shared__ float s_stage[BWD ? kWavesPerBlock * kStageWords : 1];
    uint32_t *tab_keys = s_keys;
    float *tab_rows = s_rows;
    // forward of an image at depth 0: the wave's table of blending weights (wet_add; in the kernels that carry the
    // per-lane walk it measured no gain and would take the LDS to the limit of 16 waves per CU)
    constexpr bool WET = !BWD && !MIXED && !DET;
    __shared__ uint32_t s_wet_keys[WET ? kFwdWavesPerBlock * kWetSlots : 1];
    __shared__ float s_wet_vals[WET ? kFwdWavesPerBlock * kWetSlots : 1];
    uint32_t *const wet_keys = s_wet_keys + (WET ? (threadIdx.x / DST_WAVE) * kWetSlots : 0);
    float *const wet_vals = s_wet_vals + (WET ? (threadIdx.x / DST_WAVE) * kWetSlots : 0);
    if (WET) {   // (a wave's LDS accesses keep their order: no barrier between this and the first use)
        for (int e = threadIdx.x % DST_WAVE; e < kWetSlots; e += DST_WAVE) {
            wet_keys[e] = 0xFFFFFFFFu;
            wet_vals[e] = 0.f;
        }
    }
    // Backward with a hit record: the launcher starts the replaying kernel and the re-tracing kernel one after
    // the other, and word 0 of the record (blocks the forward trace asked for) decides on the device which of
    // the two does the work: the host never has to wait for the forward trace to learn whether its record is complete.
    if (BWD && p.hit_record != nullptr) {
        const bool complete = p.hit_record[0] <= (uint64_t)p.hit_record_blocks;
        if (REC != complete) return;
    }
    if (BWD) {
        table_clear_keys<AUXM, DET>(s_keys);
        for (int k = threadIdx.x; k < kTableRows * RowLayout<AUXM>::stride; k += kWavesPerBlock * DST_WAVE)
            s_rows[k] = 0.f;
        __syncthreads();
    }
    // Backward: a block is the four waves of a 16x16 pixel tile (they share the gradient table).  Forward: the
    // waves share nothing, so each is a workgroup of its own and takes a free wave slot as soon as there is
    // one; workgroups x, x+8, x+16, x+24 (same XCD under round-robin dispatch) are the four waves of a tile.
    uint32_t bid = blockIdx.x, wv = threadIdx.x / DST_WAVE;
    if (!BWD && kFwdWavesPerBlock == 1) {
        bid = (blockIdx.x >> 5) * 8u + (blockIdx.x & 7u);
        wv = (blockIdx.x >> 3) & 3u;
    }
    // (Measured slower than the strips below, on the 1080p room scene: a band or whole rows of the image per XCD,
    // +15 % / +8 % forward - eight distant image regions in flight, eight times more distinct BVH data in the shared
    // last-level cache - and compact patches of 2x4 to 8x16 blocks per XCD inside super-tiles, +1 % to +13 %.)
    // Image grids are walked in column strips eight blocks wide, row by row inside a strip.  Workgroups go to the
    // eight XCDs in turn, so in a full strip XCD q works its way down column q: the tiles an XCD has in flight are
    // vertical neighbours and meet the same BVH nodes in that XCD's own L2 (row-major order over a 120-block-wide image
    // gave an XCD blocks eight columns apart: forward 8.5 -> 8.1 ms on the 1080p room scene).  The last strip may be
    // narrower; its blocks are spread over all XCDs like the others.  The launcher chooses the width (launch()).
    if (BWD && block_order != nullptr) bid = block_order[bid];   // replay: the longest blocks first (k_block_order)
    uint32_t bx, by;
    static_assert(!HAND || (!BWD && kFwdWavesPerBlock == 1), "tiles are handed over by forward kernels of one wave per workgroup");
    const bool taker = HAND && MIXED && handover != nullptr && hand_arg == 0u;
    block_of_position(bid, btiles_x, (tiles_y + 1u) / 2u, strip_width, th_log2 != 0, bx, by);
    if constexpr (HAND) {
        if (taker) {   // the tile comes from the list, not from the workgroup's number
            const uint32_t n = min(handover[0], gridDim.x);
            const uint32_t id = handover[kHandHeader + min(blockIdx.x, kHandCap - 1u)];
            wv = id & 3u;
            bx = (id >> 2) % btiles_x;
            by = (id >> 2) / btiles_x;
            // Every taker has read the count and its entry before it is counted itself (the fence keeps the reads in front
            // of the ticket), and no wave writes the list while takers run: the last one counted empties it.
            __threadfence();
            if (threadIdx.x == 0u) {
                const uint32_t ticket = atomicAdd(&handover[1], 1u);
                if (ticket == gridDim.x - 1u) {
                    handover[2] += n;
                    handover[1] = 0u;
                    handover[0] = 0u;
                }
            }
            if (blockIdx.x >= n) return;
        }
    }
    const bool flat = th_log2 == 0;   // a ray list: tiles of 1x64 rays, a block = four consecutive tiles
    if (flat ? by >= 1u : 2u * by >= tiles_y) return;   // padding of the forward grid (whole blocks)
    RecView rv = {nullptr, nullptr, nullptr, 0u};
    if (REC) {
        const uint32_t n_waves = btiles_x * ((tiles_y + 1u) / 2u) * kWavesPerBlock, slots_ = (uint32_t)p.mtd_alloc + 1u;
        const uint64_t dir_words = ((uint64_t)n_waves * slots_ + 1u) / 2u;
        rv.base = p.hit_record;
        rv.dir = reinterpret_cast<uint32_t *>(p.hit_record + 2) + (size_t)((by * btiles_x + bx) * kWavesPerBlock + wv) * slots_;
        rv.blocks = p.hit_record + 2 + dir_words;
        rv.capacity = p.hit_record_blocks;
    }
    const uint32_t ty = flat ? 0u : 2u * by + (wv >> 1), tx = flat ? 4u * bx + wv : 2u * bx + (wv & 1u);
    const bool wave_on = ty < tiles_y && tx < tiles_x;
    if (!BWD && !wave_on) return;   // the backward kernel keeps every wave for the block-wide flush below
    const uint32_t lane = threadIdx.x % DST_WAVE;
    const uint32_t py = (ty << th_log2) + (lane >> tw_log2);
    const uint32_t px = (tx << tw_log2) + (lane & ((1u << tw_log2) - 1u));
    const bool inside = wave_on && py < (uint32_t)p.H && px < (uint32_t)p.W;
    // ray lists are traced in a coherent order (see k_ray_keys): position in that order -> ray number
    const size_t pos = inside ? ((size_t)py * p.W + px) : 0;
    // (forward: ray lists always run the MIXED kernels, so the image kernels need not look at the order)
    const size_t r = ((MIXED || BWD) && ray_order != nullptr && inside) ? (size_t)ray_order[pos] : pos;
    const float max_abs = __uint_as_float(acc.bounds->scale);   // the size origins are compared with (rays_run_together)
    const int MID = 14 + p.aux, AUXO = 11, RGBO = 11 + p.aux;
    const int slots = p.mtd_alloc + 1, mtd = p.max_trace_depth;
    float *mid = p.mid_val + (size_t)slots * MID * r;
    const F3 ray_o = ld3(p.ray_o + 3 * r), ray_d = ld3(p.ray_d + 3 * r);
    uint32_t n_proc = 0, n_con = 0;
#ifdef DST_STATS
    WaveStats ws = {0, 0, 0, 0, 0, 0, 0, 0, 0};
#define WS_ARG , ws
#else
#define WS_ARG
#endif
    BounceAcc<AUXM> run;
    BounceIn<AUXM> in;
    F3 g_ro = f3(0, 0, 0), g_rd = f3(0, 0, 0);

    if (!BWD) {
        // reference forward.cu:318-424
        float out_rgb[3] = {0.f, 0.f, 0.f};
        F3 ot = ray_o, dt = ray_d;
        float s_prod = 1.0f;
        bool on = inside;
        uint32_t first_walk = (HAND && handover != nullptr) ? hand_arg : 0u;
        for (int i = 0; i <= mtd; ++i) {
            const float min_depth = (i == 0) ? (p.start_from_first ? kNear : 0.0f) : kStartOffset;
            F3 dist_acc = f3(0, 0, 0);
            const bool gave_up = walk_bounce<false, AUXM, REC, MIXED, DET, HAND>(p, acc, max_abs, on, ot, dt, min_depth, run, in, g_ro, g_rd, n_proc, n_con, WET ? wet_keys : nullptr, WET ? wet_vals : nullptr, nullptr, rv, i, dist_acc, taker ? kWalkPerLane : (i == 0 ? first_walk : 0u) WS_ARG);
            if constexpr (HAND) if (gave_up) {   // (bounce 0, before anything was written; no else below)
                uint32_t slot = 0u;
                if (lane == 0u) slot = atomicAdd(&handover[0], 1u);
                slot = __builtin_amdgcn_readfirstlane(slot);
                if (slot < kHandCap) {
                    if (lane == 0u) handover[kHandHeader + slot] = ((by * btiles_x + bx) << 2) | wv;
                    return;
                }
                first_walk = 0u;   // the list is full: this wave keeps its tile
                --i;
                continue;
            }
            if (on) {
                run.C[0] += run.T * p.background[0];
                run.C[1] += run.T * p.background[1];
                run.C[2] += run.T * p.background[2];
                const float A = 1 - run.T;
                const F3 E = f3(ot.x + run.D * dt.x, ot.y + run.D * dt.y, ot.z + run.D * dt.z);
                if (i == 0) {
                    p.out_dpt[r] = run.D;
                    p.out_acc[r] = A;
                    p.out_norm[3 * r + 0] = run.N[0];
                    p.out_norm[3 * r + 1] = run.N[1];
                    p.out_norm[3 * r + 2] = run.N[2];
                    p.out_dist[3 * r + 0] = dist_acc.x;   // zeros unless DST_FLAG_DISTORTION (as the reference)
                    p.out_dist[3 * r + 1] = dist_acc.y;
                    p.out_dist[3 * r + 2] = dist_acc.z;
#pragma unroll
                    for (int ch = 0; ch < AUXM; ++ch)
                        if (ch < p.aux) p.out_aux[(size_t)p.aux * r + ch] = run.O[ch];
                }
                const float f_this = (i == mtd) ? 1.0f : 1 - run.O[0];
                out_rgb[0] += run.C[0] * f_this * s_prod;
                out_rgb[1] += run.C[1] * f_this * s_prod;
                out_rgb[2] += run.C[2] * f_this * s_prod;
                s_prod *= run.O[0];
                float *m = mid + (size_t)i * MID;
                m[0] = ot.x; m[1] = ot.y; m[2] = ot.z;
                m[3] = dt.x; m[4] = dt.y; m[5] = dt.z;
                m[6] = run.D;
                m[7] = A;
                m[8] = run.N[0]; m[9] = run.N[1]; m[10] = run.N[2];
#pragma unroll
                for (int ch = 0; ch < AUXM; ++ch)
                    if (ch < p.aux) m[AUXO + ch] = run.O[ch];
                m[RGBO + 0] = run.C[0];
                m[RGBO + 1] = run.C[1];
                m[RGBO + 2] = run.C[2];
                const F3 N = f3(run.N[0], run.N[1], run.N[2]);
                const float nl = length(N);
                if (nl == 0.0f || run.O[0] <= p.specular_threshold) {
                    on = false;
                    // slots of the bounces never traced read as zeros
                    for (int k = (i + 1) * MID; k < slots * MID; ++k) mid[k] = 0.f;
                } else {
                    const F3 n = N / nl;
                    dt = dt - 2 * dot(n, dt) * n;
                    ot = E + kStartOffset * dt;
                }
            }
        }
        if (inside) {
            if (on)
                for (int k = (mtd + 1) * MID; k < slots * MID; ++k) mid[k] = 0.f;
            p.out_rgb[3 * r + 0] = out_rgb[0];
            p.out_rgb[3 * r + 1] = out_rgb[1];
            p.out_rgb[3 * r + 2] = out_rgb[2];
        }
        if (WET && p.training && p.a_weights != nullptr) {   // the wave's blending weights: one addition per surfel
            for (int e = (int)lane; e < kWetSlots; e += DST_WAVE) {
                const uint32_t k = wet_keys[e];
                const float v = wet_vals[e];
                if (k != 0xFFFFFFFFu && v != 0.f) aadd(p.a_weights + k, v);
            }
        }
        if (p.counters != nullptr) {
            uint32_t a = wave_sum(n_proc), b = wave_sum(n_con);
            if (lane == 0) {
                atomicAdd(p.counters + 0, (unsigned long long)a);
                atomicAdd(p.counters + 1, (unsigned long long)b);
#ifdef DST_STATS   // development build only: counters must then hold 8 entries
                atomicAdd(p.counters + 2, ws.nodes);
                atomicAdd(p.counters + 3, ws.leaves);
                atomicAdd(p.counters + 4, ws.t_trav);
                atomicAdd(p.counters + 5, ws.t_comp);
                atomicAdd(p.counters + 6, ws.chunks);
                atomicAdd(p.counters + 7, ws.leaf_any);
                atomicAdd(p.counters + 8, ws.t_plan);   // exact quad tests run (forward only)
                atomicAdd(p.counters + 9, ws.steps);    // compositing iterations of the wave
                atomicAdd(p.counters + 10, ws.t_hb);    // lanes with an entry, summed over those iterations
#endif
            }
        }
    } else {
        // reference backward.cu:658-853
        float C_prev[3], c_prev[3] = {0.f, 0.f, 0.f}, g_out_rgb[3];
        for (int ch = 0; ch < 3; ++ch) {
            C_prev[ch] = p.out_rgb[3 * r + ch];
            g_out_rgb[ch] = p.dL_drgb[3 * r + ch];
        }
        float s_prod = 1.0f;
        for (int i = 0; i < mtd; ++i) {
            for (int ch = 0; ch < 3; ++ch) {
                float c_curr = mid[ch + RGBO + i * MID];
                C_prev[ch] = C_prev[ch] + s_prod * (c_prev[ch] - c_curr);
                c_prev[ch] = c_curr;
            }
            s_prod *= mid[AUXO + i * MID];
        }
        for (int i = mtd; i >= 0; --i) {
            const float *m = mid + (size_t)i * MID;
            const F3 ot = ld3(m), dt = ld3(m + 3);
            const float s_prev = (i > 0) ? mid[AUXO + (i - 1) * MID] : 1.0f;
            const bool on = inside && !(length(dt) == 0.0f || s_prev <= p.specular_threshold);
            if (on) {
                for (int ch = 0; ch < 3; ++ch) in.rgb[ch] = m[RGBO + ch];
                in.dpt = m[6];
                in.acc = m[7];
                in.nrm[0] = m[8]; in.nrm[1] = m[9]; in.nrm[2] = m[10];
#pragma unroll
                for (int ch = 0; ch < AUXM; ++ch) {
                    in.aux[ch] = (ch < p.aux) ? m[AUXO + ch] : 0.f;
                    in.g_aux[ch] = 0.f;
                }
                in.g_dpt = 0.f;
                in.g_acc = 0.f;
                in.g_nrm[0] = in.g_nrm[1] = in.g_nrm[2] = 0.f;
                const float f_this = (i == mtd) ? 1.0f : 1 - in.aux[0];
                for (int ch = 0; ch < 3; ++ch) in.g_rgb[ch] = g_out_rgb[ch] * f_this * s_prod;
                s_prod /= s_prev;
                if (i != mtd) {
                    for (int ch = 0; ch < 3; ++ch) {
                        in.g_aux[0] += g_out_rgb[ch] * (C_prev[ch] / in.aux[0]);
                        c_prev[ch] = (i > 0) ? mid[ch + RGBO + (i - 1) * MID] : 0.0f;
                        C_prev[ch] = C_prev[ch] - s_prod * (c_prev[ch] - in.rgb[ch]);
                    }
                    const F3 nrm = f3(in.nrm[0], in.nrm[1], in.nrm[2]);
                    const float nl = length(nrm);
                    if (nl != 0.f) {
                        g_rd = g_rd + g_ro * (float)kStepEps;
                        const F3 n = nrm / nl;
                        in.g_dpt += g_ro.x * dt.x + g_ro.y * dt.y + g_ro.z * dt.z;
                        const F3 gn = dnormvdv(nrm, ddotndndn(n, dt, g_rd * -2.0f));
                        in.g_nrm[0] += gn.x;
                        in.g_nrm[1] += gn.y;
                        in.g_nrm[2] += gn.z;
                        g_rd = g_ro * in.dpt + g_rd + ddotndndd(n, g_rd * -2.0f);
                    }
                }
                if (i == 0) {
                    in.g_dpt += p.dL_ddpt[r];
                    in.g_acc += p.dL_dacc[r];
                    in.g_nrm[0] += p.dL_dnorm[3 * r + 0];
                    in.g_nrm[1] += p.dL_dnorm[3 * r + 1];
                    in.g_nrm[2] += p.dL_dnorm[3 * r + 2];
#pragma unroll
                    for (int ch = 0; ch < AUXM; ++ch)
                        if (ch < p.aux) in.g_aux[ch] += p.dL_daux[(size_t)p.aux * r + ch];
                }
            }
            const float min_depth = (i == 0) ? (p.start_from_first ? kNear : 0.0f) : kStartOffset;
            F3 no_dist = f3(0, 0, 0);
            (void)walk_bounce<true, AUXM, REC, MIXED, DET, false>(p, acc, max_abs, on, ot, dt, min_depth, run, in, g_ro, g_rd, n_proc, n_con, tab_keys, tab_rows, s_stage + wv * kStageWords, rv, i, no_dist, 0u WS_ARG);
        }
#ifdef DST_STATS   // development build only: counters must then hold 11 entries
        if (p.counters != nullptr && lane == 0) {
            atomicAdd(p.counters + 2, ws.steps);
            atomicAdd(p.counters + 3, ws.t_plan);
            atomicAdd(p.counters + 4, ws.t_trav);
            atomicAdd(p.counters + 5, ws.t_comp);
            atomicAdd(p.counters + 6, ws.chunks);
            atomicAdd(p.counters + 7, ws.t_hb);
            atomicAdd(p.counters + 8, ws.nodes);
            atomicAdd(p.counters + 9, ws.leaves);
            atomicAdd(p.counters + 10, ws.leaf_any);
        }
#endif
        if (inside) {
            p.dL_dray_o[3 * r + 0] = g_ro.x; p.dL_dray_o[3 * r + 1] = g_ro.y; p.dL_dray_o[3 * r + 2] = g_ro.z;
            p.dL_dray_d[3 * r + 0] = g_rd.x; p.dL_dray_d[3 * r + 1] = g_rd.y; p.dL_dray_d[3 * r + 2] = g_rd.z;
        }
        __syncthreads();
        table_flush<AUXM, DET>(p, s_keys, s_rows);
    }
}

// The two entry kernels differ only in the occupancy the register allocator is told to aim for: both are
// bound by the latency of dependent fetches, so waves in flight matter more than a few spilled values.
#ifndef DST_FWD_WAVES
#define DST_FWD_WAVES 4
#endif
#ifndef DST_BWD_WAVES
#define DST_BWD_WAVES 3
#endif
// EXTRAS: the rarely used forward options (DstParams.flags: fixed-point blending weights, distortion output) live in
// a kernel of their own, so that the usual one does not carry their registers.
template <int AUXM, bool REC, bool MIXED, bool EXTRAS>
__global__ __launch_bounds__(kFwdWavesPerBlock *DST_WAVE) __attribute__((amdgpu_waves_per_eu(DST_FWD_WAVES, DST_FWD_WAVES)))
void k_trace_fwd(const DstParams p, const DstAccelView acc, int tw_log2, int th_log2, uint32_t tiles_x,
                 uint32_t tiles_y, uint32_t btiles_x, const uint32_t *ray_order, uint32_t strip_width, uint32_t *handover,
                 uint32_t hand_arg) {
    trace_body<false, AUXM, REC, MIXED, EXTRAS, kFwdWavesPerBlock == 1>(p, acc, tw_log2, th_log2, tiles_x, tiles_y, btiles_x, ray_order, strip_width, nullptr, handover, hand_arg);
}
// The forward kernel of image grids at depth 0 without the tile hand-over: what scenes without many small quads are
// traced with (the hand-over's few extra live values cost the walk 1 to 4 % of its time through the register
// allocation, whether a tile is ever handed over or not).
template <int AUXM, bool REC>
__global__ __launch_bounds__(kFwdWavesPerBlock *DST_WAVE) __attribute__((amdgpu_waves_per_eu(DST_FWD_WAVES, DST_FWD_WAVES)))
void k_trace_fwd_plain(const DstParams p, const DstAccelView acc, int tw_log2, int th_log2, uint32_t tiles_x,
                       uint32_t tiles_y, uint32_t btiles_x, const uint32_t *ray_order, uint32_t strip_width) {
    trace_body<false, AUXM, REC, false, false, false>(p, acc, tw_log2, th_log2, tiles_x, tiles_y, btiles_x, ray_order, strip_width, nullptr, nullptr, 0u);
}
template <int AUXM, bool REC, bool MIXED, bool DET>
__global__ __launch_bounds__(kWavesPerBlock *DST_WAVE) __attribute__((amdgpu_waves_per_eu(DST_BWD_WAVES, DST_BWD_WAVES)))
void k_trace_bwd(const DstParams p, const DstAccelView acc, int tw_log2, int th_log2, uint32_t tiles_x,
                 uint32_t tiles_y, uint32_t btiles_x, const uint32_t *ray_order, uint32_t strip_width,
                 const uint32_t *block_order) {
    trace_body<true, AUXM, REC, MIXED, DET, false>(p, acc, tw_log2, th_log2, tiles_x, tiles_y, btiles_x, ray_order, strip_width, block_order, nullptr, 0u);
}

// Closing kernels of the deterministic mode: fixed point -> fp32, added to the caller's (zero-filled) tensors.
template <int AUXM>
__global__ void k_det_finish_grads(const DstParams p, uint32_t *out_of_range) {
    constexpr int cols = RowLayout<AUXM>::cols;
    const size_t n = (size_t)p.P * cols;
    for (size_t k = (size_t)blockIdx.x * blockDim.x + threadIdx.x; k < n; k += (size_t)gridDim.x * blockDim.x) {
        const long long q = (long long)p.det_workspace[k];
        if (q == 0) continue;
        if (det_out_of_range(q)) atomicAdd(out_of_range, 1u);
        const uint32_t g = (uint32_t)(k / cols);
        const int col = (int)(k - (size_t)g * cols);
        float *dst = tensor_address<AUXM>(p, g, col);
        if (dst != nullptr) *dst += from_fixed(q, det_shift(col));
    }
}
// Closing kernel of a backward trace with gradient rows: rows -> the caller's tensors.
template <int AUXM>
__global__ void k_finish_grad_rows(const DstParams p) {
    constexpr int cols = RowLayout<AUXM>::cols;
    const size_t n = (size_t)p.P * cols;
    for (size_t k = (size_t)blockIdx.x * blockDim.x + threadIdx.x; k < n; k += (size_t)gridDim.x * blockDim.x) {
        const float v = p.grad_rows[k];
        if (v == 0.f) continue;
        const uint32_t g = (uint32_t)(k / cols);
        const int col = (int)(k - (size_t)g * cols);
        float *dst = tensor_address<AUXM>(p, g, col);
        if (dst != nullptr) *dst += v;
    }
}
__global__ void k_det_finish_weights(const DstParams p, uint32_t *out_of_range) {
    for (int g = blockIdx.x * blockDim.x + threadIdx.x; g < p.P; g += gridDim.x * blockDim.x) {
        const long long q = (long long)p.det_workspace[g];
        if (q != 0) p.a_weights[g] += from_fixed(q, kDetShiftOther);
        if (det_out_of_range(q)) atomicAdd(out_of_range, 1u);
    }
}

// Sort key of a ray of a ray list, so that the 64 rays of a wave run side by side: the cell of the origin on a
// 32^3 grid over the scene (15 bits), then the direction as a Morton code of its octahedral map (2 x 8 bits).
// Rays that cannot be keyed (NaN, zero direction) get key 0.
__global__ void k_ray_keys(const float *__restrict__ ray_o, const float *__restrict__ ray_d, const DstBounds *bounds,
                           uint32_t *__restrict__ keys, uint32_t *__restrict__ vals, uint32_t n) {
    const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= n) return;
    const float ext = __uint_as_float(bounds->scale);
    const float inv = ext > 0.f ? 16.0f / ext : 0.f;
    uint32_t cell = 0u, dir = 0u;
    float d[3], l1 = 0.f;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        const float c = fminf(fmaxf(ray_o[3 * (size_t)r + a] * inv + 16.0f, 0.f), 31.f);   // NaN -> 0
        cell = (cell << 5) | (uint32_t)c;
        d[a] = ray_d[3 * (size_t)r + a];
        l1 += fabsf(d[a]);
    }
    if (l1 > 0.f && l1 < INFINITY) {
        float u = d[0] / l1, v = d[1] / l1;
        if (d[2] < 0.f) {   // fold the lower hemisphere over the square's corners
            const float fu = (1.f - fabsf(v)) * (u >= 0.f ? 1.f : -1.f), fv = (1.f - fabsf(u)) * (v >= 0.f ? 1.f : -1.f);
            u = fu;
            v = fv;
        }
        uint32_t qu = (uint32_t)fminf(fmaxf((u * 0.5f + 0.5f) * 256.f, 0.f), 255.f);
        uint32_t qv = (uint32_t)fminf(fmaxf((v * 0.5f + 0.5f) * 256.f, 0.f), 255.f);
        auto spread8 = [](uint32_t x) {
            x = (x | (x << 4)) & 0x0F0Fu;
            x = (x | (x << 2)) & 0x3333u;
            x = (x | (x << 1)) & 0x5555u;
            return x;
        };
        dir = (spread8(qu) << 1) | spread8(qv);
    }
    keys[r] = (cell << 16) | dir;
    vals[r] = r;
}

__global__ void k_pack_half(const float *__restrict__ src, uint16_t *__restrict__ dst, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x)
        dst[i] = __builtin_bit_cast(uint16_t, (_Float16)src[i]);   // round to nearest even
}

struct TileGrid {
    int tw_log2, th_log2;
    uint32_t tiles_x, tiles_y, btiles_x, btiles_y;
};

// 8x8 pixel tiles per wave, 2x2 tiles per block.  A thin grid (H < 8: a (B,N,3) ray list) is one flat list of
// H*W rays in tiles of 1x64, traced in a coherent order of its own (k_ray_keys).
constexpr int kThinRows = 8;
constexpr uint32_t kOrderMinRays = 2048;   // shorter lists are traced as they come
TileGrid tile_grid(int H, int W) {
    TileGrid t;
    if (H < kThinRows) {
        W = H * W;
        H = 1;
    }
    t.th_log2 = 3;
    while (t.th_log2 > 0 && (1 << t.th_log2) > H) --t.th_log2;
    t.tw_log2 = 6 - t.th_log2;
    t.tiles_x = ((uint32_t)W + (1u << t.tw_log2) - 1) >> t.tw_log2;
    t.tiles_y = ((uint32_t)H + (1u << t.th_log2) - 1) >> t.th_log2;
    if (t.th_log2 == 0) {   // a list: a block is four consecutive tiles
        t.btiles_x = (t.tiles_x + 3) / 4;
        t.btiles_y = 1;
    } else {
        t.btiles_x = (t.tiles_x + 1) / 2;
        t.btiles_y = (t.tiles_y + 1) / 2;
    }
    return t;
}

// `handover` / `hand_arg`: see trace_body (forward only; hand_arg steps = 0 launches the takers of the listed tiles).
template <bool BWD, bool REC>
void launch(const DstParams &p, const DstAccelView &acc, const TileGrid &t, const uint32_t *ray_order, hipStream_t stream,
            const uint32_t *block_order = nullptr, uint32_t *handover = nullptr, uint32_t hand_arg = 0u) {
    const uint32_t n_blocks = t.btiles_x * t.btiles_y;
    dim3 grid(n_blocks), block(kWavesPerBlock * DST_WAVE);
    const bool takers = !BWD && handover != nullptr && hand_arg == 0u;
    if (!BWD && kFwdWavesPerBlock == 1) {
        grid = dim3((n_blocks + 7u) / 8u * 32u);
        block = dim3(DST_WAVE);
        if (takers) grid = dim3(std::min<uint32_t>(n_blocks * (uint32_t)kWavesPerBlock, kHandCap));
    }
    // The per-lane walk is built into the kernels used where waves of unrelated rays are to be expected:
    // reflection bounces and ray lists (thin grids).  Image-shaped grids traced to depth 0 get the pure packet kernels.
    // Order of the blocks of an image grid (trace_body): column strips put vertical neighbours on one XCD.  Measured
    // forward, strips of 8 / 16 / 24 blocks / row-major: 8.12 / 8.20 / 8.53 / 8.48 ms on 120 x 68 blocks (1080p, 1M
    // surfels), but 4.68 / 4.37 / 4.19 / 4.28 ms on 50 x 50 blocks (a sphere in front of an empty background): with only
    // two or three rounds of workgroups on the chip the order decides more about the last round than about the caches.
    // The backward trace gains 1 to 3 % from strips of 8 on every grid measured.
    uint32_t strip = 0u;
    if (t.th_log2 != 0) strip = BWD ? (uint32_t)DST_STRIP_BWD : (n_blocks >= kStripMinBlocks ? (uint32_t)DST_STRIP_FWD : 0u);
    const bool mixed = takers || p.max_trace_depth > 0 || t.th_log2 < 3;
    const bool det = (p.flags & DST_FLAG_DETERMINISTIC) != 0u;
#define DST_LAUNCH_M(AUX, MIXED)                                                                                   \
    do {                                                                                                           \
        if (BWD && det)                                                                                            \
            hipLaunchKernelGGL((k_trace_bwd<AUX, REC, (MIXED) && !REC, true>), grid, block, 0, stream, p, acc,      \
                               t.tw_log2, t.th_log2, t.tiles_x, t.tiles_y, t.btiles_x, ray_order, strip, block_order);    \
        else if (BWD)                                                                                              \
            hipLaunchKernelGGL((k_trace_bwd<AUX, REC, (MIXED) && !REC, false>), grid, block, 0, stream, p, acc,     \
                               t.tw_log2, t.th_log2, t.tiles_x, t.tiles_y, t.btiles_x, ray_order, strip, block_order);    \
        else if (!(MIXED) && p.flags == 0u && handover == nullptr)                                                 \
            hipLaunchKernelGGL((k_trace_fwd_plain<AUX, REC>), grid, block, 0, stream, p, acc, t.tw_log2,           \
                               t.th_log2, t.tiles_x, t.tiles_y, t.btiles_x, ray_order, strip);                            \
        else if (p.flags != 0u)                                                                                    \
            hipLaunchKernelGGL((k_trace_fwd<AUX, REC, MIXED, true>), grid, block, 0, stream, p, acc, t.tw_log2,    \
                               t.th_log2, t.tiles_x, t.tiles_y, t.btiles_x, ray_order, strip, handover, hand_arg);        \
        else                                                                                                       \
            hipLaunchKernelGGL((k_trace_fwd<AUX, REC, MIXED, false>), grid, block, 0, stream, p, acc, t.tw_log2,   \
                               t.th_log2, t.tiles_x, t.tiles_y, t.btiles_x, ray_order, strip, handover, hand_arg);        \
    } while (0)
#define DST_LAUNCH(AUX)                                                                                            \
    do {                                                                                                           \
        if (mixed) DST_LAUNCH_M(AUX, true);                                                                        \
        else DST_LAUNCH_M(AUX, false);                                                                             \
    } while (0)
    if (p.aux <= 2) DST_LAUNCH(2);
    else if (p.aux <= 4) DST_LAUNCH(4);
    else DST_LAUNCH(8);
#undef DST_LAUNCH_M
#undef DST_LAUNCH
}

}  // namespace

int dst_launch_pack_half(const float *src, uint16_t *dst, uint64_t n, hipStream_t stream) {
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((n + 255u) / 256u, 4096u);
    hipLaunchKernelGGL(k_pack_half, dim3(blocks), dim3(256), 0, stream, src, dst, n);
    return hipGetLastError() == hipSuccess ? DST_OK : DST_E_DEVICE;
}

uint64_t dst_det_workspace_words(int32_t P, int32_t aux, int backward) {
    if (P <= 0 || aux < 1 || aux > DST_MAX_AUX) return 0;
    if (!backward) return (uint64_t)P;
    const int cols = aux <= 2 ? RowLayout<2>::cols : (aux <= 4 ? RowLayout<4>::cols : RowLayout<8>::cols);
    return (uint64_t)P * cols;
}

uint64_t dst_hit_record_layout(int32_t H, int32_t W, int32_t mtd_alloc, uint32_t blocks, uint64_t *header_words,
                               uint32_t *n_waves) {
    if (H <= 0 || W <= 0 || mtd_alloc < 0) {
        if (header_words) *header_words = 0;
        if (n_waves) *n_waves = 0;
        return 0;
    }
    const TileGrid t = tile_grid(H, W);
    const uint64_t waves = (uint64_t)t.btiles_x * t.btiles_y * kWavesPerBlock;
    const uint64_t header = 2 + (waves * (uint64_t)(mtd_alloc + 1) + 1) / 2;
    if (header_words) *header_words = header;
    if (n_waves) *n_waves = (uint32_t)waves;
    return header + (uint64_t)blocks * kRecBlockWords;
}

int dst_launch_trace(dst_ctx *ctx, const DstParams &p_in, bool backward, hipStream_t stream) {
    if (p_in.H <= 0 || p_in.W <= 0) return DST_OK;  // empty ray grid: nothing to do
    DstParams p = p_in;
    const uint32_t *ray_order = nullptr;
    if (p.H < kThinRows) {
        // a ray list: flat, and (when it is long enough to matter) in an order that puts similar rays in one wave.
        // Forward and backward derive the same order from the same rays, so a hit record stays valid.
        if ((uint64_t)p.H * p.W > 0x7FFFFFFFull) return dst_fail(ctx, DST_E_INVALID, "ray grid too large");
        p.W = p.H * p.W;
        p.H = 1;
        const uint32_t n = (uint32_t)p.W;
        if (n >= kOrderMinRays) {
            if (n > ctx->ray_capacity) {
                for (int k = 0; k < 2; ++k) {
                    if (ctx->ray_keys[k]) (void)hipFree(ctx->ray_keys[k]);
                    if (ctx->ray_vals[k]) (void)hipFree(ctx->ray_vals[k]);
                    ctx->ray_keys[k] = ctx->ray_vals[k] = nullptr;
                }
                if (ctx->ray_hist) (void)hipFree(ctx->ray_hist);
                ctx->ray_hist = nullptr;
                ctx->ray_capacity = 0;
                for (int k = 0; k < 2; ++k) {
                    DST_HIP(ctx, hipMalloc((void **)&ctx->ray_keys[k], sizeof(uint32_t) * n));
                    DST_HIP(ctx, hipMalloc((void **)&ctx->ray_vals[k], sizeof(uint32_t) * n));
                }
                DST_HIP(ctx, hipMalloc((void **)&ctx->ray_hist, sizeof(uint32_t) * dst_sort_hist_elems(n)));
                ctx->ray_capacity = n;
            }
            hipLaunchKernelGGL(k_ray_keys, dim3((n + 255u) / 256u), dim3(256), 0, stream, p.ray_o, p.ray_d, ctx->bounds,
                               ctx->ray_keys[0], ctx->ray_vals[0], n);
            dst_sort_pairs(ctx->ray_keys, ctx->ray_vals, ctx->ray_hist, n, stream);
            ray_order = ctx->ray_vals[0];
        }
    }
    const TileGrid t = tile_grid(p.H, p.W);
    if ((uint64_t)t.tiles_x * t.tiles_y > 0x3FFFFFFFull) return dst_fail(ctx, DST_E_INVALID, "ray grid too large");
    DstAccelView acc;
    acc.wide = ctx->wide;
    acc.leaves = ctx->leaves;
    acc.pre = ctx->pre;
    acc.bounds = ctx->bounds;
    acc.n_leaves = ctx->n_leaves;
    acc.root = dst_root_ref(ctx->n_leaves);
    const bool rec = p.hit_record != nullptr;
    const bool det = (p.flags & DST_FLAG_DETERMINISTIC) != 0u;
    uint32_t *const out_of_range = ctx->handover + kDstHandoverOutOfRange;   // (a spare word of the list's header)
    if (backward) {
        const uint32_t n_blocks = t.btiles_x * t.btiles_y;
        if (rec && n_blocks < kOrderMinBlocks) {
            launch<true, true>(p, acc, t, ray_order, stream);
        } else if (rec) {
            // the replay takes its blocks longest first (the forward left every wave's chunk count in the record)
            if (n_blocks > ctx->block_order_capacity) {
                if (ctx->block_order) (void)hipFree(ctx->block_order);
                ctx->block_order = nullptr;
                ctx->block_order_capacity = 0;
                DST_HIP(ctx, hipMalloc((void **)&ctx->block_order, sizeof(uint32_t) * n_blocks));
                ctx->block_order_capacity = n_blocks;
            }
            const uint32_t strip = t.th_log2 != 0 ? (uint32_t)DST_STRIP_BWD : 0u;
            hipLaunchKernelGGL(k_block_order, dim3(1), dim3(1024), 0, stream,
                               reinterpret_cast<const uint32_t *>(p.hit_record + 2), (uint32_t)p.mtd_alloc + 1u, t.btiles_x,
                               t.btiles_y, strip, t.th_log2 != 0 ? 1 : 0, n_blocks, ctx->block_order);
            launch<true, true>(p, acc, t, ray_order, stream, ctx->block_order);   // does the work if the record is complete,
        }
        launch<true, false>(p, acc, t, ray_order, stream);           // else this one does (it returns at once otherwise)
        const dim3 grid(2048), block(256);
        if (det) {
            if (p.aux <= 2) hipLaunchKernelGGL(k_det_finish_grads<2>, grid, block, 0, stream, p, out_of_range);
            else if (p.aux <= 4) hipLaunchKernelGGL(k_det_finish_grads<4>, grid, block, 0, stream, p, out_of_range);
            else hipLaunchKernelGGL(k_det_finish_grads<8>, grid, block, 0, stream, p, out_of_range);
        } else if (p.grad_rows != nullptr) {
            if (p.aux <= 2) hipLaunchKernelGGL(k_finish_grad_rows<2>, grid, block, 0, stream, p);
            else if (p.aux <= 4) hipLaunchKernelGGL(k_finish_grad_rows<4>, grid, block, 0, stream, p);
            else hipLaunchKernelGGL(k_finish_grad_rows<8>, grid, block, 0, stream, p);
        }
    } else {
        // Refits count the small quads too, on the device; the count comes over behind the first forward trace after
        // a refit (a 4-byte copy on this stream, nobody waits for it) and serves the traces after that one.
        if (ctx->bounds_host != nullptr && ctx->bounds != nullptr) {
            if (ctx->small_quads_asked) ctx->small_quads = *(volatile const uint32_t *)&ctx->bounds_host->small_quads;
            if (ctx->small_quads_refits != ctx->refits) {
                DST_HIP(ctx, hipMemcpyAsync(&ctx->bounds_host->small_quads, &ctx->bounds->small_quads, sizeof(uint32_t),
                                            hipMemcpyDeviceToHost, stream));
                ctx->small_quads_refits = ctx->refits;
                ctx->small_quads_asked = true;
            }
        }
        // the second launch of each pair traces the tiles the first one handed over (usually none: it leaves at once)
        uint32_t *const list = (kFwdWavesPerBlock == 1 && dst_handover_active(ctx)) ? ctx->handover : nullptr;
        const uint32_t steps = std::max<uint32_t>(ctx->handover_steps, 1u);
        for (int pass = 0; pass < (list != nullptr ? 2 : 1); ++pass) {
            const uint32_t arg = pass == 0 ? steps : 0u;
            if (rec) launch<false, true>(p, acc, t, ray_order, stream, nullptr, list, arg);
            else launch<false, false>(p, acc, t, ray_order, stream, nullptr, list, arg);
        }
        if (det && p.training && p.a_weights != nullptr)
            hipLaunchKernelGGL(k_det_finish_weights, dim3(1024), dim3(256), 0, stream, p, out_of_range);
    }
    DST_HIP(ctx, hipGetLastError());
    return DST_OK;
}
