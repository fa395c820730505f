// LBVH over the surfel quads: Morton codes -> LDS-staged radix sort -> Karras hierarchy ->
// bottom-up box fit, plus the refit-only path that keeps topology and leaf order.
// Replaces the OptiX GAS build / update of the reference (trace_surfels.cpp:36-159).
#include "dst_internal.h"

#include <algorithm>
#include <cstring>

namespace {

constexpr int kBlock = 256;
constexpr int kTile = 1024;        // keys per wave in the radix sort
constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;

__device__ __forceinline__ uint32_t f2ord(float f) {
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__host__ __device__ __forceinline__ float ord2f(uint32_t u) {
    u = (u & 0x80000000u) ? (u & 0x7fffffffu) : ~u;
#ifdef __HIP_DEVICE_COMPILE__
    return __uint_as_float(u);
#else
    float f;
    std::memcpy(&f, &u, 4);
    return f;
#endif
}

__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

__global__ void k_init_bounds(DstBounds *b) {
    if (threadIdx.x == 0) {
        for (int a = 0; a < 3; ++a) { b->lo[a] = 0xFFFFFFFFu; b->hi[a] = 0u; }
        b->max_abs = 0u;
        b->bad_topology = 0u;
        b->equal_keys = 0u;
        b->max_depth = 0u;
        b->small_quads = 0u;
    }
}

__global__ void k_fill_u32(uint32_t *p, uint32_t v, uint32_t n) {
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// The coordinate bound covers the finite coordinates: one corner at infinity must not void the bound of the others.
__device__ __forceinline__ float finite_max(float m, float x) { return x < INFINITY ? fmaxf(m, x) : m; }

// Largest |coordinate| of a block's quads -> bounds->max_abs: the waves meet in LDS, one atomic per block (atomics of
// many waves to one word are served one by one).  Every thread of the block calls it.
__device__ __forceinline__ void block_max_abs(float mabs, DstBounds *bounds) {
    __shared__ float s_m[kBlock / DST_WAVE];
    mabs = wave_max(mabs);
    if ((threadIdx.x & (DST_WAVE - 1)) == 0) s_m[threadIdx.x / DST_WAVE] = mabs;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x / DST_WAVE); ++w) mabs = fmaxf(mabs, s_m[w]);
        if (mabs > 0.f && mabs < INFINITY) atomicMax(&bounds->max_abs, __float_as_uint(mabs));
    }
}

// The four corners of a quad: rows ids[0..3] of the vertex buffer; rows 4g..4g+3 in order (the usual layout) are
// 48 consecutive bytes and come as three 16-byte loads.
__device__ __forceinline__ void load_corners(const float *__restrict__ vertices, int4 q, uint32_t g, float (&c)[4][3]) {
    if (q.x == (int)(4u * g) && q.y == q.x + 1 && q.z == q.x + 2 && q.w == q.x + 3 &&
        (reinterpret_cast<uintptr_t>(vertices) & 15u) == 0u) {
        const float4 *v = reinterpret_cast<const float4 *>(vertices + 12 * (size_t)g);
        const float4 a = v[0], b = v[1], d = v[2];
        c[0][0] = a.x; c[0][1] = a.y; c[0][2] = a.z; c[1][0] = a.w;
        c[1][1] = b.x; c[1][2] = b.y; c[2][0] = b.z; c[2][1] = b.w;
        c[2][2] = d.x; c[3][0] = d.y; c[3][1] = d.z; c[3][2] = d.w;
        return;
    }
    const int ids[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float *v = vertices + (size_t)ids[k] * 3;
        c[k][0] = v[0];
        c[k][1] = v[1];
        c[k][2] = v[2];
    }
}

// Build only.  Per surfel: resolve the quad's four vertex ids through the triangle buffer, then reduce the centroid
// bounds (Morton codes) and the largest |coordinate| (the trace kernels' padding).  A refit keeps the ids and gets
// the coordinate bound from the kernel that writes the leaf records.
__global__ void k_quad_setup(const float *__restrict__ vertices, uint32_t n_vertices,
                             const int32_t *__restrict__ triangles, int4 *__restrict__ quad_ids,
                             float4 *__restrict__ centroids, DstBounds *__restrict__ bounds, uint32_t P) {
    // grid-stride: a block ends with seven atomics on the same seven words, and those are served one by one,
    // so each block takes many surfels
    __shared__ float s_lo[kBlock / DST_WAVE][3], s_hi[kBlock / DST_WAVE][3];
    float cen[3] = {INFINITY, INFINITY, INFINITY}, cenh[3] = {-INFINITY, -INFINITY, -INFINITY};
    float mabs = 0.f;
    for (uint32_t g = blockIdx.x * blockDim.x + threadIdx.x; g < P; g += gridDim.x * blockDim.x) {
        float lo[3] = {INFINITY, INFINITY, INFINITY}, hi[3] = {-INFINITY, -INFINITY, -INFINITY};
        const int32_t *t = triangles + (size_t)g * 6;   // 24 bytes per surfel: three 8-byte loads where the buffer allows
        int2 ta, tb, tc;
        if ((reinterpret_cast<uintptr_t>(triangles) & 7u) == 0u) {
            const int2 *t2 = reinterpret_cast<const int2 *>(t);
            ta = t2[0]; tb = t2[1]; tc = t2[2];
        } else {
            ta = make_int2(t[0], t[1]); tb = make_int2(t[2], t[3]); tc = make_int2(t[4], t[5]);
        }
        int4 q = make_int4(ta.x, ta.y, tb.x, tc.y);
        bool bad = (tb.y != ta.y) || (tc.x != tb.x);
        bad |= (uint32_t)q.x >= n_vertices || (uint32_t)q.y >= n_vertices || (uint32_t)q.z >= n_vertices ||
               (uint32_t)q.w >= n_vertices;
        if (bad) {
            atomicOr(&bounds->bad_topology, 1u);
            q = make_int4(0, 0, 0, 0);
        } else if (q.x != (int)(4u * g) || q.y != q.x + 1 || q.z != q.x + 2 || q.w != q.x + 3) {
            atomicOr(&bounds->bad_topology, 2u);   // valid, but not rows 4g..4g+3 in order
        }
        quad_ids[g] = q;
        float c[4][3];
        load_corners(vertices, q, g, c);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
#pragma unroll
            for (int a = 0; a < 3; ++a) {
                lo[a] = fminf(lo[a], c[k][a]);
                hi[a] = fmaxf(hi[a], c[k][a]);
                mabs = finite_max(mabs, fabsf(c[k][a]));
            }
        }
        float4 c4;
        c4.x = 0.5f * (lo[0] + hi[0]);
        c4.y = 0.5f * (lo[1] + hi[1]);
        c4.z = 0.5f * (lo[2] + hi[2]);
        c4.w = 0.f;
        centroids[g] = c4;
        // a centroid at infinity (or NaN) takes no part in the grid's extent; its key is clamped to the grid's edge
        if (fabsf(c4.x) < INFINITY) { cen[0] = fminf(cen[0], c4.x); cenh[0] = fmaxf(cenh[0], c4.x); }
        if (fabsf(c4.y) < INFINITY) { cen[1] = fminf(cen[1], c4.y); cenh[1] = fmaxf(cenh[1], c4.y); }
        if (fabsf(c4.z) < INFINITY) { cen[2] = fminf(cen[2], c4.z); cenh[2] = fmaxf(cenh[2], c4.z); }
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        cen[a] = wave_min(cen[a]);
        cenh[a] = wave_max(cenh[a]);
    }
    const int w = threadIdx.x / DST_WAVE;
    if ((threadIdx.x & (DST_WAVE - 1)) == 0) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            s_lo[w][a] = cen[a];
            s_hi[w][a] = cenh[a];
        }
    }
    __syncthreads();
    if (threadIdx.x < 3) {
        const int a = threadIdx.x;
        float l = INFINITY, h = -INFINITY;
        for (int k = 0; k < (int)(blockDim.x / DST_WAVE); ++k) {
            l = fminf(l, s_lo[k][a]);
            h = fmaxf(h, s_hi[k][a]);
        }
        if (l <= h) {  // skips empty and NaN-only blocks
            atomicMin(&bounds->lo[a], f2ord(l));
            atomicMax(&bounds->hi[a], f2ord(h));
        }
    }
    block_max_abs(mabs, bounds);
}

__device__ __forceinline__ uint32_t spread10(uint32_t v) {
    v &= 0x3FFu;
    v = (v | (v << 16)) & 0x030000FFu;
    v = (v | (v << 8)) & 0x0300F00Fu;
    v = (v | (v << 4)) & 0x030C30C3u;
    v = (v | (v << 2)) & 0x09249249u;
    return v;
}

__global__ void k_morton(const float4 *__restrict__ centroids, const DstBounds *__restrict__ bounds,
                         uint32_t *__restrict__ keys, uint32_t *__restrict__ vals, uint32_t P) {
    uint32_t g = blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= P) return;
    float4 c = centroids[g];
    const float cc[3] = {c.x, c.y, c.z};
    uint32_t q[3];
    // Cubic cells: one scale for the three axes (the longest extent).  With a scale per axis a flat scene (a 200 m
    // ground with 4 m of height) gets cells of 20 cm x 20 cm x 4 mm, and the hierarchy splits in height long before
    // it has separated what lies far apart on the ground.
    float ext = 0.f;
#pragma unroll
    for (int a = 0; a < 3; ++a) ext = fmaxf(ext, ord2f(bounds->hi[a]) - ord2f(bounds->lo[a]));
    const float s = (ext > 0.f && ext < INFINITY) ? 1024.0f / ext : 0.f;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        float x = (cc[a] - ord2f(bounds->lo[a])) * s;
        x = fminf(fmaxf(x, 0.f), 1023.f);  // NaN -> 0
        q[a] = (uint32_t)x;
    }
    keys[g] = (spread10(q[0]) << 2) | (spread10(q[1]) << 1) | spread10(q[2]);
    vals[g] = g;
}

// The box the two-level keys are laid over: the centroids' bounds, cut down to mean +- 4 sigma per axis, three times
// over.  One surfel a million scene sizes away (an optimisation step gone wrong) would otherwise shrink the scene to
// a single cell even of the 2^20 grid; cut off, it lands in a cell at the grid's edge.  A uniform or a normal cloud
// keeps its bounds (4 sigma lies outside, or takes a few surfels in a hundred thousand to the edge cells).  The sums
// are integers (coordinates quantised to 16 bits of the current box), so every run cuts at the same place.
struct CoreBox {
    float lo[3], hi[3];
    unsigned long long s0[3], s1[3], s2[3];
};
__global__ void k_core_init(CoreBox *core, const DstBounds *__restrict__ bounds) {
    const int a = threadIdx.x;
    if (a < 3) {
        core->lo[a] = ord2f(bounds->lo[a]);
        core->hi[a] = ord2f(bounds->hi[a]);
        core->s0[a] = core->s1[a] = core->s2[a] = 0ull;
    }
}
__global__ void k_core_stats(const float4 *__restrict__ centroids, CoreBox *core, uint32_t P) {
    __shared__ unsigned long long s_sum[kBlock / DST_WAVE][9];
    float lo[3], sc[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        lo[a] = core->lo[a];
        const float ext = core->hi[a] - lo[a];
        sc[a] = (ext > 0.f && ext < INFINITY) ? 65535.0f / ext : 0.f;
    }
    unsigned long long acc[9] = {0ull, 0ull, 0ull, 0ull, 0ull, 0ull, 0ull, 0ull, 0ull};
    for (uint32_t g = blockIdx.x * blockDim.x + threadIdx.x; g < P; g += gridDim.x * blockDim.x) {
        const float4 c = centroids[g];
        const float cc[3] = {c.x, c.y, c.z};
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            const float x = (cc[a] - lo[a]) * sc[a];
            if (x >= 0.f && x <= 65535.f) {   // inside the current box (and not NaN)
                const unsigned long long q = (unsigned long long)x;
                acc[a] += 1ull;
                acc[3 + a] += q;
                acc[6 + a] += q * q;
            }
        }
    }
#pragma unroll
    for (int k = 0; k < 9; ++k) {
#pragma unroll
        for (int o = DST_WAVE / 2; o > 0; o >>= 1) acc[k] += __shfl_xor(acc[k], o);
    }
    const int w = threadIdx.x / DST_WAVE;
    if ((threadIdx.x & (DST_WAVE - 1)) == 0) {
#pragma unroll
        for (int k = 0; k < 9; ++k) s_sum[w][k] = acc[k];
    }
    __syncthreads();
    if (threadIdx.x < 9) {
        unsigned long long t = 0ull;
        for (int k = 0; k < (int)(blockDim.x / DST_WAVE); ++k) t += s_sum[k][threadIdx.x];
        unsigned long long *dst = threadIdx.x < 3 ? &core->s0[threadIdx.x] : (threadIdx.x < 6 ? &core->s1[threadIdx.x - 3] : &core->s2[threadIdx.x - 6]);
        if (t != 0ull) atomicAdd(dst, t);
    }
}
__global__ void k_core_cut(CoreBox *core) {
    const int a = threadIdx.x;
    if (a >= 3) return;
    const double n = (double)core->s0[a];
    if (n > 0.0) {
        const double mean = (double)core->s1[a] / n;
        const double var = fmax((double)core->s2[a] / n - mean * mean, 0.0);
        const double half = 4.0 * sqrt(var) + 1.0;   // and one cell of the 16-bit grid
        const double q_lo = fmax(mean - half, 0.0), q_hi = fmin(mean + half, 65535.0);
        const double lo = (double)core->lo[a], ext = (double)core->hi[a] - lo;
        core->lo[a] = (float)(lo + q_lo / 65535.0 * ext);
        core->hi[a] = (float)(lo + q_hi / 65535.0 * ext);
    }
    core->s0[a] = core->s1[a] = core->s2[a] = 0ull;
}

// Size of the scene's bulk: the largest coordinate of the keys' box (two-level keys: the cut box), else of any vertex.
__global__ void k_scene_scale(DstBounds *bounds, const CoreBox *core) {
    if (threadIdx.x != 0) return;
    float m = __uint_as_float(bounds->max_abs);
    if (core != nullptr) {
        float c = 0.f;
        for (int a = 0; a < 3; ++a) c = finite_max(c, fmaxf(fabsf(core->lo[a]), fabsf(core->hi[a])));
        if (c > 0.f) m = fminf(m, c);
    }
    bounds->scale = __float_as_uint(m);
}

// Two-level keys for scenes whose centroids crowd into few cells of the 1024^3 grid (a few surfels far outside an
// otherwise compact scene stretch the grid over the whole extent): 20 bits per axis, the upper ten interleaved
// into `hi` (the same cells as k_morton's), the lower ten into `lo`.  Sorted as two stable 32-bit sorts, by `lo`
// first and then by `hi`, with the same kernels as the one-level keys.
__global__ void k_morton_fine(const float4 *__restrict__ centroids, const CoreBox *__restrict__ core,
                              uint32_t *__restrict__ keys, uint32_t *__restrict__ lo_of, uint32_t *__restrict__ hi_of,
                              uint32_t *__restrict__ vals, uint32_t P) {
    uint32_t g = blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= P) return;
    float4 c = centroids[g];
    const float cc[3] = {c.x, c.y, c.z};
    float ext = 0.f;
#pragma unroll
    for (int a = 0; a < 3; ++a) ext = fmaxf(ext, core->hi[a] - core->lo[a]);
    const float s = (ext > 0.f && ext < INFINITY) ? 1048576.0f / ext : 0.f;
    uint32_t qh[3], ql[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        float x = (cc[a] - core->lo[a]) * s;   // a surfel outside the box goes to the cell at its edge
        x = fminf(fmaxf(x, 0.f), 1048575.f);  // NaN -> 0
        const uint32_t q = (uint32_t)x;
        qh[a] = q >> 10;
        ql[a] = q & 1023u;
    }
    const uint32_t lo = (spread10(ql[0]) << 2) | (spread10(ql[1]) << 1) | spread10(ql[2]);
    keys[g] = lo;
    lo_of[g] = lo;
    hi_of[g] = (spread10(qh[0]) << 2) | (spread10(qh[1]) << 1) | spread10(qh[2]);
    vals[g] = g;
}
__global__ void k_gather_u32(uint32_t *__restrict__ dst, const uint32_t *__restrict__ src,
                             const uint32_t *__restrict__ index, uint32_t n) {
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[index[i]];
}

// ---- radix sort: one wave owns a contiguous tile of kTile keys ------------------------------------
__global__ void k_radix_hist(const uint32_t *__restrict__ keys, uint32_t *__restrict__ tile_hist, uint32_t n,
                             uint32_t n_tiles, int shift) {
    __shared__ uint32_t hist[kBlock / DST_WAVE][kRadix];
    const int w = threadIdx.x / DST_WAVE, lane = threadIdx.x % DST_WAVE;
    const uint32_t tile = blockIdx.x * (kBlock / DST_WAVE) + w;
    for (int d = lane; d < kRadix; d += DST_WAVE) hist[w][d] = 0;
    __syncthreads();
    if (tile < n_tiles) {
        for (int r = 0; r < kTile / DST_WAVE; ++r) {
            uint32_t i = tile * kTile + r * DST_WAVE + lane;
            if (i < n) atomicAdd(&hist[w][(keys[i] >> shift) & (kRadix - 1)], 1u);
        }
    }
    __syncthreads();
    if (tile < n_tiles)
        for (int d = lane; d < kRadix; d += DST_WAVE) tile_hist[(size_t)d * n_tiles + tile] = hist[w][d];
}

// Exclusive scan of the tile counters in two steps: block d scans the row of digit d (one counter per tile) in place
// and leaves the row's total in row_total[d]; a second, tiny kernel turns the 256 totals into the digits' start
// positions, which the scatter adds to a tile's entry.  (One block walking all 256 x tiles counters took 0.14 ms per
// pass at a million keys: a fifth of the whole build.)
__global__ void k_scan_rows(uint32_t *tile_hist, uint32_t *row_total, uint32_t n_tiles) {
    __shared__ uint32_t wave_sum[1024 / DST_WAVE];
    __shared__ uint32_t carry_s;
    uint32_t *data = tile_hist + (size_t)blockIdx.x * n_tiles;
    const uint32_t t = threadIdx.x, nt = blockDim.x, lane = t % DST_WAVE, w = t / DST_WAVE;
    if (t == 0) carry_s = 0u;
    __syncthreads();
    for (uint32_t base = 0; base < n_tiles; base += nt) {
        const uint32_t i = base + t;
        const uint32_t mine = i < n_tiles ? data[i] : 0u;
        uint32_t incl = mine;   // inclusive scan over the wave
#pragma unroll
        for (int off = 1; off < DST_WAVE; off <<= 1) {
            const uint32_t up = __shfl_up(incl, off);
            if ((int)lane >= off) incl += up;
        }
        if (lane == DST_WAVE - 1) wave_sum[w] = incl;
        __syncthreads();
        uint32_t before = carry_s;
        for (uint32_t k = 0; k < w; ++k) before += wave_sum[k];
        if (i < n_tiles) data[i] = before + incl - mine;
        __syncthreads();
        if (t == nt - 1) carry_s = before + incl;   // the last thread's running total is the slab's
        __syncthreads();
    }
    if (t == 0) row_total[blockIdx.x] = carry_s;
}
__global__ void k_scan_digits(uint32_t *row_total) {   // one block of kRadix threads, in place, exclusive
    __shared__ uint32_t s[kRadix];
    const uint32_t t = threadIdx.x;
    s[t] = row_total[t];
    __syncthreads();
    for (uint32_t off = 1; off < kRadix; off <<= 1) {
        const uint32_t add = t >= off ? s[t - off] : 0u;
        __syncthreads();
        s[t] += add;
        __syncthreads();
    }
    row_total[t] = s[t] - row_total[t];
}

__global__ void k_radix_scatter(const uint32_t *__restrict__ keys_in, const uint32_t *__restrict__ vals_in,
                                uint32_t *__restrict__ keys_out, uint32_t *__restrict__ vals_out,
                                const uint32_t *__restrict__ tile_hist, const uint32_t *__restrict__ digit_start,
                                uint32_t n, uint32_t n_tiles, int shift) {
    __shared__ uint32_t base[kBlock / DST_WAVE][kRadix];
    const int w = threadIdx.x / DST_WAVE, lane = threadIdx.x % DST_WAVE;
    const uint32_t tile = blockIdx.x * (kBlock / DST_WAVE) + w;
    if (tile < n_tiles)
        for (int d = lane; d < kRadix; d += DST_WAVE) base[w][d] = tile_hist[(size_t)d * n_tiles + tile] + digit_start[d];
    __syncthreads();
    if (tile >= n_tiles) return;
    const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    for (int r = 0; r < kTile / DST_WAVE; ++r) {
        uint32_t i = tile * kTile + r * DST_WAVE + lane;
        bool valid = i < n;
        uint32_t key = valid ? keys_in[i] : 0u, val = valid ? vals_in[i] : 0u;
        uint32_t digit = (key >> shift) & (kRadix - 1);
        uint64_t same = __ballot(valid);
#pragma unroll
        for (int b = 0; b < kRadixBits; ++b) {
            bool bit = (digit >> b) & 1u;
            uint64_t bb = __ballot(bit);
            same &= bit ? bb : ~bb;
        }
        uint32_t rank = __popcll(same & lt);
        uint32_t off = 0;
        if (valid) off = base[w][digit];
        __builtin_amdgcn_wave_barrier();   // every lane has read its digit's position before the first of the digit moves it on
        if (valid) {
            keys_out[off + rank] = key;
            vals_out[off + rank] = val;
            if (rank == 0) base[w][digit] = off + (uint32_t)__popcll(same);
        }
    }
}

// ---- Karras 2012 hierarchy over the sorted keys -----------------------------------------------------
// Length of the common prefix of keys i and j; equal keys go on with the second-level keys (FINE) and then with the
// positions themselves, which keeps the hierarchy balanced over any run of equal keys.
template <bool FINE>
__device__ __forceinline__ int delta_of(const uint32_t *__restrict__ keys, const uint32_t *__restrict__ lo, int n, int i, int j) {
    if (j < 0 || j >= n) return -1;
    uint32_t a = keys[i], b = keys[j];
    if (a != b) return __clz(a ^ b);
    if (FINE) {
        a = lo[i];
        b = lo[j];
        if (a != b) return 32 + __clz(a ^ b);
        return 64 + __clz((uint32_t)i ^ (uint32_t)j);
    }
    return 32 + __clz((uint32_t)i ^ (uint32_t)j);
}

constexpr uint32_t kEqualKeysEvery = 16;
// FINE = false also counts the neighbours with equal keys (bounds->equal_keys): the host reads the count with the
// bounds and goes over to two-level keys when the grid turns out too coarse for the scene.
template <bool FINE>
__global__ void k_karras(const uint32_t *__restrict__ keys, const uint32_t *__restrict__ keys_lo, DstNode *__restrict__ nodes,
                         uint32_t *__restrict__ node_parent, uint32_t *__restrict__ leaf_parent, int n,
                         DstBounds *__restrict__ bounds) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n - 1) return;
    auto delta = [&](const uint32_t *, int, int a, int b) { return delta_of<FINE>(keys, keys_lo, n, a, b); };
    if (!FINE && (blockIdx.x % kEqualKeysEvery) == 0u) {
        // a sample: every sixteenth block counts (one atomic per wave to one word - a million keys counted in full
        // added 0.1 ms to the build)
        const uint64_t active = __ballot(true), equal = __ballot(keys[i] == keys[i + 1]);
        if (equal != 0ull && (int)__lane_id() == __builtin_ctzll(active)) atomicAdd(&bounds->equal_keys, (uint32_t)__popcll(equal));
    }
    int d = (delta(keys, n, i, i + 1) - delta(keys, n, i, i - 1)) >= 0 ? 1 : -1;
    int dmin = delta(keys, n, i, i - d);
    int lmax = 2;
    while (delta(keys, n, i, i + lmax * d) > dmin) lmax <<= 1;
    int l = 0;
    for (int t = lmax >> 1; t >= 1; t >>= 1)
        if (delta(keys, n, i, i + (l + t) * d) > dmin) l += t;
    int j = i + l * d;
    int dnode = delta(keys, n, i, j);
    int s = 0;
    int t = l;
    do {
        t = (t + 1) >> 1;
        if (delta(keys, n, i, i + (s + t) * d) > dnode) s += t;
    } while (t > 1);
    int gamma = i + s * d + min(d, 0);
    int lo = min(i, j), hi = max(i, j);
    uint32_t c0, c1;
    if (lo == gamma) {
        c0 = DST_LEAF_BIT | (uint32_t)gamma;
        leaf_parent[gamma] = ((uint32_t)i << 1) | 0u;
    } else {
        c0 = (uint32_t)gamma;
        node_parent[gamma] = ((uint32_t)i << 1) | 0u;
    }
    if (hi == gamma + 1) {
        c1 = DST_LEAF_BIT | (uint32_t)(gamma + 1);
        leaf_parent[gamma + 1] = ((uint32_t)i << 1) | 1u;
    } else {
        c1 = (uint32_t)(gamma + 1);
        node_parent[gamma + 1] = ((uint32_t)i << 1) | 1u;
    }
    nodes[i].c0 = c0;
    nodes[i].c1 = c1;
    nodes[i].first = (uint32_t)lo;
    nodes[i].last = (uint32_t)hi;
    if (i == 0) node_parent[0] = DST_NO_PARENT;
}

// The same sample of equal neighbours for builds that do not run k_karras<false> (agglomerated hierarchies).
__global__ void k_count_equal_keys(const uint32_t *__restrict__ keys, int n, DstBounds *__restrict__ bounds) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n - 1 || (blockIdx.x % kEqualKeysEvery) != 0u) return;
    const uint64_t active = __ballot(true), equal = __ballot(keys[i] == keys[i + 1]);
    if (equal != 0ull && (int)__lane_id() == __builtin_ctzll(active)) atomicAdd(&bounds->equal_keys, (uint32_t)__popcll(equal));
}

// Deepest leaf of the hierarchy (number of nodes above it), for the builds with two-level keys: their depth is no
// longer bounded by 30 key bits + the bits of a position, and the walks' stacks are sized for that bound.
__global__ void k_tree_depth(const uint32_t *__restrict__ node_parent, const uint32_t *__restrict__ leaf_parent,
                             DstBounds *__restrict__ bounds, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t depth = 0u;
    if (i < n) {
        uint32_t p = leaf_parent[i];
        while (p != DST_NO_PARENT && depth < 4096u) {
            ++depth;
            p = node_parent[p >> 1];
        }
    }
#pragma unroll
    for (int off = DST_WAVE / 2; off >= 1; off >>= 1) depth = max(depth, (uint32_t)__shfl_xor((int)depth, off));
    if (__lane_id() == 0u && depth != 0u) atomicMax(&bounds->max_depth, depth);
}

#include "ploc.inc"

// The quads as the first clusters, in Morton order.
__global__ void k_ploc_init(const float *__restrict__ vertices, const int4 *__restrict__ quad_ids,
                            const uint32_t *__restrict__ sorted_ids, PlocBufs pb, uint32_t n) {
    const uint32_t m = blockIdx.x * blockDim.x + threadIdx.x;
    if (m == 0) {
        pb.state[0] = pb.state[1] = n;
        pb.state[2] = pb.state[3] = 0u;
        pb.state[4] = pb.state[5] = pb.state[6] = 0u;
    }
    if (m >= n) return;
    const uint32_t g = sorted_ids[m];
    float c[4][3];
    load_corners(vertices, quad_ids[g], g, c);
    float *out = pb.box[0] + 6 * (size_t)m;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        out[a] = fminf(fminf(c[0][a], c[1][a]), fminf(c[2][a], c[3][a]));
        out[3 + a] = fmaxf(fmaxf(c[0][a], c[1][a]), fmaxf(c[2][a], c[3][a]));
    }
    pb.id[0][m] = DST_LEAF_BIT | m;
}

// The trace kernels widen every box and every stand-in limit by a multiple of the magnitudes of the numbers that meet
// in the test: the ray origin's (added per ray) and the quad's own coordinates' (added here, once, to the quad's box
// and limits).  A scene-wide bound in the quad's place would make the slack of every test grow with the farthest surfel:
// one of them a thousand scene sizes away and every box of the scene is wider than the surfel inside it.
constexpr float kBoxPad = 4e-6f;      // box faces, per unit of coordinate magnitude (make_slab has the ray's share)
constexpr float kPlanePad = 1.5e-4f;  // in-plane slack of the stand-in (make_pre: padw)
constexpr float kDistPad = 1e-4f;     // slack of the stand-in's distance along the ray (make_pre: tp)
__device__ __forceinline__ float quad_magnitude(const float (&c)[4][3]) {
    float m = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int a = 0; a < 3; ++a) m = finite_max(m, fabsf(c[k][a]));
    return m;
}

// Leaf record + conservative stand-in of one quad (corners c[0..3] = A,B,C,D, surfel id g) at leaf position i.
// The plane normals use the fused form the hit test is defined with: cross(x,y).x = fma(x.y, y.z, -(x.z*y.y)), ...
__device__ __forceinline__ void write_leaf(const float (&c)[4][3], uint32_t g, uint32_t i, DstLeaf *__restrict__ leaves,
                                           DstLeafPre *__restrict__ pre) {
    auto cross_f = [](const float *x, const float *y, float *out) {
        out[0] = __builtin_fmaf(x[1], y[2], -(x[2] * y[1]));
        out[1] = __builtin_fmaf(x[2], y[0], -(x[0] * y[2]));
        out[2] = __builtin_fmaf(x[0], y[1], -(x[1] * y[0]));
    };
    float e1[3], e2[3], e3[3], f1[3], f2[3], n0[3], n1[3], n2[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        e1[a] = c[1][a] - c[0][a];   // B - A
        e2[a] = c[2][a] - c[0][a];   // C - A
        e3[a] = c[3][a] - c[0][a];   // D - A
        f1[a] = c[2][a] - c[1][a];   // C - B
        f2[a] = c[3][a] - c[1][a];   // D - B
    }
    cross_f(e1, e2, n0);
    cross_f(f1, f2, n1);
    cross_f(e2, e3, n2);
    const float c1 = __builtin_fmaf(n1[2], e1[2], __builtin_fmaf(n1[1], e1[1], n1[0] * e1[0]));
    float out[24];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        out[a] = c[0][a];
        out[3 + a] = e1[a];
        out[6 + a] = e2[a];
        out[9 + a] = e3[a];
        out[12 + a] = n1[a];
        out[16 + a] = n0[a];
        out[19 + a] = n2[a];
    }
    out[15] = __uint_as_float(g);
    out[22] = c1;
    out[23] = 0.f;
    float4 *dst = reinterpret_cast<float4 *>(&leaves[i]);
#pragma unroll
    for (int k = 0; k < 6; ++k) dst[k] = make_float4(out[4 * k], out[4 * k + 1], out[4 * k + 2], out[4 * k + 3]);

    // the conservative stand-in (see DstLeafPre): mean plane, averaged half edges, their dual vectors
    float cen[3], nrm[3], h1[3], h2[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        cen[a] = 0.25f * ((c[0][a] + c[1][a]) + (c[2][a] + c[3][a]));
        nrm[a] = n0[a] - n1[a];   // the strip's second triangle winds the other way
        h1[a] = 0.25f * ((c[1][a] - c[0][a]) + (c[3][a] - c[2][a]));   // half of the averaged edge A->B / C->D
        h2[a] = 0.25f * ((c[2][a] - c[0][a]) + (c[3][a] - c[1][a]));   // half of the averaged edge A->C / B->D
    }
    const float nl = sqrtf(nrm[0] * nrm[0] + nrm[1] * nrm[1] + nrm[2] * nrm[2]);
    float fu[3], fv[3], t1[3], t2[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) nrm[a] = nrm[a] / nl;
    cross_f(h2, nrm, t1);    // perpendicular to h2 and the normal
    cross_f(nrm, h1, t2);
    const float d1 = h1[0] * t1[0] + h1[1] * t1[1] + h1[2] * t1[2];
    const float d2 = h2[0] * t2[0] + h2[1] * t2[1] + h2[2] * t2[2];
    float mfu = 0.f, lim0 = 0.f, dev = 0.f, rad2 = 0.f;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        fu[a] = t1[a] / d1;
        fv[a] = t2[a] / d2;
    }
    mfu = fmaxf(sqrtf(fu[0] * fu[0] + fu[1] * fu[1] + fu[2] * fu[2]), sqrtf(fv[0] * fv[0] + fv[1] * fv[1] + fv[2] * fv[2]));
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float w[3] = {c[k][0] - cen[0], c[k][1] - cen[1], c[k][2] - cen[2]};
        lim0 = fmaxf(lim0, fabsf(fu[0] * w[0] + fu[1] * w[1] + fu[2] * w[2]));
        lim0 = fmaxf(lim0, fabsf(fv[0] * w[0] + fv[1] * w[1] + fv[2] * w[2]));
        dev = fmaxf(dev, fabsf(nrm[0] * w[0] + nrm[1] * w[1] + nrm[2] * w[2]));
        rad2 = fmaxf(rad2, w[0] * w[0] + w[1] * w[1] + w[2] * w[2]);
    }
    const float rad = sqrtf(rad2) * 1.002f;   // every point of the quad is within this distance of the centroid
    // A ray that meets the quad at less than 0.05 rad-ish from its plane skips the stand-in (trace kernels), so a
    // corner that is `dev` off the mean plane moves a hit by at most 20 dev along the plane; margins of 2.
    float tdev = 40.0f * dev;
    lim0 = lim0 * 1.002f + tdev * mfu;
    // the quad's share of the coordinate-dependent slack (the ray's share is added per ray)
    const float mag = quad_magnitude(c);
    lim0 += (kPlanePad * mag) * mfu;
    tdev += kDistPad * mag;
    const float rad_padded = rad + kPlanePad * mag;
    const bool ok = isfinite(mfu) && isfinite(lim0) && isfinite(tdev) && isfinite(rad_padded) && isfinite(cen[0] + cen[1] + cen[2]) &&
                    isfinite(nrm[0] + nrm[1] + nrm[2]) && nl > 0.f;
    float pr[16];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        pr[a] = ok ? cen[a] : 0.f;
        pr[3 + a] = ok ? nrm[a] : 0.f;
        pr[6 + a] = ok ? fu[a] : 0.f;
        pr[9 + a] = ok ? fv[a] : 0.f;
    }
    pr[12] = ok ? mfu : INFINITY;
    pr[13] = ok ? lim0 : INFINITY;
    pr[14] = ok ? tdev : INFINITY;
    pr[15] = ok ? rad_padded : INFINITY;
    float4 *pdst = reinterpret_cast<float4 *>(&pre[i]);
#pragma unroll
    for (int k = 0; k < 4; ++k) pdst[k] = make_float4(pr[4 * k], pr[4 * k + 1], pr[4 * k + 2], pr[4 * k + 3]);
}

// ---- boxes of leaf ranges without climbing the tree ---------------------------------------------------------
// A node of the hierarchy covers a contiguous range of leaves, so its children's boxes are range unions of leaf
// boxes, and those can be looked up instead of being carried up the tree by threads that wait for each other:
// leaves are cut into blocks of 64 (one wave of the kernels that write the leaf records); every leaf stores the
// union of its block up to itself (`pbox`) and from itself on (`sbox`), a table holds the unions of 2^l consecutive
// blocks for every l, and a range is: rest of its first block + start of its last block + two table entries for
// the blocks between - or, inside one block, a loop over at most 62 leaf boxes.  min/max are exact, so the boxes
// are the same bits as those of the climbing fit.
constexpr int kRangeBlock = DST_WAVE;
struct RangeBoxes {
    float *lbox, *pbox, *sbox;   // 6 floats per leaf: lo[3], hi[3]
    float *table;                // [level][block][6]
};
__device__ __forceinline__ void box_join(float (&a)[6], const float *b) {
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        a[k] = fminf(a[k], b[k]);
        a[3 + k] = fmaxf(a[3 + k], b[3 + k]);
    }
}
__device__ __forceinline__ void box_store(float *dst, const float (&b)[6]) {
    float2 *d = reinterpret_cast<float2 *>(dst);
    d[0] = make_float2(b[0], b[1]);
    d[1] = make_float2(b[2], b[3]);
    d[2] = make_float2(b[4], b[5]);
}
// Called by ALL 64 lanes of a wave whose lane l holds leaf position base + l (`valid`: that position exists).
__device__ __forceinline__ void wave_range_boxes(const float (&c)[4][3], bool valid, uint32_t i, uint32_t n,
                                                 const RangeBoxes &rb) {
    const uint32_t lane = threadIdx.x % DST_WAVE;
    float box[6], pre[6], suf[6];
    const float pad = kBoxPad * quad_magnitude(c);
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        box[a] = valid ? fminf(fminf(c[0][a], c[1][a]), fminf(c[2][a], c[3][a])) - pad : INFINITY;
        box[3 + a] = valid ? fmaxf(fmaxf(c[0][a], c[1][a]), fmaxf(c[2][a], c[3][a])) + pad : -INFINITY;
    }
#pragma unroll
    for (int k = 0; k < 6; ++k) pre[k] = suf[k] = box[k];
#pragma unroll
    for (int off = 1; off < DST_WAVE; off <<= 1) {
#pragma unroll
        for (int k = 0; k < 6; ++k) {
            const float up = __shfl_up(pre[k], off), down = __shfl_down(suf[k], off);
            if ((int)lane >= off) pre[k] = k < 3 ? fminf(pre[k], up) : fmaxf(pre[k], up);
            if ((int)lane + off < DST_WAVE) suf[k] = k < 3 ? fminf(suf[k], down) : fmaxf(suf[k], down);
        }
    }
    if (!valid) return;
    box_store(rb.lbox + 6 * (size_t)i, box);
    box_store(rb.pbox + 6 * (size_t)i, pre);
    box_store(rb.sbox + 6 * (size_t)i, suf);
    if (lane == DST_WAVE - 1 || i == n - 1u) box_store(rb.table + 6 * (size_t)(i / kRangeBlock), pre);   // level 0: whole blocks
}
// table[level][b] = union of blocks b .. b + 2^level - 1 (entries that would run past the last block stay unused)
__global__ void k_range_table_level(float *table, uint32_t n_blocks, int level) {
    const uint32_t b = blockIdx.x * blockDim.x + threadIdx.x, half = 1u << (level - 1);
    if (b + 2u * half > n_blocks) return;
    const float *lo = table + ((size_t)(level - 1) * n_blocks + b) * 6, *hi = lo + 6 * (size_t)half;
    float box[6];
#pragma unroll
    for (int k = 0; k < 6; ++k) box[k] = lo[k];
    box_join(box, hi);
    box_store(table + ((size_t)level * n_blocks + b) * 6, box);
}
__device__ __forceinline__ void range_box(const RangeBoxes &rb, uint32_t n_blocks, uint32_t a, uint32_t b, float (&box)[6]) {
    const uint32_t ba = a / kRangeBlock, bb = b / kRangeBlock;
    if (ba == bb) {
        const float *src = rb.lbox + 6 * (size_t)a;
#pragma unroll
        for (int k = 0; k < 6; ++k) box[k] = src[k];
        for (uint32_t j = a + 1u; j <= b; ++j) box_join(box, rb.lbox + 6 * (size_t)j);
        return;
    }
    const float *s = rb.sbox + 6 * (size_t)a;
#pragma unroll
    for (int k = 0; k < 6; ++k) box[k] = s[k];
    box_join(box, rb.pbox + 6 * (size_t)b);
    if (bb > ba + 1u) {
        const uint32_t x = ba + 1u, y = bb - 1u;
        const int l = 31 - __clz(y - x + 1u);
        box_join(box, rb.table + ((size_t)l * n_blocks + x) * 6);
        box_join(box, rb.table + ((size_t)l * n_blocks + (y + 1u - (1u << l))) * 6);
    }
}
// Fit by look-up: node i's children cover leaves first..split and split+1..last (split = the child reference itself,
// see k_karras).
__global__ void k_fit_ranges(DstNode *nodes, RangeBoxes rb, uint32_t n_blocks, uint32_t n_internal) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_internal) return;
    DstNode &nd = nodes[i];
    const uint32_t first = nd.first, last = nd.last, split = nd.c0 & ~DST_LEAF_BIT;
    float b0[6], b1[6];
    range_box(rb, n_blocks, first, split, b0);
    range_box(rb, n_blocks, split + 1u, last, b1);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        nd.lo0[k] = b0[k]; nd.hi0[k] = b0[3 + k];
        nd.lo1[k] = b1[k]; nd.hi1[k] = b1[3 + k];
    }
}

// Is this quad far smaller than the scene (DstBounds::small_quads)?  `scale` = the scene's size as set by the last build.
__device__ __forceinline__ bool quad_is_small(const float (&c)[4][3], float scale) {
    float ab = 0.f, ac = 0.f;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        ab += (c[1][a] - c[0][a]) * (c[1][a] - c[0][a]);
        ac += (c[2][a] - c[0][a]) * (c[2][a] - c[0][a]);
    }
    const float lim = scale * kDstSmallQuad;
    return fmaxf(ab, ac) < lim * lim;
}
// One addition per wave that has any (scenes without small quads add nothing).
__device__ __forceinline__ void count_small_quads(bool small, DstBounds *bounds) {
    const unsigned long long m = __ballot(small);
    if ((threadIdx.x & (DST_WAVE - 1)) == 0 && m != 0ull) atomicAdd(&bounds->small_quads, (uint32_t)__popcll(m));
}

// Leaf records in Morton order (also the whole of a refit's geometry update).
__global__ void k_leaf_fill(const float *__restrict__ vertices, const int4 *__restrict__ quad_ids,
                            const uint32_t *__restrict__ sorted_ids, DstLeaf *__restrict__ leaves,
                            DstLeafPre *__restrict__ pre, RangeBoxes rb, DstBounds *__restrict__ bounds,
                            DstBounds *__restrict__ count_small, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    const bool valid = i < n;   // every lane stays for the wave-wide scans of the boxes
    float c[4][3] = {};
    float mabs = 0.f;
    bool small = false;
    if (valid) {
        const uint32_t g = sorted_ids[i];
        load_corners(vertices, quad_ids[g], g, c);
        write_leaf(c, g, i, leaves, pre);
        small = quad_is_small(c, __uint_as_float(count_small->scale));
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int a = 0; a < 3; ++a) mabs = finite_max(mabs, fabsf(c[k][a]));
    }
    if (rb.lbox != nullptr) wave_range_boxes(c, valid, i, n, rb);
    if (bounds != nullptr) block_max_abs(mabs, bounds);   // a refit: the coordinate bound of the moved quads
    count_small_quads(small, count_small);
}

// The same for a refit straight from the surfel parameters: the four corners of surfel g are
//   v_k = (mean + a_k * (sx * R[:,0])) + b_k * (sy * R[:,1]),  (a,b) = (-3,3), (-3,-3), (3,3), (3,-3),
// R the rotation of the quaternion (w,x,y,z) divided by its norm sqrt(((w*w + x*x) + y*y) + z*z): the quads of
// the 2DGS convention (reference example/utils/gaussian_utils.py:176-210), every operation in fp32, rounded once,
// in exactly this order (this file is compiled without contraction).  Optionally writes the corners to
// `vertices_out` (4P,3) in the canonical order (rows 4g..4g+3) for the trace calls, and reduces the largest
// |coordinate| the trace kernels size their padding with.
__global__ void k_leaf_fill_from_surfels(const float *__restrict__ means, const float *__restrict__ scales,
                                         const float *__restrict__ rotations, const uint32_t *__restrict__ sorted_ids,
                                         DstLeaf *__restrict__ leaves, DstLeafPre *__restrict__ pre,
                                         float *__restrict__ vertices_out, DstBounds *__restrict__ bounds,
                                         RangeBoxes rb, uint32_t n) {
    float mabs = 0.f;
    // wave-uniform trip count: every lane stays for the wave-wide scans of the boxes
    for (uint32_t base = blockIdx.x * blockDim.x + (threadIdx.x & ~(DST_WAVE - 1u)); base < n; base += gridDim.x * blockDim.x) {
        const uint32_t i = base + (threadIdx.x & (DST_WAVE - 1u));
        const bool valid = i < n;
        float c[4][3] = {};
        if (valid) {
        const uint32_t g = sorted_ids[i];
        const float q0 = rotations[4 * (size_t)g], q1 = rotations[4 * (size_t)g + 1], q2 = rotations[4 * (size_t)g + 2],
                    q3 = rotations[4 * (size_t)g + 3];
        const float nrm = sqrtf(((q0 * q0 + q1 * q1) + q2 * q2) + q3 * q3);
        const float w = q0 / nrm, x = q1 / nrm, y = q2 / nrm, z = q3 / nrm;
        const float sx = scales[2 * (size_t)g], sy = scales[2 * (size_t)g + 1];
        const float u[3] = {(1.f - 2.f * (y * y + z * z)) * sx, (2.f * (x * y + w * z)) * sx, (2.f * (x * z - w * y)) * sx};
        const float v[3] = {(2.f * (x * y - w * z)) * sy, (1.f - 2.f * (x * x + z * z)) * sy, (2.f * (y * z + w * x)) * sy};
        const float m[3] = {means[3 * (size_t)g], means[3 * (size_t)g + 1], means[3 * (size_t)g + 2]};
        const float sa[4] = {-3.f, -3.f, 3.f, 3.f}, sb[4] = {3.f, -3.f, 3.f, -3.f};
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int a = 0; a < 3; ++a) {
                c[k][a] = (m[a] + sa[k] * u[a]) + sb[k] * v[a];
                mabs = finite_max(mabs, fabsf(c[k][a]));
            }
        if (vertices_out != nullptr) {
            float4 *dst = reinterpret_cast<float4 *>(vertices_out + 12 * (size_t)g);   // 48 bytes per surfel
            dst[0] = make_float4(c[0][0], c[0][1], c[0][2], c[1][0]);
            dst[1] = make_float4(c[1][1], c[1][2], c[2][0], c[2][1]);
            dst[2] = make_float4(c[2][2], c[3][0], c[3][1], c[3][2]);
        }
        write_leaf(c, g, i, leaves, pre);
        }
        count_small_quads(valid && quad_is_small(c, __uint_as_float(bounds->scale)), bounds);
        if (rb.lbox != nullptr) wave_range_boxes(c, valid, i, n, rb);
    }
    mabs = wave_max(mabs);
    if ((threadIdx.x & (DST_WAVE - 1)) == 0 && mabs > 0.f && mabs < INFINITY)
        atomicMax(&bounds->max_abs, __float_as_uint(mabs));
}

// Bottom-up fit: each leaf climbs; the second thread to reach a node merges the two child boxes and goes on.
// A node's leaves are contiguous and its index is the first or the last of them, so every node whose leaves
// all belong to this block of kFitBlock consecutive leaves is reached only by threads of this block: those meet in
// LDS (workgroup-scope ordering, no cache maintenance).  Only the few nodes that span blocks use the
// agent-scope protocol through memory, whose fences write back and invalidate the L2 of the XCD.
constexpr int kFitBlock = 1024;
__global__ __launch_bounds__(kFitBlock) void k_fit(DstNode *nodes, const uint32_t *__restrict__ node_parent,
                      const uint32_t *__restrict__ leaf_parent, uint32_t *flags, const float *__restrict__ vertices,
                      const int4 *__restrict__ quad_ids, const uint32_t *__restrict__ sorted_ids, uint32_t n) {
    __shared__ float s_box[kFitBlock][12];      // per local node: box of child 0, box of child 1
    __shared__ uint32_t s_arrived[kFitBlock];
    s_arrived[threadIdx.x] = 0u;
    __syncthreads();
    const uint32_t blk_lo = blockIdx.x * blockDim.x, blk_hi = min(blk_lo + blockDim.x, n) - 1u;
    uint32_t i = blk_lo + threadIdx.x;
    if (i >= n) return;
    float box[6];
    float c[4][3];
    const uint32_t g = sorted_ids[i];
    load_corners(vertices, quad_ids[g], g, c);   // (the leaf records hold edge vectors, not the corners)
    const float pad = kBoxPad * quad_magnitude(c);   // as in wave_range_boxes: the two fits give the same bits
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        box[a] = fminf(fminf(c[0][a], c[1][a]), fminf(c[2][a], c[3][a])) - pad;
        box[3 + a] = fmaxf(fmaxf(c[0][a], c[1][a]), fmaxf(c[2][a], c[3][a])) + pad;
    }
    uint32_t pp = leaf_parent[i];
    bool local = true;
    while (pp != DST_NO_PARENT) {
        const uint32_t p = pp >> 1, which = pp & 1u;
        float *mine = which ? nodes[p].lo1 : nodes[p].lo0;
        if (local) local = nodes[p].first >= blk_lo && nodes[p].last <= blk_hi;
        if (local) {
            const uint32_t slot = p - blk_lo;
#pragma unroll
            for (int k = 0; k < 6; ++k) {
                mine[k] = box[k];                      // for the kernels that follow
                s_box[slot][6 * which + k] = box[k];   // for the sibling's thread
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");   // the LDS stores come before the arrival count
            const uint32_t arrived = __hip_atomic_fetch_add(&s_arrived[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (arrived == 0) return;
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                box[k] = fminf(box[k], s_box[slot][6 * (1u - which) + k]);
                box[3 + k] = fmaxf(box[3 + k], s_box[slot][6 * (1u - which) + 3 + k]);
            }
        } else {
            const float *other = which ? nodes[p].lo0 : nodes[p].lo1;
#pragma unroll
            for (int k = 0; k < 6; ++k) __hip_atomic_store(mine + k, box[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __threadfence();
            uint32_t arrived = atomicAdd(&flags[p], 1u);
            if (arrived == 0) return;
            __threadfence();
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                float olo = __hip_atomic_load(other + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                float ohi = __hip_atomic_load(other + 3 + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                box[k] = fminf(box[k], olo);
                box[3 + k] = fmaxf(box[3 + k], ohi);
            }
        }
        pp = node_parent[p];
    }
}

// Reference the trace kernels follow for a child of a binary node: a subtree of at most DST_GROUP leaves
// (contiguous in Morton order) is one leaf group, anything larger is the wide node of the same index.
// The child's leaves first .. last are known from its parent (first .. split and split + 1 .. last): no look at the
// child's own record.
__device__ __forceinline__ uint32_t traversal_ref(uint32_t c, uint32_t first, uint32_t last) {
    if (c & DST_LEAF_BIT) return DST_LEAF_BIT | (c & DST_REF_FIRST_MASK);
    const uint32_t count = last - first + 1u;
    if (count <= DST_GROUP) return DST_LEAF_BIT | ((count - 1u) << 28) | first;
    return c;
}
// Both children of a node as traversal references.
__device__ __forceinline__ void child_refs(const DstNode &nd, uint32_t &r0, uint32_t &r1) {
    const uint32_t split = nd.c0 & ~DST_LEAF_BIT;
    r0 = traversal_ref(nd.c0, nd.first, split);
    r1 = traversal_ref(nd.c1, split + 1u, nd.last);
}

// Collapse the fitted binary hierarchy into 4-wide traversal nodes.  Two ways: node i offers its grandchildren (a child
// that is already a leaf group is offered itself), or - `depth_word` says the hierarchy is shallow enough - it starts
// from its two children and opens the one with the largest surface, twice: big boxes are the ones rays meet, so
// looking inside them at once saves the visit (6 to 9 % fewer node visits on the scenes measured).  A step of the
// second kind may go down a single level of the binary hierarchy, so the walks' stacks (128 entries, three deferred
// children per step) bound its use to hierarchies of at most kAreaCollapseDepth levels; the grandchildren rule goes
// down two levels per step and serves up to kMaxDepth.  The choice depends on the boxes, so a refit may make it anew.
constexpr uint32_t kAreaCollapseDepth = 42;
__global__ void k_widen(const DstNode *__restrict__ nodes, DstWideNode *__restrict__ wide, uint32_t n_internal,
                        const uint32_t *__restrict__ depth_word) {
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_internal) return;
    const DstNode nd = nodes[i];
    if (nd.last - nd.first + 1u <= DST_GROUP) return;   // inside a leaf group: never visited
    const bool by_area = depth_word != nullptr && *depth_word <= kAreaCollapseDepth;
    DstWideNode w;
    uint32_t k = 0;
    auto put = [&](const float *lo, const float *hi, uint32_t ref) {
        w.lox[k] = lo[0]; w.loy[k] = lo[1]; w.loz[k] = lo[2];
        w.hix[k] = hi[0]; w.hiy[k] = hi[1]; w.hiz[k] = hi[2];
        w.ref[k] = ref;
        ++k;
    };
    uint32_t own[2];
    child_refs(nd, own[0], own[1]);
    if (!by_area) {
        const float *los[2] = {nd.lo0, nd.lo1}, *his[2] = {nd.hi0, nd.hi1};
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const uint32_t r = own[s];
            if (r & DST_LEAF_BIT) {
                put(los[s], his[s], r);
            } else {
                const DstNode ch = nodes[r];
                uint32_t g0, g1;
                child_refs(ch, g0, g1);
                put(ch.lo0, ch.hi0, g0);
                put(ch.lo1, ch.hi1, g1);
            }
        }
    } else {
        float lo[DST_WIDE][3], hi[DST_WIDE][3];
        uint32_t ref[DST_WIDE];   // traversal references, in the order of the leaves below them
        int m = 2;
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            lo[0][a] = nd.lo0[a]; hi[0][a] = nd.hi0[a];
            lo[1][a] = nd.lo1[a]; hi[1][a] = nd.hi1[a];
        }
        ref[0] = own[0];
        ref[1] = own[1];
        while (m < DST_WIDE) {
            int best = -1;
            float best_area = -1.f;
            for (int c = 0; c < m; ++c) {
                if (ref[c] & DST_LEAF_BIT) continue;
                const float dx = hi[c][0] - lo[c][0], dy = hi[c][1] - lo[c][1], dz = hi[c][2] - lo[c][2];
                float area = dx * dy + dy * dz + dz * dx;
                if (!(area >= 0.f)) area = INFINITY;   // a box of non-finite corners: open it
                if (area > best_area) {
                    best_area = area;
                    best = c;
                }
            }
            if (best < 0) break;
            const DstNode ch = nodes[ref[best]];
            for (int c = m; c > best + 1; --c) {   // make room behind the opened child
#pragma unroll
                for (int a = 0; a < 3; ++a) {
                    lo[c][a] = lo[c - 1][a];
                    hi[c][a] = hi[c - 1][a];
                }
                ref[c] = ref[c - 1];
            }
#pragma unroll
            for (int a = 0; a < 3; ++a) {
                lo[best][a] = ch.lo0[a]; hi[best][a] = ch.hi0[a];
                lo[best + 1][a] = ch.lo1[a]; hi[best + 1][a] = ch.hi1[a];
            }
            child_refs(ch, ref[best], ref[best + 1]);
            ++m;
        }
        for (int c = 0; c < m; ++c) put(lo[c], hi[c], ref[c]);
    }
    w.count = k;
    for (; k < DST_WIDE; ++k) {   // unused slots: the traversal masks them by `count`
        w.lox[k] = w.loy[k] = w.loz[k] = 0.f;
        w.hix[k] = w.hiy[k] = w.hiz[k] = 0.f;
        w.ref[k] = DST_LEAF_BIT;  // would be a harmless one-quad group, never another node
    }
    w.pad[0] = w.pad[1] = w.pad[2] = 0u;
    wide[i] = w;
}

inline dim3 grid_for(uint32_t n, int block = kBlock) { return dim3((n + block - 1) / block); }

// One-level keys are kept while at most DST_FINE_KEYS_NUM / DST_FINE_KEYS_DEN of the neighbours in Morton order share
// a cell.  Measured at a million surfels: with half of them sharing (a 200 m ground in 20 cm cells) the finer keys
// change nothing in the trace; with 97 % sharing (a 10 m room and a hundred surfels 150 m away) they make the
// trace 1.15x faster, with the far surfels 1.5 km away 7x; the second level costs 0.05 to 0.1 ms per build.
#ifndef DST_FINE_KEYS_NUM
#define DST_FINE_KEYS_NUM 3
#define DST_FINE_KEYS_DEN 4
#endif
constexpr uint32_t kMaxDepth = 60;   // nodes above a leaf; one-level keys stay below 30 + 27
bool fine_keys_wanted(uint32_t equal_keys, uint32_t n) {
    // `equal_keys` was counted over the pairs (i, i+1), i < n-1, of every kEqualKeysEvery-th block of kBlock pairs
    const uint64_t pairs = n - 1u, span = (uint64_t)kBlock * kEqualKeysEvery;
    const uint64_t sampled = pairs / span * kBlock + std::min<uint64_t>(pairs % span, kBlock);
    return (uint64_t)equal_keys * DST_FINE_KEYS_DEN > sampled * DST_FINE_KEYS_NUM;
}

int ensure_capacity(dst_ctx *ctx, uint32_t P) {
    if (P <= ctx->capacity) return DST_OK;
    dst_lbvh_free(ctx);
    const size_t n = P;
    const size_t tiles = (n + kTile - 1) / kTile;
    DST_HIP(ctx, hipMalloc((void **)&ctx->nodes, sizeof(DstNode) * std::max<size_t>(n - 1, 1)));
    DST_HIP(ctx, hipMalloc((void **)&ctx->wide, sizeof(DstWideNode) * std::max<size_t>(n - 1, 1)));
    // (two spare records: the per-lane walk reads a leaf group as eight or ten 16-byte words whatever its size)
    DST_HIP(ctx, hipMalloc((void **)&ctx->leaves, sizeof(DstLeaf) * (n + 2)));
    DST_HIP(ctx, hipMemset(ctx->leaves + n, 0, 2 * sizeof(DstLeaf)));
    DST_HIP(ctx, hipMalloc((void **)&ctx->pre, sizeof(DstLeafPre) * (n + 1)));   // the trace kernels fetch them in pairs
    DST_HIP(ctx, hipMemset(ctx->pre + n, 0, sizeof(DstLeafPre)));
    DST_HIP(ctx, hipMalloc((void **)&ctx->node_parent, sizeof(uint32_t) * n));
    DST_HIP(ctx, hipMalloc((void **)&ctx->leaf_parent, sizeof(uint32_t) * n));
    DST_HIP(ctx, hipMalloc((void **)&ctx->flags, sizeof(uint32_t) * n));
    DST_HIP(ctx, hipMalloc((void **)&ctx->quad_ids, sizeof(int32_t) * 4 * n));
    DST_HIP(ctx, hipMalloc((void **)&ctx->centroids, sizeof(float) * 4 * n));
    DST_HIP(ctx, hipMalloc((void **)&ctx->range_lbox, sizeof(float) * 6 * n));
    DST_HIP(ctx, hipMalloc((void **)&ctx->range_pbox, sizeof(float) * 6 * n));
    DST_HIP(ctx, hipMalloc((void **)&ctx->range_sbox, sizeof(float) * 6 * n));
    {
        const size_t n_blocks = (n + kRangeBlock - 1) / kRangeBlock;
        size_t levels = 1;
        while ((size_t(2) << (levels - 1)) <= n_blocks) ++levels;
        DST_HIP(ctx, hipMalloc((void **)&ctx->range_table, sizeof(float) * 6 * n_blocks * levels));
    }
    for (int k = 0; k < 2; ++k) {
        DST_HIP(ctx, hipMalloc((void **)&ctx->keys[k], sizeof(uint32_t) * n));
        DST_HIP(ctx, hipMalloc((void **)&ctx->vals[k], sizeof(uint32_t) * n));
    }
    ctx->tile_hist_elems = tiles * kRadix + kRadix;
    DST_HIP(ctx, hipMalloc((void **)&ctx->tile_hist, sizeof(uint32_t) * ctx->tile_hist_elems));
    ctx->ploc_blocks = (uint32_t)((n + kPlocBlock - 1) / kPlocBlock);
    DST_HIP(ctx, hipMalloc((void **)&ctx->ploc_state, sizeof(uint32_t) * (kPlocStateWords + 2 * ((size_t)ctx->ploc_blocks + 1))));
    DST_HIP(ctx, hipMemset(ctx->ploc_state, 0xFF, sizeof(uint32_t) * kPlocStateWords));   // depth word: "too deep" until a build says otherwise
    if (!ctx->ploc_host) DST_HIP(ctx, hipHostMalloc((void **)&ctx->ploc_host, sizeof(uint32_t) * kPlocStateWords, hipHostMallocDefault));
    if (!ctx->bounds) DST_HIP(ctx, hipMalloc((void **)&ctx->bounds, sizeof(DstBounds)));
    if (!ctx->core_box) DST_HIP(ctx, hipMalloc((void **)&ctx->core_box, sizeof(CoreBox)));
    if (!ctx->bounds_host) DST_HIP(ctx, hipHostMalloc((void **)&ctx->bounds_host, sizeof(DstBounds), hipHostMallocDefault));
    ctx->capacity = P;
    return DST_OK;
}

// Scratch of dst_refit_accel_static: the arrival counters of the bottom-up fit, one per surfel.  One copy per
// GPU, held until the process ends; host code reaches it only through the address hipGetSymbolAddress returns
// on that GPU (the array's name is not a device address on the host side).
__device__ __align__(256) uint32_t g_refit_scratch[DST_STATIC_REFIT_MAX_SURFELS];
constexpr int kMaxDevices = 64;
uint32_t *g_refit_scratch_ptr[kMaxDevices] = {};

// Hierarchy by agglomeration (see above).  Scratch comes from buffers that are idle between the sort and the leaf
// records: the range boxes (cluster boxes, per-cluster words), the centroids (temporary nodes), the sort's second
// value buffer and the fit's arrival counters (cluster ids).  Reads the cluster count back every few rounds, to know
// when one workgroup can finish; leaves the sorted surfel ids of the new leaf order in ctx->vals[0].
int ploc_hierarchy(dst_ctx *ctx, const float *vertices, uint32_t n, hipStream_t stream) {
    PlocBufs pb;
    pb.box[0] = ctx->range_pbox;
    pb.box[1] = ctx->range_sbox;
    pb.id[0] = ctx->vals[1];
    pb.id[1] = ctx->flags;
    uint32_t *words = reinterpret_cast<uint32_t *>(ctx->range_lbox);
    pb.nn = words;
    pb.pre = words + (size_t)n;
    pb.lpar = words + 2 * (size_t)n;
    uint32_t *tmp = reinterpret_cast<uint32_t *>(ctx->centroids);
    pb.tc0 = tmp;
    pb.tc1 = tmp + (size_t)n;
    pb.tsize = tmp + 2 * (size_t)n;
    pb.tpar = tmp + 3 * (size_t)n;
    pb.state = ctx->ploc_state;
    pb.n_blocks = ctx->ploc_blocks;
    hipLaunchKernelGGL(k_ploc_init, grid_for(n), dim3(kBlock), 0, stream, vertices, reinterpret_cast<const int4 *>(ctx->quad_ids),
                       ctx->vals[0], pb, n);
    int it = 0;
    uint32_t count = n;
    int batch = 32;
    while (count > kPlocTail) {
        const dim3 grid((count + kPlocBlock - 1) / kPlocBlock);   // enough for the largest count this batch can see
        for (int k = 0; k < batch; ++k, ++it) {
            hipLaunchKernelGGL(k_ploc_nn, grid, dim3(kPlocBlock), 0, stream, pb, it);
            hipLaunchKernelGGL(k_ploc_flags, grid, dim3(kPlocBlock), 0, stream, pb, it);
            hipLaunchKernelGGL(k_ploc_scan, dim3(1), dim3(kPlocBlock), 0, stream, pb, it);
            hipLaunchKernelGGL(k_ploc_apply, grid, dim3(kPlocBlock), 0, stream, pb, it);
        }
        DST_HIP(ctx, hipMemcpyAsync(ctx->ploc_host, ctx->ploc_state, sizeof(uint32_t) * kPlocStateWords, hipMemcpyDeviceToHost, stream));
        DST_HIP(ctx, hipStreamSynchronize(stream));
        const uint32_t now = ctx->ploc_host[it & 1];
        if (now >= count || (uint32_t)it > kPlocMaxRounds) {   // no progress in a whole batch: cannot happen (every round merges)
            ctx->ploc_refused = true;
            return kPlocRefused;
        }
        count = now;
        batch = 8;
    }
    hipLaunchKernelGGL(k_ploc_tail, dim3(1), dim3(kPlocBlock), 0, stream, pb, it);
    // the layout below follows the links of a finished hierarchy: make sure it is one
    DST_HIP(ctx, hipMemcpyAsync(ctx->ploc_host, ctx->ploc_state, sizeof(uint32_t) * kPlocStateWords, hipMemcpyDeviceToHost, stream));
    DST_HIP(ctx, hipStreamSynchronize(stream));
    if (ctx->ploc_host[4] != 0u || ctx->ploc_host[0] != 1u || ctx->ploc_host[2] != n - 1u) {
        ctx->ploc_refused = true;
        return kPlocRefused;
    }
    hipLaunchKernelGGL(k_ploc_leaf_positions, grid_for(n), dim3(kBlock), 0, stream, pb, ctx->vals[0], ctx->vals[1], n);
    hipLaunchKernelGGL(k_ploc_node_numbers, grid_for(n - 1), dim3(kBlock), 0, stream, pb, ctx->nodes, n);
    hipLaunchKernelGGL(k_ploc_links, grid_for(n - 1), dim3(kBlock), 0, stream, pb, ctx->nodes, ctx->node_parent, ctx->leaf_parent, n);
    DST_HIP(ctx, hipGetLastError());
    DST_HIP(ctx, hipMemcpyAsync(ctx->ploc_host, ctx->ploc_state, sizeof(uint32_t) * kPlocStateWords, hipMemcpyDeviceToHost, stream));
    DST_HIP(ctx, hipStreamSynchronize(stream));
    if (ctx->ploc_host[4] != 0u) {   // the links did not form one hierarchy over all leaves: nothing may read its order
        ctx->ploc_refused = true;
        return kPlocRefused;
    }
    std::swap(ctx->vals[0], ctx->vals[1]);   // the surfel ids in leaf order
    return DST_OK;
}

}  // namespace

int dst_static_scratch_init(dst_ctx *ctx) {
    const int dev = ctx->device;
    if (dev < 0 || dev >= kMaxDevices) return dst_fail(ctx, DST_E_UNSUPPORTED, "device ordinal beyond 63");
    if (g_refit_scratch_ptr[dev] != nullptr) return DST_OK;
    uint32_t *ptr = nullptr;
    DST_HIP(ctx, hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(g_refit_scratch)));
    if (ptr == nullptr) return dst_fail(ctx, DST_E_DEVICE, "hipGetSymbolAddress returned no address");
    g_refit_scratch_ptr[dev] = ptr;
    return DST_OK;
}

uint32_t *dst_static_scratch(const dst_ctx *ctx) {
    return (ctx->device >= 0 && ctx->device < kMaxDevices) ? g_refit_scratch_ptr[ctx->device] : nullptr;
}

// Stable LSD radix sort of (key, value) pairs, 32-bit keys, four 8-bit passes; the sorted pairs end in buffer 0.
// tile_hist holds 256 counters per 1024 keys and 256 more for the digits' start positions (dst_sort_hist_elems).  Used by the BVH build (Morton codes) and by the ray ordering.
void dst_sort_pairs(uint32_t *keys[2], uint32_t *vals[2], uint32_t *tile_hist, uint32_t n, hipStream_t stream) {
    const uint32_t tiles = (n + kTile - 1) / kTile;
    const uint32_t tile_blocks = (tiles + (kBlock / DST_WAVE) - 1) / (kBlock / DST_WAVE);
    int src = 0;
    for (int shift = 0; shift < 32; shift += kRadixBits) {
        hipLaunchKernelGGL(k_radix_hist, dim3(tile_blocks), dim3(kBlock), 0, stream, keys[src], tile_hist, n, tiles, shift);
        uint32_t *digit_start = tile_hist + (size_t)tiles * kRadix;   // kRadix words behind the tile counters
        hipLaunchKernelGGL(k_scan_rows, dim3(kRadix), dim3(1024), 0, stream, tile_hist, digit_start, tiles);
        hipLaunchKernelGGL(k_scan_digits, dim3(1), dim3(kRadix), 0, stream, digit_start);
        hipLaunchKernelGGL(k_radix_scatter, dim3(tile_blocks), dim3(kBlock), 0, stream, keys[src], vals[src],
                           keys[1 - src], vals[1 - src], tile_hist, digit_start, n, tiles, shift);
        src = 1 - src;
    }
}
size_t dst_sort_hist_elems(uint32_t n) { return (size_t)((n + kTile - 1) / kTile) * kRadix + kRadix; }

void dst_lbvh_free(dst_ctx *ctx) {
    auto rel = [](auto *&p) {
        if (p) (void)hipFree(p);
        p = nullptr;
    };
    rel(ctx->nodes);
    rel(ctx->wide);
    rel(ctx->leaves);
    rel(ctx->pre);
    rel(ctx->node_parent);
    rel(ctx->leaf_parent);
    rel(ctx->flags);
    rel(ctx->quad_ids);
    rel(ctx->centroids);
    rel(ctx->range_lbox);
    rel(ctx->range_pbox);
    rel(ctx->range_sbox);
    rel(ctx->range_table);
    rel(ctx->keys[0]);
    rel(ctx->keys[1]);
    rel(ctx->vals[0]);
    rel(ctx->vals[1]);
    rel(ctx->tile_hist);
    rel(ctx->ploc_state);
    rel(ctx->ray_keys[0]);
    rel(ctx->ray_keys[1]);
    rel(ctx->ray_vals[0]);
    rel(ctx->ray_vals[1]);
    rel(ctx->ray_hist);
    rel(ctx->block_order);
    ctx->block_order_capacity = 0;
    ctx->ray_capacity = 0;
    ctx->capacity = 0;
    ctx->built = false;
    ctx->n_leaves = 0;
}

int dst_lbvh_build(dst_ctx *ctx, const float *vertices, uint32_t n_vertices, const int32_t *triangles, uint32_t P,
                   bool rebuild, hipStream_t stream, uint32_t *fit_flags, const DstSurfelSource *surfels) {
    if (rebuild) {
        ctx->built = false;
        int rc = ensure_capacity(ctx, P);
        if (rc) return rc;
        ctx->n_leaves = P;
    }
    // The fit looks the boxes up (k_fit_ranges); a caller that brings its own arrival counters (the refit that
    // allocates nothing) gets the climbing fit, which needs nothing else.
    const bool by_ranges = fit_flags == nullptr;
    RangeBoxes rb = {nullptr, nullptr, nullptr, nullptr};
    if (by_ranges) rb = RangeBoxes{ctx->range_lbox, ctx->range_pbox, ctx->range_sbox, ctx->range_table};
    if (fit_flags == nullptr) fit_flags = ctx->flags;   // after ensure_capacity: a first build allocates them there
    if (fit_flags == nullptr || ctx->nodes == nullptr || ctx->leaves == nullptr || ctx->pre == nullptr ||
        ctx->vals[0] == nullptr)
        return dst_fail(ctx, DST_E_DEVICE, "acceleration structure buffers are not allocated");
    const uint32_t n = P;
    int4 *quad_ids = reinterpret_cast<int4 *>(ctx->quad_ids);
    float4 *centroids = reinterpret_cast<float4 *>(ctx->centroids);
    bool use_ploc = false;

    hipLaunchKernelGGL(k_init_bounds, dim3(1), dim3(64), 0, stream, ctx->bounds);
    const dim3 setup_grid(std::min<uint32_t>(grid_for(n).x, 1024u));   // 4 blocks per CU, each thread takes several surfels
    if (surfels != nullptr) {
        // refit from the surfel parameters: corners, leaf records and the coordinate bound in one kernel
        hipLaunchKernelGGL(k_leaf_fill_from_surfels, setup_grid, dim3(kBlock), 0, stream, surfels->means, surfels->scales,
                           surfels->rotations, ctx->vals[0], ctx->leaves, ctx->pre, surfels->vertices_out, ctx->bounds, rb, n);
    } else if (rebuild)
        hipLaunchKernelGGL(k_quad_setup, setup_grid, dim3(kBlock), 0, stream, vertices, n_vertices, triangles,
                           quad_ids, centroids, ctx->bounds, n);

    if (rebuild) {
        if (ctx->fine_keys) {
            // second-level keys in original order wait in two buffers that are idle until the hierarchy is made
            uint32_t *lo_of = ctx->node_parent, *hi_of = ctx->flags;
            CoreBox *core = reinterpret_cast<CoreBox *>(ctx->core_box);
            hipLaunchKernelGGL(k_core_init, dim3(1), dim3(64), 0, stream, core, ctx->bounds);
            for (int pass = 0; pass < 3; ++pass) {
                hipLaunchKernelGGL(k_core_stats, dim3(std::min<uint32_t>(grid_for(n).x, 256u)), dim3(kBlock), 0, stream,
                                   centroids, core, n);
                hipLaunchKernelGGL(k_core_cut, dim3(1), dim3(64), 0, stream, core);
            }
            hipLaunchKernelGGL(k_scene_scale, dim3(1), dim3(64), 0, stream, ctx->bounds, core);
            hipLaunchKernelGGL(k_morton_fine, grid_for(n), dim3(kBlock), 0, stream, centroids, core, ctx->keys[0],
                               lo_of, hi_of, ctx->vals[0], n);
            dst_sort_pairs(ctx->keys, ctx->vals, ctx->tile_hist, n, stream);
            hipLaunchKernelGGL(k_gather_u32, grid_for(n), dim3(kBlock), 0, stream, ctx->keys[0], hi_of, ctx->vals[0], n);
            dst_sort_pairs(ctx->keys, ctx->vals, ctx->tile_hist, n, stream);   // stable: equal cells stay in `lo` order
            hipLaunchKernelGGL(k_gather_u32, grid_for(n), dim3(kBlock), 0, stream, ctx->keys[1], lo_of, ctx->vals[0], n);
        } else {
            hipLaunchKernelGGL(k_scene_scale, dim3(1), dim3(64), 0, stream, ctx->bounds, (const CoreBox *)nullptr);
            hipLaunchKernelGGL(k_morton, grid_for(n), dim3(kBlock), 0, stream, centroids, ctx->bounds, ctx->keys[0],
                               ctx->vals[0], n);
            dst_sort_pairs(ctx->keys, ctx->vals, ctx->tile_hist, n, stream);   // the sorted pairs end in buffer 0
        }
        use_ploc = ctx->use_ploc && !ctx->ploc_refused && n >= kPlocMinSurfels && vertices != nullptr;
        if (use_ploc) {
            if (!ctx->fine_keys)
                hipLaunchKernelGGL(k_count_equal_keys, grid_for(n - 1), dim3(kBlock), 0, stream, ctx->keys[0], (int)n, ctx->bounds);
            int rc = ploc_hierarchy(ctx, vertices, n, stream);
            if (rc == kPlocRefused)
                return dst_lbvh_build(ctx, vertices, n_vertices, triangles, P, true, stream, by_ranges ? nullptr : fit_flags, surfels);
            if (rc) return rc;
        } else if (n > 1) {
            hipLaunchKernelGGL(k_fill_u32, dim3(1), dim3(64), 0, stream, ctx->ploc_state + 5, 0xFFFFFFFFu, 1u);   // depth unknown: grandchildren
            hipLaunchKernelGGL(k_fill_u32, grid_for(n), dim3(kBlock), 0, stream, ctx->node_parent, DST_NO_PARENT, n);
            if (ctx->fine_keys) {
                hipLaunchKernelGGL(k_karras<true>, grid_for(n - 1), dim3(kBlock), 0, stream, ctx->keys[0], ctx->keys[1],
                                   ctx->nodes, ctx->node_parent, ctx->leaf_parent, (int)n, ctx->bounds);
                hipLaunchKernelGGL(k_tree_depth, grid_for(n), dim3(kBlock), 0, stream, ctx->node_parent, ctx->leaf_parent,
                                   ctx->bounds, n);
            } else
                hipLaunchKernelGGL(k_karras<false>, grid_for(n - 1), dim3(kBlock), 0, stream, ctx->keys[0], nullptr,
                                   ctx->nodes, ctx->node_parent, ctx->leaf_parent, (int)n, ctx->bounds);
        } else {
            hipLaunchKernelGGL(k_fill_u32, dim3(1), dim3(kBlock), 0, stream, ctx->leaf_parent, DST_NO_PARENT, 1u);
        }
    }
    if (surfels == nullptr)
        hipLaunchKernelGGL(k_leaf_fill, grid_for(n), dim3(kBlock), 0, stream, vertices, quad_ids, ctx->vals[0],
                           ctx->leaves, ctx->pre, rb, rebuild ? nullptr : ctx->bounds, ctx->bounds, n);
    if (by_ranges) {
        const uint32_t n_blocks = (n + kRangeBlock - 1) / kRangeBlock;
        for (int level = 1; (2u << (level - 1)) <= n_blocks; ++level)
            hipLaunchKernelGGL(k_range_table_level, grid_for(n_blocks), dim3(kBlock), 0, stream, ctx->range_table, n_blocks, level);
        if (n > 1)
            hipLaunchKernelGGL(k_fit_ranges, grid_for(n - 1), dim3(kBlock), 0, stream, ctx->nodes, rb, n_blocks, n - 1);
    } else {
        hipLaunchKernelGGL(k_fill_u32, grid_for(n), dim3(kBlock), 0, stream, fit_flags, 0u, n);
        if (vertices == nullptr) return dst_fail(ctx, DST_E_INVALID, "the fit by arrival counters reads the corners from a vertex buffer");
        hipLaunchKernelGGL(k_fit, dim3((n + kFitBlock - 1) / kFitBlock), dim3(kFitBlock), 0, stream, ctx->nodes, ctx->node_parent, ctx->leaf_parent,
                           fit_flags, vertices, quad_ids, ctx->vals[0], n);
    }
    if (n > DST_GROUP)
        hipLaunchKernelGGL(k_widen, grid_for(n - 1), dim3(kBlock), 0, stream, ctx->nodes, ctx->wide, n - 1, ctx->ploc_state + 5);
    DST_HIP(ctx, hipGetLastError());

    if (rebuild) {
        DST_HIP(ctx, hipMemcpyAsync(ctx->bounds_host, ctx->bounds, sizeof(DstBounds), hipMemcpyDeviceToHost, stream));
        DST_HIP(ctx, hipMemcpyAsync(ctx->ploc_host, ctx->ploc_state, sizeof(uint32_t) * kPlocStateWords, hipMemcpyDeviceToHost, stream));
        DST_HIP(ctx, hipStreamSynchronize(stream));
        if (use_ploc && (ctx->ploc_host[4] != 0u || ctx->ploc_host[5] > kMaxDepth)) {
            // the agglomeration did not finish, or its hierarchy is deeper than the walks' stacks are sized for (clusters
            // nested at every scale): this context keeps the Morton hierarchy from now on
            ctx->ploc_refused = true;
            return dst_lbvh_build(ctx, vertices, n_vertices, triangles, P, true, stream, by_ranges ? nullptr : fit_flags, surfels);
        }
        ctx->hierarchy_depth = use_ploc ? ctx->ploc_host[5] : 0u;
        ctx->agglomerated = use_ploc;
        ctx->canonical = (ctx->bounds_host->bad_topology & 2u) == 0u;
        if (ctx->bounds_host->bad_topology & 1u)
            return dst_fail(ctx, DST_E_TOPOLOGY,
                            "triangles must come in pairs [a,b,c],[b,c,d] per surfel with ids inside vertices");
        for (int a = 0; a < 3; ++a) {
            ctx->scene_lo[a] = ord2f(ctx->bounds_host->lo[a]);
            ctx->scene_hi[a] = ord2f(ctx->bounds_host->hi[a]);
        }
        std::memcpy(&ctx->max_abs, &ctx->bounds_host->max_abs, 4);
        ctx->small_quads = ctx->bounds_host->small_quads;
        ctx->small_quads_refits = ctx->refits;
        ctx->small_quads_asked = false;
        if (ctx->fine_keys && ctx->bounds_host->max_depth > kMaxDepth) {
            // deeper than the walks' stacks are sized for (nested clusters at every scale): one-level keys, for good
            ctx->fine_keys = false;
            ctx->fine_keys_refused = true;
            return dst_lbvh_build(ctx, vertices, n_vertices, triangles, P, true, stream, by_ranges ? nullptr : fit_flags, surfels);
        }
        if (!ctx->fine_keys && !ctx->fine_keys_refused && fine_keys_wanted(ctx->bounds_host->equal_keys, n)) {
            // too many surfels per cell of the grid: build once more with two-level keys, and keep them from now on
            ctx->fine_keys = true;
            return dst_lbvh_build(ctx, vertices, n_vertices, triangles, P, true, stream, by_ranges ? nullptr : fit_flags, surfels);
        }
        ctx->built_vertices = n_vertices;
        ctx->built = true;
        ctx->builds++;
    } else {
        ctx->refits++;
    }
    return DST_OK;
}
