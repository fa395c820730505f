// The BVH builder (csrc/lbvh.hip with csrc/ploc.inc), compiled for the CPU and run on small scenes: every kernel's
// indexing is exercised under the host's memory checks (build with -fsanitize=address) and the finished structure is
// held against its invariants - before any of it runs on a GPU.  Test infrastructure; see hip/hip_runtime.h here.
#include "hip/hip_runtime.h"

#include "../../diff-surfel-tracing_amd/csrc/lbvh.hip"

#include <cstdio>
#include <random>
#include <set>

namespace {

struct Scene {
    std::vector<float> v;     // (4P,3)
    std::vector<int32_t> f;   // (2P,3)
    uint32_t P;
};

Scene make_scene(uint32_t P, int kind, uint32_t seed) {
    // kind 0: uniform cube, random orientations; 1: all centres at one point; 2: identical quads but a few; 3: some
    // quads with NaN / infinite corners; 4: a plane of overlapping quads plus a dense cluster
    Scene s;
    s.P = P;
    s.v.resize(12 * (size_t)P);
    s.f.resize(6 * (size_t)P);
    std::mt19937 rng(seed);
    std::uniform_real_distribution<float> U(-1.f, 1.f);
    std::normal_distribution<float> N(0.f, 1.f);
    float first[12];
    for (uint32_t g = 0; g < P; ++g) {
        float m[3] = {U(rng), U(rng), U(rng)};
        if (kind == 1) m[0] = m[1] = m[2] = 0.25f;
        if (kind == 4) {
            if (g % 3) m[2] = -1.f;
            else { m[0] = 0.3f + 0.05f * N(rng); m[1] = 0.05f * N(rng); m[2] = 0.05f * N(rng); }
        }
        float q[4] = {N(rng), N(rng), N(rng), N(rng)};
        if (kind == 4 && g % 3) { q[0] = 1.f; q[1] = q[2] = 0.f; q[3] = N(rng); }
        const float nq = std::sqrt(q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3]);
        const float w = q[0] / nq, x = q[1] / nq, y = q[2] / nq, z = q[3] / nq;
        const float sx = std::exp(-3.5f + 0.5f * N(rng)), sy = std::exp(-3.5f + 0.5f * N(rng));
        const float u[3] = {(1 - 2 * (y * y + z * z)) * sx, 2 * (x * y + w * z) * sx, 2 * (x * z - w * y) * sx};
        const float t[3] = {2 * (x * y - w * z) * sy, (1 - 2 * (x * x + z * z)) * sy, 2 * (y * z + w * x) * sy};
        const float sa[4] = {-3, -3, 3, 3}, sb[4] = {3, -3, 3, -3};
        for (int k = 0; k < 4; ++k)
            for (int a = 0; a < 3; ++a) s.v[12 * (size_t)g + 3 * k + a] = m[a] + sa[k] * u[a] + sb[k] * t[a];
        if (g == 0) std::memcpy(first, &s.v[0], sizeof(first));
        if (kind == 2 && g + 40 < P) std::memcpy(&s.v[12 * (size_t)g], first, sizeof(first));
        if (kind == 3 && g % 97 == 5) s.v[12 * (size_t)g + (g % 12)] = (g % 2) ? NAN : INFINITY;
        if (kind == 3 && g % 211 == 7)
            for (int k = 0; k < 12; ++k) s.v[12 * (size_t)g + k] = NAN;
        for (int k = 0; k < 3; ++k) {
            s.f[6 * (size_t)g + k] = 4 * g + k;
            s.f[6 * (size_t)g + 3 + k] = 4 * g + 1 + k;
        }
    }
    return s;
}

int failures = 0;
#define CHECK(cond, ...)                                   \
    do {                                                   \
        if (!(cond)) {                                     \
            if (++failures < 20) {                         \
                std::printf("FAILED %s:%d: ", __FILE__, __LINE__); \
                std::printf(__VA_ARGS__);                  \
                std::printf("\n");                         \
            }                                              \
        }                                                  \
    } while (0)

struct Box { float lo[3], hi[3]; };
bool same_box(const float *lo, const float *hi, const Box &b) {
    for (int a = 0; a < 3; ++a)
        if (std::memcmp(&lo[a], &b.lo[a], 4) != 0 || std::memcmp(&hi[a], &b.hi[a], 4) != 0) return false;
    return true;
}

// The invariants the fit by look-up, the refit, the collapse and the walks rely on.  Returns the depth (nodes above the
// deepest leaf).
uint32_t check_structure(const dst_ctx &c, const Scene &s, const char *what) {
    const uint32_t n = c.n_leaves;
    CHECK(n == s.P, "%s: leaves", what);
    // every surfel exactly once, corners copied
    std::vector<int> seen(n, 0);
    std::vector<Box> lbox(n);
    for (uint32_t i = 0; i < n; ++i) {
        const DstLeaf &L = c.leaves[i];
        CHECK(L.g < n, "%s: leaf %u holds surfel %u", what, i, L.g);
        if (L.g >= n) continue;
        seen[L.g]++;
        {   // corner A and the edge vectors to B, C, D, as the fp32 differences of the corners
            const float *v = &s.v[12 * (size_t)L.g];
            float want[12];
            for (int a = 0; a < 3; ++a) {
                want[a] = v[a];
                for (int k = 1; k < 4; ++k) want[3 * k + a] = v[3 * k + a] - v[a];
            }
            CHECK(std::memcmp(L.A, want, 48) == 0, "%s: corner and edges of leaf %u", what, i);
        }
        float cc[4][3];
        std::memcpy(cc, &s.v[12 * (size_t)L.g], 48);
        float mag = 0.f;
        for (int k = 0; k < 4; ++k)
            for (int a = 0; a < 3; ++a)
                if (std::fabs(cc[k][a]) < INFINITY) mag = std::max(mag, std::fabs(cc[k][a]));
        const float pad = 4e-6f * mag;
        for (int a = 0; a < 3; ++a) {
            lbox[i].lo[a] = std::fmin(std::fmin(cc[0][a], cc[1][a]), std::fmin(cc[2][a], cc[3][a])) - pad;
            lbox[i].hi[a] = std::fmax(std::fmax(cc[0][a], cc[1][a]), std::fmax(cc[2][a], cc[3][a])) + pad;
        }
    }
    for (uint32_t g = 0; g < n; ++g) CHECK(seen[g] == 1, "%s: surfel %u appears %d times", what, g, seen[g]);
    if (n < 2) return 0;
    // walk from the root
    std::vector<int> node_seen(n - 1, 0), leaf_seen(n, 0);
    std::vector<Box> nbox(n - 1);
    std::vector<std::pair<uint32_t, uint32_t>> stack{{0u, 1u}};
    std::vector<uint32_t> order;
    uint32_t depth = 0;
    CHECK(c.node_parent[0] == DST_NO_PARENT, "%s: root parent", what);
    while (!stack.empty()) {
        auto [i, d] = stack.back();
        stack.pop_back();
        if (i + 1 >= n) { CHECK(false, "%s: node index %u", what, i); continue; }
        if (node_seen[i]++) { CHECK(false, "%s: node %u reached twice", what, i); continue; }
        order.push_back(i);
        depth = std::max(depth, d);
        const DstNode &nd = c.nodes[i];
        const uint32_t split = nd.c0 & ~DST_LEAF_BIT;
        CHECK(nd.first <= split && split < nd.last && nd.last < n, "%s: node %u range %u %u %u", what, i, nd.first, split, nd.last);
        CHECK((nd.c1 & ~DST_LEAF_BIT) == split + 1, "%s: node %u right child", what, i);
        CHECK(((nd.c0 & DST_LEAF_BIT) != 0) == (split == nd.first), "%s: node %u left leaf flag", what, i);
        CHECK(((nd.c1 & DST_LEAF_BIT) != 0) == (split + 1 == nd.last), "%s: node %u right leaf flag", what, i);
        CHECK(i == 0 || i == nd.first || i == nd.last, "%s: node %u is neither end of its range", what, i);
        const uint32_t cs[2] = {nd.c0, nd.c1};
        for (uint32_t w = 0; w < 2; ++w) {
            if (cs[w] & DST_LEAF_BIT) {
                const uint32_t j = cs[w] & ~DST_LEAF_BIT;
                if (j >= n) { CHECK(false, "%s: leaf index", what); continue; }
                CHECK(leaf_seen[j]++ == 0, "%s: leaf %u twice", what, j);
                CHECK(c.leaf_parent[j] == ((i << 1) | w), "%s: leaf %u parent", what, j);
            } else {
                if (cs[w] + 1 >= n) { CHECK(false, "%s: child index", what); continue; }
                CHECK(c.node_parent[cs[w]] == ((i << 1) | w), "%s: node %u parent", what, cs[w]);
                const DstNode &ch = c.nodes[cs[w]];
                CHECK(w == 0 ? (ch.first == nd.first && ch.last == split) : (ch.first == split + 1 && ch.last == nd.last),
                      "%s: child range of node %u", what, i);
                stack.push_back({cs[w], d + 1});
            }
        }
    }
    for (uint32_t i = 0; i + 1 < n; ++i) CHECK(node_seen[i] == 1, "%s: node %u reached %d times", what, i, node_seen[i]);
    for (uint32_t i = 0; i < n; ++i) CHECK(leaf_seen[i] == 1, "%s: leaf %u reached %d times", what, i, leaf_seen[i]);
    if (failures) return depth;
    // boxes: exact unions, bottom-up
    for (size_t k = order.size(); k-- > 0;) {
        const uint32_t i = order[k];
        const DstNode &nd = c.nodes[i];
        Box b[2];
        const uint32_t cs[2] = {nd.c0, nd.c1};
        for (int w = 0; w < 2; ++w) b[w] = (cs[w] & DST_LEAF_BIT) ? lbox[cs[w] & ~DST_LEAF_BIT] : nbox[cs[w]];
        CHECK(same_box(nd.lo0, nd.hi0, b[0]) && same_box(nd.lo1, nd.hi1, b[1]), "%s: boxes of node %u", what, i);
        for (int a = 0; a < 3; ++a) {
            nbox[i].lo[a] = std::fmin(b[0].lo[a], b[1].lo[a]);
            nbox[i].hi[a] = std::fmax(b[0].hi[a], b[1].hi[a]);
        }
    }
    // the wide nodes: from the root every leaf is reached once; a child's box is its binary node's (or leaf group's)
    if (n > DST_GROUP) {
        std::vector<int> hit(n, 0);
        struct Item { uint32_t ref, depth; };
        std::vector<Item> st{{0u, 1u}};
        uint32_t wdepth = 0, steps = 0;
        while (!st.empty() && steps++ < 4 * n) {
            Item it = st.back();
            st.pop_back();
            if (it.ref & DST_LEAF_BIT) {
                const uint32_t first = it.ref & DST_REF_FIRST_MASK, count = ((it.ref >> 28) & 7u) + 1u;
                CHECK(first + count <= n && count <= DST_GROUP, "%s: leaf group %u+%u", what, first, count);
                for (uint32_t q = 0; q < count && first + q < n; ++q) hit[first + q]++;
                continue;
            }
            if (it.ref + 1 >= n) { CHECK(false, "%s: wide index", what); continue; }
            wdepth = std::max(wdepth, it.depth);
            const DstWideNode &w = c.wide[it.ref];
            CHECK(w.count >= 2 && w.count <= DST_WIDE, "%s: wide node %u has %u children", what, it.ref, w.count);
            const DstNode &nd = c.nodes[it.ref];
            uint32_t at = nd.first;
            for (uint32_t k = 0; k < w.count && k < DST_WIDE; ++k) {
                const uint32_t r = w.ref[k];
                uint32_t f, l;
                if (r & DST_LEAF_BIT) { f = r & DST_REF_FIRST_MASK; l = f + ((r >> 28) & 7u); }
                else if (r + 1 < n) { f = c.nodes[r].first; l = c.nodes[r].last; }
                else { CHECK(false, "%s: wide child", what); continue; }
                CHECK(f == at, "%s: children of wide node %u are not in leaf order", what, it.ref);
                at = l + 1;
                Box u = lbox[f];
                for (uint32_t j = f + 1; j <= l && j < n; ++j)
                    for (int a = 0; a < 3; ++a) { u.lo[a] = std::fmin(u.lo[a], lbox[j].lo[a]); u.hi[a] = std::fmax(u.hi[a], lbox[j].hi[a]); }
                const float lo[3] = {w.lox[k], w.loy[k], w.loz[k]}, hi[3] = {w.hix[k], w.hiy[k], w.hiz[k]};
                CHECK(same_box(lo, hi, u), "%s: box of child %u of wide node %u", what, k, it.ref);
                st.push_back({r, it.depth + 1});
            }
            CHECK(at == nd.last + 1, "%s: wide node %u does not cover its range", what, it.ref);
        }
        for (uint32_t i = 0; i < n; ++i) CHECK(hit[i] == 1, "%s: leaf %u is in %d leaf groups", what, i, hit[i]);
        CHECK(3 * wdepth <= 126, "%s: wide hierarchy %u deep, the walks' stacks hold 128 entries", what, wdepth);
    }
    return depth;
}

void run_case(uint32_t P, int kind, bool agglomerate, uint32_t seed) {
    char what[128];
    std::snprintf(what, sizeof(what), "P=%u kind=%d %s", P, kind, agglomerate ? "agglomerated" : "morton");
    Scene s = make_scene(P, kind, seed);
    dst_ctx ctx;
    ctx.use_ploc = agglomerate;
    int rc = dst_lbvh_build(&ctx, s.v.data(), 4 * P, s.f.data(), P, true, nullptr);
    CHECK(rc == DST_OK, "%s: build returned %d (%s)", what, rc, ctx.err.c_str());
    if (rc != DST_OK) return;
    const uint32_t depth = check_structure(ctx, s, what);
    std::printf("%-40s depth %2u agglomerated %d refused %d key levels %d\n", what, depth, (int)ctx.agglomerated,
                (int)ctx.ploc_refused, ctx.fine_keys ? 2 : 1);
    CHECK(!agglomerate || P < 64 || ctx.agglomerated || ctx.ploc_refused, "%s: not agglomerated", what);
    CHECK(!ctx.agglomerated || ctx.hierarchy_depth == depth, "%s: reported depth %u", what, ctx.hierarchy_depth);
    // a refit on moved geometry keeps order and topology and fits the boxes again (both fits)
    std::vector<uint32_t> order(P);
    for (uint32_t i = 0; i < P; ++i) order[i] = ctx.leaves[i].g;
    Scene moved = s;
    std::mt19937 rng(seed + 1);
    std::normal_distribution<float> N(0.f, 0.1f);
    for (uint32_t g = 0; g < P; g += 2) {
        const float d[3] = {N(rng), N(rng), N(rng)};
        for (int k = 0; k < 4; ++k)
            for (int a = 0; a < 3; ++a) moved.v[12 * (size_t)g + 3 * k + a] += d[a];
    }
    rc = dst_lbvh_build(&ctx, moved.v.data(), 4 * P, nullptr, P, false, nullptr);
    CHECK(rc == DST_OK, "%s: refit returned %d", what, rc);
    check_structure(ctx, moved, what);
    for (uint32_t i = 0; i < P; ++i) CHECK(order[i] == ctx.leaves[i].g, "%s: refit moved leaf %u", what, i);
    if (P <= DST_STATIC_REFIT_MAX_SURFELS && P > 1) {   // the climbing fit with caller-provided counters
        std::vector<uint32_t> counters(P);
        rc = dst_lbvh_build(&ctx, s.v.data(), 4 * P, nullptr, P, false, nullptr, counters.data());
        CHECK(rc == DST_OK, "%s: climbing refit returned %d", what, rc);
        check_structure(ctx, s, what);
    }
    dst_lbvh_free(&ctx);
    std::free(ctx.bounds);
    std::free(ctx.core_box);
    std::free(ctx.bounds_host);
    std::free(ctx.ploc_host);
}

}  // namespace

int main(int argc, char **argv) {
    std::setvbuf(stdout, nullptr, _IONBF, 0);
    if (argc == 4) {   // one case: surfels, kind of scene, agglomerate
        run_case((uint32_t)std::atoi(argv[1]), std::atoi(argv[2]), std::atoi(argv[3]) != 0, 1);
        std::printf(failures ? "FAILED: %d checks\n" : "ALL OK\n", failures);
        return failures ? 1 : 0;
    }
    const bool quick = argc > 1 && std::string(argv[1]) == "quick";
    const uint32_t sizes[] = {1, 2, 3, 63, 64, 65, 100, 1024, 1025, 2500, 5000};
    for (int agg = 1; agg >= 0; --agg) {
        for (uint32_t P : sizes) {
            if (quick && P > 2500) continue;
            run_case(P, 0, agg != 0, 11 + P);
        }
        run_case(3000, 1, agg != 0, 5);
        run_case(3000, 2, agg != 0, 6);
        run_case(3000, 3, agg != 0, 7);
        run_case(4000, 4, agg != 0, 8);
    }
    std::printf(failures ? "FAILED: %d checks\n" : "ALL OK\n", failures);
    return failures ? 1 : 0;
}
