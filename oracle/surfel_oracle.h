/*
 * CPU oracle for the differentiable surfel ray tracer -- TEST INFRASTRUCTURE ONLY.
 *
 * This is a CPU restatement of the reference device programs
 * (optix_tracer/forward.cu, optix_tracer/backward.cu, the live part of
 * optix_tracer/auxiliary.h).  Only tests, the smoke check and the benchmark's
 * cpu_baseline leg may load it; the shipped library never does.
 *
 * Hit enumeration (owned by NVIDIA OptiX in the reference, which is not part
 * of the reference tree) is DEFINED here, see surfel_oracle.cpp: parity of
 * that part against OptiX itself is unpinned.
 *
 * Parity unpinned (transcribed from the cited lines and reviewed, but checked
 * by no independent test, because the reference deviates from the true
 * gradient there and nothing but the reference itself says how):
 *   - bounce_backward(): the flow of dL/dacc (the reference never accumulates
 *     the weight sum W, backward.cu:568);
 *   - path_backward(): the part of a bounce's gradient that reaches the
 *     previous bounce through the reflected ray's origin and direction
 *     (backward.cu:700-790).
 * Everything else is pinned by tests/test_oracle_*.py: scalar functions against
 * numpy/scipy, the ray/quad test against float64 Moeller-Trumbore, hit ordering
 * against brute force, compositing against closed forms, gradients (depth 0
 * and the bounce weighting at depth 1) against torch autograd of an
 * independent float64 forward.
 */
#ifndef SURFEL_ORACLE_H
#define SURFEL_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* How candidate hits are enumerated and inserted into the 16-entry buffer. */
enum {
    ORACLE_HITS_BRUTE_LITERAL = 0, /* all quads in ascending primitive order, reference any-hit rule */
    ORACLE_HITS_BRUTE_LEXI = 1,    /* all quads, (t, idx) lexicographic rule (arrival-order independent) */
    ORACLE_HITS_BVH_LEXI = 2       /* median-split CPU BVH, lexicographic rule (fast; used for the CPU baseline) */
};

typedef struct OracleParams {
    /* sizes */
    int32_t P, H, W;       /* surfels, ray grid */
    int32_t D, M;          /* SH degree, SH coefficients per surfel (0 if colors_precomp) */
    int32_t aux;           /* auxiliary channels (reference AUX_CHANNELS = 2) */
    int32_t mtd_alloc;     /* mid_val holds (mtd_alloc + 1) slots per ray (reference MAX_TRACE_DEPTH = 1) */
    int32_t training, start_from_first, max_trace_depth;
    float specular_threshold;
    /* oracle controls */
    int32_t hit_mode;      /* ORACLE_HITS_* */
    int32_t literal_stale; /* 1: keep the reference's stale slot on a repeated surfel (forward.cu:207-208) */
    int32_t n_threads;     /* OpenMP threads, 0 = default */
    /* inputs */
    const float *ray_o, *ray_d;   /* (H,W,3) */
    const float *vertices;        /* (4P,3) */
    const int32_t *faces;         /* (2P,3) */
    const float *background;      /* (3) */
    const float *means3D;         /* (P,3) */
    const float *shs;             /* (P,M,3) or NULL */
    const float *colors_precomp;  /* (P,3) or NULL */
    const float *others_precomp;  /* (P,aux) or NULL */
    const float *opacities;       /* (P,1) */
    const float *scales;          /* (P,2) */
    const float *rotations;       /* (P,4) */
    /* forward outputs (backward inputs) */
    float *out_rgb, *out_dpt, *out_acc, *out_norm, *out_dist, *out_aux; /* (H,W,{3,1,1,3,3,aux}) */
    float *mid_val;               /* (H,W,(mtd_alloc+1)*(14+aux)) */
    float *a_weights;             /* (P) or NULL */
    /* optional per-ray counters (forward): entries that reach the uv evaluation / composited hits */
    int32_t *n_proc, *n_con;      /* (H*W) or NULL */
    double *trace_seconds;        /* optional: wall time of the ray loop alone (set-up and CPU BVH build excluded) */
    /* upstream gradients */
    const float *dL_drgb, *dL_ddpt, *dL_dacc, *dL_ddist, *dL_dnorm, *dL_daux;
    /* gradient outputs */
    float *dL_dray_o, *dL_dray_d;                     /* (H,W,3) */
    float *dL_dmeans3D, *dL_dgrads3D;                 /* (P,3) */
    float *dL_dshs;                                   /* (P,M,3) */
    float *dL_dcolors, *dL_dothers, *dL_dopacities;   /* (P,3) (P,aux) (P,1) */
    float *dL_dscales, *dL_drotations;                /* (P,2) (P,4) */
} OracleParams;

/* Both return 0 on success, nonzero on a malformed request. */
int oracle_trace_forward(const OracleParams *p);
int oracle_trace_backward(const OracleParams *p);

/* Scalar building blocks, exported so tests can pin them one by one. */
float oracle_expf(float x);
void oracle_sh_color(int deg, const float *sh /* (M,3) */, const float *dir, float *rgb, float *clamped);
void oracle_quat_to_rows(const float *rot, float *R /* 9, row-major rows u,v,n */);
/* Ray/quad test.  Returns 1 and fills t, tri (0/1) on a hit. */
int oracle_ray_quad(const float *o, const float *d, const float *A, const float *B, const float *C,
                    const float *Dv, float *t, int *tri);
/* k nearest hits of one ray: fills up to 16 (t, idx) pairs, returns the admission count. */
int oracle_k_nearest(const OracleParams *p, const float *o, const float *d, float *t16, uint32_t *idx16);
int oracle_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
