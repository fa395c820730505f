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
 * Parity unpinned: only the hit enumeration named above (the set of hits, the value
 * of t and the order of exactly tied depths as NVIDIA's OptiX would report them).
 * Everything else is pinned by tests/test_oracle_*.py: scalar functions against
 * numpy/scipy, the ray/quad test against float64 Moeller-Trumbore, hit ordering
 * against brute force, compositing against closed forms, and every gradient
 * against torch autograd of an independent float64 forward: depth 0, the flow of
 * dL/dacc (the reference never accumulates the weight sum W, backward.cu:568:
 * differentiated as the surrogate it is the exact gradient of), the helpers of
 * the reflection chain rule as Jacobians, and the whole multi-bounce chain with
 * the reflected rays left free (backward.cu:700-790; depth 1 and depth 2).
 * The kernel's text of the small formulas (exp, quaternion frame, SH
 * polynomials, ray/quad test) is the same as the text here, not an independent
 * derivation; those four are the ones pinned against numpy/scipy for that reason.
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
    int32_t compute_dist;  /* forward only.  0: out_dist stays zero, as in the reference (forward.cu:286 leaves the
                            * accumulation open).  1: out_dist = (depth distortion, M1, M2) of the primary ray as 2DGS
                            * defines them: dist += (m*m*(1-T) + M2 - 2*m*M1)*w, M1 += m*w, M2 += m*m*w with
                            * m = far/(far-near)*(1-near/depth), near 0.2, far 100 (auxiliary.h:20-21) */
    int32_t grad_f64;      /* backward only.  0: gradient algebra in float, operation by operation as the reference
                            * writes it (the restatement).  1: the same formulas in double on the same fp32 inputs,
                            * hits and decisions; the difference between the two shows how much of a float gradient
                            * value is rounding noise of an ill-conditioned formula (grazing hits, sums that cancel) */
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
    /* optional, backward with grad_f64 only (all six or none): per element, the summed first-order change of the
     * geometric gradients when the rounded intermediates of the plane-hit chain (v1 - o, n.(v1-o), n.d) move by one
     * unit of fp32 rounding of their operands; how far two correct fp32 evaluations of the reference's formula can
     * be apart on that element.  Shapes as the gradients they belong to. */
    float *noise_ray_o, *noise_ray_d, *noise_means3D, *noise_grads3D, *noise_scales, *noise_rotations;
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
/* The three helpers of the reflection chain rule (auxiliary.h:111-121,234-252): which = 0 dnormvdv(v=a, dv=g),
 * 1 ddotndndn(n=a, d=b, g), 2 ddotndndd(n=a, d=b, g). */
void oracle_reflection_vjp(int which, const float *a, const float *b, const float *g, float *out);
/* k nearest hits of one ray: fills up to 16 (t, idx) pairs, returns the admission count. */
int oracle_k_nearest(const OracleParams *p, const float *o, const float *d, float *t16, uint32_t *idx16);
int oracle_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
