/*
 * CPU oracle for the fused camera->BEV pooling path.  TEST INFRASTRUCTURE ONLY:
 * tests, the smoke check and the benchmark's CPU-baseline leg link this file; the
 * product library never does.
 *
 * It restates, as one scalar loop nest in fp32 with every operation individually
 * rounded (build with -ffp-contract=off), the algorithm of the reference's fused
 * forward kernel and of its dense PyTorch pooling path:
 *   voxel centres, projection, perspective divide
 *       flashbev/flashbevpool/src/flash_bevpool_cuda.cu:45-46,102-132
 *       flashbev/flashbevpool/sampling_vt.py:364-378,449-466
 *   field-of-view mask, bilinear corner indices and weights
 *       flash_bevpool_cuda.cu:137-159, sampling_vt.py:56-63
 *   depth-parameter interpolation and Gaussian/Laplace likelihood, threshold
 *       flash_bevpool_cuda.cu:161-188, sampling_vt.py:82-112
 *   feature interpolation, accumulation, mean over valid (camera, height) samples
 *       flash_bevpool_cuda.cu:190-216, sampling_vt.py:74-80,114-121
 * The backward pass is the exact derivative of that forward (what autograd gives on
 * sampling_vt.py:36-123), NOT the reference CUDA backward
 * (flash_bevpool_cuda.cu:665-674), which adds the same term to the mean and sigma
 * slots and omits d(weight)/d(mean), d(weight)/d(sigma).
 *
 * Depth model 2 ("categorical": per-pixel probabilities over D depth bins,
 * interpolated linearly along depth) has no counterpart in the reference:
 * parity unpinned by the reference; it is pinned only by the dense restatement and
 * the invariants in tests/.
 *
 * Pinning of this file (tests/test_oracle_pinning.py): closed-form projections in
 * binary-friendly numbers (optical-axis point, behind the camera, the last-column clamp),
 * textbook likelihood values at the mean and at one sigma, threshold and categorical-bin
 * cases, torch grid_sample(bilinear, border, align_corners=True) as the library routine
 * the interpolation reduces to (this file against the dense path, up to the benchmark's
 * largest shapes), linearity / constant-feature / camera-permutation invariants, and for
 * the gradients float64 autograd, gradcheck, central differences and the adjoint identity.
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <stdlib.h>

typedef struct {
    int32_t B, N, H, W, C;
    int32_t Hi, Wi;
    int32_t gx, gy, gz;
    float roi[6];      /* xmin xmax ymin ymax zmin zmax */
    float eps;
    float thr;
    int32_t dist;      /* 0 gaussian, 1 laplace, 2 categorical */
    int32_t D;         /* channels of the depth tensor: 2, or number of bins */
    float dmin, dstep; /* categorical: bin k sits at dmin + k*dstep */
    int32_t reduce_sum;/* 0: mean over valid samples (reference), 1: plain sum */
    double step[3];    /* cell size along x, y, z; 0: (hi - lo) / n in float64 (the canonical one) */
} oracle_problem;

typedef struct {
    int valid;          /* projection / field-of-view validity */
    int u0, u1, v0, v1;
    float du, dv;
    float w00, w01, w10, w11; /* (v0,u0) (v1,u0) (v0,u1) (v1,u1) */
    float depth;        /* raw projected depth D */
    float fu, fv;
} sample_geom;

static inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* One (cell, camera, height-bin) sample in the canonical operation order. */
static inline void project_sample(const oracle_problem *p, const float *P,
                                  float x, float y, float z, sample_geom *g)
{
    float U = ((P[0] * x + P[1] * y) + P[2] * z) + P[3];
    float V = ((P[4] * x + P[5] * y) + P[6] * z) + P[7];
    float Dp = ((P[8] * x + P[9] * y) + P[10] * z) + P[11];
    memset(g, 0, sizeof(*g));
    g->depth = Dp;
    if (!(Dp > 0.0f)) return;
    float dc = fmaxf(Dp, p->eps);
    float ui = U / dc;
    float vi = V / dc;
    float fu = (ui / (float)p->Wi) * (float)p->W;
    float fv = (vi / (float)p->Hi) * (float)p->H;
    g->fu = fu; g->fv = fv;
    if (!(fu >= 0.0f && fu < (float)p->W && fv >= 0.0f && fv < (float)p->H)) return;
    float u0f = floorf(fu), v0f = floorf(fv);
    g->du = fu - u0f;
    g->dv = fv - v0f;
    g->u0 = clampi((int)u0f, 0, p->W - 1);
    g->u1 = clampi(g->u0 + 1, 0, p->W - 1);
    g->v0 = clampi((int)v0f, 0, p->H - 1);
    g->v1 = clampi(g->v0 + 1, 0, p->H - 1);
    g->w00 = (1.0f - g->du) * (1.0f - g->dv);
    g->w01 = (1.0f - g->du) * g->dv;
    g->w10 = g->du * (1.0f - g->dv);
    g->w11 = g->du * g->dv;
    g->valid = 1;
}

/*
 * Centre of cell i along one axis: the float64 value lo + (i + 0.5) * (hi - lo) / n, rounded once
 * to fp32 (the roi bounds are fp32 values, widened exactly).  The reference's dense path takes
 * linspace(lo, hi, n + 1)[:-1] + step / 2 (sampling_vt.py:364-378), its fused kernel
 * lo + (i + 0.5) * fp32(step) (flash_bevpool_cuda.cu:45-46); the second accumulates the rounding
 * of the fp32 step along the axis (0.8 m is not an fp32 number), which a Gaussian tail weight
 * magnifies beyond the parity tolerance, so the correctly rounded centre is the canonical one.
 */
static inline float voxel_centre(float lo, float hi, int n, int i, double given_step)
{
    /* (a caller of the operator's extension may hand over its own cell size, e.g. the fp32 quotient the
     * reference's Python forms, flash_bevpool.py:62-64: then that size is the step) */
    double step = given_step > 0.0 ? given_step : ((double)hi - (double)lo) / (double)n;
    return (float)((double)lo + ((double)i + 0.5) * step);
}

static inline float bilerp(const sample_geom *g, float a00, float a01, float a10, float a11)
{
    return ((g->w00 * a00 + g->w01 * a01) + g->w10 * a10) + g->w11 * a11;
}

typedef struct {
    float wgt;      /* depth weight */
    float dmu, dsg; /* parametric: d wgt / d mean, d wgt / d sigma */
    int k0, k1;     /* categorical: the two bins and the mix */
    float r;
    int keep;       /* passes the categorical range test and the weight threshold */
} depth_eval;

/* depth points at the [H,W,D] block of camera (b,n). */
static inline void eval_depth(const oracle_problem *p, const float *depth,
                              const sample_geom *g, depth_eval *e)
{
    const int W = p->W, Dd = p->D;
    const float *c00 = depth + ((size_t)g->v0 * W + g->u0) * Dd;
    const float *c01 = depth + ((size_t)g->v1 * W + g->u0) * Dd;
    const float *c10 = depth + ((size_t)g->v0 * W + g->u1) * Dd;
    const float *c11 = depth + ((size_t)g->v1 * W + g->u1) * Dd;
    memset(e, 0, sizeof(*e));
    if (p->dist == 2) {
        float t = (g->depth - p->dmin) / p->dstep;
        if (!(t >= 0.0f && t <= (float)(Dd - 1))) return;
        float k0f = floorf(t);
        e->k0 = clampi((int)k0f, 0, Dd - 1);
        e->k1 = clampi(e->k0 + 1, 0, Dd - 1);
        e->r = t - k0f;
        float p0 = bilerp(g, c00[e->k0], c01[e->k0], c10[e->k0], c11[e->k0]);
        float p1 = bilerp(g, c00[e->k1], c01[e->k1], c10[e->k1], c11[e->k1]);
        e->wgt = (1.0f - e->r) * p0 + e->r * p1;
    } else {
        float mu = bilerp(g, c00[0], c01[0], c10[0], c11[0]);
        float sg = bilerp(g, c00[1], c01[1], c10[1], c11[1]);
        float s = sg + p->eps;
        float zs = (g->depth - mu) / s;
        if (p->dist == 0) {
            e->wgt = expf((-0.5f * zs) * zs) / s;
            e->dmu = e->wgt * zs / s;
            e->dsg = e->wgt * (zs * zs - 1.0f) / s;
        } else {
            e->wgt = (0.5f * expf(-fabsf(zs))) / s;
            float sgn = (zs > 0.0f) ? 1.0f : ((zs < 0.0f) ? -1.0f : 0.0f);
            e->dmu = e->wgt * sgn / s;
            e->dsg = e->wgt * (fabsf(zs) - 1.0f) / s;
        }
    }
    e->keep = !(e->wgt < p->thr);
}

/*
 * Per-sample geometry, sample order [B, gy, gx, N, gz].
 * mask: uint8; idx: int32 x4 (u0,u1,v0,v1); frac: float x2 (du,dv); depth: float.
 * Any output may be NULL.
 */
void fbev_oracle_geometry(const oracle_problem *p, const float *proj /* [B,N,12] */,
                          uint8_t *mask, int32_t *idx, float *frac, float *depth_out)
{
    size_t s = 0;
    for (int b = 0; b < p->B; ++b)
        for (int iy = 0; iy < p->gy; ++iy)
            for (int ix = 0; ix < p->gx; ++ix) {
                float x = voxel_centre(p->roi[0], p->roi[1], p->gx, ix, p->step[0]);
                float y = voxel_centre(p->roi[2], p->roi[3], p->gy, iy, p->step[1]);
                for (int n = 0; n < p->N; ++n)
                    for (int iz = 0; iz < p->gz; ++iz, ++s) {
                        float z = voxel_centre(p->roi[4], p->roi[5], p->gz, iz, p->step[2]);
                        sample_geom g;
                        project_sample(p, proj + ((size_t)b * p->N + n) * 12, x, y, z, &g);
                        if (mask) mask[s] = (uint8_t)g.valid;
                        if (idx) {
                            idx[4 * s + 0] = g.valid ? g.u0 : -1;
                            idx[4 * s + 1] = g.valid ? g.u1 : -1;
                            idx[4 * s + 2] = g.valid ? g.v0 : -1;
                            idx[4 * s + 3] = g.valid ? g.v1 : -1;
                        }
                        if (frac) {
                            frac[2 * s + 0] = g.valid ? g.du : 0.0f;
                            frac[2 * s + 1] = g.valid ? g.dv : 0.0f;
                        }
                        if (depth_out) depth_out[s] = g.depth;
                    }
            }
}

/*
 * Forward.  depth [B,N,H,W,D], feats [B,N,H,W,C], proj [B,N,12], out [B,gy,gx,C].
 * count (optional) [B,gy,gx]: number of samples that entered the mean.
 * keep (optional) uint8 [B,gy,gx,N,gz]: sample passed FOV and threshold tests.
 */
void fbev_oracle_forward(const oracle_problem *p, const float *depth, const float *feats,
                         const float *proj, float *out, float *count, uint8_t *keep)
{
    const int C = p->C, H = p->H, W = p->W;
    float *acc = (float *)malloc(sizeof(float) * (size_t)C);
    size_t s = 0;
    for (int b = 0; b < p->B; ++b)
        for (int iy = 0; iy < p->gy; ++iy)
            for (int ix = 0; ix < p->gx; ++ix) {
                float x = voxel_centre(p->roi[0], p->roi[1], p->gx, ix, p->step[0]);
                float y = voxel_centre(p->roi[2], p->roi[3], p->gy, iy, p->step[1]);
                for (int c = 0; c < C; ++c) acc[c] = 0.0f;
                float cnt = 0.0f;
                for (int n = 0; n < p->N; ++n) {
                    size_t cam = (size_t)b * p->N + n;
                    const float *dcam = depth + cam * H * W * p->D;
                    const float *fcam = feats + cam * H * W * C;
                    for (int iz = 0; iz < p->gz; ++iz, ++s) {
                        float z = voxel_centre(p->roi[4], p->roi[5], p->gz, iz, p->step[2]);
                        sample_geom g;
                        if (keep) keep[s] = 0;
                        project_sample(p, proj + cam * 12, x, y, z, &g);
                        if (!g.valid) continue;
                        depth_eval e;
                        eval_depth(p, dcam, &g, &e);
                        if (!e.keep) continue;
                        if (keep) keep[s] = 1;
                        const float *f00 = fcam + ((size_t)g.v0 * W + g.u0) * C;
                        const float *f01 = fcam + ((size_t)g.v1 * W + g.u0) * C;
                        const float *f10 = fcam + ((size_t)g.v0 * W + g.u1) * C;
                        const float *f11 = fcam + ((size_t)g.v1 * W + g.u1) * C;
                        for (int c = 0; c < C; ++c) {
                            float f = bilerp(&g, f00[c], f01[c], f10[c], f11[c]);
                            acc[c] += f * e.wgt;
                        }
                        cnt += 1.0f;
                    }
                }
                float *o = out + (((size_t)b * p->gy + iy) * p->gx + ix) * C;
                for (int c = 0; c < C; ++c)
                    o[c] = p->reduce_sum ? acc[c] : (cnt > 0.0f ? acc[c] / cnt : 0.0f);
                if (count) count[((size_t)b * p->gy + iy) * p->gx + ix] = cnt;
            }
    free(acc);
}

/*
 * Backward: true gradient of fbev_oracle_forward w.r.t. feats and depth.
 * Sums are carried in float64 and rounded once, because the summation order of a
 * scatter is not part of the contract.  d_depth [B,N,H,W,D], d_feats [B,N,H,W,C].
 */
void fbev_oracle_backward(const oracle_problem *p, const float *grad_out, const float *depth,
                          const float *feats, const float *proj, float *d_depth, float *d_feats)
{
    const int C = p->C, H = p->H, W = p->W, Dd = p->D, NZ = p->N * p->gz;
    size_t n_feat = (size_t)p->B * p->N * H * W * C;
    size_t n_dep = (size_t)p->B * p->N * H * W * Dd;
    double *af = (double *)calloc(n_feat, sizeof(double));
    double *ad = (double *)calloc(n_dep, sizeof(double));
    sample_geom *gs = (sample_geom *)malloc(sizeof(sample_geom) * (size_t)NZ);
    depth_eval *es = (depth_eval *)malloc(sizeof(depth_eval) * (size_t)NZ);
    for (int b = 0; b < p->B; ++b)
        for (int iy = 0; iy < p->gy; ++iy)
            for (int ix = 0; ix < p->gx; ++ix) {
                float x = voxel_centre(p->roi[0], p->roi[1], p->gx, ix, p->step[0]);
                float y = voxel_centre(p->roi[2], p->roi[3], p->gy, iy, p->step[1]);
                int cnt = 0;
                for (int n = 0; n < p->N; ++n) {
                    size_t cam = (size_t)b * p->N + n;
                    for (int iz = 0; iz < p->gz; ++iz) {
                        int k = n * p->gz + iz;
                        float z = voxel_centre(p->roi[4], p->roi[5], p->gz, iz, p->step[2]);
                        project_sample(p, proj + cam * 12, x, y, z, &gs[k]);
                        es[k].keep = 0;
                        if (!gs[k].valid) continue;
                        eval_depth(p, depth + cam * H * W * Dd, &gs[k], &es[k]);
                        cnt += es[k].keep;
                    }
                }
                if (cnt == 0) continue;
                double inv = p->reduce_sum ? 1.0 : 1.0 / (double)cnt;
                const float *go = grad_out + (((size_t)b * p->gy + iy) * p->gx + ix) * C;
                for (int k = 0; k < NZ; ++k) {
                    if (!es[k].keep) continue;
                    const sample_geom *g = &gs[k];
                    const depth_eval *e = &es[k];
                    size_t cam = (size_t)b * p->N + k / p->gz;
                    size_t t00 = (cam * H + g->v0) * W + g->u0, t01 = (cam * H + g->v1) * W + g->u0;
                    size_t t10 = (cam * H + g->v0) * W + g->u1, t11 = (cam * H + g->v1) * W + g->u1;
                    double G = 0.0;
                    for (int c = 0; c < C; ++c) {
                        double gc = (double)go[c] * inv;
                        double f = (double)g->w00 * feats[t00 * C + c] + (double)g->w01 * feats[t01 * C + c]
                                 + (double)g->w10 * feats[t10 * C + c] + (double)g->w11 * feats[t11 * C + c];
                        G += gc * f;
                        double gw = gc * (double)e->wgt;
                        af[t00 * C + c] += gw * g->w00;
                        af[t01 * C + c] += gw * g->w01;
                        af[t10 * C + c] += gw * g->w10;
                        af[t11 * C + c] += gw * g->w11;
                    }
                    if (p->dist == 2) {
                        double a = G * (1.0 - (double)e->r), bq = G * (double)e->r;
                        ad[t00 * Dd + e->k0] += a * g->w00; ad[t00 * Dd + e->k1] += bq * g->w00;
                        ad[t01 * Dd + e->k0] += a * g->w01; ad[t01 * Dd + e->k1] += bq * g->w01;
                        ad[t10 * Dd + e->k0] += a * g->w10; ad[t10 * Dd + e->k1] += bq * g->w10;
                        ad[t11 * Dd + e->k0] += a * g->w11; ad[t11 * Dd + e->k1] += bq * g->w11;
                    } else {
                        double a = G * (double)e->dmu, bq = G * (double)e->dsg;
                        ad[t00 * 2] += a * g->w00; ad[t00 * 2 + 1] += bq * g->w00;
                        ad[t01 * 2] += a * g->w01; ad[t01 * 2 + 1] += bq * g->w01;
                        ad[t10 * 2] += a * g->w10; ad[t10 * 2 + 1] += bq * g->w10;
                        ad[t11 * 2] += a * g->w11; ad[t11 * 2 + 1] += bq * g->w11;
                    }
                }
            }
    for (size_t i = 0; i < n_feat; ++i) d_feats[i] = (float)af[i];
    for (size_t i = 0; i < n_dep; ++i) d_depth[i] = (float)ad[i];
    free(af); free(ad); free(gs); free(es);
}

size_t fbev_oracle_problem_size(void) { return sizeof(oracle_problem); }
