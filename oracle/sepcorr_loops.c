/*
 * CPU loop restatement of the memory-saving separation ops.  TEST INFRASTRUCTURE ONLY:
 * it checks the HIP kernels and the torch oracle; the shipped library never links it.
 *
 * Each function follows one of the reference's straight-loop ("unoptimized") kernels,
 * one image-1 pixel (b,i,j) per outer iteration, with the same update rules:
 *   sep_max_argmax_avg_forward_*  <- MemorySaver_kernel_forward.cu:766-819 (max/avg) and
 *                                    :498-507 (strict '<' update => lowest index wins ties)
 *   sep_compression_forward_*     <- MemorySaver_kernel_forward.cu:834-889
 *   sep_max_argmax_avg_backward_* <- MemorySaver_kernel_max_avg_argmax_backward.cu:785-923
 *   sep_compression_backward_*    <- MemorySaver_kernel_compression_backward.cu:417-508
 * Differences on purpose: dF2 is accumulated per (u,v) owner instead of atomicAdd (the sum
 * is the same, the order is fixed); outputs are written, not accumulated into pre-initialised
 * buffers; argmax entries outside the axis select nothing instead of indexing out of range.
 *
 * Built twice by the Makefile: REAL=float (suffix _f32) and REAL=double (suffix _f64).
 * Layouts (all contiguous): f1 (B,H1,W1,C), f2 (B,H2,W2,C), *_u (B,H1,W1,ch,H2),
 * *_v (B,H1,W1,ch,W2), argmax int32 with ch=1.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef REAL
#define REAL float
#endif
#ifndef SUFFIX
#define SUFFIX _f32
#endif
#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUFFIX)

static REAL dotc(const REAL *a, const REAL *b, int C) {
    REAL s = 0;
    for (int c = 0; c < C; ++c) s += a[c] * b[c];
    return s;
}

void FN(sep_max_argmax_avg_forward)(const REAL *f1, const REAL *f2, REAL *out_u, REAL *out_v,
                                    int32_t *am_u, int32_t *am_v, int B, int H1, int W1, int H2,
                                    int W2, int C) {
    const long N1 = (long)H1 * W1;
#pragma omp parallel for schedule(static)
    for (long bp = 0; bp < B * N1; ++bp) {
        const int b = (int)(bp / N1);
        const REAL *g1 = f1 + bp * C;
        REAL *mu = out_u + bp * 2 * H2, *au = mu + H2;
        REAL *mv = out_v + bp * 2 * W2, *av = mv + W2;
        int32_t *iu = am_u ? am_u + bp * H2 : NULL;
        int32_t *iv = am_v ? am_v + bp * W2 : NULL;
        for (int u = 0; u < H2; ++u) { mu[u] = -INFINITY; au[u] = 0; if (iu) iu[u] = 0; }
        for (int v = 0; v < W2; ++v) { mv[v] = -INFINITY; av[v] = 0; if (iv) iv[v] = 0; }
        for (int v = 0; v < W2; ++v)
            for (int u = 0; u < H2; ++u) {
                const REAL c = dotc(g1, f2 + (((long)b * H2 + u) * W2 + v) * C, C);
                if (mu[u] < c) { mu[u] = c; if (iu) iu[u] = v; }
                if (mv[v] < c) { mv[v] = c; if (iv) iv[v] = u; }
                au[u] += c / W2;
                av[v] += c / H2;
            }
    }
}

void FN(sep_compression_forward)(const REAL *f1, const REAL *f2, const REAL *a_u, const REAL *a_v,
                                 REAL *comp_u, REAL *comp_v, int B, int H1, int W1, int H2, int W2,
                                 int C, int K) {
    const long N1 = (long)H1 * W1;
#pragma omp parallel for schedule(static)
    for (long bp = 0; bp < B * N1; ++bp) {
        const int b = (int)(bp / N1);
        const REAL *g1 = f1 + bp * C;
        const REAL *wu = a_u + bp * K * W2, *wv = a_v + bp * K * H2;
        REAL *cu = comp_u + bp * K * H2, *cv = comp_v + bp * K * W2;
        memset(cu, 0, sizeof(REAL) * K * H2);
        memset(cv, 0, sizeof(REAL) * K * W2);
        for (int v = 0; v < W2; ++v)
            for (int u = 0; u < H2; ++u) {
                const REAL c = dotc(g1, f2 + (((long)b * H2 + u) * W2 + v) * C, C);
                for (int k = 0; k < K; ++k) {
                    cu[k * H2 + u] += c * wu[k * W2 + v];
                    cv[k * W2 + v] += c * wv[k * H2 + u];
                }
            }
    }
}

/* dF1[p,:] = sum_q G[p,q] f2[q,:]; dF2[q,:] = sum_p G[p,q] f1[p,:] for a caller-supplied G row. */
typedef void (*grow_fn)(const void *ctx, long bp, REAL *grow);

static void route_volume_grad(const REAL *f1, const REAL *f2, REAL *d1, REAL *d2, int B, int H1,
                              int W1, int H2, int W2, int C, grow_fn fill, const void *ctx) {
    const long N1 = (long)H1 * W1, N2 = (long)H2 * W2;
    /* G for one batch at a time, (N1,N2); tiny inputs only */
    REAL *G = (REAL *)malloc(sizeof(REAL) * N1 * N2);
    for (int b = 0; b < B; ++b) {
#pragma omp parallel for schedule(static)
        for (long p = 0; p < N1; ++p) {
            REAL *gr = G + p * N2;
            fill(ctx, b * N1 + p, gr);
            REAL *o = d1 + (b * N1 + p) * C;
            for (int c = 0; c < C; ++c) o[c] = 0;
            for (long q = 0; q < N2; ++q) {
                const REAL *g2 = f2 + (b * N2 + q) * C;
                for (int c = 0; c < C; ++c) o[c] += g2[c] * gr[q];
            }
        }
#pragma omp parallel for schedule(static)
        for (long q = 0; q < N2; ++q) {
            REAL *o = d2 + (b * N2 + q) * C;
            for (int c = 0; c < C; ++c) o[c] = 0;
            for (long p = 0; p < N1; ++p) {
                const REAL *g1 = f1 + (b * N1 + p) * C;
                const REAL g = G[p * N2 + q];
                for (int c = 0; c < C; ++c) o[c] += g1[c] * g;
            }
        }
    }
    free(G);
}

struct maxavg_ctx { const int32_t *am_u, *am_v; const REAL *g_u, *g_v; int H2, W2; };

static void maxavg_grow(const void *vctx, long bp, REAL *gr) {
    const struct maxavg_ctx *c = (const struct maxavg_ctx *)vctx;
    const int H2 = c->H2, W2 = c->W2;
    const int32_t *iu = c->am_u + bp * H2, *iv = c->am_v + bp * W2;
    const REAL *gmu = c->g_u + bp * 2 * H2, *gau = gmu + H2;
    const REAL *gmv = c->g_v + bp * 2 * W2, *gav = gmv + W2;
    for (int u = 0; u < H2; ++u)
        for (int v = 0; v < W2; ++v) {
            REAL g = gau[u] / W2 + gav[v] / H2;
            if (iu[u] == v) g += gmu[u];
            if (iv[v] == u) g += gmv[v];
            gr[(long)u * W2 + v] = g;
        }
}

void FN(sep_max_argmax_avg_backward)(const REAL *f1, const REAL *f2, const int32_t *am_u,
                                     const int32_t *am_v, const REAL *g_u, const REAL *g_v, REAL *d1,
                                     REAL *d2, int B, int H1, int W1, int H2, int W2, int C) {
    struct maxavg_ctx ctx = {am_u, am_v, g_u, g_v, H2, W2};
    route_volume_grad(f1, f2, d1, d2, B, H1, W1, H2, W2, C, maxavg_grow, &ctx);
}

struct comp_ctx { const REAL *a_u, *a_v, *g_cu, *g_cv; int H2, W2, K; };

static void comp_grow(const void *vctx, long bp, REAL *gr) {
    const struct comp_ctx *c = (const struct comp_ctx *)vctx;
    const int H2 = c->H2, W2 = c->W2, K = c->K;
    const REAL *wu = c->a_u + bp * K * W2, *wv = c->a_v + bp * K * H2;
    const REAL *gu = c->g_cu + bp * K * H2, *gv = c->g_cv + bp * K * W2;
    for (int u = 0; u < H2; ++u)
        for (int v = 0; v < W2; ++v) {
            REAL g = 0;
            for (int k = 0; k < K; ++k) g += wu[k * W2 + v] * gu[k * H2 + u] + wv[k * H2 + u] * gv[k * W2 + v];
            gr[(long)u * W2 + v] = g;
        }
}

void FN(sep_compression_backward)(const REAL *f1, const REAL *f2, const REAL *a_u, const REAL *a_v,
                                  const REAL *g_cu, const REAL *g_cv, REAL *d1, REAL *d2, REAL *da_u,
                                  REAL *da_v, int B, int H1, int W1, int H2, int W2, int C, int K) {
    struct comp_ctx ctx = {a_u, a_v, g_cu, g_cv, H2, W2, K};
    route_volume_grad(f1, f2, d1, d2, B, H1, W1, H2, W2, C, comp_grow, &ctx);
    const long N1 = (long)H1 * W1;
#pragma omp parallel for schedule(static)
    for (long bp = 0; bp < B * N1; ++bp) {
        const int b = (int)(bp / N1);
        const REAL *g1 = f1 + bp * C;
        const REAL *gu = g_cu + bp * K * H2, *gv = g_cv + bp * K * W2;
        REAL *du = da_u + bp * K * W2, *dv = da_v + bp * K * H2;
        memset(du, 0, sizeof(REAL) * K * W2);
        memset(dv, 0, sizeof(REAL) * K * H2);
        for (int u = 0; u < H2; ++u)
            for (int v = 0; v < W2; ++v) {
                const REAL cval = dotc(g1, f2 + (((long)b * H2 + u) * W2 + v) * C, C);
                for (int k = 0; k < K; ++k) {
                    du[k * W2 + v] += cval * gu[k * H2 + u];
                    dv[k * H2 + u] += cval * gv[k * W2 + v];
                }
            }
    }
}
