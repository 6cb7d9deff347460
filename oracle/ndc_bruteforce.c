/*
 * Brute-force float64 restatement of the NDC source update and its gradients.
 *
 * TEST INFRASTRUCTURE ONLY: loaded by tests/ (through oracle/bruteforce.py) to pin the
 * PyTorch oracle; never linked into or called from the shipped library.
 *
 * Plain nested loops, no library convolution, so that a mistake in how the PyTorch
 * oracle drives conv{1,2,3}d (a transposed channel pair, a flipped tap, a wrong pad)
 * cannot be shared.  Operator conventions follow
 * deconver/deconvolution/kernels.py:32-39 of the reference:
 *
 *   K(u)[o,p] = sum_{i,tau} u[i, p + tau - pad] * h[o,i,tau]     (cross-correlation)
 *   A(v)[i,p] = sum_{o,tau} v[o, p + pad - tau] * h[o,i,tau]     (adjoint of K)
 *
 * and the update / gradient formulas follow deconver/deconvolution/reference.py:169-173
 * and deconver/deconvolution/functional.py:97-182.
 *
 * Layout: x (B, G*m, D,H,W); z/out (B, G*sc, D,H,W); h (G, m, sc, kD,kH,kW); zero
 * padding k/2, stride 1.  Rank-1/2 inputs use leading extents of 1.
 */
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
    int B, G, m, sc, D, H, W, kD, kH, kW;
} bf_geom;

static inline size_t sp_of(const bf_geom *g) { return (size_t)g->D * g->H * g->W; }

static inline double at(const double *t, const bf_geom *g, int nch, int b, int ch, int d,
                        int h, int w)
{
    if (d < 0 || d >= g->D || h < 0 || h >= g->H || w < 0 || w >= g->W) return 0.0;
    return t[(((size_t)b * nch + ch) * g->D + d) * g->H * g->W + (size_t)h * g->W + w];
}

static inline double wt(const double *hf, const bf_geom *g, int grp, int o, int i, int td,
                        int th, int tw)
{
    return hf[((((size_t)grp * g->m + o) * g->sc + i) * g->kD + td) * g->kH * g->kW +
              (size_t)th * g->kW + tw];
}

/* out (B, G*m, S) = K(u), u (B, G*sc, S) */
void ndc_bf_K(const bf_geom *g, const double *u, const double *hf, double *out)
{
    const int pD = g->kD / 2, pH = g->kH / 2, pW = g->kW / 2;
    const int cin = g->G * g->sc, cout = g->G * g->m;
    for (int b = 0; b < g->B; ++b)
        for (int grp = 0; grp < g->G; ++grp)
            for (int o = 0; o < g->m; ++o)
                for (int d = 0; d < g->D; ++d)
                    for (int h = 0; h < g->H; ++h)
                        for (int w = 0; w < g->W; ++w) {
                            double acc = 0.0;
                            for (int i = 0; i < g->sc; ++i)
                                for (int td = 0; td < g->kD; ++td)
                                    for (int th = 0; th < g->kH; ++th)
                                        for (int tw = 0; tw < g->kW; ++tw)
                                            acc += at(u, g, cin, b, grp * g->sc + i,
                                                      d + td - pD, h + th - pH, w + tw - pW) *
                                                   wt(hf, g, grp, o, i, td, th, tw);
                            out[(((size_t)b * cout + grp * g->m + o) * g->D + d) * g->H * g->W +
                                (size_t)h * g->W + w] = acc;
                        }
}

/* out (B, G*sc, S) = A(v), v (B, G*m, S) */
void ndc_bf_A(const bf_geom *g, const double *v, const double *hf, double *out)
{
    const int pD = g->kD / 2, pH = g->kH / 2, pW = g->kW / 2;
    const int cin = g->G * g->m, cout = g->G * g->sc;
    for (int b = 0; b < g->B; ++b)
        for (int grp = 0; grp < g->G; ++grp)
            for (int i = 0; i < g->sc; ++i)
                for (int d = 0; d < g->D; ++d)
                    for (int h = 0; h < g->H; ++h)
                        for (int w = 0; w < g->W; ++w) {
                            double acc = 0.0;
                            for (int o = 0; o < g->m; ++o)
                                for (int td = 0; td < g->kD; ++td)
                                    for (int th = 0; th < g->kH; ++th)
                                        for (int tw = 0; tw < g->kW; ++tw)
                                            acc += at(v, g, cin, b, grp * g->m + o,
                                                      d + pD - td, h + pH - th, w + pW - tw) *
                                                   wt(hf, g, grp, o, i, td, th, tw);
                            out[(((size_t)b * cout + grp * g->sc + i) * g->D + d) * g->H * g->W +
                                (size_t)h * g->W + w] = acc;
                        }
}

static void rectify(const bf_geom *g, const double *z, const double *bias, int relu, double *s,
                    double *pre)
{
    const size_t sp = sp_of(g);
    const int cs = g->G * g->sc;
    for (int b = 0; b < g->B; ++b)
        for (int c = 0; c < cs; ++c)
            for (size_t p = 0; p < sp; ++p) {
                size_t idx = ((size_t)b * cs + c) * sp + p;
                double v = z[idx] + (bias ? bias[c] : 0.0);
                if (pre) pre[idx] = v;
                s[idx] = (relu && v < 0.0) ? 0.0 : v;
            }
}

/* out = s * (A(x)+eps) / (A(K(s))+eps), s = relu?(z + bias); t1 = K(s) also returned */
void ndc_bf_update(const bf_geom *g, const double *x, const double *z, const double *hf,
                   const double *bias, double eps, int relu, double *out, double *t1)
{
    const size_t sp = sp_of(g);
    const size_t ns = (size_t)g->B * g->G * g->sc * sp;
    double *s = (double *)malloc(ns * sizeof(double));
    double *n = (double *)malloc(ns * sizeof(double));
    double *d = (double *)malloc(ns * sizeof(double));
    rectify(g, z, bias, relu, s, NULL);
    ndc_bf_K(g, s, hf, t1);
    ndc_bf_A(g, x, hf, n);
    ndc_bf_A(g, t1, hf, d);
    for (size_t k = 0; k < ns; ++k) out[k] = s[k] * (n[k] + eps) / (d[k] + eps);
    free(s);
    free(n);
    free(d);
}

/* gradients of the update w.r.t. x, z, h, bias for an upstream gradient gout */
void ndc_bf_backward(const bf_geom *g, const double *x, const double *z, const double *hf,
                     const double *bias, const double *gout, double eps, int relu, double *gx,
                     double *gz, double *gh, double *gb)
{
    const size_t sp = sp_of(g);
    const int cs = g->G * g->sc, cx = g->G * g->m;
    const size_t ns = (size_t)g->B * cs * sp, nx = (size_t)g->B * cx * sp;
    const int pD = g->kD / 2, pH = g->kH / 2, pW = g->kW / 2;
    double *s = (double *)malloc(ns * sizeof(double));
    double *pre = (double *)malloc(ns * sizeof(double));
    double *n = (double *)malloc(ns * sizeof(double));
    double *d = (double *)malloc(ns * sizeof(double));
    double *gn = (double *)malloc(ns * sizeof(double));
    double *gd = (double *)malloc(ns * sizeof(double));
    double *agt1 = (double *)malloc(ns * sizeof(double));
    double *t1 = (double *)malloc(nx * sizeof(double));
    double *gt1 = (double *)malloc(nx * sizeof(double));
    rectify(g, z, bias, relu, s, pre);
    ndc_bf_K(g, s, hf, t1);
    ndc_bf_A(g, x, hf, n);
    ndc_bf_A(g, t1, hf, d);
    for (size_t k = 0; k < ns; ++k) {
        n[k] += eps;
        d[k] += eps;
        gn[k] = gout[k] * s[k] / d[k];
        gd[k] = -gn[k] * n[k] / d[k];
    }
    ndc_bf_K(g, gd, hf, gt1);
    ndc_bf_K(g, gn, hf, gx);
    ndc_bf_A(g, gt1, hf, agt1);
    for (int c = 0; c < cs; ++c) gb[c] = 0.0;
    for (int b = 0; b < g->B; ++b)
        for (int c = 0; c < cs; ++c)
            for (size_t p = 0; p < sp; ++p) {
                size_t idx = ((size_t)b * cs + c) * sp + p;
                double v = gout[idx] * n[idx] / d[idx] + agt1[idx];
                if (relu && !(pre[idx] > 0.0)) v = 0.0;
                gz[idx] = v;
                gb[c] += v;
            }
    /* gh[grp,o,i,tau] */
    for (int grp = 0; grp < g->G; ++grp)
        for (int o = 0; o < g->m; ++o)
            for (int i = 0; i < g->sc; ++i)
                for (int td = 0; td < g->kD; ++td)
                    for (int th = 0; th < g->kH; ++th)
                        for (int tw = 0; tw < g->kW; ++tw) {
                            double acc = 0.0;
                            for (int b = 0; b < g->B; ++b)
                                for (int dd = 0; dd < g->D; ++dd)
                                    for (int hh = 0; hh < g->H; ++hh)
                                        for (int ww = 0; ww < g->W; ++ww) {
                                            acc += at(gt1, g, cx, b, grp * g->m + o, dd, hh, ww) *
                                                   at(s, g, cs, b, grp * g->sc + i, dd + td - pD,
                                                      hh + th - pH, ww + tw - pW);
                                            acc += at(gn, g, cs, b, grp * g->sc + i, dd, hh, ww) *
                                                   at(x, g, cx, b, grp * g->m + o, dd + pD - td,
                                                      hh + pH - th, ww + pW - tw);
                                            acc += at(gd, g, cs, b, grp * g->sc + i, dd, hh, ww) *
                                                   at(t1, g, cx, b, grp * g->m + o, dd + pD - td,
                                                      hh + pH - th, ww + pW - tw);
                                        }
                            gh[((((size_t)grp * g->m + o) * g->sc + i) * g->kD + td) * g->kH *
                                   g->kW +
                               (size_t)th * g->kW + tw] = acc;
                        }
    free(s);
    free(pre);
    free(n);
    free(d);
    free(gn);
    free(gd);
    free(agt1);
    free(t1);
    free(gt1);
}
