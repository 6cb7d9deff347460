// Direct kernels: one thread per output element, global loads with bounds checks, any
// rank / grouping / kernel extent.  They are the envelope path (geometries the fused
// LDS-tiled kernels do not cover) and the on-GPU cross-check of the fused kernels.
//
// Tap conventions (deconver/deconvolution/kernels.py:32-39 of the reference):
//   K(u)[o,p] = sum_{i,tau} u[i, p + tau - pad] * h[o,i,tau]
//   A(v)[i,p] = sum_{o,tau} v[o, p + pad - tau] * h[o,i,tau]
#pragma once

#include "ndc_common.h"

namespace ndc {
namespace direct {

struct Pos {
    int b, g, ch, d, h, w;
};

// idx enumerates (b, g, ch in [0,nch), d, h, w) in row-major order
NDC_HD Pos decode(long long idx, const KGeom &q, int nch)
{
    Pos p;
    p.w = (int)(idx % q.W);
    idx /= q.W;
    p.h = (int)(idx % q.H);
    idx /= q.H;
    p.d = (int)(idx % q.D);
    idx /= q.D;
    p.ch = (int)(idx % nch);
    idx /= nch;
    p.g = (int)(idx % q.G);
    p.b = (int)(idx / q.G);
    return p;
}

NDC_HD bool inside(const KGeom &q, int d, int h, int w)
{
    return (unsigned)d < (unsigned)q.D && (unsigned)h < (unsigned)q.H && (unsigned)w < (unsigned)q.W;
}

NDC_HD long long plane_off(const KGeom &q, int d, int h, int w)
{
    return ((long long)d * q.H + h) * q.W + w;
}

// rectified, biased source value at an in-bounds position
template <typename T>
NDC_HD float source_at(const KGeom &q, const T *z, const float *bias, long long off, int chan)
{
    float v = Elem<T>::load(z + off);
    if (bias) v += bias[chan];
    if (q.relu) v = v < 0.f ? 0.f : v;   // a NaN stays a NaN, as in torch.relu
    return v;
}

// ---------------------------------------------------------------- grouped convolution
// ADJ = false: out (B,G*m,S) = K(in (B,G*sc,S));  ADJ = true: out (B,G*sc,S) = A(in (B,G*m,S)).
// When `rectify` is set the input is read as relu?(in + bias) (zero outside the volume).
template <typename TI, typename TO, bool ADJ>
NDC_HD void gconv(long long idx, const KGeom &q, const TI *in, const float *hf, const float *bias,
                  bool rectify, TO *out)
{
    const int cin = ADJ ? q.m : q.sc, cout = ADJ ? q.sc : q.m;
    const Pos p = decode(idx, q, cout);
    const long long in_base = ((long long)p.b * q.G + p.g) * cin * q.SP;
    const float *hg = hf + (long long)p.g * q.m * q.sc * q.KT;
    float acc = 0.f;
    for (int ci = 0; ci < cin; ++ci) {
        const int o = ADJ ? ci : p.ch, i = ADJ ? p.ch : ci;
        const float *hw = hg + ((long long)o * q.sc + i) * q.KT;
        for (int td = 0; td < q.kD; ++td)
            for (int th = 0; th < q.kH; ++th)
                for (int tw = 0; tw < q.kW; ++tw) {
                    const int dd = ADJ ? p.d + q.pD - td : p.d + td - q.pD;
                    const int hh = ADJ ? p.h + q.pH - th : p.h + th - q.pH;
                    const int ww = ADJ ? p.w + q.pW - tw : p.w + tw - q.pW;
                    if (!inside(q, dd, hh, ww)) continue;
                    const long long off = in_base + (long long)ci * q.SP + plane_off(q, dd, hh, ww);
                    float v;
                    if (rectify) {
                        v = Elem<TI>::load(in + off);
                        if (bias) v += bias[p.g * cin + ci];
                        if (q.relu) v = v < 0.f ? 0.f : v;   // a NaN stays a NaN, as in torch.relu
                    } else {
                        v = Elem<TI>::load(in + off);
                    }
                    acc += v * hw[(td * q.kH + th) * q.kW + tw];
                }
    }
    Elem<TO>::store(out + idx, acc);
}

// numerator / denominator at one source element: n = A(x)+eps, d = A(t1)+eps
template <typename T>
NDC_HD void num_den(const KGeom &q, const Pos &p, const T *x, const T *t1, const float *hf,
                    float &n, float &d)
{
    const long long base = ((long long)p.b * q.G + p.g) * q.m * q.SP;
    const float *hg = hf + (long long)p.g * q.m * q.sc * q.KT;
    float an = 0.f, ad = 0.f;
    for (int o = 0; o < q.m; ++o) {
        const float *hw = hg + ((long long)o * q.sc + p.ch) * q.KT;
        for (int td = 0; td < q.kD; ++td)
            for (int th = 0; th < q.kH; ++th)
                for (int tw = 0; tw < q.kW; ++tw) {
                    const int dd = p.d + q.pD - td, hh = p.h + q.pH - th, ww = p.w + q.pW - tw;
                    if (!inside(q, dd, hh, ww)) continue;
                    const long long off = base + (long long)o * q.SP + plane_off(q, dd, hh, ww);
                    const float wv = hw[(td * q.kH + th) * q.kW + tw];
                    an += Elem<T>::load(x + off) * wv;
                    ad += Elem<T>::load(t1 + off) * wv;
                }
    }
    n = an + q.eps;
    d = ad + q.eps;
}

// ---------------------------------------------------------------- forward epilogue
// out = s * (A(x)+eps) / (A(t1)+eps), idx over (B, G*sc, S)
template <typename T>
NDC_HD void fwd(long long idx, const KGeom &q, const T *x, const T *t1, const T *z,
                const float *hf, const float *bias, T *out, T *s_over_den, T *ratio)
{
    const Pos p = decode(idx, q, q.sc);
    float n, d;
    num_den<T>(q, p, x, t1, hf, n, d);
    const float s = source_at<T>(q, z, bias, idx, p.g * q.sc + p.ch);
    Elem<T>::store(out + idx, s * n / d);
    if (s_over_den) Elem<T>::store(s_over_den + idx, s / d);
    if (ratio) Elem<T>::store(ratio + idx, n / d);
}

// ---------------------------------------------------------------- backward, elementwise part
// gn = g*s/d, gd = -gn*n/d (float scratch), idx over (B, G*sc, S)
template <typename T>
NDC_HD void bwd_gn_gd(long long idx, const KGeom &q, const T *x, const T *t1, const T *z,
                      const T *gout, const float *hf, const float *bias, float *gn, float *gd)
{
    const Pos p = decode(idx, q, q.sc);
    float n, d;
    num_den<T>(q, p, x, t1, hf, n, d);
    const float s = source_at<T>(q, z, bias, idx, p.g * q.sc + p.ch);
    const float inv = 1.0f / d;
    const float a = Elem<T>::load(gout + idx) * s * inv;
    gn[idx] = a;
    gd[idx] = -(a * n) * inv;
}

// gz = [z+b>0] * (g*n/d + A(gt1)), idx over (B, G*sc, S); gt1 is float scratch (B,G*m,S)
template <typename T>
NDC_HD void bwd_gz(long long idx, const KGeom &q, const T *x, const T *t1, const T *z,
                   const T *gout, const float *gt1, const float *hf, const float *bias, T *gz)
{
    const Pos p = decode(idx, q, q.sc);
    float n, d;
    num_den<T>(q, p, x, t1, hf, n, d);
    // A(gt1)
    const long long base = ((long long)p.b * q.G + p.g) * q.m * q.SP;
    const float *hg = hf + (long long)p.g * q.m * q.sc * q.KT;
    float ag = 0.f;
    for (int o = 0; o < q.m; ++o) {
        const float *hw = hg + ((long long)o * q.sc + p.ch) * q.KT;
        for (int td = 0; td < q.kD; ++td)
            for (int th = 0; th < q.kH; ++th)
                for (int tw = 0; tw < q.kW; ++tw) {
                    const int dd = p.d + q.pD - td, hh = p.h + q.pH - th, ww = p.w + q.pW - tw;
                    if (!inside(q, dd, hh, ww)) continue;
                    ag += gt1[base + (long long)o * q.SP + plane_off(q, dd, hh, ww)] *
                          hw[(td * q.kH + th) * q.kW + tw];
                }
    }
    float r = Elem<T>::load(gout + idx) * n / d + ag;
    if (q.relu) {
        float pre = Elem<T>::load(z + idx);
        if (bias) pre += bias[p.g * q.sc + p.ch];
        if (pre <= 0.f) r = 0.f;   // a NaN passes, as through torch.relu's backward
    }
    Elem<T>::store(gz + idx, r);
}

// ---------------------------------------------------------------- reductions
// One block per output; each thread returns its strided partial, the block sums them.

// gb[c] = sum_{b,p} gz[b,c,p]
template <typename T>
NDC_HD float gb_partial(int out_idx, int tid, int nthreads, const KGeom &q, const T *gz)
{
    const long long total = (long long)q.B * q.SP;
    float acc = 0.f;
    for (long long k = tid; k < total; k += nthreads) {
        const long long b = k / q.SP, p = k - b * q.SP;
        acc += Elem<T>::load(gz + (b * q.CS() + out_idx) * q.SP + p);
    }
    return acc;
}

// gh[g,o,i,tau] = sum_{b,p} gt1[o,p] s[i,p+tau-pad] + gn[i,p] x[o,p+pad-tau] + gd[i,p] t1[o,p+pad-tau]
template <typename T>
NDC_HD float gh_partial(int out_idx, int tid, int nthreads, const KGeom &q, const T *x,
                        const T *t1, const T *z, const float *bias, const float *gn,
                        const float *gd, const float *gt1)
{
    int r = out_idx;
    const int tw = r % q.kW;
    r /= q.kW;
    const int th = r % q.kH;
    r /= q.kH;
    const int td = r % q.kD;
    r /= q.kD;
    const int i = r % q.sc;
    r /= q.sc;
    const int o = r % q.m;
    const int g = r / q.m;
    const long long total = (long long)q.B * q.SP;
    float acc = 0.f;
    for (long long k = tid; k < total; k += nthreads) {
        const long long b = k / q.SP;
        long long p = k - b * q.SP;
        const int w = (int)(p % q.W);
        p /= q.W;
        const int h = (int)(p % q.H);
        const int d = (int)(p / q.H);
        const long long xb = ((b * q.G + g) * q.m + o) * q.SP;
        const long long sb = ((b * q.G + g) * q.sc + i) * q.SP;
        const long long here = plane_off(q, d, h, w);
        // K-side term: s at p + tau - pad
        {
            const int dd = d + td - q.pD, hh = h + th - q.pH, ww = w + tw - q.pW;
            if (inside(q, dd, hh, ww))
                acc += gt1[xb + here] *
                       source_at<T>(q, z, bias, sb + plane_off(q, dd, hh, ww), g * q.sc + i);
        }
        // A-side terms: x and t1 at p + pad - tau
        {
            const int dd = d + q.pD - td, hh = h + q.pH - th, ww = w + q.pW - tw;
            if (inside(q, dd, hh, ww)) {
                const long long off = xb + plane_off(q, dd, hh, ww);
                acc += gn[sb + here] * Elem<T>::load(x + off);
                acc += gd[sb + here] * Elem<T>::load(t1 + off);
            }
        }
    }
    return acc;
}

}  // namespace direct
}  // namespace ndc
