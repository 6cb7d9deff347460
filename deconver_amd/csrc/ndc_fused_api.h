// Host side of the fused kernels: which geometries they cover, launch shapes, scratch
// layout, and the launch sequence of a forward / backward call.  Needs a `Backend` with
// `block_kernel<Kernel>(params, nblocks, nthreads, lds_floats, stream)` and `elementwise`.
#pragma once

#include "../../include/deconver_ndc.h"
#include <stdlib.h>

#include "ndc_fused.h"

namespace ndc {
namespace fused {

// Filter geometries with compiled instances, in the marching view (2-D k x k runs as
// (k, 1, k)).  One row per (KD, KH, KW, SC, RHF, RHB); RHF / RHB are the rows per thread of
// the forward and backward kernels.  Several rows may share a filter geometry: the first
// one whose row counts match the tuning choice (or, failing that, the first one) is used.
#define NDC_FUSED_VARIANTS(X)  \
    X(3, 3, 3, 4, 4, 2)        \
    X(3, 3, 3, 4, 2, 1)        \
    X(5, 1, 5, 4, 1, 1)        \
    X(3, 1, 3, 4, 1, 1)

struct Variant {
    int KD, KH, KW, SC, RHF, RHB;
};

// Launch-shape choices that are not dictated by the geometry.  Defaults are the measured
// best; the environment variables exist for tuning runs only.
struct Tuning {
    int rhf, rhb, threads_f, threads_b;
};

static inline int env_int(const char *name, int dflt)
{
    const char *v = getenv(name);
    return v && *v ? atoi(v) : dflt;
}

static inline Tuning tuning()
{
    Tuning t;
    t.rhf = env_int("NDC_TUNE_RHF", 4);
    t.rhb = env_int("NDC_TUNE_RHB", 2);
    t.threads_f = env_int("NDC_TUNE_NTF", 256);
    t.threads_b = env_int("NDC_TUNE_NTB", 256);
    return t;
}

static inline bool find_variant(const KGeom &q, const March &m, Variant &v)
{
    if (q.m != 1) return false;
    const Tuning tn = tuning();
    bool found = false;
#define X(kd_, kh_, kw_, sc_, rhf_, rhb_)                                       \
    if (m.KD == kd_ && m.KH == kh_ && m.KW == kw_ && q.sc == sc_) {             \
        const bool exact = rhf_ == tn.rhf && rhb_ == tn.rhb;                    \
        if (!found || exact) v = Variant{kd_, kh_, kw_, sc_, rhf_, rhb_};       \
        if (exact) return true;                                                 \
        found = true;                                                           \
    }
    NDC_FUSED_VARIANTS(X)
#undef X
    return found;
}

struct Plan {
    Variant v;
    March m;
    Tile tf, tb;          // forward / backward launch shapes
    int lds_f, lds_b1, lds_b2;
    int nblk_f, nblk_b;
};

template <int KD, int KH, int KW, int SC, int RHF, int RHB>
static inline void plan_lds(Plan &pl)
{
    pl.lds_f = FwdKernel<KD, KH, KW, SC, RHF, float>::lds_floats(pl.tf);
    pl.lds_b1 = Bwd1Kernel<KD, KH, KW, SC, RHB, float>::lds_floats(pl.tb);
    pl.lds_b2 = Bwd2Kernel<KD, KH, KW, SC, RHB, float>::lds_floats(pl.tb);
}

static inline bool make_plan(const KGeom &q, Plan &pl)
{
    pl.m = march_of(q);
    if (!find_variant(q, pl.m, pl.v)) return false;
    const Tuning tn = tuning();
    if (!make_tile(pl.m, pl.v.RHF, tn.threads_f, pl.tf)) return false;
    if (!make_tile(pl.m, pl.v.RHB, tn.threads_b, pl.tb)) return false;
#define X(kd_, kh_, kw_, sc_, rhf_, rhb_)                                                     \
    if (pl.v.KD == kd_ && pl.v.KH == kh_ && pl.v.KW == kw_ && pl.v.SC == sc_ && pl.v.RHF == rhf_ &&  \
        pl.v.RHB == rhb_)               \
        plan_lds<kd_, kh_, kw_, sc_, rhf_, rhb_>(pl);
    NDC_FUSED_VARIANTS(X)
#undef X
    const int cap = kMaxLdsBytes / 4;
    if (pl.lds_f > cap || pl.lds_b1 > cap || pl.lds_b2 > cap) return false;
    const long long nbc = (long long)q.B * q.G;
    if (nbc * pl.tf.ntile > 0x7fffffffLL || nbc * pl.tb.ntile > 0x7fffffffLL) return false;
    pl.nblk_f = (int)(nbc * pl.tf.ntile);
    pl.nblk_b = (int)(nbc * pl.tb.ntile);
    return true;
}

static inline bool supported(const KGeom &q)
{
    Plan pl;
    return make_plan(q, pl);
}

static inline size_t align256(size_t v) { return (v + 255) / 256 * 256; }

// scratch: gt1 (activation dtype) | pass-1 partials | pass-2 partials
static inline size_t backward_ws(const KGeom &q, int dtype, int /*need_gh*/, int /*need_gb*/)
{
    Plan pl;
    if (!make_plan(q, pl)) return 0;
    const size_t esz = dtype == NDC_BF16 ? 2 : 4;
    const size_t n_x = (size_t)q.B * q.G * q.SP;
    const size_t kt = (size_t)q.sc * q.KT;
    return align256(n_x * esz) + align256((size_t)pl.nblk_b * kt * 4) +
           align256((size_t)pl.nblk_b * (kt + q.sc) * 4);
}

template <class BE, typename T>
static int forward(const KGeom &q, const T *x, const T *z, const float *h, const float *bias,
                   T *out, T *t1, void *stream)
{
    Plan pl;
    if (!make_plan(q, pl)) return NDC_ERR_GEOMETRY;
    FwdParams<T> p;
    p.x = x;
    p.z = z;
    p.h = h;
    p.bias = bias;
    p.out = out;
    p.t1 = t1;
    p.B = q.B;
    p.C = q.G;
    p.D = pl.m.D;
    p.H = pl.m.H;
    p.W = pl.m.W;
    p.relu = q.relu;
    p.eps = q.eps;
    p.t = pl.tf;
#define X(kd_, kh_, kw_, sc_, rhf_, rhb_)                                                        \
    if (pl.v.KD == kd_ && pl.v.KH == kh_ && pl.v.KW == kw_ && pl.v.SC == sc_ && pl.v.RHF == rhf_ &&  \
        pl.v.RHB == rhb_)                  \
        return BE::template block_kernel<FwdKernel<kd_, kh_, kw_, sc_, rhf_, T>>(               \
            p, pl.nblk_f, pl.tf.NT, pl.lds_f, stream);
    NDC_FUSED_VARIANTS(X)
#undef X
    return NDC_ERR_GEOMETRY;
}

template <class BE, typename T>
static int backward(const KGeom &q, const T *x, const T *z, const T *t1, const float *h,
                    const float *bias, const T *gout, T *gx, T *gz, float *gh, float *gb,
                    void *ws, void *stream, float *pass_ms = nullptr)
{
    // pass_ms (optional, 3 floats): device time of pass 1, pass 2 and the partial-sum
    // reduction, taken with events on `stream`; makes the call synchronous
    typename BE::Timer tm(pass_ms != nullptr, stream);
    Plan pl;
    if (!make_plan(q, pl)) return NDC_ERR_GEOMETRY;
    const size_t n_x = (size_t)q.B * q.G * q.SP;
    const int kt = q.sc * q.KT;
    char *w = (char *)ws;
    T *gt1 = (T *)w;
    w += align256(n_x * sizeof(T));
    float *part1 = (float *)w;
    w += align256((size_t)pl.nblk_b * kt * 4);
    float *part2 = (float *)w;

    BwdParams<T> p;
    p.x = x;
    p.z = z;
    p.t1 = t1;
    p.gout = gout;
    p.h = h;
    p.bias = bias;
    p.gx = gx;
    p.gz = gz;
    p.gt1 = gt1;
    p.need_gh = gh != nullptr;
    p.need_gb = gb != nullptr;
    p.B = q.B;
    p.C = q.G;
    p.D = pl.m.D;
    p.H = pl.m.H;
    p.W = pl.m.W;
    p.relu = q.relu;
    p.eps = q.eps;
    p.t = pl.tb;

    int st = NDC_ERR_GEOMETRY;
    p.part = part1;
    p.part_stride = kt;
#define X(kd_, kh_, kw_, sc_, rhf_, rhb_)                                                        \
    if (pl.v.KD == kd_ && pl.v.KH == kh_ && pl.v.KW == kw_ && pl.v.SC == sc_ && pl.v.RHF == rhf_ &&  \
        pl.v.RHB == rhb_)                  \
        st = BE::template block_kernel<Bwd1Kernel<kd_, kh_, kw_, sc_, rhb_, T>>(                \
            p, pl.nblk_b, pl.tb.NT, pl.lds_b1, stream);
    NDC_FUSED_VARIANTS(X)
#undef X
    if (st) return st;
    tm.mark();
    if (!gz && !gh && !gb) {
        tm.finish(pass_ms, 3);
        return NDC_OK;
    }

    p.part = part2;
    p.part_stride = kt + q.sc;
    st = NDC_ERR_GEOMETRY;
#define X(kd_, kh_, kw_, sc_, rhf_, rhb_)                                                        \
    if (pl.v.KD == kd_ && pl.v.KH == kh_ && pl.v.KW == kw_ && pl.v.SC == sc_ && pl.v.RHF == rhf_ &&  \
        pl.v.RHB == rhb_)                  \
        st = BE::template block_kernel<Bwd2Kernel<kd_, kh_, kw_, sc_, rhb_, T>>(                \
            p, pl.nblk_b, pl.tb.NT, pl.lds_b2, stream);
    NDC_FUSED_VARIANTS(X)
#undef X
    if (st) return st;
    tm.mark();

    // combine the per-workgroup partial sums: fixed order, so results are reproducible
    const int C = q.G, SC = q.sc, ntile = pl.tb.ntile, B = q.B;
    if (gh) {
        st = BE::elementwise((long long)C * kt, stream, [=] NDC_LAMBDA(long long idx) {
            const int c = (int)(idx / kt), r = (int)(idx % kt);
            float acc = 0.f;
            for (int b = 0; b < B; ++b)
                for (int tl = 0; tl < ntile; ++tl) {
                    const long long blk = ((long long)b * C + c) * ntile + tl;
                    acc += part1[blk * kt + r] + part2[blk * (kt + SC) + r];
                }
            gh[idx] = acc;
        });
        if (st) return st;
    }
    if (gb) {
        st = BE::elementwise((long long)C * SC, stream, [=] NDC_LAMBDA(long long idx) {
            const int c = (int)(idx / SC), i = (int)(idx % SC);
            float acc = 0.f;
            for (int b = 0; b < B; ++b)
                for (int tl = 0; tl < ntile; ++tl) {
                    const long long blk = ((long long)b * C + c) * ntile + tl;
                    acc += part2[blk * (kt + SC) + kt + i];
                }
            gb[idx] = acc;
        });
        if (st) return st;
    }
    tm.mark();
    tm.finish(pass_ms, 3);
    return NDC_OK;
}

}  // namespace fused
}  // namespace ndc
