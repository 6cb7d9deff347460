// Host side of the fused kernels: which geometries they cover, launch shapes, scratch
// layout, and the launch sequence of a forward / backward call.  Needs a `Backend` with
// `block_kernel<Kernel>(params, nblocks, nthreads, lds_floats, stream)` and `elementwise`.
#pragma once

#include "../../include/deconver_ndc.h"
#include <stdlib.h>

#include <atomic>

#include "ndc_fused.h"
#include "ndc_fused_mfma.h"

namespace ndc {
namespace fused {

// Compiled instances, in the marching view (2-D k x k runs as (k, 1, k)).  One row per
// (KD, KH, KW, SC, RHF, RWF, RHB, RWB): RHF x RWF is the register tile (rows x columns per
// thread) of the forward kernel, RHB x RWB that of the two backward kernels.  Rows of one
// filter geometry are listed in order of preference; a row with RW = 2 needs an even W and
// tensors aligned to two elements, so every geometry also has an RW = 1 row.
#define NDC_FUSED_VARIANTS(X)        \
    X(3, 3, 3, 4, 2, 2, 2, 2)        \
    X(3, 3, 3, 4, 2, 2, 1, 2)        \
    X(3, 3, 3, 4, 4, 1, 2, 1)        \
    X(3, 3, 3, 4, 2, 1, 1, 1)        \
    X(5, 1, 5, 4, 1, 2, 1, 2)        \
    X(5, 1, 5, 4, 1, 1, 1, 1)        \
    X(3, 1, 3, 4, 1, 2, 1, 2)        \
    X(3, 1, 3, 4, 1, 1, 1, 1)

struct Variant {
    int KD, KH, KW, SC, RHF, RWF, RHB, RWB;
};

// Launch-shape choices that are not dictated by the geometry: the measured best, fixed at
// compile time.  A tuning build (-DNDC_TUNING, never the shipped library) reads them from
// NDC_TUNE_* environment variables once, at the first call.
struct Tuning {
    int rhf, rwf, rhb, rwb;      // forced register tiles (0: the table's order of preference)
    int threads_f, threads_b;    // workgroup sizes of the FMA kernels, forward / backward
    int threads_f2, threads_b2;  // ... of the bf16 dot2 kernels
    int split, dot2;             // march segments on / bf16 dot2 kernels on
    int mfma;                    // bf16 matrix-instruction kernels on (where they cover the geometry)
};

#ifdef NDC_TUNING
static inline int env_int(const char *name, int dflt)
{
    const char *v = getenv(name);
    return v && *v ? atoi(v) : dflt;
}
static inline const Tuning &tuning()
{
    static const Tuning t = {env_int("NDC_TUNE_RHF", 0),  env_int("NDC_TUNE_RWF", 0),
                             env_int("NDC_TUNE_RHB", 0),  env_int("NDC_TUNE_RWB", 0),
                             env_int("NDC_TUNE_NTF", 256), env_int("NDC_TUNE_NTB", 512),
                             env_int("NDC_TUNE_NTF2", 256), env_int("NDC_TUNE_NTB2", 256),
                             env_int("NDC_TUNE_SPLIT", 1), env_int("NDC_TUNE_DOT2", 1),
                             env_int("NDC_TUNE_MFMA", 1)};
    return t;
}
#else
static inline Tuning tuning() { return Tuning{0, 0, 0, 0, 256, 512, 256, 256, 1, 1, 1}; }
#endif

// first listed row of this filter geometry that the width / alignment allow (and, in a
// tuning run, that matches the requested register tiles)
static inline bool find_variant(const KGeom &q, const March &m, bool pairs_ok, Variant &v)
{
    if (q.m != 1) return false;
    const Tuning tn = tuning();
    // 2-D problems march along the image rows with one strip of lanes across a row: below
    // 128 columns a lane per column (not per column pair) keeps more of the wavefront busy
    // (measured 16-32 % faster from 16 to 100 columns, 4-15 % slower from 128 on)
    const bool narrow_2d = m.H == 1 && m.W < 128 && !tn.rwf && !tn.rwb;
    const bool even = pairs_ok && m.W % 2 == 0 && !narrow_2d;
    bool found = false;
#define X(kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_)                                        \
    if (!found && m.KD == kd_ && m.KH == kh_ && m.KW == kw_ && q.sc == sc_ &&                \
        (even || (rwf_ == 1 && rwb_ == 1)) && (!tn.rhf || tn.rhf == rhf_) &&                 \
        (!tn.rwf || tn.rwf == rwf_) && (!tn.rhb || tn.rhb == rhb_) &&                        \
        (!tn.rwb || tn.rwb == rwb_)) {                                                       \
        v = Variant{kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_};                             \
        found = true;                                                                        \
    }
    NDC_FUSED_VARIANTS(X)
#undef X
    if (found) return true;
    // no row matches a tuning request: fall back to the plain order of preference
#define X(kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_)                                        \
    if (!found && m.KD == kd_ && m.KH == kh_ && m.KW == kw_ && q.sc == sc_ &&                \
        (even || (rwf_ == 1 && rwb_ == 1))) {                                                \
        v = Variant{kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_};                             \
        found = true;                                                                        \
    }
    NDC_FUSED_VARIANTS(X)
#undef X
    return found;
}

// The process-wide default of the kernel family for calls that do not name one
// (ndc_matrix_kernels): 0 = vector unit, 1 = the kernels built on the 4x4x4 matrix instruction
// (ndc_fused_mfma.h) where they cover the geometry.  Off unless a caller turns it on: the path
// is specified as a depthwise stencil that keeps matrix instructions out of it.  Atomic, so
// that a thread that sets it and threads that launch do not race; a call that must not depend
// on it names its family in ndc_geom.path.
static inline std::atomic<int> &matrix_default()
{
    static std::atomic<int> on{0};
    return on;
}

#ifndef NDC_SPLIT_F
#define NDC_SPLIT_F 4096
#endif
#ifndef NDC_SPLIT_B
#define NDC_SPLIT_B 2048
#endif
static const long long kSplitWavesF = NDC_SPLIT_F, kSplitWavesB = NDC_SPLIT_B;

struct Plan {
    Variant v;
    March m;
    bool dot2;            // bf16 dot2 kernels (3x3x3, SC = 4, even W, aligned pairs)
    bool mfma1, mfma2;    // ... with pass 1 / pass 2 on the matrix instruction when they read the forward's ratios
    bool mfmaf;           // ... with the forward on the matrix instruction
    Tile tf, tb;          // forward / backward launch shapes
    int lds_f, lds_b1, lds_b2;
    int nblk_f, nblk_b;
};

template <int KD, int KH, int KW, int SC, int RHF, int RWF, int RHB, int RWB>
static inline void plan_lds(Plan &pl)
{
    pl.lds_f = FwdKernel<KD, KH, KW, SC, RHF, RWF, float>::lds_floats(pl.tf);
    pl.lds_b1 = Bwd1Kernel<KD, KH, KW, SC, RHB, RWB, float>::lds_floats(pl.tb);
    pl.lds_b2 = Bwd2Kernel<KD, KH, KW, SC, RHB, RWB, float>::lds_floats(pl.tb);
}

#define NDC_IS_VARIANT(pl, kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_)                          \
    ((pl).v.KD == kd_ && (pl).v.KH == kh_ && (pl).v.KW == kw_ && (pl).v.SC == sc_ &&            \
     (pl).v.RHF == rhf_ && (pl).v.RWF == rwf_ && (pl).v.RHB == rhb_ && (pl).v.RWB == rwb_)

// pairs_ok: every activation pointer of the call is aligned to two elements
static const int kDot2RH = 2;   // rows per thread of the bf16 dot2 kernels (columns: 2)

static inline bool make_plan_for(const KGeom &q, Plan &pl, bool pairs_ok, int dtype, bool matrix)
{
    pl.m = march_of(q);
    pl.dot2 = false;
    pl.mfma1 = pl.mfma2 = pl.mfmaf = false;
    // 32-bit offsets inside one (sample, channel) volume
    if ((long long)q.sc * q.SP >= (1LL << 31)) return false;
    if (!find_variant(q, pl.m, pairs_ok, pl.v)) return false;
    const Tuning tn = tuning();
    if (!make_tile(pl.m, pl.v.RHF, pl.v.RWF, tn.threads_f, pl.tf)) return false;
    if (!make_tile(pl.m, pl.v.RHB, pl.v.RWB, tn.threads_b, pl.tb)) return false;
    if (tn.split) {
        // the forward keeps four wavefronts per SIMD resident, the backward kernels two
        split_march(pl.m, (long long)q.B * q.G * pl.tf.ntile, pl.tf, kSplitWavesF);
        split_march(pl.m, (long long)q.B * q.G * pl.tb.ntile, pl.tb, kSplitWavesB);
    }
#define X(kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_)                                        \
    if (NDC_IS_VARIANT(pl, kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_))                      \
        plan_lds<kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_>(pl);
    NDC_FUSED_VARIANTS(X)
#undef X
    // (their buffer addressing wants every (sample, channel group) slice below 2^31 bytes)
    if (dtype == NDC_BF16 && pairs_ok && pl.m.W % 2 == 0 && q.sc == 4 && pl.m.KD == 3 &&
        (long long)q.sc * q.SP * 2 < (1LL << 31) &&
        pl.m.KH == 3 && pl.m.KW == 3 && tn.dot2) {
        Tile tf, tb;
        if (make_tile(pl.m, kDot2RH, 2, tn.threads_f2, tf, FwdKernelB<kDot2RH>::kMinStrips) &&
            make_tile(pl.m, kDot2RH, 2, tn.threads_b2, tb)) {
            const int lf = FwdKernelB<kDot2RH>::lds_floats(tf);
            const int l1 = Bwd1KernelB<kDot2RH>::lds_floats(tb);
            const int l2 = Bwd2KernelB<kDot2RH>::lds_floats(tb);
            const int cap2 = kMaxLdsBytes / 4;
            if (lf <= cap2 && l1 <= cap2 && l2 <= cap2) {
                pl.dot2 = true;
                pl.tf = tf;
                pl.tb = tb;
                pl.lds_f = lf;
                pl.lds_b1 = l1;
                pl.lds_b2 = l2;
                // (pass 1 only where two of its workgroups fit a CU: with 128 columns its LDS
                // need leaves room for one, and the dot2 kernel is faster, 2.73 against 2.96 ms
                // at 64 channels of 128^3)
                pl.mfma1 = tn.mfma && matrix && Bwd1KernelM<kDot2RH>::covers(pl.m.W) &&
                           Bwd1KernelM<kDot2RH>::lds_floats(tb) <= cap2 / 2;
                pl.mfmaf = tn.mfma && matrix && FwdKernelM<kDot2RH>::covers(pl.m.W) &&
                           FwdKernelM<kDot2RH>::lds_floats(tf) <= cap2;
                pl.mfma2 = tn.mfma && matrix && Bwd2KernelM<kDot2RH>::covers(pl.m.W) &&
                           Bwd2KernelM<kDot2RH>::lds_floats(tb) <= cap2;
            }
        }
    }
    const int cap = kMaxLdsBytes / 4;
    if (pl.lds_f > cap || pl.lds_b1 > cap || pl.lds_b2 > cap) return false;
    const long long nbc = (long long)q.B * q.G;
    const long long nf = nbc * pl.tf.ntile * pl.tf.nseg, nb = nbc * pl.tb.ntile * pl.tb.nseg;
    if (nf > 0x7fffffffLL || nb > 0x7fffffffLL) return false;
    pl.nblk_f = (int)nf;
    pl.nblk_b = (int)nb;
    return true;
}

// The column-pair variants hold more of a row per workgroup: where their LDS need exceeds a
// workgroup's share (wide rows of a tall image) the one-column variants may still fit, and
// those are what supported() answers for.
// matrix: the call runs the matrix-instruction family where it covers the geometry (the
// launch shapes, workspace sizes and table sizes are the same for both families)
static inline bool make_plan(const KGeom &q, Plan &pl, bool pairs_ok = true, int dtype = NDC_F32,
                             bool matrix = false)
{
    if (make_plan_for(q, pl, pairs_ok, dtype, matrix)) return true;
    return pairs_ok && make_plan_for(q, pl, false, dtype, matrix);
}

static inline bool supported(const KGeom &q)
{
    Plan pl;
    return make_plan(q, pl, false);
}

template <typename T> static inline bool pair_aligned(const void *p)
{
    return p == nullptr || ((uintptr_t)p % (2 * sizeof(T))) == 0;
}

static inline size_t align256(size_t v) { return (v + 255) / 256 * 256; }

// scratch: gt1 (activation dtype) | pass-1 partials | pass-2 partials
static inline size_t backward_ws(const KGeom &q, int dtype, int /*need_gh*/, int /*need_gb*/)
{
    // sized for whichever variant the call ends up with (aligned pairs or not)
    Plan a, b;
    if (!make_plan(q, a, false, dtype)) return 0;
    const bool has_b = make_plan(q, b, true, dtype);
    const size_t nblk = has_b && b.nblk_b > a.nblk_b ? b.nblk_b : a.nblk_b;
    const size_t esz = dtype == NDC_BF16 ? 2 : 4;
    const size_t n_x = (size_t)q.B * q.G * q.SP;
    const size_t kt = (size_t)q.sc * q.KT;
    const size_t tabs = has_b && b.dot2 ? align256((size_t)q.G * kTabWords * 4) : 0;
    return align256(n_x * esz) + align256(nblk * kt * 4) + align256(nblk * (kt + q.sc) * 4) + tabs;
}

// bytes of scratch the forward call needs (the packed tap tables of the bf16 dot2 kernels)
static inline size_t forward_ws(const KGeom &q, int dtype)
{
    Plan pl;
    if (!make_plan(q, pl, true, dtype) || !pl.dot2) return 0;
    return align256((size_t)q.G * kTabWords * 4);
}

// whether backward() reads the forward's s/d and n/d for this geometry: every fused kernel
// family has that form
static inline bool backward_uses_saved(const KGeom &q, int dtype)
{
    Plan pl;
    return make_plan(q, pl, true, dtype);
}

template <class BE, typename T> struct Dot2Launch {
    static int fwd(const FwdParams<T> &, const Plan &, void *) { return NDC_ERR_GEOMETRY; }
    static int bwd1(const BwdParams<T> &, const Plan &, void *, bool) { return NDC_ERR_GEOMETRY; }
    static int bwd2(const BwdParams<T> &, const Plan &, void *, bool) { return NDC_ERR_GEOMETRY; }
};
template <class BE> struct Dot2Launch<BE, bf16_t> {
    static int fwd(const FwdParams<bf16_t> &p, const Plan &pl, void *stream)
    {
        if (pl.mfmaf)
            return BE::template block_kernel<FwdKernelM<kDot2RH>>(p, pl.nblk_f, pl.tf.NT,
                                                                   FwdKernelM<kDot2RH>::lds_floats(pl.tf), stream);
        if (p.s_over_den && p.ratio)
            return BE::template block_kernel<FwdKernelB<kDot2RH, true>>(p, pl.nblk_f, pl.tf.NT, pl.lds_f, stream);
        return BE::template block_kernel<FwdKernelB<kDot2RH>>(p, pl.nblk_f, pl.tf.NT, pl.lds_f, stream);
    }
    // saved: the call brought the forward's s/d and n/d
    static int bwd1(const BwdParams<bf16_t> &p, const Plan &pl, void *stream, bool saved)
    {
        if (saved && pl.mfma1)
            return BE::template block_kernel<Bwd1KernelM<kDot2RH>>(
                p, pl.nblk_b, pl.tb.NT, Bwd1KernelM<kDot2RH>::lds_floats(pl.tb), stream);
        if (saved)
            return BE::template block_kernel<Bwd1KernelB<kDot2RH, true>>(
                p, pl.nblk_b, pl.tb.NT, Bwd1KernelB<kDot2RH, true>::lds_floats(pl.tb), stream);
        return BE::template block_kernel<Bwd1KernelB<kDot2RH>>(p, pl.nblk_b, pl.tb.NT, pl.lds_b1, stream);
    }
    static int bwd2(const BwdParams<bf16_t> &p, const Plan &pl, void *stream, bool saved)
    {
        if (saved && pl.mfma2)
            return BE::template block_kernel<Bwd2KernelM<kDot2RH>>(
                p, pl.nblk_b, pl.tb.NT, Bwd2KernelM<kDot2RH>::lds_floats(pl.tb), stream);
        if (saved)
            return BE::template block_kernel<Bwd2KernelB<kDot2RH, true>>(
                p, pl.nblk_b, pl.tb.NT, Bwd2KernelB<kDot2RH, true>::lds_floats(pl.tb), stream);
        return BE::template block_kernel<Bwd2KernelB<kDot2RH>>(p, pl.nblk_b, pl.tb.NT, pl.lds_b2, stream);
    }
};

// the packed filter tables of the bf16 dot2 kernels: G * kTabWords words from h
template <class BE> static int prepare_taps(const KGeom &q, const float *h, float *tab, void *stream)
{
    return BE::elementwise((long long)q.G * kTabWords, stream,
                           [=] NDC_LAMBDA(long long idx) { prep_tables(idx, h, tab); });
}

template <class BE, typename T>
static int forward(const KGeom &q, const T *x, const T *z, const float *h, const float *bias,
                   T *out, T *t1, T *s_over_den, T *ratio, const float *taps, void *ws,
                   void *stream)
{
    // taps: packed filter tables prepared earlier for this h (prepare_taps), or null: then
    // they are packed into ws by a small launch ahead of the kernel
    Plan pl;
    const bool pairs = pair_aligned<T>(x) && pair_aligned<T>(z) && pair_aligned<T>(out) &&
                       pair_aligned<T>(t1) && pair_aligned<T>(s_over_den) && pair_aligned<T>(ratio);
    const int dtype = sizeof(T) == 2 ? NDC_BF16 : NDC_F32;
    if (!make_plan(q, pl, pairs, (ws || taps) ? dtype : NDC_F32, q.matrix != 0)) return NDC_ERR_GEOMETRY;
    FwdParams<T> p;
    p.wtab = nullptr;
    p.x = x;
    p.z = z;
    p.h = h;
    p.bias = bias;
    p.out = out;
    p.t1 = t1;
    p.s_over_den = s_over_den;
    p.ratio = ratio;
    p.B = q.B;
    p.C = q.G;
    p.D = pl.m.D;
    p.H = pl.m.H;
    p.W = pl.m.W;
    p.relu = q.relu;
    p.eps = q.eps;
    p.t = pl.tf;
    if (pl.dot2) {
        if (taps) {
            p.wtab = taps;
        } else {
            float *tab = (float *)ws;
            const int st = prepare_taps<BE>(q, h, tab, stream);
            if (st) return st;
            p.wtab = tab;
        }
        return Dot2Launch<BE, T>::fwd(p, pl, stream);
    }
#define X(kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_)                                          \
    if (NDC_IS_VARIANT(pl, kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_))                        \
        return BE::template block_kernel<FwdKernel<kd_, kh_, kw_, sc_, rhf_, rwf_, T>>(        \
            p, pl.nblk_f, pl.tf.NT, pl.lds_f, stream);
    NDC_FUSED_VARIANTS(X)
#undef X
    return NDC_ERR_GEOMETRY;
}

template <class BE, typename T>
static int backward(const KGeom &q, const T *x, const T *z, const T *t1, const T *s_over_den,
                    const T *ratio, const float *h, const float *bias, const T *gout, T *gx,
                    T *gz, float *gh, float *gb, const float *taps, void *ws, void *stream,
                    float *pass_ms = nullptr)
{
    // pass_ms (optional, 3 floats): device time of pass 1, pass 2 and the partial-sum
    // reduction, taken with events on `stream`; makes the call synchronous
    typename BE::Timer tm(pass_ms != nullptr, stream);
    Plan pl;
    const bool pairs = pair_aligned<T>(x) && pair_aligned<T>(z) && pair_aligned<T>(t1) &&
                       pair_aligned<T>(gout) && pair_aligned<T>(gx) && pair_aligned<T>(gz) &&
                       pair_aligned<T>(s_over_den) && pair_aligned<T>(ratio);
    const bool saved = s_over_den != nullptr && ratio != nullptr;
    const int dtype = sizeof(T) == 2 ? NDC_BF16 : NDC_F32;
    if (!make_plan(q, pl, pairs, dtype, q.matrix != 0)) return NDC_ERR_GEOMETRY;
    const size_t n_x = (size_t)q.B * q.G * q.SP;
    const int kt = q.sc * q.KT;
    char *w = (char *)ws;
    T *gt1 = (T *)w;
    w += align256(n_x * sizeof(T));
    float *part1 = (float *)w;
    w += align256((size_t)pl.nblk_b * kt * 4);
    float *part2 = (float *)w;
    w += align256((size_t)pl.nblk_b * (kt + q.sc) * 4);
    float *tab = (float *)w;

    BwdParams<T> p;
    p.x = x;
    p.z = z;
    p.t1 = t1;
    p.gout = gout;
    p.s_over_den = s_over_den;
    p.ratio = ratio;
    p.h = h;
    p.bias = bias;
    p.gx = gx;
    p.gz = gz;
    p.gt1 = gt1;
    p.wtab = nullptr;
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
    if (pl.dot2) {
        if (taps) {
            p.wtab = taps;
        } else {
            st = prepare_taps<BE>(q, h, tab, stream);
            if (st) return st;
            p.wtab = tab;
        }
        st = Dot2Launch<BE, T>::bwd1(p, pl, stream, saved);
    } else {
#define X(kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_)                                          \
    if (NDC_IS_VARIANT(pl, kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_)) {                      \
        if (saved)                                                                             \
            st = BE::template block_kernel<Bwd1Kernel<kd_, kh_, kw_, sc_, rhb_, rwb_, T, true>>(\
                p, pl.nblk_b, pl.tb.NT, pl.lds_b1, stream);                                    \
        else                                                                                   \
            st = BE::template block_kernel<Bwd1Kernel<kd_, kh_, kw_, sc_, rhb_, rwb_, T>>(     \
                p, pl.nblk_b, pl.tb.NT, pl.lds_b1, stream);                                    \
    }
        NDC_FUSED_VARIANTS(X)
#undef X
    }
    if (st) return st;
    tm.mark();
    if (!gz && !gh && !gb) {
        tm.finish(pass_ms, 3);
        return NDC_OK;
    }

    p.part = part2;
    p.part_stride = kt + q.sc;
    st = NDC_ERR_GEOMETRY;
    if (pl.dot2) {
        st = Dot2Launch<BE, T>::bwd2(p, pl, stream, saved);
    } else {
#define X(kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_)                                          \
    if (NDC_IS_VARIANT(pl, kd_, kh_, kw_, sc_, rhf_, rwf_, rhb_, rwb_)) {                      \
        typedef Bwd2Kernel<kd_, kh_, kw_, sc_, rhb_, rwb_, T, true> KS;                        \
        if (saved)                                                                             \
            st = BE::template block_kernel<KS>(p, pl.nblk_b, pl.tb.NT, KS::lds_floats(pl.tb),  \
                                               stream);                                        \
        else                                                                                   \
            st = BE::template block_kernel<Bwd2Kernel<kd_, kh_, kw_, sc_, rhb_, rwb_, T>>(     \
                p, pl.nblk_b, pl.tb.NT, pl.lds_b2, stream);                                    \
    }
        NDC_FUSED_VARIANTS(X)
#undef X
    }
    if (st) return st;
    tm.mark();

    // combine the per-workgroup partial sums: a fixed association, so results are reproducible
    const int C = q.G, SC = q.sc, ntile = pl.tb.ntile * pl.tb.nseg, B = q.B;
    // (gh and gb in one launch: outputs [0, C kt) are gh, the C SC after them gb)
    const int n_gh = gh ? C * kt : 0, n_gb = gb ? C * SC : 0;
    if (n_gh + n_gb) {
        st = BE::strided_sum(n_gh + n_gb, B * ntile, stream, [=] NDC_LAMBDA(int o, float v) {
            if (o < n_gh) gh[o] = v; else gb[o - n_gh] = v;
        }, [=] NDC_LAMBDA(int o, int pi) {
            if (o < n_gh) {
                const int c = o / kt, r = o % kt;
                const long long blk = ((long long)(pi / ntile) * C + c) * ntile + pi % ntile;
                return part1[blk * kt + r] + part2[blk * (kt + SC) + r];
            }
            const int c = (o - n_gh) / SC, i = (o - n_gh) % SC;
            const long long blk = ((long long)(pi / ntile) * C + c) * ntile + pi % ntile;
            return part2[blk * (kt + SC) + kt + i];
        });
        if (st) return st;
    }
    tm.mark();
    tm.finish(pass_ms, 3);
    return NDC_OK;
}

}  // namespace fused
}  // namespace ndc
