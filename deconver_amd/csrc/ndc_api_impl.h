// Host-side logic of the C ABI (include/deconver_ndc.h): argument checks, path choice,
// workspace carving, launch sequence.  Included by exactly two translation units, each of
// which first defines a `Backend` with the launch primitives:
//   ndc_capi.hip       -> HIP launches on gfx950 (the product)
//   ndc_hostcheck.cpp  -> sequential host execution of the same kernel bodies (CPU tests)
#pragma once

#include "../../include/deconver_ndc.h"
#include "ndc_common.h"
#include "ndc_direct.h"
#include "ndc_fused_api.h"

namespace ndc {

static inline int make_kgeom(const ndc_geom *g, KGeom &q)
{
    if (!g) return NDC_ERR_NULL;
    if (g->dtype != NDC_F32 && g->dtype != NDC_BF16) return NDC_ERR_DTYPE;
    if (g->batch < 1 || g->groups < 1 || g->m < 1 || g->sc < 1) return NDC_ERR_GEOMETRY;
    long long taps = 1, sp = 1;
    for (int a = 0; a < 3; ++a) {
        if (g->size[a] < 1 || g->kernel[a] < 1 || (g->kernel[a] & 1) == 0) return NDC_ERR_GEOMETRY;
        taps *= g->kernel[a];
        sp *= g->size[a];
    }
    if (taps > 4096 || g->m > 1024 || g->sc > 1024) return NDC_ERR_GEOMETRY;
    // element counts must stay well inside int64 and block counts inside int32
    const long long cmax = (long long)g->groups * (g->m > g->sc ? g->m : g->sc);
    if (sp > (1LL << 40) || (long double)sp * cmax * g->batch > 9.0e15L) return NDC_ERR_GEOMETRY;
    if (g->path < NDC_PATH_AUTO || g->path > NDC_PATH_FUSED_VECTOR) return NDC_ERR_GEOMETRY;
    q.B = g->batch;
    q.G = g->groups;
    q.m = g->m;
    q.sc = g->sc;
    q.D = g->size[0];
    q.H = g->size[1];
    q.W = g->size[2];
    q.kD = g->kernel[0];
    q.kH = g->kernel[1];
    q.kW = g->kernel[2];
    q.pD = q.kD / 2;
    q.pH = q.kH / 2;
    q.pW = q.kW / 2;
    q.KT = (int)taps;
    q.relu = g->relu_input ? 1 : 0;
    // the kernel family is fixed here, once per call: named by the call, or the process default
    q.matrix = g->path == NDC_PATH_FUSED_MATRIX   ? 1
               : g->path == NDC_PATH_FUSED_VECTOR ? 0
                                                  : fused::matrix_default().load(std::memory_order_relaxed);
    q.eps = g->eps;
    q.SP = sp;
    return NDC_OK;
}

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Decide which implementation serves a call.  Returns NDC_PATH_DIRECT / NDC_PATH_FUSED, or
// a negative status when the caller forced a path that does not cover the geometry.
static inline int choose_path(const ndc_geom *g, const KGeom &q)
{
    const bool fused_ok = fused::supported(q);
    if (g->path == NDC_PATH_DIRECT) return NDC_PATH_DIRECT;
    if (g->path == NDC_PATH_FUSED || g->path == NDC_PATH_FUSED_MATRIX || g->path == NDC_PATH_FUSED_VECTOR)
        return fused_ok ? (int)NDC_PATH_FUSED : (int)NDC_ERR_GEOMETRY;
    return fused_ok ? (int)NDC_PATH_FUSED : (int)NDC_PATH_DIRECT;
}

// ------------------------------------------------------------------ direct path

template <typename T>
static int direct_forward(const KGeom &q, const T *x, const T *z, const float *h,
                          const float *bias, T *out, T *t1, T *s_over_den, T *ratio, void *stream)
{
    // t1 = K(relu(z + b)) lands in the caller's t1; without one there is nowhere to put
    // it, so the direct path asks for it (the fused path does not need it)
    if (!t1) return NDC_ERR_NULL;
    const long long n_x = (long long)q.B * q.C() * q.SP, n_s = (long long)q.B * q.CS() * q.SP;
    int st = Backend::elementwise(n_x, stream, [=] NDC_LAMBDA(long long idx) {
        direct::gconv<T, T, false>(idx, q, z, h, bias, true, t1);
    });
    if (st) return st;
    return Backend::elementwise(n_s, stream, [=] NDC_LAMBDA(long long idx) {
        direct::fwd<T>(idx, q, x, t1, z, h, bias, out, s_over_den, ratio);
    });
}

static inline size_t direct_backward_ws(const KGeom &q)
{
    const size_t n_x = (size_t)q.B * q.C() * q.SP, n_s = (size_t)q.B * q.CS() * q.SP;
    return align_up(n_s * 4, 256) * 2 + align_up(n_x * 4, 256);
}

template <typename T>
static int direct_backward(const KGeom &q, const T *x, const T *z, const T *t1, const float *h,
                           const float *bias, const T *gout, T *gx, T *gz, float *gh, float *gb,
                           void *ws, void *stream)
{
    const long long n_x = (long long)q.B * q.C() * q.SP, n_s = (long long)q.B * q.CS() * q.SP;
    char *w = (char *)ws;
    float *gn = (float *)w;
    w += align_up((size_t)n_s * 4, 256);
    float *gd = (float *)w;
    w += align_up((size_t)n_s * 4, 256);
    float *gt1 = (float *)w;
    KGeom qn = q;  // gn/gd/gt1 are plain tensors: no bias, no rectification on load
    qn.relu = 0;
    int st = Backend::elementwise(n_s, stream, [=] NDC_LAMBDA(long long idx) {
        direct::bwd_gn_gd<T>(idx, q, x, t1, z, gout, h, bias, gn, gd);
    });
    if (st) return st;
    st = Backend::elementwise(n_x, stream, [=] NDC_LAMBDA(long long idx) {
        direct::gconv<float, float, false>(idx, qn, gd, h, nullptr, false, gt1);
    });
    if (st) return st;
    if (gx) {
        st = Backend::elementwise(n_x, stream, [=] NDC_LAMBDA(long long idx) {
            direct::gconv<float, T, false>(idx, qn, gn, h, nullptr, false, gx);
        });
        if (st) return st;
    }
    if (gh) {
        st = Backend::block_reduce(q.G * q.m * q.sc * q.KT, stream, gh,
                                   [=] NDC_LAMBDA(int o, int tid, int nt) {
                                       return direct::gh_partial<T>(o, tid, nt, q, x, t1, z, bias,
                                                                    gn, gd, gt1);
                                   });
        if (st) return st;
    }
    if (gz || gb) {
        // gz is needed to form gb; when the caller does not want gz it goes to the gn
        // scratch (gn is dead by now), typed as T
        T *gz_out = gz ? gz : (T *)gn;
        st = Backend::elementwise(n_s, stream, [=] NDC_LAMBDA(long long idx) {
            direct::bwd_gz<T>(idx, q, x, t1, z, gout, gt1, h, bias, gz_out);
        });
        if (st) return st;
        if (gb) {
            st = Backend::block_reduce(q.CS(), stream, gb, [=] NDC_LAMBDA(int o, int tid, int nt) {
                return direct::gb_partial<T>(o, tid, nt, q, gz_out);
            });
            if (st) return st;
        }
    }
    return NDC_OK;
}

template <typename TI, typename TO>
static int direct_gconv(const KGeom &q, const TI *in, const float *h, const float *bias,
                        int adjoint, TO *out, void *stream)
{
    const bool rectify = (bias != nullptr) || q.relu;
    if (adjoint) {
        const long long n = (long long)q.B * q.CS() * q.SP;
        return Backend::elementwise(n, stream, [=] NDC_LAMBDA(long long idx) {
            direct::gconv<TI, TO, true>(idx, q, in, h, bias, rectify, out);
        });
    }
    const long long n = (long long)q.B * q.C() * q.SP;
    return Backend::elementwise(n, stream, [=] NDC_LAMBDA(long long idx) {
        direct::gconv<TI, TO, false>(idx, q, in, h, bias, rectify, out);
    });
}

}  // namespace ndc

// ============================================================================ C ABI

extern "C" {

int ndc_version(void) { return 300; }   // 0.3.0: the projections themselves (streaming GEMM)

const char *ndc_status_string(int status)
{
    switch (status) {
    case NDC_OK: return "ok";
    case NDC_ERR_NULL: return "a required pointer is null";
    case NDC_ERR_GEOMETRY: return "geometry not covered by the requested path";
    case NDC_ERR_DTYPE: return "unknown dtype tag";
    case NDC_ERR_WORKSPACE: return "workspace too small or misaligned";
    case NDC_ERR_LAUNCH: return "kernel launch failed";
    case NDC_ERR_SCRATCH_LIMIT:
        return "geometry needs more scratch than the no-allocation entry point's device array holds";
    default: return "unknown status";
    }
}

int ndc_fused_supported(const ndc_geom *g)
{
    ndc::KGeom q;
    if (ndc::make_kgeom(g, q) != NDC_OK) return 0;
    return ndc::fused::supported(q) ? 1 : 0;
}

int ndc_check_geometry(const ndc_geom *g)
{
    ndc::KGeom q;
    int st = ndc::make_kgeom(g, q);
    if (st) return st;
    st = ndc::choose_path(g, q);
    return st < 0 ? st : NDC_OK;
}

size_t ndc_forward_workspace_bytes(const ndc_geom *g)
{
    using namespace ndc;
    KGeom q;
    if (make_kgeom(g, q) != NDC_OK) return 0;
    const int path = choose_path(g, q);
    if (path != NDC_PATH_FUSED) return 0;
    return fused::forward_ws(q, g->dtype);
}

size_t ndc_taps_bytes(const ndc_geom *g) { return ndc_forward_workspace_bytes(g); }

int ndc_prepare_taps(const ndc_geom *g, const float *h, void *taps, size_t taps_bytes, void *stream)
{
    using namespace ndc;
    KGeom q;
    const int st = make_kgeom(g, q);
    if (st) return st;
    const size_t need = ndc_taps_bytes(g);
    if (!need) return NDC_OK;
    if (!h) return NDC_ERR_NULL;
    if (!taps || taps_bytes < need || ((uintptr_t)taps & 255u)) return NDC_ERR_WORKSPACE;
    return fused::prepare_taps<Backend>(q, h, (float *)taps, stream);
}

static int forward_impl(const ndc_geom *g, const void *x, const void *z, const float *h,
                        const float *bias, void *out, void *t1, void *s_over_den, void *ratio,
                        const void *taps, void *workspace, size_t workspace_bytes, void *stream)
{
    using namespace ndc;
    KGeom q;
    int st = make_kgeom(g, q);
    if (st) return st;
    if (!x || !z || !h || !out) return NDC_ERR_NULL;
    if ((s_over_den == nullptr) != (ratio == nullptr)) return NDC_ERR_NULL;
    const int path = choose_path(g, q);
    if (path < 0) return path;
    if (path == NDC_PATH_FUSED) {
        const size_t need = taps ? 0 : fused::forward_ws(q, g->dtype);
        if (need && (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255u)))
            return NDC_ERR_WORKSPACE;
        void *ws = need ? workspace : nullptr;
        const float *tp = fused::forward_ws(q, g->dtype) ? (const float *)taps : nullptr;
        return g->dtype == NDC_F32
                   ? fused::forward<Backend, float>(q, (const float *)x, (const float *)z, h, bias,
                                                    (float *)out, (float *)t1, (float *)s_over_den,
                                                    (float *)ratio, tp, ws, stream)
                   : fused::forward<Backend, bf16_t>(q, (const bf16_t *)x, (const bf16_t *)z, h,
                                                     bias, (bf16_t *)out, (bf16_t *)t1,
                                                     (bf16_t *)s_over_den, (bf16_t *)ratio, tp, ws,
                                                     stream);
    }
    return g->dtype == NDC_F32
               ? direct_forward<float>(q, (const float *)x, (const float *)z, h, bias,
                                       (float *)out, (float *)t1, (float *)s_over_den,
                                       (float *)ratio, stream)
               : direct_forward<bf16_t>(q, (const bf16_t *)x, (const bf16_t *)z, h, bias,
                                        (bf16_t *)out, (bf16_t *)t1, (bf16_t *)s_over_den,
                                        (bf16_t *)ratio, stream);
}

int ndc_forward(const ndc_geom *g, const void *x, const void *z, const float *h,
                const float *bias, void *out, void *t1, void *s_over_den, void *ratio,
                void *workspace, size_t workspace_bytes, void *stream)
{
    return forward_impl(g, x, z, h, bias, out, t1, s_over_den, ratio, nullptr, workspace,
                        workspace_bytes, stream);
}

int ndc_forward_taps(const ndc_geom *g, const void *x, const void *z, const float *h,
                     const void *taps, const float *bias, void *out, void *t1, void *s_over_den,
                     void *ratio, void *stream)
{
    if (ndc_taps_bytes(g) && (!taps || ((uintptr_t)taps & 255u))) return NDC_ERR_WORKSPACE;
    return forward_impl(g, x, z, h, bias, out, t1, s_over_den, ratio, taps, nullptr, 0, stream);
}

int ndc_matrix_kernels(int on)
{
    if (on >= 0) ndc::fused::matrix_default().store(on ? 1 : 0, std::memory_order_relaxed);
    return ndc::fused::matrix_default().load(std::memory_order_relaxed);
}

int ndc_backward_uses_saved(const ndc_geom *g)
{
    using namespace ndc;
    KGeom q;
    if (!g || make_kgeom(g, q) != NDC_OK) return 0;
    if (choose_path(g, q) != NDC_PATH_FUSED) return 0;
    return fused::backward_uses_saved(q, g->dtype) ? 1 : 0;
}

size_t ndc_backward_workspace_bytes(const ndc_geom *g, int need_gx, int need_gz, int need_gh,
                                    int need_gb)
{
    using namespace ndc;
    KGeom q;
    if (make_kgeom(g, q) != NDC_OK) return 0;
    const int path = choose_path(g, q);
    if (path < 0) return 0;
    (void)need_gx;
    (void)need_gz;
    if (path == NDC_PATH_FUSED) return fused::backward_ws(q, g->dtype, need_gh, need_gb);
    return direct_backward_ws(q);
}

static int backward_impl(const ndc_geom *g, const void *x, const void *z, const void *t1,
                         const void *s_over_den, const void *ratio, const float *h, const float *bias,
                         const void *gout, void *gx, void *gz, float *gh, float *gb, const void *taps,
                         void *workspace, size_t workspace_bytes, void *stream, float *pass_ms)
{
    using namespace ndc;
    KGeom q;
    int st = make_kgeom(g, q);
    if (st) return st;
    if (!x || !z || !t1 || !h || !gout) return NDC_ERR_NULL;
    if ((s_over_den == nullptr) != (ratio == nullptr)) return NDC_ERR_NULL;
    if (!gx && !gz && !gh && !gb) return NDC_OK;
    const int path = choose_path(g, q);
    if (path < 0) return path;
    const size_t need = ndc_backward_workspace_bytes(g, gx != nullptr, gz != nullptr,
                                                     gh != nullptr, gb != nullptr);
    if (need && (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255u)))
        return NDC_ERR_WORKSPACE;
    if (path == NDC_PATH_FUSED) {
        const float *tp = fused::forward_ws(q, g->dtype) ? (const float *)taps : nullptr;
        return g->dtype == NDC_F32
                   ? fused::backward<Backend, float>(q, (const float *)x, (const float *)z,
                                                     (const float *)t1, (const float *)s_over_den,
                                                     (const float *)ratio, h, bias,
                                                     (const float *)gout, (float *)gx,
                                                     (float *)gz, gh, gb, tp, workspace, stream, pass_ms)
                   : fused::backward<Backend, bf16_t>(q, (const bf16_t *)x, (const bf16_t *)z,
                                                      (const bf16_t *)t1, (const bf16_t *)s_over_den,
                                                      (const bf16_t *)ratio, h, bias,
                                                      (const bf16_t *)gout, (bf16_t *)gx,
                                                      (bf16_t *)gz, gh, gb, tp, workspace, stream,
                                                      pass_ms);
    }
    return g->dtype == NDC_F32
               ? direct_backward<float>(q, (const float *)x, (const float *)z, (const float *)t1,
                                        h, bias, (const float *)gout, (float *)gx, (float *)gz,
                                        gh, gb, workspace, stream)
               : direct_backward<bf16_t>(q, (const bf16_t *)x, (const bf16_t *)z,
                                         (const bf16_t *)t1, h, bias, (const bf16_t *)gout,
                                         (bf16_t *)gx, (bf16_t *)gz, gh, gb, workspace, stream);
}

int ndc_backward(const ndc_geom *g, const void *x, const void *z, const void *t1,
                 const void *s_over_den, const void *ratio, const float *h, const float *bias,
                 const void *gout, void *gx, void *gz, float *gh, float *gb, void *workspace,
                 size_t workspace_bytes, void *stream)
{
    return backward_impl(g, x, z, t1, s_over_den, ratio, h, bias, gout, gx, gz, gh, gb, nullptr,
                         workspace, workspace_bytes, stream, nullptr);
}

int ndc_backward_taps(const ndc_geom *g, const void *x, const void *z, const void *t1,
                      const void *s_over_den, const void *ratio, const float *h, const void *taps,
                      const float *bias, const void *gout, void *gx, void *gz, float *gh, float *gb,
                      void *workspace, size_t workspace_bytes, void *stream)
{
    if (ndc_taps_bytes(g) && (!taps || ((uintptr_t)taps & 255u))) return NDC_ERR_WORKSPACE;
    return backward_impl(g, x, z, t1, s_over_den, ratio, h, bias, gout, gx, gz, gh, gb, taps,
                         workspace, workspace_bytes, stream, nullptr);
}

int ndc_backward_profiled(const ndc_geom *g, const void *x, const void *z, const void *t1,
                          const void *s_over_den, const void *ratio, const float *h,
                          const float *bias, const void *gout, void *gx, void *gz, float *gh,
                          float *gb, void *workspace, size_t workspace_bytes, void *stream,
                          float *pass_ms)
{
    if (!pass_ms) return NDC_ERR_NULL;
    pass_ms[0] = pass_ms[1] = pass_ms[2] = 0.f;
    return backward_impl(g, x, z, t1, s_over_den, ratio, h, bias, gout, gx, gz, gh, gb, nullptr,
                         workspace, workspace_bytes, stream, pass_ms);
}

int ndc_relayout(const void *src, void *dst, int64_t batch, int64_t channels, int64_t spatial,
                 int dtype, int to_channels_last, void *stream)
{
    if (!src || !dst) return NDC_ERR_NULL;
    if (dtype != NDC_F32 && dtype != NDC_BF16) return NDC_ERR_DTYPE;
    if (batch < 1 || channels < 1 || spatial < 1 ||
        (long double)batch * channels * spatial > 9.0e15L)
        return NDC_ERR_GEOMETRY;
    if (src == dst) return NDC_ERR_GEOMETRY;
    // channels-last (B, S, C) -> channel-first (B, C, S) transposes S x C matrices, the other
    // direction C x S ones
    const long long R = to_channels_last ? channels : spatial, K = to_channels_last ? spatial : channels;
    const int st = ndc::Backend::transpose(src, dst, batch, R, K, dtype == NDC_BF16 ? 2 : 4, stream);
    return st == -2 ? (int)NDC_ERR_GEOMETRY : st;
}

// How a row of n elements is cut for the row normalisation: about 4096 workgroups in all, parts
// of at least 8192 elements and a multiple of 2048 (every thread's 16-byte vectors stay whole),
// at most 64 parts (one wavefront adds a row's partial sums).
static void rownorm_split(long long rows, long long n, int &nsplit, long long &chunk)
{
    long long want = (4096 + rows - 1) / rows;
    if (want > 64) want = 64;
    if (want > n / 8192) want = n / 8192;
    if (want < 1) want = 1;
    chunk = (n + want - 1) / want;
    chunk = (chunk + 2047) / 2048 * 2048;
    nsplit = (int)((n + chunk - 1) / chunk);
}

static int rownorm_check(long long rows, long long n, int dtype)
{
    if (dtype != NDC_F32 && dtype != NDC_BF16) return NDC_ERR_DTYPE;
    if (rows < 1 || n < 1 || (long double)rows * n > 9.0e15L) return NDC_ERR_GEOMETRY;
    int nsplit;
    long long chunk;
    rownorm_split(rows, n, nsplit, chunk);
    if (rows * nsplit > 0x7fffffffLL) return NDC_ERR_GEOMETRY;
    return NDC_OK;
}

size_t ndc_rownorm_workspace_bytes(int64_t rows, int64_t n)
{
    if (rows < 1 || n < 1) return 0;
    int nsplit;
    long long chunk;
    rownorm_split(rows, n, nsplit, chunk);
    return (size_t)rows * nsplit * 2 * sizeof(float);
}

static bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

int ndc_rownorm_forward(const void *x, void *y, float *stats, int64_t rows, int64_t n, int dtype,
                        float eps, void *workspace, size_t workspace_bytes, void *stream)
{
    if (!x || !y || !stats || !workspace) return NDC_ERR_NULL;
    int st = rownorm_check(rows, n, dtype);
    if (st) return st;
    if (x == (const void *)y || !(eps >= 0.f)) return NDC_ERR_GEOMETRY;
    if (workspace_bytes < ndc_rownorm_workspace_bytes(rows, n) || ((uintptr_t)workspace & 7u))
        return NDC_ERR_WORKSPACE;
    int nsplit;
    long long chunk;
    rownorm_split(rows, n, nsplit, chunk);
    const int esz = dtype == NDC_BF16 ? 2 : 4;
    const bool vec = n % (16 / esz) == 0 && aligned16(x) && aligned16(y);
    return ndc::Backend::rownorm(false, x, nullptr, nullptr, (float *)workspace, stats, y, rows, n, nsplit,
                                 chunk, esz, vec, eps, stream);
}

int ndc_rownorm_backward(const void *gy, const void *y, const float *stats, const void *addend, void *gx,
                         int64_t rows, int64_t n, int dtype, void *workspace, size_t workspace_bytes,
                         void *stream)
{
    if (!gy || !y || !stats || !gx || !workspace) return NDC_ERR_NULL;
    int st = rownorm_check(rows, n, dtype);
    if (st) return st;
    if (gx == y) return NDC_ERR_GEOMETRY;
    if (workspace_bytes < ndc_rownorm_workspace_bytes(rows, n) || ((uintptr_t)workspace & 7u))
        return NDC_ERR_WORKSPACE;
    int nsplit;
    long long chunk;
    rownorm_split(rows, n, nsplit, chunk);
    const int esz = dtype == NDC_BF16 ? 2 : 4;
    const bool vec = n % (16 / esz) == 0 && aligned16(gy) && aligned16(y) && aligned16(gx) &&
                     (!addend || aligned16(addend));
    return ndc::Backend::rownorm(true, gy, y, addend, (float *)workspace, const_cast<float *>(stats), gx, rows,
                                 n, nsplit, chunk, esz, vec, 0.f, stream);
}

static int bias_act_check(long long batch, long long channels, long long n, int act, int dtype)
{
    if (dtype != NDC_F32 && dtype != NDC_BF16) return NDC_ERR_DTYPE;
    if (batch < 1 || channels < 1 || channels > 0x7fffffffLL || n < 1 || act < NDC_ACT_NONE || act > NDC_ACT_GELU)
        return NDC_ERR_GEOMETRY;
    if ((long double)batch * channels * n > 9.0e15L) return NDC_ERR_GEOMETRY;
    return rownorm_check(batch * channels, n, dtype);
}

int64_t ndc_bias_act_parts(int64_t rows, int64_t n)
{
    if (rows < 1 || n < 1) return 0;
    int nsplit;
    long long chunk;
    rownorm_split(rows, n, nsplit, chunk);
    return nsplit;
}

int ndc_bias_act(const void *z, const float *bias, const void *residual, void *y, int64_t batch,
                 int64_t channels, int64_t n, int act, int dtype, void *stream)
{
    if (!z || !y) return NDC_ERR_NULL;
    int st = bias_act_check(batch, channels, n, act, dtype);
    if (st) return st;
    int nsplit;
    long long chunk;
    rownorm_split(batch * channels, n, nsplit, chunk);
    const int esz = dtype == NDC_BF16 ? 2 : 4;
    const bool vec = n % (16 / esz) == 0 && aligned16(z) && aligned16(y) && (!residual || aligned16(residual));
    return ndc::Backend::bias_act(z, bias, residual, y, batch * channels, (int)channels, n, nsplit, chunk, act,
                                  esz, vec, stream);
}

int ndc_bias_act_backward(const void *gy, const void *z, const float *bias, void *gz, float *gpart,
                          int64_t batch, int64_t channels, int64_t n, int act, int dtype, void *stream)
{
    if (!gy || !z || !gz) return NDC_ERR_NULL;
    int st = bias_act_check(batch, channels, n, act, dtype);
    if (st) return st;
    if (act == NDC_ACT_NONE) return NDC_ERR_GEOMETRY;   // gz = gy: nothing to compute
    int nsplit;
    long long chunk;
    rownorm_split(batch * channels, n, nsplit, chunk);
    const int esz = dtype == NDC_BF16 ? 2 : 4;
    const bool vec = n % (16 / esz) == 0 && aligned16(gy) && aligned16(z) && aligned16(gz);
    return ndc::Backend::bias_act_backward(gy, z, bias, gz, gpart, batch * channels, (int)channels, n, nsplit,
                                           chunk, act, esz, vec, stream);
}

// ---- streaming GEMM of the 1x1 projections (ndc_pwgemm.h)

int ndc_pointwise_gemm_supported(int64_t cin, int64_t cout, int64_t n, int dtype)
{
    if (dtype != NDC_BF16) return 0;
    // up to 256 input channels held whole in registers, any width of output; or many input
    // channels in chunks of 64 with the accumulators of at most 128 output channels
    const bool whole = cin == 64 || cin == 128 || cin == 256;
    const bool deep = cin > 256 && cin % 64 == 0 && cin <= 4096 && cout <= 128;
    if (!whole && !deep) return 0;
    if (cout < 32 || cout % 32 || cout > 4096) return 0;
    if (cin * cout * 2 > 128 * 1024) return 0;        // the packed weights stay in LDS,
    if (cin * cout * 2 + cout * 36 > 160 * 1024) return 0;   // with the bias and eight rows of sums
    if (n < 64 || n % 64) return 0;
    return 1;
}

size_t ndc_pointwise_weight_bytes(int64_t cin, int64_t cout)
{
    return cin > 0 && cout > 0 ? (size_t)cin * (size_t)cout * 2 : 0;
}

int ndc_pointwise_pack(const void *w, int w_dtype, int transposed, void *wfrag, int64_t cin, int64_t cout,
                       void *stream)
{
    if (!w || !wfrag) return NDC_ERR_NULL;
    if (w_dtype != NDC_F32 && w_dtype != NDC_BF16) return NDC_ERR_DTYPE;
    if (cin < 16 || cin % 16 || cout < 32 || cout % 32 || cin > 4096 || cout > 4096) return NDC_ERR_GEOMETRY;
    if ((uintptr_t)wfrag & 15u) return NDC_ERR_WORKSPACE;
    return ndc::Backend::pwgemm_pack(w, w_dtype == NDC_BF16, transposed != 0, wfrag, (int)cout, (int)cin, stream);
}

int ndc_pointwise_gemm(const void *x, const void *wfrag, const float *bias, const void *residual, void *y,
                       void *zkeep, int64_t batch, int64_t cin, int64_t cout, int64_t n, int act, int dtype,
                       void *stream)
{
    if (!x || !wfrag || !y) return NDC_ERR_NULL;
    if (dtype != NDC_BF16) return NDC_ERR_DTYPE;
    if (batch < 1 || act < NDC_ACT_NONE || act > NDC_ACT_GELU) return NDC_ERR_GEOMETRY;
    if (!ndc_pointwise_gemm_supported(cin, cout, n, dtype)) return NDC_ERR_GEOMETRY;
    if ((long double)batch * (cin > cout ? cin : cout) * n > 9.0e15L) return NDC_ERR_GEOMETRY;
    if (batch * (n / 64) > 0x7fffff00LL || n > 0x3fffffffLL) return NDC_ERR_GEOMETRY;   // 32-bit tile count and lane offsets
    // word accesses on voxel pairs, 16-byte reads of the weights
    if (((uintptr_t)x & 3u) || ((uintptr_t)y & 3u) || (residual && ((uintptr_t)residual & 3u)) ||
        (zkeep && ((uintptr_t)zkeep & 3u)) || ((uintptr_t)wfrag & 15u) || (bias && ((uintptr_t)bias & 3u)))
        return NDC_ERR_WORKSPACE;
    if (y == x || zkeep == x || (zkeep && zkeep == y)) return NDC_ERR_GEOMETRY;
    if (cin > 256 && (act != NDC_ACT_NONE || zkeep)) return NDC_ERR_GEOMETRY;   // see the header
    if (act == NDC_ACT_NONE && zkeep) return NDC_ERR_GEOMETRY;   // without an activation y - bias is the product
    return ndc::Backend::pwgemm(x, wfrag, bias, residual, y, zkeep, nullptr, nullptr, batch, (int)cin, (int)cout, n, act,
                                stream);
}

int ndc_pointwise_gemm_masked(const void *x, const void *wfrag, const float *bias, const void *residual,
                              const void *mask, void *y, int64_t batch, int64_t cin, int64_t cout, int64_t n,
                              int dtype, void *stream)
{
    if (!x || !wfrag || !y || !mask) return NDC_ERR_NULL;
    if (dtype != NDC_BF16) return NDC_ERR_DTYPE;
    if (batch < 1 || !ndc_pointwise_gemm_supported(cin, cout, n, dtype)) return NDC_ERR_GEOMETRY;
    if ((long double)batch * (cin > cout ? cin : cout) * n > 9.0e15L) return NDC_ERR_GEOMETRY;
    if (batch * (n / 64) > 0x7fffff00LL || n > 0x3fffffffLL) return NDC_ERR_GEOMETRY;
    if (((uintptr_t)x & 3u) || ((uintptr_t)y & 3u) || ((uintptr_t)mask & 3u) || (residual && ((uintptr_t)residual & 3u)) ||
        ((uintptr_t)wfrag & 15u) || (bias && ((uintptr_t)bias & 3u)))
        return NDC_ERR_WORKSPACE;
    if (y == x || y == mask) return NDC_ERR_GEOMETRY;
    return ndc::Backend::pwgemm(x, wfrag, bias, residual, y, nullptr, nullptr, mask, batch, (int)cin, (int)cout, n, 5, stream);
}

int64_t ndc_pointwise_gemm_parts(void)
{
    return 4096;
}

int ndc_pointwise_gemm_actgrad(const void *gy, const void *wfrag, const float *bias, const void *z, void *gz,
                               float *gpart, int64_t batch, int64_t cin, int64_t cout, int64_t n, int act,
                               int dtype, void *stream)
{
    if (!gy || !wfrag || !z || !gz) return NDC_ERR_NULL;
    if (dtype != NDC_BF16) return NDC_ERR_DTYPE;
    if (batch < 1 || (act != NDC_ACT_RELU && act != NDC_ACT_GELU)) return NDC_ERR_GEOMETRY;
    if (!ndc_pointwise_gemm_supported(cin, cout, n, dtype) || cin > 256) return NDC_ERR_GEOMETRY;
    if ((long double)batch * (cin > cout ? cin : cout) * n > 9.0e15L) return NDC_ERR_GEOMETRY;
    if (batch * (n / 64) > 0x7fffff00LL || n > 0x3fffffffLL) return NDC_ERR_GEOMETRY;
    if (((uintptr_t)gy & 3u) || ((uintptr_t)gz & 3u) || ((uintptr_t)z & 3u) || ((uintptr_t)wfrag & 15u) ||
        (bias && ((uintptr_t)bias & 3u)) || (gpart && ((uintptr_t)gpart & 3u)))
        return NDC_ERR_WORKSPACE;
    if (gz == gy || gz == z) return NDC_ERR_GEOMETRY;
    return ndc::Backend::pwgemm(gy, wfrag, bias, z, gz, nullptr, gpart, nullptr, batch, (int)cin, (int)cout, n, act + 2, stream);
}

static int chnorm_check(long long B, long long C, long long n, int dtype)
{
    if (dtype != NDC_F32 && dtype != NDC_BF16) return NDC_ERR_DTYPE;
    if (B < 1 || C < 1 || C > 0x7fffffffLL || n < 1 || (long double)B * C * n > 9.0e15L) return NDC_ERR_GEOMETRY;
    return NDC_OK;
}

// 16-byte accesses (8 or 4 voxels per thread) where that still leaves a few hundred workgroups;
// on small grids one voxel per thread, so that the launch spreads over the chip
static bool chnorm_wide(long long batch, long long n, int esz)
{
    return n % (16 / esz) == 0 && batch * ndc::Backend::chnorm_blocks(n, esz, true) >= 256;
}

int64_t ndc_chnorm_parts(int64_t batch, int64_t n, int dtype)
{
    if (batch < 1 || n < 1 || (dtype != NDC_F32 && dtype != NDC_BF16)) return 0;
    const int esz = dtype == NDC_BF16 ? 2 : 4;
    // (the count for the access width the entry points use when the buffers are aligned; an
    // unaligned call where the wide form applies needs more rows and is refused)
    return batch * ndc::Backend::chnorm_blocks(n, esz, chnorm_wide(batch, n, esz)) * ndc::Backend::kChnormWaves;
}

int ndc_chnorm_forward(const void *x, const float *weight, const float *bias, void *y, float *stats,
                       int64_t batch, int64_t channels, int64_t n, int dtype, float eps, void *stream)
{
    if (!x || !y || !stats) return NDC_ERR_NULL;
    int st = chnorm_check(batch, channels, n, dtype);
    if (st) return st;
    if (x == (const void *)y || !(eps >= 0.f)) return NDC_ERR_GEOMETRY;
    const int esz = dtype == NDC_BF16 ? 2 : 4;
    const bool vec = chnorm_wide(batch, n, esz) && aligned16(x) && aligned16(y);
    st = ndc::Backend::chnorm(false, nullptr, x, stats, weight, bias, y, nullptr, batch, (int)channels, n, esz, vec,
                              eps, stream);
    return st == -2 ? (int)NDC_ERR_GEOMETRY : st;
}

int ndc_chnorm_backward(const void *gy, const void *x, const float *stats, const float *weight, void *gx,
                        float *partial, int64_t batch, int64_t channels, int64_t n, int dtype, void *stream)
{
    if (!gy || !x || !stats || !gx) return NDC_ERR_NULL;
    int st = chnorm_check(batch, channels, n, dtype);
    if (st) return st;
    if (gx == x) return NDC_ERR_GEOMETRY;
    const int esz = dtype == NDC_BF16 ? 2 : 4;
    const bool fits = chnorm_wide(batch, n, esz);
    const bool vec = fits && aligned16(gy) && aligned16(x) && aligned16(gx);
    // the partial rows are laid out for the path ndc_chnorm_parts counted
    if (partial && fits && !vec) return NDC_ERR_WORKSPACE;
    st = ndc::Backend::chnorm(true, gy, x, stats, weight, nullptr, gx, partial, batch, (int)channels, n, esz, vec,
                              0.f, stream);
    return st == -2 ? (int)NDC_ERR_GEOMETRY : st;
}

int ndc_row_sums(const void *x, float *partial, int64_t rows, int64_t n, int dtype, void *stream)
{
    if (!x || !partial) return NDC_ERR_NULL;
    int st = rownorm_check(rows, n, dtype);
    if (st) return st;
    int nsplit;
    long long chunk;
    rownorm_split(rows, n, nsplit, chunk);
    const int esz = dtype == NDC_BF16 ? 2 : 4;
    const bool vec = n % (16 / esz) == 0 && aligned16(x);
    return ndc::Backend::row_sums(x, partial, rows, n, nsplit, chunk, esz, vec, stream);
}

int ndc_regroup(const void *src, void *dst, const float *bias, int64_t rows, int64_t channels, int64_t D,
                 int64_t H, int64_t W, int depth2, int dtype, int to_channels, void *stream)
{
    if (!src || !dst) return NDC_ERR_NULL;
    if (dtype != NDC_F32 && dtype != NDC_BF16) return NDC_ERR_DTYPE;
    const int esz = dtype == NDC_BF16 ? 2 : 4;
    if (rows < 1 || channels < 1 || D < 1 || H < 2 || W < 2 || D > 0x3fffffff || H > 0x3fffffff ||
        W > 0x3fffffff || channels > 0x7fffffff || (long double)rows * D * H * W > 9.0e15L)
        return NDC_ERR_GEOMETRY;
    // even windows, whole 16-byte vectors per row, aligned buffers; a bias only on the way back
    if (H % 2 || W % (16 / esz) || (depth2 && D % 2) || src == dst || !aligned16(src) || !aligned16(dst) ||
        (bias && to_channels))
        return NDC_ERR_GEOMETRY;
    const int st = ndc::Backend::regroup2(src, dst, bias, rows, (int)channels, (int)D, (int)H, (int)W,
                                          depth2 ? 1 : 0, esz, to_channels ? 1 : 0, stream);
    return st == -2 ? (int)NDC_ERR_GEOMETRY : st;
}

int ndc_gconv(const ndc_geom *g, const void *in, const float *h, const float *bias, int adjoint,
              void *out, void *stream)
{
    using namespace ndc;
    KGeom q;
    int st = make_kgeom(g, q);
    if (st) return st;
    if (!in || !h || !out) return NDC_ERR_NULL;
    return g->dtype == NDC_F32
               ? direct_gconv<float, float>(q, (const float *)in, h, bias, adjoint, (float *)out,
                                            stream)
               : direct_gconv<bf16_t, bf16_t>(q, (const bf16_t *)in, h, bias, adjoint,
                                              (bf16_t *)out, stream);
}

}  // extern "C"
