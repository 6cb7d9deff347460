// Fused, LDS-tiled kernels of the NDC update for depthwise filters (m = 1).
//
// Work decomposition (all three kernels):
//   - one workgroup owns one (sample, channel) volume and a band of TH = S*RH output rows
//     over the FULL width W, and marches along the slowest spatial axis ("planes", k);
//   - lanes run along W (coalesced global traffic, conflict-free LDS rows); a thread owns
//     column `col` of row strip `strip` (RH consecutive rows);
//   - operands that are read with spatial neighbours live in LDS rings of a few planes
//     with zero halo columns / rows (so the tap loops carry no bounds checks); operands
//     that are only read at the thread's own position come straight from global memory;
//   - filter taps of the channel are wave-uniform and read through a uniform pointer
//     (scalar loads / SGPR operands); the tap loops are rolled over the source channel or
//     the tap plane so that only one slice of the filter is resident at a time.
//
//   A-type applications (1 -> SC channels: A(x), A(t1), A(gt1)) are gathered from the
//   rings; K-type applications (SC -> 1 channel: K(s), K(gn), K(gd)) are scattered plane by
//   plane into per-thread accumulators of the KD pending output planes, so each staged
//   value is read from LDS once per (row, tap-column) and reused for all tap planes.
//   The PH halo rows a band needs above and below are produced by the first 2*PH strips as
//   one extra row each (a wave-uniform branch), so no strip computes rows nobody reads.
//
// 2-D problems (D = 1) are run as (D', H', W') = (H, 1, W) with kernel (kH, 1, kW): the
// march then goes along H.
//
// Forward  (FwdKernel):  out = s (A(x)+eps) / (A(K(s))+eps), optional side output t1 = K(s)
// Backward pass 1 (Bwd1Kernel): gn = g s/d, gd = -gn n/d (never stored), gx = K(gn),
//          gt1 = K(gd) (scratch), and the two A-side filter-gradient terms
// Backward pass 2 (Bwd2Kernel): gz = [z+b>0] (g n/d + A(gt1)), gb, and the K-side
//          filter-gradient term
// The per-workgroup filter/bias partial sums are combined by a small deterministic
// reduction (no atomics).
#pragma once

#include "ndc_common.h"
#include "ndc_exec.h"

#if NDC_DEVICE_BUILD
#define NDC_ROLLED _Pragma("unroll 1")
#define NDC_UNROLL _Pragma("unroll")
#else
#define NDC_ROLLED
#define NDC_UNROLL
#endif

namespace ndc {
namespace fused {

// ------------------------------------------------------------------ launch shape

struct Tile {
    int S;       // row strips per workgroup
    int NT;      // threads per workgroup (multiple of 64, >= S*W)
    int TH;      // output rows per workgroup
    int ntile;   // row bands per volume
    int P;       // LDS row pitch in floats (W + 2*PW)
};

// the marching view of a problem: 2-D inputs march along H
struct March {
    int D, H, W, KD, KH, KW;
};

static inline March march_of(const KGeom &q)
{
    March m;
    if (q.D == 1 && q.kD == 1) {
        m.D = q.H;
        m.H = 1;
        m.W = q.W;
        m.KD = q.kH;
        m.KH = 1;
        m.KW = q.kW;
    } else {
        m.D = q.D;
        m.H = q.H;
        m.W = q.W;
        m.KD = q.kD;
        m.KH = q.kH;
        m.KW = q.kW;
    }
    return m;
}

static inline int round_up(int v, int a) { return (v + a - 1) / a * a; }

static const int kMaxThreads = 512;
static const int kMaxLdsBytes = 160 * 1024;

// S strips of RH rows; S >= 2*PH so that the halo rows fit the fixed per-thread bounds
static inline bool make_tile(const March &m, int RH, int target_threads, Tile &t)
{
    const int PH = m.KH / 2, PW = m.KW / 2;
    if (m.W > kMaxThreads) return false;
    int smin = PH > 0 ? 2 * PH : 1;
    int s = target_threads / m.W;
    const int srows = (m.H + RH - 1) / RH;
    if (s > srows) s = srows;
    if (s < smin) s = smin;
    if (s * m.W > kMaxThreads) return false;
    t.S = s;
    t.NT = round_up(s * m.W, 64);
    t.TH = s * RH;
    t.ntile = (m.H + t.TH - 1) / t.TH;
    t.P = m.W + 2 * PW;
    return true;
}

// ------------------------------------------------------------------ parameters

template <typename T> struct FwdParams {
    const T *x, *z;
    const float *h, *bias;
    T *out, *t1;
    int B, C, D, H, W;
    int relu;
    float eps;
    Tile t;
};

template <typename T> struct BwdParams {
    const T *x, *z, *t1, *gout;
    const float *h, *bias;
    T *gx, *gz;
    T *gt1;        // scratch (B, C, S): written by pass 1, read by pass 2
    float *part;   // per-workgroup partial sums, [nblocks][part_stride]
    int part_stride;
    int need_gh, need_gb;
    int B, C, D, H, W;
    int relu;
    float eps;
    Tile t;
};

struct BlockId {
    int b, c, r0;
};

NDC_HD BlockId decode_block(int block_id, int C, const Tile &t)
{
    BlockId id;
    const int tile = block_id % t.ntile;
    const int bc = block_id / t.ntile;
    id.b = bc / C;
    id.c = bc % C;
    id.r0 = tile * t.TH;
    return id;
}

NDC_HD int wrap(int v, int n)  // v mod n for v >= -n
{
    return (v + n) % n;
}

NDC_HD int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// Tile row of the extra halo row that strip `s` (< 2*PH) produces, in a tile whose row j
// is image row r0 - PH + j: the PH rows above the band, then the PH rows below it.
NDC_HD int halo_row(int s, int PH, int TH) { return s < PH ? s : TH + s; }

// One K-type pass over NR consecutive output rows: `base` addresses, in a staged plane of
// ONE source channel, the element (first output row, own column - PW); the input rows
// base .. base + NR + 2*PH - 1 feed the NR output rows, and every tap plane jd of the KD
// pending output planes.  w = taps of that source channel, (KD, KH, KW) order.
template <int KD, int KH, int KW, int NR, int STRIDE, class Exec>
NDC_D void k_rows(Exec &ex, int base, int P, UniformF w, float (*acc)[STRIDE], int r_off)
{
    NDC_UNROLL
    for (int q = 0; q < NR + KH - 1; ++q) {
        NDC_UNROLL
        for (int tw = 0; tw < KW; ++tw) {
            const float v = ex.ld(base + q * P + tw);
            NDC_UNROLL
            for (int th = 0; th < KH; ++th) {
                const int rr = q - th;
                if (rr < 0 || rr >= NR) continue;
                NDC_UNROLL
                for (int jd = 0; jd < KD; ++jd)
                    acc[jd][r_off + rr] += v * w[((KD - 1 - jd) * KH + th) * KW + tw];
            }
        }
    }
}

// =================================================================== forward

template <int KD_, int KH_, int KW_, int SC_, int RH_, typename T> struct FwdKernel {
    static constexpr int KD = KD_, KH = KH_, KW = KW_, SC = SC_, RH = RH_;
    static constexpr int PD = KD / 2, PH = KH / 2, PW = KW / 2, KT = KD * KH * KW;
    static constexpr int XT = PH > 0 ? 1 : 0;            // one extra halo row for strips < 2*PH
    static constexpr int RHK = RH + XT;
    static constexpr int NZR = RH + (PH > 0 ? 2 : 0);    // rows of s a thread stages
    static constexpr int NXR = RH + (PH > 0 ? 1 : 0);    // rows of x a thread stages
    static constexpr int XR = KD + 1;                    // x ring slots
    typedef FwdParams<T> Params;

    struct State {
        int strip, col, active;
        float t1acc[KD][RHK];
        float pz[SC][NZR];
        float px[NXR];
    };

    // tile rows: s has TH + 4*PH (row j = image r0 - 2*PH + j); x and t1 have TH + 2*PH
    // (row j = image r0 - PH + j)
    static NDC_HD int rows_s(int TH) { return TH + 4 * PH; }
    static NDC_HD int rows_x(int TH) { return TH + 2 * PH; }
    static NDC_HD int lds_floats(const Tile &t)
    {
        return (SC * rows_s(t.TH) + (XR + KD) * rows_x(t.TH)) * t.P;
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t);
        const int S = t.S, P = t.P, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RS = rows_s(TH), RX = rows_x(TH);
        const int off_s = 0, off_x = SC * RS * P, off_t = off_x + XR * RX * P;
        const int total = off_t + KD * RX * P;
        const long long plane = (long long)H * W;
        const long long cplane = (long long)D * plane;   // one channel volume
        const T *xg = p.x + ((long long)id.b * p.C + id.c) * cplane;
        const T *zg = p.z + ((long long)id.b * p.C + id.c) * SC * cplane;
        T *og = p.out + ((long long)id.b * p.C + id.c) * SC * cplane;
        T *t1g = p.t1 ? p.t1 + ((long long)id.b * p.C + id.c) * cplane : nullptr;
        UniformF hw = as_uniform(p.h + (long long)id.c * SC * KT);
        UniformF bias = as_uniform(p.bias ? p.bias + id.c * SC : nullptr);
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const int relu = p.relu;
        const float eps = p.eps;

        // global -> registers: plane k of s (bias / ReLU applied) and plane k - PD of x.
        // Rows outside the image read a clamped address and are zeroed by a select.
        auto load_plane = [&](State &st, int k) {
            if (!st.active) return;
            if (k < D) {
                const T *zk = zg + (long long)k * plane;
                NDC_UNROLL
                for (int n = 0; n < NZR; ++n) {
                    const int j = st.strip + n * S, row = r0 - 2 * PH + j;
                    const bool ok = j < RS && row >= 0 && row < H;
                    const int o = clampi(row, 0, H - 1) * W + st.col;
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        float v = Elem<T>::load(zk + i * cplane + o) + (bias ? bias[i] : 0.f);
                        if (relu) v = v > 0.f ? v : 0.f;
                        st.pz[i][n] = ok ? v : 0.f;
                    }
                }
            } else {
                NDC_UNROLL
                for (int n = 0; n < NZR; ++n)
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) st.pz[i][n] = 0.f;
            }
            const int kx = k - PD;
            if (kx >= 0 && kx < D) {
                const T *xk = xg + (long long)kx * plane;
                NDC_UNROLL
                for (int n = 0; n < NXR; ++n) {
                    const int j = st.strip + n * S, row = r0 - PH + j;
                    const bool ok = j < RX && row >= 0 && row < H;
                    const float v = Elem<T>::load(xk + clampi(row, 0, H - 1) * W + st.col);
                    st.px[n] = ok ? v : 0.f;
                }
            } else {
                NDC_UNROLL
                for (int n = 0; n < NXR; ++n) st.px[n] = 0.f;
            }
        };

        auto store_plane = [&](State &st, int k) {
            if (!st.active) return;
            NDC_UNROLL
            for (int n = 0; n < NZR; ++n) {
                const int j = st.strip + n * S;
                if (j < RS) {
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i)
                        ex.st_(off_s + (i * RS + j) * P + PW + st.col, st.pz[i][n]);
                }
            }
            const int slot = wrap((k - PD) % XR, XR);
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const int j = st.strip + n * S;
                if (j < RX) ex.st_(off_x + (slot * RX + j) * P + PW + st.col, st.px[n]);
            }
        };

        // ---- set-up: thread coordinates, zeroed accumulators, zeroed LDS (halo columns and
        //      never-staged rows stay zero for the whole march)
        ex.each([&](State &st, int tid) {
            st.strip = tid / W;
            st.col = tid - st.strip * W;
            st.active = st.strip < S;
            NDC_UNROLL
            for (int a = 0; a < KD; ++a)
                NDC_UNROLL
                for (int r = 0; r < RHK; ++r) st.t1acc[a][r] = 0.f;
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, 0);
        });
        ex.sync();

        for (int k = 0; k < D + 2 * PD; ++k) {
            ex.each([&](State &st, int) { store_plane(st, k); });
            ex.sync();

            // ---- K-scatter: plane k of s feeds the KD pending planes of t1
            ex.each([&](State &st, int) {
                if (!st.active) return;
                const bool extra = XT && st.strip < 2 * PH;
                const int jx = halo_row(st.strip, PH, TH);
                if (k < D) {
                    NDC_ROLLED
                    for (int i = 0; i < SC; ++i) {
                        UniformF wi = hw + i * KT;
                        const int sb = off_s + i * RS * P + st.col;
                        k_rows<KD, KH, KW, RH, RHK>(ex, sb + (PH + st.strip * RH) * P, P, wi, st.t1acc, 0);
                        if (extra) k_rows<KD, KH, KW, 1, RHK>(ex, sb + jx * P, P, wi, st.t1acc, RH);
                    }
                }
                // plane k - PD of t1 is complete: publish it (zero outside the volume)
                const int pf = k - PD;
                const bool inplane = pf >= 0 && pf < D;
                const int tb = off_t + wrap(pf % KD, KD) * RX * P + PW + st.col;
                NDC_UNROLL
                for (int r = 0; r < RHK; ++r) {
                    const bool mine = r < RH || extra;
                    const int j = r < RH ? PH + st.strip * RH + r : jx;
                    const int row = r0 - PH + j;
                    const bool live = inplane && row >= 0 && row < H;
                    const float v = live ? st.t1acc[0][r] : 0.f;
                    if (mine) ex.st_(tb + j * P, v);
                    if (r < RH && t1g && live)
                        Elem<T>::store(t1g + (long long)pf * plane + row * W + st.col, v);
                    NDC_UNROLL
                    for (int a = 0; a + 1 < KD; ++a) st.t1acc[a][r] = st.t1acc[a + 1][r];
                    st.t1acc[KD - 1][r] = 0.f;
                }
            });
            ex.sync();

            // ---- prefetch of the next plane, then A-gather + epilogue for plane k - 2*PD
            ex.each([&](State &st, int) {
                if (!st.active) return;
                load_plane(st, k + 1);
                const int j0 = k - 2 * PD;
                if (j0 < 0) return;
                // the thread's own source values: re-read from global (an L2 hit) rather
                // than carried in registers across 2*PD planes
                float sv[SC][RH];
                const T *zk = zg + (long long)j0 * plane;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    const int row = r0 + st.strip * RH + r;
                    const int o = clampi(row, 0, H - 1) * W + st.col;
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        float v = Elem<T>::load(zk + i * cplane + o) + (bias ? bias[i] : 0.f);
                        if (relu) v = v > 0.f ? v : 0.f;
                        sv[i][r] = v;
                    }
                }
                float an[SC][RH], ad[SC][RH];
                NDC_UNROLL
                for (int i = 0; i < SC; ++i)
                    NDC_UNROLL
                    for (int r = 0; r < RH; ++r) an[i][r] = ad[i][r] = 0.f;
                NDC_ROLLED
                for (int td = 0; td < KD; ++td) {
                    const int pl = j0 + PD - td;
                    const int ob = (st.strip * RH) * P + st.col + 2 * PW;
                    const int bx = off_x + wrap(pl % XR, XR) * RX * P + ob;
                    const int bt = off_t + wrap(pl % KD, KD) * RX * P + ob;
                    UniformF wt = hw + td * KH * KW;
                    NDC_UNROLL
                    for (int q = 0; q < RH + 2 * PH; ++q)
                        NDC_UNROLL
                        for (int tw = 0; tw < KW; ++tw) {
                            const float vx = ex.ld(bx + q * P - tw), vt = ex.ld(bt + q * P - tw);
                            NDC_UNROLL
                            for (int th = 0; th < KH; ++th) {
                                const int rr = q - 2 * PH + th;
                                if (rr < 0 || rr >= RH) continue;
                                NDC_UNROLL
                                for (int i = 0; i < SC; ++i) {
                                    const float wv = wt[i * KT + th * KW + tw];
                                    an[i][rr] += vx * wv;
                                    ad[i][rr] += vt * wv;
                                }
                            }
                        }
                }
                T *ok_ = og + (long long)j0 * plane;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    const int row = r0 + st.strip * RH + r;
                    if (row >= H) continue;
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        const float v = sv[i][r] * (an[i][r] + eps) * fast_rcp(ad[i][r] + eps);
                        Elem<T>::store(ok_ + i * cplane + row * W + st.col, v);
                    }
                }
            });
        }
    }
};

// =================================================================== backward, pass 1

template <int KD_, int KH_, int KW_, int SC_, int RH_, typename T> struct Bwd1Kernel {
    static constexpr int KD = KD_, KH = KH_, KW = KW_, SC = SC_, RH = RH_;
    static constexpr int PD = KD / 2, PH = KH / 2, PW = KW / 2, KT = KD * KH * KW;
    static constexpr int XT = PH > 0 ? 1 : 0;
    static constexpr int NXR = RH + (PH > 0 ? 2 : 0);   // rows of x/t1 a thread stages
    static constexpr int XR = KD + 1;
    static constexpr int NRED = SC * KT;
    typedef BwdParams<T> Params;

    struct State {
        int strip, col, active;
        float gacc[SC][KT];      // A-side filter-gradient terms
        float accx[KD][RH];      // pending planes of gx
        float acct[KD][RH];      // pending planes of gt1
        float px[NXR], pt[NXR];
    };

    // tile rows: x / t1 have TH + 4*PH (row j = image r0 - 2*PH + j); gn / gd have
    // TH + 2*PH (row j = image r0 - PH + j)
    static NDC_HD int rows_x(int TH) { return TH + 4 * PH; }
    static NDC_HD int rows_g(int TH) { return TH + 2 * PH; }
    static NDC_HD int lds_floats(const Tile &t)
    {
        const int main_ = (2 * XR * rows_x(t.TH) + 2 * SC * rows_g(t.TH)) * t.P;
        const int red = (t.NT / 64) * NRED;
        return main_ > red ? main_ : red;
    }

    // n, d (numerator / denominator sums) of NR rows whose first x/t1 tile row is `base`
    template <int NR, class Exec>
    static NDC_D void gather_nd(Exec &ex, int bx, int bt, int P, UniformF wt,
                                float (&an)[SC][NR], float (&ad)[SC][NR])
    {
        NDC_UNROLL
        for (int q = 0; q < NR + 2 * PH; ++q)
            NDC_UNROLL
            for (int tw = 0; tw < KW; ++tw) {
                const float vx = ex.ld(bx + q * P - tw), vt = ex.ld(bt + q * P - tw);
                NDC_UNROLL
                for (int th = 0; th < KH; ++th) {
                    const int rr = q - 2 * PH + th;
                    if (rr < 0 || rr >= NR) continue;
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        const float wv = wt[i * KT + th * KW + tw];
                        an[i][rr] += vx * wv;
                        ad[i][rr] += vt * wv;
                    }
                }
            }
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t);
        const int S = t.S, P = t.P, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RX = rows_x(TH), RG = rows_g(TH);
        const int off_x = 0, off_t = XR * RX * P, off_g = 2 * XR * RX * P;
        const int total = off_g + 2 * SC * RG * P;
        const long long plane = (long long)H * W;
        const long long cplane = (long long)D * plane;
        const long long cbase = ((long long)id.b * p.C + id.c) * cplane;
        const T *xg = p.x + cbase, *t1g = p.t1 + cbase;
        const T *zg = p.z + cbase * SC, *gg = p.gout + cbase * SC;
        T *gxg = p.gx ? p.gx + cbase : nullptr;
        T *gt1g = p.gt1 + cbase;
        UniformF hw = as_uniform(p.h + (long long)id.c * SC * KT);
        UniformF bias = as_uniform(p.bias ? p.bias + id.c * SC : nullptr);
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const int relu = p.relu;
        const float eps = p.eps;
        const int need_gh = p.need_gh;

        auto load_plane = [&](State &st, int k) {
            if (!st.active) return;
            if (k < D) {
                const long long ko = (long long)k * plane;
                NDC_UNROLL
                for (int n = 0; n < NXR; ++n) {
                    const int j = st.strip + n * S, row = r0 - 2 * PH + j;
                    const bool ok = j < RX && row >= 0 && row < H;
                    const long long o = ko + clampi(row, 0, H - 1) * W + st.col;
                    const float vx = Elem<T>::load(xg + o), vt = Elem<T>::load(t1g + o);
                    st.px[n] = ok ? vx : 0.f;
                    st.pt[n] = ok ? vt : 0.f;
                }
            } else {
                NDC_UNROLL
                for (int n = 0; n < NXR; ++n) st.px[n] = st.pt[n] = 0.f;
            }
        };
        auto store_plane = [&](State &st, int k) {
            if (!st.active) return;
            const int slot = wrap(k % XR, XR);
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const int j = st.strip + n * S;
                if (j < RX) {
                    ex.st_(off_x + (slot * RX + j) * P + PW + st.col, st.px[n]);
                    ex.st_(off_t + (slot * RX + j) * P + PW + st.col, st.pt[n]);
                }
            }
        };

        // gn, gd of NR rows starting at gn/gd tile row j; published to LDS; returned in an/ad
        auto gn_gd_rows = [&](State &st, int j1, int j, auto nr_tag, float (&an)[SC][decltype(nr_tag)::value],
                              float (&ad)[SC][decltype(nr_tag)::value]) {
            constexpr int NR = decltype(nr_tag)::value;
            float sv[SC][NR], gv[SC][NR];
            const long long ko = (long long)j1 * plane;
            NDC_UNROLL
            for (int r = 0; r < NR; ++r) {
                const int row = r0 - PH + j + r;
                const bool ok = row >= 0 && row < H;
                const long long o = ko + clampi(row, 0, H - 1) * W + st.col;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    float s = Elem<T>::load(zg + i * cplane + o) + (bias ? bias[i] : 0.f);
                    if (relu) s = s > 0.f ? s : 0.f;
                    const float g = Elem<T>::load(gg + i * cplane + o);
                    sv[i][r] = s;
                    gv[i][r] = ok ? g : 0.f;
                }
            }
            NDC_UNROLL
            for (int i = 0; i < SC; ++i)
                NDC_UNROLL
                for (int r = 0; r < NR; ++r) an[i][r] = ad[i][r] = 0.f;
            NDC_ROLLED
            for (int td = 0; td < KD; ++td) {
                const int slot = wrap((j1 + PD - td) % XR, XR);
                const int ob = (slot * RX + j) * P + st.col + 2 * PW;
                gather_nd<NR>(ex, off_x + ob, off_t + ob, P, hw + td * KH * KW, an, ad);
            }
            NDC_UNROLL
            for (int r = 0; r < NR; ++r)
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    const float inv = fast_rcp(ad[i][r] + eps);
                    const float gn = gv[i][r] * sv[i][r] * inv;
                    const float gd = -(gn * (an[i][r] + eps)) * inv;
                    ex.st_(off_g + (i * RG + j + r) * P + PW + st.col, gn);
                    ex.st_(off_g + ((SC + i) * RG + j + r) * P + PW + st.col, gd);
                    an[i][r] = gn;
                    ad[i][r] = gd;
                }
        };

        ex.each([&](State &st, int tid) {
            st.strip = tid / W;
            st.col = tid - st.strip * W;
            st.active = st.strip < S;
            NDC_UNROLL
            for (int i = 0; i < SC; ++i)
                NDC_UNROLL
                for (int a = 0; a < KT; ++a) st.gacc[i][a] = 0.f;
            NDC_UNROLL
            for (int a = 0; a < KD; ++a)
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) st.accx[a][r] = st.acct[a][r] = 0.f;
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, 0);
        });
        ex.sync();

        for (int k = 0; k < D + 2 * PD; ++k) {
            ex.each([&](State &st, int) { store_plane(st, k); });
            ex.sync();

            // ---- gather: gn, gd of plane k - PD on the band plus PH halo rows each side
            const int j1 = k - PD;
            const bool live1 = j1 >= 0 && j1 < D;
            ex.each([&](State &st, int) {
                if (!st.active || !live1) return;
                {
                    float an[SC][RH], ad[SC][RH];
                    const int j = PH + st.strip * RH;
                    gn_gd_rows(st, j1, j, IntTag<RH>(), an, ad);
                    if (need_gh) {
                        // own rows: A-side filter-gradient terms, re-reading the x / t1 windows
                        NDC_UNROLL
                        for (int td = 0; td < KD; ++td) {
                            const int slot = wrap((j1 + PD - td) % XR, XR);
                            const int ob = (slot * RX + j) * P + st.col + 2 * PW;
                            NDC_UNROLL
                            for (int q = 0; q < RH + 2 * PH; ++q)
                                NDC_UNROLL
                                for (int tw = 0; tw < KW; ++tw) {
                                    const float vx = ex.ld(off_x + ob + q * P - tw);
                                    const float vt = ex.ld(off_t + ob + q * P - tw);
                                    NDC_UNROLL
                                    for (int th = 0; th < KH; ++th) {
                                        const int rr = q - 2 * PH + th;
                                        if (rr < 0 || rr >= RH) continue;
                                        NDC_UNROLL
                                        for (int i = 0; i < SC; ++i)
                                            st.gacc[i][(td * KH + th) * KW + tw] +=
                                                an[i][rr] * vx + ad[i][rr] * vt;
                                    }
                                }
                        }
                    }
                }
                if (XT && st.strip < 2 * PH) {
                    float an[SC][1], ad[SC][1];
                    gn_gd_rows(st, j1, halo_row(st.strip, PH, TH), IntTag<1>(), an, ad);
                }
            });
            ex.sync();

            // ---- prefetch, then scatter: plane k - PD of gn/gd feeds pending planes of gx / gt1
            ex.each([&](State &st, int) {
                if (!st.active) return;
                load_plane(st, k + 1);
                if (live1) {
                    NDC_ROLLED
                    for (int i = 0; i < SC; ++i) {
                        UniformF wi = hw + i * KT;
                        const int gb_ = off_g + (st.strip * RH) * P + st.col;
                        k_rows<KD, KH, KW, RH, RH>(ex, gb_ + i * RG * P, P, wi, st.accx, 0);
                        k_rows<KD, KH, KW, RH, RH>(ex, gb_ + (SC + i) * RG * P, P, wi, st.acct, 0);
                    }
                }
                const int pf = k - 2 * PD;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    const int row = r0 + st.strip * RH + r;
                    if (pf >= 0 && row < H) {
                        const long long o = (long long)pf * plane + row * W + st.col;
                        if (gxg) Elem<T>::store(gxg + o, st.accx[0][r]);
                        Elem<T>::store(gt1g + o, st.acct[0][r]);
                    }
                    NDC_UNROLL
                    for (int a = 0; a + 1 < KD; ++a) {
                        st.accx[a][r] = st.accx[a + 1][r];
                        st.acct[a][r] = st.acct[a + 1][r];
                    }
                    st.accx[KD - 1][r] = 0.f;
                    st.acct[KD - 1][r] = 0.f;
                }
            });
        }

        if (need_gh) {
            float *dst = p.part + (long long)block_id * p.part_stride;
            ex.template block_reduce<NRED>(
                [](State &st, int i) { return st.gacc[i / KT][i % KT]; },
                [&](int i, float v) { dst[i] = v; });
        }
    }
};

// =================================================================== backward, pass 2

template <int KD_, int KH_, int KW_, int SC_, int RH_, typename T> struct Bwd2Kernel {
    static constexpr int KD = KD_, KH = KH_, KW = KW_, SC = SC_, RH = RH_;
    static constexpr int PD = KD / 2, PH = KH / 2, PW = KW / 2, KT = KD * KH * KW;
    static constexpr int NXR = RH + (PH > 0 ? 1 : 0);
    static constexpr int XR = KD + 1;
    static constexpr int NRED = SC * KT + SC;
    typedef BwdParams<T> Params;

    struct State {
        int strip, col, active;
        float gacc[SC][KT];   // K-side filter-gradient term
        float gbacc[SC];
        float px[NXR], pt[NXR], pg[NXR];
    };

    static NDC_HD int rows_x(int TH) { return TH + 2 * PH; }
    static NDC_HD int lds_floats(const Tile &t)
    {
        const int main_ = 3 * XR * rows_x(t.TH) * t.P;
        const int red = (t.NT / 64) * NRED;
        return main_ > red ? main_ : red;
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t);
        const int S = t.S, P = t.P, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RX = rows_x(TH);
        const int off_x = 0, off_t = XR * RX * P, off_g = 2 * XR * RX * P;
        const int total = 3 * XR * RX * P;
        const long long plane = (long long)H * W;
        const long long cplane = (long long)D * plane;
        const long long cbase = ((long long)id.b * p.C + id.c) * cplane;
        const T *xg = p.x + cbase, *t1g = p.t1 + cbase, *gt1g = p.gt1 + cbase;
        const T *zg = p.z + cbase * SC, *gg = p.gout + cbase * SC;
        T *gzg = p.gz ? p.gz + cbase * SC : nullptr;
        UniformF hw = as_uniform(p.h + (long long)id.c * SC * KT);
        UniformF bias = as_uniform(p.bias ? p.bias + id.c * SC : nullptr);
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const int relu = p.relu;
        const float eps = p.eps;
        const int need_gh = p.need_gh;

        auto load_plane = [&](State &st, int k) {
            if (!st.active) return;
            if (k < D) {
                const long long ko = (long long)k * plane;
                NDC_UNROLL
                for (int n = 0; n < NXR; ++n) {
                    const int j = st.strip + n * S, row = r0 - PH + j;
                    const bool ok = j < RX && row >= 0 && row < H;
                    const long long o = ko + clampi(row, 0, H - 1) * W + st.col;
                    const float vx = Elem<T>::load(xg + o), vt = Elem<T>::load(t1g + o),
                                vg = Elem<T>::load(gt1g + o);
                    st.px[n] = ok ? vx : 0.f;
                    st.pt[n] = ok ? vt : 0.f;
                    st.pg[n] = ok ? vg : 0.f;
                }
            } else {
                NDC_UNROLL
                for (int n = 0; n < NXR; ++n) st.px[n] = st.pt[n] = st.pg[n] = 0.f;
            }
        };
        auto store_plane = [&](State &st, int k) {
            if (!st.active) return;
            const int slot = wrap(k % XR, XR);
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const int j = st.strip + n * S;
                if (j < RX) {
                    const int o = (slot * RX + j) * P + PW + st.col;
                    ex.st_(off_x + o, st.px[n]);
                    ex.st_(off_t + o, st.pt[n]);
                    ex.st_(off_g + o, st.pg[n]);
                }
            }
        };

        ex.each([&](State &st, int tid) {
            st.strip = tid / W;
            st.col = tid - st.strip * W;
            st.active = st.strip < S;
            NDC_UNROLL
            for (int i = 0; i < SC; ++i) {
                st.gbacc[i] = 0.f;
                NDC_UNROLL
                for (int a = 0; a < KT; ++a) st.gacc[i][a] = 0.f;
            }
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, 0);
        });
        ex.sync();

        for (int k = 0; k < D + PD; ++k) {
            ex.each([&](State &st, int) { store_plane(st, k); });
            ex.sync();

            const int j0 = k - PD;
            ex.each([&](State &st, int) {
                if (!st.active) return;
                load_plane(st, k + 1);
                if (j0 < 0) return;
                float sv[SC][RH], gv[SC][RH];
                const long long ko = (long long)j0 * plane;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    const int row = r0 + st.strip * RH + r;
                    const bool ok = row < H;
                    const long long o = ko + clampi(row, 0, H - 1) * W + st.col;
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        // s <= 0 marks "masked" (ReLU inactive); with relu off nothing is masked
                        float s = Elem<T>::load(zg + i * cplane + o) + (bias ? bias[i] : 0.f);
                        const float g = Elem<T>::load(gg + i * cplane + o);
                        if (relu) s = s > 0.f ? s : 0.f;
                        sv[i][r] = ok ? s : 0.f;
                        gv[i][r] = ok ? g : 0.f;
                    }
                }
                float an[SC][RH], ad[SC][RH], ag[SC][RH];
                NDC_UNROLL
                for (int i = 0; i < SC; ++i)
                    NDC_UNROLL
                    for (int r = 0; r < RH; ++r) an[i][r] = ad[i][r] = ag[i][r] = 0.f;
                NDC_UNROLL
                for (int td = 0; td < KD; ++td) {
                    const int slot = wrap((j0 + PD - td) % XR, XR);
                    const int ob = (slot * RX + st.strip * RH) * P + st.col + 2 * PW;
                    NDC_UNROLL
                    for (int q = 0; q < RH + 2 * PH; ++q)
                        NDC_UNROLL
                        for (int tw = 0; tw < KW; ++tw) {
                            const int o = ob + q * P - tw;
                            const float vx = ex.ld(off_x + o), vt = ex.ld(off_t + o), vg = ex.ld(off_g + o);
                            NDC_UNROLL
                            for (int th = 0; th < KH; ++th) {
                                const int rr = q - 2 * PH + th;
                                if (rr < 0 || rr >= RH) continue;
                                NDC_UNROLL
                                for (int i = 0; i < SC; ++i) {
                                    const float wv = hw[((i * KD + td) * KH + th) * KW + tw];
                                    an[i][rr] += vx * wv;
                                    ad[i][rr] += vt * wv;
                                    ag[i][rr] += vg * wv;
                                    if (need_gh) st.gacc[i][(td * KH + th) * KW + tw] += sv[i][rr] * vg;
                                }
                            }
                        }
                }
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    const int row = r0 + st.strip * RH + r;
                    if (row >= H) continue;
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        float v = gv[i][r] * (an[i][r] + eps) * fast_rcp(ad[i][r] + eps) + ag[i][r];
                        if (relu && !(sv[i][r] > 0.f)) v = 0.f;
                        st.gbacc[i] += v;
                        if (gzg) Elem<T>::store(gzg + i * cplane + ko + row * W + st.col, v);
                    }
                }
            });
        }

        if (p.need_gh || p.need_gb) {
            float *dst = p.part + (long long)block_id * p.part_stride;
            ex.template block_reduce<NRED>(
                [](State &st, int i) {
                    return i < SC * KT ? st.gacc[(i < SC * KT ? i : 0) / KT][i % KT]
                                       : st.gbacc[i >= SC * KT ? i - SC * KT : 0];
                },
                [&](int i, float v) { dst[i] = v; });
        }
    }
};

}  // namespace fused
}  // namespace ndc
